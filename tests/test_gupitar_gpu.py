"""The Gupitar decoder on the GPU against the plain implementation (tests/plain_gupitar.py): every mechanism alone
through its kernels, then the engine whole, token by token, in portions down to two tokens, in mixed batches on reused
pages and slots, long decoding, and greedy generation through the scheduler. The configurations are made here
(tests/gupitar_tiny.py) and differ from each other in every size."""
import io
import os

import numpy as np
import pytest
import torch

import plain_gupitar as plain
from gupitar_tiny import make_gupitar_folder
from replay_tools import collect, mixed, portions, prefill_then_decode, round_up, to_lines, whole

pytestmark = pytest.mark.gpu

F32_BOUND = 2e-5        # of the logits' scale: float32 against float64, sums in other orders
BF16_BOUND = 0.06       # of the logits' scale: what the format costs on these models; a fault costs far more
_models = {}


def model_for(tmp_path_factory, which):
    if which not in _models:
        folder = make_gupitar_folder(tmp_path_factory.mktemp(f"gupitar_{which}"), which)
        _models[which] = (folder, plain.read_config(folder), plain.read_safetensors(os.path.join(folder, "model.safetensors")))
    return _models[which]


def tokens_for(seed, count, vocab):
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def row_errors(got, want):
    difference = got - want
    difference = difference - difference.mean(-1, keepdims=True)
    return np.sqrt((difference ** 2).mean(-1)) / np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean())


def run_trace(folder, dtype, steps, out_dir, max_tokens, max_requests=4, **options):
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, max_requests=max_requests, **options)
    report = io.StringIO()
    replay(engine, io.StringIO(to_lines(steps)), str(out_dir), report)
    assert report.getvalue().split() == [word for step in steps for word in ("done", str(step["step"]))]
    engine.cache.check()
    assert not engine.cache.requests and all(free == group.pool.num_pages for free, group in zip(engine.cache.free_pages(), engine.cache.groups))
    return engine


_plain_logits = {}
CLOSE_CALL = 0.03       # a router's margin below which a bfloat16 engine may send the token to another expert


def plain_logits(config, weights, tokens, with_margins=False):
    key = (id(weights), tuple(tokens))
    if key not in _plain_logits:
        margins = []
        logits = plain.forward(config, weights, tokens, margins=margins)
        _plain_logits[key] = (logits, np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf))
    return _plain_logits[key] if with_margins else _plain_logits[key][0]


def decided(config, weights, tokens, places, dtype):
    """Which of the places a bfloat16 engine is held to: those where no router of the plain run had a close call."""
    if dtype == "float32":
        return np.ones(len(places), dtype=bool)
    margins = plain_logits(config, weights, tokens, with_margins=True)[1][places]
    assert len(places) < 40 or (margins >= CLOSE_CALL).mean() > 0.5      # the comparison still covers most of a long sequence
    return margins >= CLOSE_CALL


def within_bound(errors, dtype):
    """Float32: every position within the bound. bfloat16: a token that went to another expert than in the plain run
    (left out itself, ``decided``) also moves what the positions after it read from the cache and the state; nine in
    ten positions are held to the bound and none may be off by three times as much. What a fault of a kernel does
    (a window off by one, a lost state, a wrong page) shows in float32, where every position is held, and costs far
    more than this in either format."""
    if dtype == "float32" or len(errors) < 10:
        return errors.max() < (F32_BOUND if dtype == "float32" else BF16_BOUND)
    return np.quantile(errors, 0.9) < BF16_BOUND and errors.max() < 3 * BF16_BOUND


def check_against_plain(steps, out_dir, requests, config, weights, dtype):
    got = collect(steps, str(out_dir), config["vocab"])
    for rid, tokens in requests.items():
        want = plain_logits(config, weights, tokens)
        places = sorted(place for (request, place) in got if request == rid)
        assert places, f"no logits came back for {rid}"
        errors = row_errors(np.stack([got[(rid, place)] for place in places]), want[places])
        errors = np.where(decided(config, weights, tokens, places, dtype), errors, 0.0)
        assert within_bound(errors, dtype), f"{rid}: position {places[int(errors.argmax())]} is off by {errors.max():.3g} of the scale"


def device(array, dtype=torch.float32):
    return torch.as_tensor(np.asarray(array), dtype=dtype).cuda().contiguous()


def as_bf16(array):
    return torch.as_tensor(np.asarray(array), dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


# ---- mechanisms alone -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [64, 50, 7])
def test_norm_with_a_weight_around_zero(width):
    from microllm_rocm_amd.parts import PartSpec, Runtime, build_part
    rng = np.random.default_rng(width)
    x, delta, weight = rng.normal(size=(5, width)) * 3, rng.normal(size=(5, width)), as_bf16(rng.normal(size=width) * 0.3)
    norm = build_part("norm", PartSpec("rms_norm", {"size": width, "eps": 1e-5, "unit_offset": True}, {"weight": "w"}),
                      Runtime(torch.float32, torch.device("cuda")))
    norm.bind({"w": device(weight)})
    h = device(x)
    got = norm.forward(h, delta=device(delta), write_h=True).cpu().numpy()
    assert np.abs(got - plain.norm_around_zero(x + delta, weight, 1e-5)).max() < 1e-5
    assert np.abs(h.cpu().numpy() - (x + delta)).max() < 1e-6
    # a weight of zero is a gain of one, not of zero
    norm.bind({"w": device(np.zeros(width))})
    assert np.abs(norm.forward(device(x)).cpu().numpy() - plain.unit_rms(x, 1e-5)).max() < 1e-5


@pytest.mark.parametrize("q_rank,kv_rank,rot,tiled,dtype", [(24, 40, 8, False, torch.float32), (10, 18, 4, False, torch.float32),
                                                            (48, 224, 32, True, torch.bfloat16), (16, 36, 6, False, torch.bfloat16),
                                                            (24, 40, 8, True, torch.bfloat16)])
def test_latents_norm_rotation_and_page_write(q_rank, kv_rank, rot, tiled, dtype):
    """Both latents of tokens at far positions; the cached row through plain pages and through the tiled pages."""
    from microllm_rocm_amd.cache.layout import key_page_shape, key_rows, value_page_shape, value_rows
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(kv_rank)
    n, page_size, pages, base = 11, 16, 5, 300.0
    positions = np.array([0, 1, 2, 3, 1000, 1001, 5, 6, 7, 77777, 15])
    proj = rng.normal(size=(n, 3 + q_rank + kv_rank + rot)) * 2
    q_weight, kv_weight = rng.normal(size=q_rank) + 1, rng.normal(size=kv_rank) + 1
    slots = np.array([page_size * 3 + 15, page_size * 4, 0, 1, 2, -1, 20, 21, 22, 23, 40])
    inv_freq = device(base ** (-2.0 * np.arange(rot // 2) / rot), torch.float64)
    cos_sin = kernels.rope_table(device(positions, torch.int32), inv_freq)
    kwargs = {}
    if tiled:
        kwargs = dict(k_pages=torch.zeros(key_page_shape(pages, 1, page_size, kv_rank + rot), dtype=dtype, device="cuda"),
                      v_pages=torch.zeros(value_page_shape(pages, 1, page_size, kv_rank + rot), dtype=dtype, device="cuda"),
                      tiled_page_size=page_size)
    else:
        kwargs = dict(pages=torch.zeros((pages, page_size, kv_rank + rot), dtype=dtype, device="cuda"))
    cq = kernels.latent_prepare(device(proj), 3, q_rank, device(q_weight), 3 + q_rank, kv_rank, rot, device(kv_weight), 1e-5, cos_sin,
                                device(slots, torch.int32), dtype, **kwargs)
    bound = 1e-5 if dtype == torch.float32 else 0.03
    assert np.abs(cq.float().cpu().numpy() - plain.norm_plain(proj[:, 3:3 + q_rank], q_weight, 1e-5)).max() < bound * 4
    want = np.concatenate([plain.norm_plain(proj[:, 3 + q_rank:3 + q_rank + kv_rank], kv_weight, 1e-5),
                           plain.rotate_half(proj[:, 3 + q_rank + kv_rank:], positions, rot, base)], axis=1)
    if tiled:
        as_keys = key_rows(kwargs["k_pages"], kv_rank + rot)[:, 0].reshape(pages * page_size, -1).float().cpu().numpy()
        as_values = value_rows(kwargs["v_pages"], kv_rank + rot)[:, 0].reshape(pages * page_size, -1).float().cpu().numpy()
        assert np.array_equal(as_keys, as_values)
        stored = as_keys
    else:
        stored = kwargs["pages"].reshape(pages * page_size, -1).float().cpu().numpy()
    for row, slot in enumerate(slots):
        if slot >= 0:
            assert np.abs(stored[slot] - want[row]).max() < bound * 8, row
    untouched = np.ones(pages * page_size, dtype=bool)
    untouched[slots[slots >= 0]] = False
    assert np.abs(stored[untouched]).max() == 0.0      # a negative slot stores nothing, and nothing lands elsewhere


@pytest.mark.parametrize("types", [(torch.float32, torch.float32, torch.float32), (torch.float32, torch.bfloat16, torch.bfloat16),
                                   (torch.bfloat16, torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("n,heads,n_in,n_out", [(1, 1, 5, 3), (9, 3, 16, 40), (20, 2, 70, 130), (3, 2, 1500, 70)])
def test_product_per_head(types, n, heads, n_in, n_out):
    """Views with strides of their own on both sides, a gate, rows that do not fill a workgroup's tile."""
    from microllm_rocm_amd.ops import kernels
    x_type, w_type, out_type = types
    rng = np.random.default_rng(n_in)
    x = as_bf16(rng.normal(size=(n, heads, n_in + 3)))
    w = as_bf16(rng.normal(size=(heads, n_in, n_out)) * 0.3)
    gate = rng.normal(size=(n, heads * n_out + 2))
    want = np.einsum("nhi,hio->nho", x[:, :, :n_in], w)
    x_device = device(x, x_type)
    out = torch.zeros((n, heads, n_out + 5), dtype=out_type, device="cuda")
    kernels.head_product(x_device[:, :, :n_in], device(w, w_type), out[:, :, 2:2 + n_out])
    bound = 1e-5 if out_type == torch.float32 else 0.01
    assert np.abs(out[:, :, 2:2 + n_out].float().cpu().numpy() - want).max() < bound * max(1.0, np.abs(want).max())
    assert float(out[:, :, :2].abs().max()) == 0.0 and float(out[:, :, 2 + n_out:].abs().max()) == 0.0
    gate_device = device(gate)
    kernels.head_product(x_device[:, :, :n_in], device(w, w_type), out[:, :, 2:2 + n_out], gate=gate_device[:, :heads * n_out])
    gated = want * plain.sigmoid(gate[:, :heads * n_out]).reshape(n, heads, n_out)
    assert np.abs(out[:, :, 2:2 + n_out].float().cpu().numpy() - gated).max() < bound * max(1.0, np.abs(want).max())
    if x_type == torch.float32:       # a row's sums do not depend on the rows beside it, nor on which of the two kernels a step's size takes
        alone = torch.zeros((1, heads, n_out), dtype=out_type, device="cuda")
        kernels.head_product(x_device[n - 1:, :, :n_in], device(w, w_type), alone, gate=gate_device[n - 1:, :heads * n_out])
        assert torch.equal(alone[0], out[n - 1, :, 2:2 + n_out])
        many = torch.zeros((70, heads, n_out), dtype=out_type, device="cuda")
        kernels.head_product(x_device[n - 1:, :, :n_in].expand(70, heads, n_in), device(w, w_type), many)
        kernels.head_product(x_device[n - 1:, :, :n_in], device(w, w_type), alone)
        assert torch.equal(many[69], alone[0]) and torch.equal(many[0], alone[0])


def test_queries_are_folded_and_turned():
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(5)
    n, heads, dim, rot, rank, base = 7, 3, 10, 6, 12, 50.0
    positions = np.array([0, 1, 2, 500, 501, 9, 10])
    q = rng.normal(size=(n, heads, dim + rot))
    fold = rng.normal(size=(heads, dim, rank))
    cos_sin = kernels.rope_table(device(positions, torch.int32), device(base ** (-2.0 * np.arange(rot // 2) / rot), torch.float64))
    want = np.concatenate([np.einsum("nhd,hdr->nhr", q[:, :, :dim], fold), plain.rotate_half(q[:, :, dim:], positions, rot, base)], axis=2)
    q_device = device(q.reshape(n, -1))
    direct = torch.zeros((n, heads * (rank + rot)), device="cuda")
    kernels.head_product(q_device.view(n, heads, dim + rot)[:, :, :dim], device(fold), direct.view(n, heads, rank + rot)[:, :, :rank])
    kernels.latent_query(q_device, heads, dim, rot, rank, cos_sin, direct)
    assert np.abs(direct.cpu().numpy().reshape(n, heads, -1) - want).max() < 2e-5
    # the way of steps with many rows: the unrotated parts out, a batched product, the result joined in
    joined = torch.zeros_like(direct)
    flat = kernels.latent_query(q_device, heads, dim, rot, rank, cos_sin, joined, want_flat=True)
    assert np.abs(flat.cpu().numpy() - q[:, :, :dim].transpose(1, 0, 2)).max() < 1e-6
    kernels.latent_query(q_device, heads, dim, rot, rank, cos_sin, joined, folded=torch.bmm(flat, device(fold)))
    assert np.abs(joined.cpu().numpy().reshape(n, heads, -1) - want).max() < 2e-5


def test_heads_side_by_side_and_gated():
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(8)
    values, gate = as_bf16(rng.normal(size=(3, 11, 20))), rng.normal(size=(11, 70))
    want = values.transpose(1, 0, 2).reshape(11, 60)
    for dtype, bound in ((torch.float32, 1e-6), (torch.bfloat16, 0.02)):
        assert np.abs(kernels.gate_heads(device(values, dtype), None).float().cpu().numpy() - want).max() == 0.0
        got = kernels.gate_heads(device(values, dtype), device(gate)[:, 5:65]).float().cpu().numpy()
        assert np.abs(got - want * plain.sigmoid(gate[:, 5:65])).max() < bound


def attention_over_rows(q_full, rows, rank, window, scale, portions_of, mfma, page_size=16):
    """One request through the attention over cached rows, its pages scattered and out of order, in the given portions:
    through the kernel for plain pages (float32) or through the tiled pages and the MFMA kernels (bfloat16)."""
    from types import SimpleNamespace
    from microllm_rocm_amd.cache.layout import key_page_shape, value_page_shape, write_key_rows, write_value_rows
    from microllm_rocm_amd.ops import kernels
    from microllm_rocm_amd.parts.attention import QueryTilePlanner
    n, heads, width = q_full.shape
    rot = width - rank
    dtype = torch.bfloat16 if mfma else torch.float32
    blocks = -(-n // page_size)
    pages = [2 + 3 * block for block in reversed(range(blocks))]
    table = device([pages], torch.int32)
    count = 3 * blocks + 2
    filler = 0.0 if mfma else 1e4       # plain pages: what is not this request's must not count
    held = torch.full((count, 1, page_size, width), filler, dtype=dtype, device="cuda")
    if mfma:
        k_pages = torch.zeros(key_page_shape(count, 1, page_size, width), dtype=dtype, device="cuda")
        v_pages = torch.zeros(value_page_shape(count, 1, page_size, width), dtype=dtype, device="cuda")
    out = []
    first = 0
    for portion in portions_of:
        positions = np.arange(first, first + portion)
        slots = np.array([pages[p // page_size] * page_size + p % page_size for p in positions])
        held.view(-1, width)[device(slots, torch.int64)] = device(rows[positions], dtype)
        if mfma:        # (the page write has a test of its own; here the rows are placed through the layout's views)
            write_key_rows(k_pages, held)
            write_value_rows(v_pages, held)
        else:
            plain_pages = held.view(count, page_size, width)
        q = device(q_full[first:first + portion].reshape(portion, -1), dtype)
        seq_of_token, pos = device(np.zeros(portion), torch.int32), device(positions, torch.int32)
        if mfma:
            planner = QueryTilePlanner(window > 0)
            host = SimpleNamespace(counts=[portion], cu=np.array([0, portion]), starts=[first], totals=[first + portion],
                                   single_tokens_only=portion == 1, n_tokens=portion, n_seqs=1, page_size=page_size)
            ctx = SimpleNamespace(max_count=portion, planned_total=first + portion, max_total=first + portion, n_tokens=portion,
                                  seq_of_token=seq_of_token, positions=pos, fixed=False, host=host, tokens=pos, planned={})
            arrays, values = planner.plan(host)
            plan = SimpleNamespace(**values, **{name: device(array, torch.int32) for name, array in arrays.items()})
            ctx.plan_of = lambda _planner: plan
            view = SimpleNamespace(block_table=table, page_size=page_size)
            found = kernels.paged_attention(q, k_pages, v_pages, view, ctx, scale, window, heads, 1, width, planner=planner)
            out.append(found.view(portion, heads, width)[:, :, :rank].float().cpu().numpy())
        else:
            out.append(kernels.latent_attention(q, plain_pages, table, seq_of_token, pos, scale, window, heads, rank, rot).cpu().numpy())
        first += portion
    return np.concatenate(out)


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("window", [1, 15, 16, 17, 41, 64, 65, 0])
def test_window_edges_far_keys_and_first_tokens(mfma, window):
    """One key's score is made to stand out: the key just inside the window takes all the weight, the key just outside
    it none, wherever the edge falls in a page or a tile of keys; in a prompt, decoded, and in portions of two."""
    rng = np.random.default_rng(window)
    n, heads, rank, rot = 150, 2, 32, 16
    rows = as_bf16(rng.normal(size=(n, rank + rot)) * 0.1)
    q_full = as_bf16(rng.normal(size=(n, heads, rank + rot)) * 0.1)
    bound = 0.02 if mfma else 1e-4
    for portions_of in ([n], [n - 40] + [1] * 40, [2] * (n // 2), [1] * 5 + [n - 5]):
        want = plain.folded_attention(q_full, rows, rank, window, 1.0)
        got = attention_over_rows(q_full, rows, rank, window, 1.0, portions_of, mfma)
        assert np.abs(got - want).max() < bound, portions_of
    # the first tokens: position 0 sees itself alone
    assert np.abs(got[0] - rows[0, :rank]).max() < bound
    span = window if window else n
    for query in (n - 1, 100, 64, 16):
        for back in (span - 1, span):            # the oldest key still seen, and the first one no longer seen
            key = query - back
            if key < 0:
                continue
            sharp_rows, sharp_q = rows.copy(), q_full.copy()
            sharp_q[query, 0] = 0.0
            sharp_q[query, 0, 3] = 8.0
            sharp_rows[key, 3] = 8.0
            want = plain.folded_attention(sharp_q, sharp_rows, rank, window, 1.0)
            seen = back < span
            assert (np.abs(want[query, 0] - sharp_rows[key, :rank]).max() < 1e-6) == seen      # the plain run itself shows the edge
            for portions_of in ([query + 1], [query, 1]):       # the query as a prompt's last token, and decoded alone
                got = attention_over_rows(sharp_q[:query + 1], sharp_rows[:query + 1], rank, window, 1.0, portions_of, mfma)
                assert np.abs(got[query] - want[query]).max() < bound, (query, back, portions_of)


def test_recurrence_in_steps_with_carried_state():
    """Convolution, gates and the recurrence: two requests in one step, then continued one and two tokens at a time
    beside a third that starts, in slots that are not in order and hold what the last user left."""
    from microllm_rocm_amd.ops import kernels
    for width, blocks, taps in ((96, 3, 4), (70, 5, 2), (64, 1, 1), (130, 2, 3)):
        rng = np.random.default_rng(width)
        size = width // blocks
        lengths = {"a": 213, "b": 9, "c": 6}
        t = {"y.b": rng.normal(size=width), "x.b": rng.normal(size=width), "conv": rng.normal(size=(width, taps)),
             "conv.b": rng.normal(size=width), "ra": rng.normal(size=(blocks, size, size)) * 0.3, "ra.b": rng.normal(size=(blocks, size)),
             "ri": rng.normal(size=(blocks, size, size)) * 0.3, "ri.b": rng.normal(size=(blocks, size)), "lam": rng.normal(size=width)}
        rows = {name: rng.normal(size=(length, 2 * width)) for name, length in lengths.items()}

        def plain_run(proj):
            y = plain.gelu_tanh(proj[:, :width] + t["y.b"])
            u = plain.causal_conv(proj[:, width:] + t["x.b"], t["conv"], t["conv.b"])
            r, i = plain.block_gate(u, t["ra"], t["ra.b"]), plain.block_gate(u, t["ri"], t["ri.b"])
            a = np.exp(-8.0 * r * plain.softplus(t["lam"]))
            state, out = np.zeros(width), np.zeros_like(u)
            for step in range(proj.shape[0]):
                state = a[step] * state + np.sqrt(1.0 - a[step] ** 2) * i[step] * u[step]
                out[step] = state * y[step]
            return out

        want = {name: plain_run(proj) for name, proj in rows.items()}
        state = torch.full((6, width), 7.0, device="cuda")
        kept = torch.full((6, taps - 1, width), 7.0, device="cuda")
        slot_of = {"a": 4, "b": 1, "c": 5}
        got = {name: [] for name in rows}
        fed = {name: 0 for name in rows}
        gate_weight = device(np.concatenate([t["ra"].transpose(0, 2, 1), t["ri"].transpose(0, 2, 1)], axis=2))

        def step(portions_of):
            names = list(portions_of)
            for name in names:
                if fed[name] == 0:
                    state[slot_of[name]].zero_()
                    kept[slot_of[name]].zero_()
            proj = device(np.concatenate([rows[name][fed[name]:fed[name] + portions_of[name]] for name in names]))
            counts = [portions_of[name] for name in names]
            cu = device(np.concatenate([[0], np.cumsum(counts)]), torch.int32)
            seq_of_token = device(np.repeat(np.arange(len(names)), counts), torch.int32)
            slots = device([slot_of[name] for name in names], torch.int32)
            u = kernels.rglru_conv(proj, width, device(t["x.b"]), device(t["conv"]), device(t["conv.b"]), kept, seq_of_token, cu, slots)
            gates = torch.empty((proj.shape[0], blocks, 2 * size), device="cuda")
            kernels.head_product(u.view(-1, blocks, size), gate_weight, gates)
            arguments = (proj, width, device(t["x.b"]), 0, device(t["y.b"]), u, gates.view(-1, 2 * width), device(t["ra.b"].reshape(-1)),
                         device(t["ri.b"].reshape(-1)), device(t["lam"]), 8.0)
            state_before, kept_before = state.clone(), kept.clone()      # the walk in chunks must leave what the plain walk leaves
            in_chunks = kernels.rglru_scan(*arguments, state_before, kept_before, cu, slots, len(names), blocks, taps, torch.float32, chunked=True)
            out = kernels.rglru_scan(*arguments, state, kept, cu, slots, len(names), blocks, taps, torch.float32)
            assert float((in_chunks - out).abs().max()) < 2e-5 * max(1.0, float(out.abs().max()))
            assert float((state_before - state).abs().max()) < 2e-5 * max(1.0, float(state.abs().max())) and torch.equal(kept_before, kept)
            out = out.cpu().numpy()
            first = 0
            for name in names:
                got[name].append(out[first:first + portions_of[name]])
                first += portions_of[name]
                fed[name] += portions_of[name]

        step({"a": 200, "b": 2})
        step({"b": 1, "a": 1})
        step({"a": 2, "c": 4, "b": 1})
        for _ in range(5):
            step({"a": 1, "c": 1} if fed["c"] < lengths["c"] else {"a": 1})
        step({"b": 5, "a": 5})
        for name in rows:
            result = np.concatenate(got[name])
            assert result.shape[0] == lengths[name]
            assert np.abs(result - want[name]).max() < 3e-5 * max(1.0, np.abs(want[name]).max()), (width, name)
        assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0      # slots of no request were not touched


@pytest.mark.parametrize("experts,top,softmax,renormalize", [(6, 2, False, False), (3, 3, False, False), (12, 1, False, False),
                                                             (5, 2, True, True), (8, 4, True, False)])
def test_choice_of_experts(experts, top, softmax, renormalize):
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(experts)
    z = rng.normal(size=(37, experts + 1)) * 2
    z[3, :experts] = 0.25        # every score equal: the lowest indices win
    z[4, 1] = z[4, min(2, experts - 1)] = 5.0
    ids, weights, shared = kernels.moe_route(device(z), experts, top, softmax_scores=softmax, renormalize=renormalize, shared_at=experts)
    want_ids, want_weights = plain.choose_experts(z[:, :experts], top, softmax, renormalize)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    assert np.abs(weights.cpu().numpy() - want_weights).max() < 1e-6
    assert np.abs(shared.cpu().numpy() - plain.sigmoid(z[:, experts])).max() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("on_input", [True, False])
def test_experts_of_every_pair(dtype, on_input):
    """Each (token, choice) through its own expert; the weight on the expert's input is not the weight on its output."""
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(11)
    n, width, ff, experts, top = 13, 50, 36, 5, 2
    x = as_bf16(rng.normal(size=(n, width)))
    gate_up, down = as_bf16(rng.normal(size=(experts, 2 * ff, width)) * 0.2), as_bf16(rng.normal(size=(experts, width, ff)) * 0.2)
    ids = np.stack([rng.permutation(experts)[:top] for _ in range(n)])
    weights = rng.uniform(0.2, 1.5, size=(n, top))
    parts = kernels.moe_experts(device(x, dtype), device(ids, torch.int32), device(weights), device(gate_up, dtype), device(down, dtype),
                                on_input).cpu().numpy()
    for token in range(n):
        for choice in range(top):
            e, w = ids[token, choice], weights[token, choice]
            t = {"gate": gate_up[e, :ff], "up": gate_up[e, ff:], "down": down[e]}
            want = plain.gated_ff((w * x[token:token + 1]) if on_input else x[token:token + 1], t, "")[0] * (1.0 if on_input else w)
            bound = 1e-5 if dtype == torch.float32 else 0.03
            assert np.abs(parts[choice, token] - want).max() < bound * max(1.0, np.abs(want).max()), (token, choice)
    limit, kernels.MOE_PAIRS_A_LAUNCH = kernels.MOE_PAIRS_A_LAUNCH, 7        # a step of more pairs than a launch takes goes in several
    try:
        in_pieces = kernels.moe_experts(device(x, dtype), device(ids, torch.int32), device(weights), device(gate_up, dtype), device(down, dtype), on_input)
    finally:
        kernels.MOE_PAIRS_A_LAUNCH = limit
    assert np.array_equal(in_pieces.cpu().numpy(), parts)


@pytest.mark.parametrize("n,width,ff,experts,top", [(300, 64, 40, 6, 2), (70, 200, 136, 3, 3), (513, 96, 264, 16, 1), (5, 48, 8, 4, 2)])
def test_experts_in_tiles_of_sorted_rows(n, width, ff, experts, top):
    """The tiled kernels against the kernels that take a pair at a time (which the test above holds against the plain
    run): experts with no rows, with one, with more than a tile's; widths that do not fill the tiles."""
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(n)
    x = device(rng.normal(size=(n, width)), torch.bfloat16)
    gate_up = device(rng.normal(size=(experts, 2 * ff, width)) * 0.2, torch.bfloat16)
    down = device(rng.normal(size=(experts, width, ff)) * 0.2, torch.bfloat16)
    busy = rng.permutation(experts)[:max(top, experts - 2)]          # the other experts get no row at all
    ids = np.stack([rng.permutation(busy)[:top] for _ in range(n)])
    ids[0, 0] = busy[0]
    weights = device(rng.uniform(0.2, 1.5, size=(n, top)))
    for on_input in (True, False):
        one_by_one = kernels.moe_experts(x, device(ids, torch.int32), weights, gate_up, down, on_input, grouped=False)
        tiled = kernels.moe_experts(x, device(ids, torch.int32), weights, gate_up, down, on_input, grouped=True)
        scale = float(one_by_one.abs().max())
        assert float((tiled - one_by_one).abs().max()) < 0.02 * scale      # the intermediate is rounded to bfloat16 from sums in another order
        again = kernels.moe_experts(x[:n // 2 + 1], device(ids[:n // 2 + 1], torch.int32), weights[:n // 2 + 1], gate_up, down, on_input, grouped=True)
        assert torch.equal(again, tiled[:, :n // 2 + 1])      # a row does not depend on the rows beside it


# ---- the engine ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_decode_and_portions(tmp_path_factory, tmp_path, which, dtype):
    folder, config, weights = model_for(tmp_path_factory, which)
    requests = {"long": tokens_for(1, 150, config["vocab"]), "short": tokens_for(2, 37, config["vocab"]), "one": tokens_for(3, 1, config["vocab"])}
    run_trace(folder, dtype, whole(requests), tmp_path / "whole", max_tokens=256)
    check_against_plain(whole(requests), tmp_path / "whole", requests, config, weights, dtype)
    for rid, tail in (("long", 70), ("short", 34)):      # the decoded tokens cross pages' edges and pass every window but the widest
        steps = prefill_then_decode(rid, requests[rid], tail=tail)
        run_trace(folder, dtype, steps, tmp_path / f"decode_{rid}", max_tokens=round_up(len(requests[rid]), 64))
        check_against_plain(steps, tmp_path / f"decode_{rid}", {rid: requests[rid]}, config, weights, dtype)
    for sizes in ([2], [3, 16, 1, 2, 31], [64, 2, 17]):
        steps = portions("long", requests["long"], sizes)
        run_trace(folder, dtype, steps, tmp_path / f"portions_{sizes[0]}", max_tokens=192)
        check_against_plain(steps, tmp_path / f"portions_{sizes[0]}", {"long": requests["long"]}, config, weights, dtype)
    steps = portions("short", requests["short"], [1])       # from its first token on, one token a step
    run_trace(folder, dtype, steps, tmp_path / "one_by_one", max_tokens=64)
    check_against_plain(steps, tmp_path / "one_by_one", {"short": requests["short"]}, config, weights, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_mixed_batches_on_reused_pages_and_slots(tmp_path_factory, tmp_path, which, dtype):
    folder, config, weights = model_for(tmp_path_factory, which)
    lengths = [90, 41, 130, 2, 67, 25, 110, 58]
    requests = {f"r{index}": tokens_for(10 + index, length, config["vocab"]) for index, length in enumerate(lengths)}
    steps, peak = mixed(requests, seed=4, max_live=3, decode_tail=12, max_portion=23)
    engine = run_trace(folder, dtype, steps, tmp_path / "mixed", max_tokens=peak, max_requests=3)
    assert engine.cache.groups[0].pool.total_taken > engine.cache.groups[0].pool.num_pages      # pages were used again
    assert engine.cache.slots.total_taken > 3                                                    # and so were slots
    check_against_plain(steps, tmp_path / "mixed", requests, config, weights, dtype)


def test_a_row_does_not_depend_on_the_batch(tmp_path_factory):
    """Float32: a request's logits are the same bits alone and beside others, whole and in portions."""
    from microllm_rocm_amd.engine import Engine, StepEntry
    folder, config, _ = model_for(tmp_path_factory, "A")
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=4)
    a, b, c = (tokens_for(seed, length, config["vocab"]) for seed, length in ((1, 45), (2, 20), (3, 33)))
    engine.open("alone")
    alone = engine.step([StepEntry("alone", a, list(range(len(a))))]).clone()
    engine.close("alone")
    for name in "abc":
        engine.open(name)
    first = engine.step([StepEntry("b", b[:7], []), StepEntry("a", a[:30], list(range(30))), StepEntry("c", c[:2], [])])
    second = engine.step([StepEntry("a", a[30:44], list(range(14))), StepEntry("c", c[2:], []), StepEntry("b", b[7:8], [])])
    third = engine.step([StepEntry("b", b[8:9], [0]), StepEntry("a", a[44:], [0])])
    together = torch.cat([first, second, third[1:]])
    assert torch.equal(alone, together)


@pytest.mark.parametrize("which", ["A", "B"])
def test_long_decoding_through_graphs(tmp_path_factory, which):
    """A short prompt, then 140 tokens one by one (steps replayed from captured graphs, state carried in slots, cached
    rows crossing many pages and leaving every window), two requests at once with unequal lengths."""
    from microllm_rocm_amd.engine import Engine, StepEntry
    folder, config, weights = model_for(tmp_path_factory, which)
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=2)
    assert engine.use_graphs
    sequences = {"x": tokens_for(7, 150, config["vocab"]), "y": tokens_for(8, 160, config["vocab"])}
    starts = {"x": 10, "y": 3}
    rows = {name: [] for name in sequences}
    for name in sequences:
        engine.open(name)
    logits = engine.step([StepEntry(name, sequences[name][:starts[name]], [starts[name] - 1]) for name in sequences])
    for index, name in enumerate(sequences):
        rows[name].append(logits[index].cpu().numpy())
    for offset in range(140):
        entries = [StepEntry(name, [sequences[name][starts[name] + offset]], [0]) for name in sequences]
        logits = engine.step(entries)
        for index, name in enumerate(sequences):
            rows[name].append(logits[index].cpu().numpy())
    assert engine.graph_replays >= 139
    for name, tokens in sequences.items():
        want = plain.forward(config, weights, tokens[:starts[name] + 140])[starts[name] - 1:]
        assert row_errors(np.stack(rows[name]), want).max() < F32_BOUND


@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tmp_path_factory, which):
    from microllm_rocm_amd import Engine, GenerationConfig, generate, generate_serial
    folder, config, weights = model_for(tmp_path_factory, which)
    prompts = [tokens_for(20 + index, length, config["vocab"]) for index, length in enumerate((5, 31, 12))]
    expected = [prompt + plain.generate_greedy(config, weights, prompt, 10) for prompt in prompts]
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=4)
    got = generate(engine, prompts, GenerationConfig(max_new_tokens=10, temperature=0.0), prefill_chunk=7, max_batched_tokens=16)
    assert got == expected
    assert generate_serial(engine, prompts[0], GenerationConfig(max_new_tokens=10, temperature=0.0)) == expected[0]
    bf16 = Engine.from_folder(folder, dtype="bfloat16", max_tokens=512, max_requests=4)
    close = generate(bf16, prompts, GenerationConfig(max_new_tokens=10, temperature=0.0), prefill_chunk=7)
    assert [len(tokens) for tokens in close] == [len(tokens) for tokens in expected]
    assert all(tokens[:len(prompt)] == prompt for tokens, prompt in zip(close, prompts))


def test_residual_stream_after_every_layer(tmp_path_factory, tmp_path):
    folder, config, weights = model_for(tmp_path_factory, "A")
    tokens = tokens_for(5, 19, config["vocab"])
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": tokens, "want": list(range(19))}], "end": ["q"]}]
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=64, max_requests=1)
    replay(engine, io.StringIO(to_lines(steps)), str(tmp_path), io.StringIO(), dump_layers=True)
    runs = []
    plain.forward(config, weights, tokens, runs)
    got = np.fromfile(os.path.join(str(tmp_path), "0.layers.f32"), dtype="<f4").reshape(len(runs), 19, config["width"])
    assert np.abs(got - np.stack(runs)).max() < 1e-4 * np.abs(np.stack(runs)).max()


def test_plain_pages_in_bfloat16_and_the_kernels_for_few_rows(tmp_path_factory, tmp_path):
    """A bfloat16 engine whose attention layers are told not to take the MFMA kernels runs the same model on plain
    pages; both engines stay within the format's cost of the plain run."""
    from microllm_rocm_amd.config.registry import load_config
    from microllm_rocm_amd.engine import Engine, StepEntry
    from microllm_rocm_amd.parts import PartSpec
    from microllm_rocm_amd.weights import load_folder
    import dataclasses
    folder, config, weights = model_for(tmp_path_factory, "C")
    architecture, typed = load_config(folder)
    spec = architecture.build_spec(typed)
    layers = tuple(dataclasses.replace(layer, mixer=PartSpec(layer.mixer.kind, {**layer.mixer.params, "mfma": False}, layer.mixer.names))
                   if layer.mixer.kind == "latent_attention" else layer for layer in spec.layers)
    spec = dataclasses.replace(spec, layers=layers)
    from microllm_rocm_amd.parts import Model, Runtime
    probe = Model(spec, Runtime(torch.bfloat16, torch.device("cpu")))
    tensors = load_folder(folder, probe.tensors(), torch.bfloat16, torch.device("cuda:0"))
    engine = Engine(spec, tensors, dtype="bfloat16", max_tokens=256, max_requests=2, tensors_placed=True)
    tokens = tokens_for(9, 120, config["vocab"])
    engine.open("p")
    first = engine.step([StepEntry("p", tokens[:100], list(range(100)))]).cpu().numpy()
    rest = [engine.step([StepEntry("p", [token], [0])]).cpu().numpy() for token in tokens[100:]]
    got = np.concatenate([first] + rest)
    errors = np.where(decided(config, weights, tokens, list(range(len(tokens))), "bfloat16"), row_errors(got, plain_logits(config, weights, tokens)), 0.0)
    assert within_bound(errors, "bfloat16")


def test_command_line_and_trace_runner_as_programs(tmp_path_factory, tmp_path, capsys):
    import json
    import subprocess
    import sys
    from microllm_rocm_amd.cli import hf_infer
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, config, weights = model_for(tmp_path_factory, "A")
    prompt = tokens_for(31, 13, config["vocab"])
    expected = plain.generate_greedy(config, weights, prompt, 6)
    base = ["--model", folder, "--tokens", ",".join(map(str, prompt)), "--new-tokens", "6", "--dtype", "float32"]

    def run(*more):
        capsys.readouterr()
        assert hf_infer.main(base + list(more)) == 0
        return json.loads(capsys.readouterr().out.strip().splitlines()[-1])

    report = run()
    assert report["architecture"] == "Gupitar" and report["generated_tokens"] == expected
    for more in (["--use-cache", "false"], ["--cache-prefill-mode", "token"], ["--batch", "2", "--batch-argmax-mode", "host"]):
        assert run(*more)["generated_tokens"] == expected, more
    sampled = [run("--temperature", "0.9", "--sample-top-k", "5", "--seed", "7")["generated_tokens"] for _ in range(2)]
    assert sampled[0] == sampled[1] and len(sampled[0]) == 6
    steps = portions("p", prompt + expected, [5, 2, 1])
    result = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
                             str(tmp_path / "trace"), "--max-tokens", "64"], input=to_lines(steps), capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr
    assert [line for line in result.stdout.splitlines() if line.startswith("done")] == [f"done {step['step']}" for step in steps]
    check_against_plain(steps, tmp_path / "trace", {"p": prompt + expected}, config, weights, "float32")
