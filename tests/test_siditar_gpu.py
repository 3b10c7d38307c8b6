"""The Siditar decoder on the GPU against the plain implementation (tests/plain_siditar.py): every mechanism alone
through its kernel, then the engine whole, token by token, in portions, in mixed batches on reused pages and slots,
long decoding, and greedy generation through the scheduler. The configurations are made here and differ from each
other in every size: grouped and single kv heads, key and value widths that differ and are no multiples of 8, one,
three and no streams, layers without a feed-forward, a loop from the first layer and none at all."""
import io
import math
import os

import numpy as np
import pytest
import torch

import plain_siditar as plain
from replay_tools import collect, mixed, portions, prefill_then_decode, round_up, to_lines, whole
from siditar_tiny import CONFIGS, make_siditar_folder

pytestmark = pytest.mark.gpu

F32_BOUND = 2e-5        # of the logits' scale: float32 against float64, sums in other orders
BF16_BOUND = 0.06       # of the logits' scale: what the format costs on these models; a fault costs far more
_models = {}


def model_for(tmp_path_factory, which):
    if which not in _models:
        folder = make_siditar_folder(tmp_path_factory.mktemp(f"siditar_{which}"), which)
        _models[which] = (folder, plain.read_config(folder), plain.read_safetensors(os.path.join(folder, "model.safetensors")))
    return _models[which]


def tokens_for(seed, count, vocab):
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def row_errors(got, want):
    """Per row: the root mean square of the difference (means taken off) over that of the wanted logits."""
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


def plain_logits(config, weights, tokens):
    key = (id(weights), tuple(tokens))
    if key not in _plain_logits:
        _plain_logits[key] = plain.forward(config, weights, tokens)
    return _plain_logits[key]


def check_against_plain(steps, out_dir, requests, config, weights, dtype):
    got = collect(steps, str(out_dir), config["vocab"])
    bound = F32_BOUND if dtype == "float32" else BF16_BOUND
    worst = 0.0
    for rid, tokens in requests.items():
        want = plain_logits(config, weights, tokens)
        places = sorted(place for (request, place) in got if request == rid)
        assert places, f"no logits came back for {rid}"
        errors = row_errors(np.stack([got[(rid, place)] for place in places]), want[places])
        assert errors.max() < bound, f"{rid}: position {places[int(errors.argmax())]} is off by {errors.max():.3g} of the scale"
        worst = max(worst, float(errors.max()))
    return worst


# ---- mechanisms alone -------------------------------------------------------------------------------------------
def device(array, dtype=torch.float32):
    return torch.as_tensor(np.asarray(array), dtype=dtype).cuda().contiguous()


@pytest.mark.parametrize("width,first", [(64, 0), (50, 1000), (6, 7), (37, 3)])
def test_embedding_adds_sine_and_cosine(width, first):
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(0)
    table = rng.normal(size=(17, width)).astype(np.float32)
    ids = rng.integers(0, 17, size=9)
    positions = np.arange(first, first + 9)
    rates = device(10000.0 ** (-2.0 * np.arange((width + 1) // 2) / width), torch.float64)
    got = kernels.embedding_sinusoid(device(table), device(ids, torch.int32), device(positions, torch.int32), rates)
    want = table[ids] + plain.position_waves(9, width, first)
    assert np.abs(got.cpu().numpy() - want).max() < 1e-6


@pytest.mark.parametrize("streams,width,parts,rms", [(1, 40, 1, False), (2, 64, 2, False), (3, 50, 1, True), (8, 600, 3, False)])
def test_stream_write_read_and_norm(streams, width, parts, rms):
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(streams)
    x = rng.normal(size=(5, streams, width)) * 3 + 1.5       # a mean that a norm without centring would keep
    y = rng.normal(size=(parts, 5, width))
    mix, give, take = rng.normal(size=(streams, streams)), rng.normal(size=streams), rng.normal(size=streams)
    weight = rng.normal(size=width) + 1
    old = [x[:, s] for s in range(streams)]
    new = plain.streams_write(old, mix, give, y.sum(0))
    read = plain.streams_read(new, take)
    want = plain.unit_rms(read, weight, 1e-5) if rms else plain.layer_norm(read, weight, 1e-5)
    x_device = device(x)
    got = kernels.stream_norm(x_device, device(weight), 1e-5, torch.float32, rms=rms, delta=device(y if parts > 1 else y[0]),
                              mix=device(mix), give=device(give), take=device(take), write_x=True)
    assert np.abs(got.cpu().numpy() - want).max() < 2e-5
    assert np.abs(x_device.cpu().numpy() - np.stack(new, axis=1)).max() < 2e-5
    # the read alone, of chosen rows, with every stream counted once: what the model's last norm does
    rows = device([4, 0, 2], torch.int32)
    got = kernels.stream_norm(x_device, device(weight), 1e-5, torch.float32, rms=rms, rows=rows)
    total = sum(new)[[4, 0, 2]]
    want = plain.unit_rms(total, weight, 1e-5) if rms else plain.layer_norm(total, weight, 1e-5)
    assert np.abs(got.cpu().numpy() - want).max() < 2e-5


def test_clamped_gated_activation():
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(3)
    gate_up = rng.normal(size=(7, 2 * 24)) * 3       # many values beyond the limit on both sides
    got = kernels.clamped_glu(device(gate_up), 1.25, 1.702, torch.float32).cpu().numpy()
    gate, up = np.minimum(gate_up[:, :24], 1.25), np.clip(gate_up[:, 24:], -1.25, 1.25)
    assert np.abs(got - gate * plain.sigmoid(1.702 * gate) * (up + 1)).max() < 1e-6


def attention_through_kernels(q, k, v, scale, table, longest, sink, dtype=torch.float32, page_size=16, first_page=3,
                              q_weight=None, k_weight=None, temp=(0.0, 1), portions_of=None):
    """One request of n tokens through qk_norm_store and bias_attention, its pages scattered; in portions if asked."""
    from microllm_rocm_amd.ops import kernels
    n, heads, dim = q.shape
    kv_heads, vdim = k.shape[1], v.shape[2]
    blocks = -(-n // page_size)
    pages = [first_page + 2 * block for block in reversed(range(blocks))]      # out of order, with holes
    k_pages = torch.zeros((first_page + 2 * blocks, page_size, kv_heads, dim), dtype=dtype, device="cuda")
    v_pages = torch.zeros((first_page + 2 * blocks, page_size, kv_heads, vdim), dtype=dtype, device="cuda")
    bias = None
    if table is not None:
        unrolled = np.stack([table[plain.bucket_of(distance, table.shape[0], longest)] for distance in range(longest + 1)])
        bias = device(unrolled)
    block_table = device([pages], torch.int32)
    outputs = []
    position = 0
    for count in (portions_of or [n]):
        count = min(count, n - position)
        if count <= 0:
            break
        rows = slice(position, position + count)
        qkv = np.concatenate([q[rows].reshape(count, -1), k[rows].reshape(count, -1), v[rows].reshape(count, -1)], axis=1)
        positions = np.arange(position, position + count)
        slots = [pages[p // page_size] * page_size + p % page_size for p in positions]
        queries = kernels.qk_norm_store(device(qkv), q_weight, k_weight, 1e-6, device(positions, torch.int32),
                                        device(slots, torch.int32), temp[0], temp[1], k_pages, v_pages, heads, kv_heads, dim,
                                        vdim, dtype)
        out = kernels.bias_attention(queries, k_pages, v_pages, block_table, device(np.zeros(count), torch.int32),
                                     device(positions, torch.int32), bias, device(sink) if sink is not None else None,
                                     scale, 1.0, heads, kv_heads, dim, vdim)
        outputs.append(out.float().cpu().numpy().reshape(count, heads, vdim))
        position += count
    return np.concatenate(outputs)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,n", [(4, 2, 24, 16, 70), (2, 1, 20, 40, 33), (3, 3, 8, 72, 130), (1, 1, 128, 200, 65)])
def test_attention_with_bias_and_sink(heads, kv_heads, dim, vdim, n):
    rng = np.random.default_rng(n)
    q, k, v = rng.normal(size=(n, heads, dim)), rng.normal(size=(n, kv_heads, dim)), rng.normal(size=(n, kv_heads, vdim))
    table, sink = rng.normal(size=(10, heads)) * 2, rng.normal(size=heads)
    want = plain.bias_sink_attention(q, k, v, 0.2, table, 27, sink)
    got = attention_through_kernels(q, k, v, 0.2, table, 27, sink)
    assert np.abs(got - want).max() < 2e-5
    again = attention_through_kernels(q, k, v, 0.2, table, 27, sink, portions_of=[2, 5, 64, 1, 1, 3, 200])
    assert np.array_equal(got, again)       # a row does not depend on how the request was cut
    # neither the bias nor the sink: plain causal attention
    want = plain.bias_sink_attention(q, k, v, 0.2, None, 0, None)
    assert np.abs(attention_through_kernels(q, k, v, 0.2, None, 0, None) - want).max() < 2e-5


@pytest.mark.parametrize("far", [0, 1, 63, 64, 65, 200, 299])
def test_one_far_key_decides(far):
    """Among 300 keys one has a score far above the others: the last query must return that key's value, wherever
    the key lies (the first tokens, a tile's edge, a page's edge)."""
    rng = np.random.default_rng(far)
    n, dim, vdim = 300, 16, 8
    q, k, v = rng.normal(size=(n, 1, dim)) * 0.1, rng.normal(size=(n, 1, dim)) * 0.1, rng.normal(size=(n, 1, vdim))
    q[-1, 0] = 0.0
    q[-1, 0, 3] = 6.0
    k[far, 0, 3] = 6.0
    got = attention_through_kernels(q, k, v, 1.0, None, 0, np.zeros(1))
    want = plain.bias_sink_attention(q, k, v, 1.0, None, 0, np.zeros(1))
    assert np.abs(got[-1] - want[-1]).max() < 1e-5 and np.abs(got[-1, 0] - v[far, 0]).max() < 1e-3


def test_bias_buckets_at_their_edges():
    """All scores are zero, so the weights are the bias alone; the table rises steeply from row to row, so a key
    that lands in a neighbouring bucket changes the result. Every distance up to beyond the longest is met, in a
    prompt and token by token."""
    rows, longest, n = 8, 21, 40
    table = (np.arange(rows)[:, None] * 1.7) * np.array([[1.0, -1.0]])
    q, k = np.zeros((n, 2, 8)), np.zeros((n, 1, 8))
    v = np.random.default_rng(0).normal(size=(n, 1, 4))
    want = plain.bias_sink_attention(q, k, v, 1.0, table, longest, np.array([0.5, -0.5]))
    got = attention_through_kernels(q, k, v, 1.0, table, longest, np.array([0.5, -0.5]))
    assert np.abs(got - want).max() < 1e-5
    got = attention_through_kernels(q, k, v, 1.0, table, longest, np.array([0.5, -0.5]), portions_of=[17] + [1] * 23)
    assert np.abs(got - want).max() < 1e-5
    from microllm_rocm_amd.parts.bias_attention import distance_bucket
    for total, far in ((8, 21), (16, 120), (12, 40), (6, 9), (2, 5), (32, 1000)):
        assert [distance_bucket(d, total, far) for d in range(2 * far)] == [plain.bucket_of(d, total, far) for d in range(2 * far)]


def test_sink_takes_weight_without_a_value():
    n = 5
    q, k, v = np.zeros((n, 1, 8)), np.zeros((n, 1, 8)), np.ones((n, 1, 4))
    got = attention_through_kernels(q, k, v, 1.0, None, 0, np.array([math.log(3.0)]))
    # i + 1 keys of weight 1 and a sink of weight 3
    assert np.abs(got[:, 0, 0] - np.array([(i + 1) / (i + 4) for i in range(n)])).max() < 1e-6
    got = attention_through_kernels(q, k, v, 1.0, None, 0, np.array([40.0]))
    assert np.abs(got).max() < 1e-15      # a sink far above every score leaves nothing


def test_query_and_key_norm_and_factor_by_position():
    rng = np.random.default_rng(5)
    n, heads, dim = 20, 2, 12
    q, k, v = rng.normal(size=(n, heads, dim)) * 4, rng.normal(size=(n, 1, dim)) * 0.3, rng.normal(size=(n, 1, 6))
    q_weight, k_weight = rng.normal(size=dim) + 1, rng.normal(size=dim) + 1
    q_normed, k_normed = plain.unit_rms(q, q_weight, 1e-6), plain.unit_rms(k, k_weight, 1e-6)
    for i in range(n):
        q_normed[i] *= plain.query_factor(i, 0.8, 3)
    want = plain.bias_sink_attention(q_normed, k_normed, v, 0.5, None, 0, None)
    got = attention_through_kernels(q, k, v, 0.5, None, 0, None, q_weight=device(q_weight), k_weight=device(k_weight), temp=(0.8, 3))
    assert np.abs(got - want).max() < 2e-5


def attention_through_mfma(q, k, v, scale, table, longest, sink, portions_of, page_size=16, splits=None, out_scale=1.0):
    """The same through the paged attention's pages and MFMA kernels (bfloat16, one width for keys and values):
    portions of several tokens go to the tiled kernel, single tokens to the kernel that splits the keys."""
    from microllm_rocm_amd.cache.layout import key_page_shape, value_page_shape
    from microllm_rocm_amd.ops import kernels
    n, heads, dim = q.shape
    kv_heads = k.shape[1]
    blocks = -(-n // page_size)
    pages = [2 + 3 * block for block in reversed(range(blocks))]
    k_pages = torch.zeros(key_page_shape(3 * blocks + 2, kv_heads, page_size, dim), dtype=torch.bfloat16, device="cuda")
    v_pages = torch.zeros(value_page_shape(3 * blocks + 2, kv_heads, page_size, dim), dtype=torch.bfloat16, device="cuda")
    bias = None
    if table is not None:
        bias = device(np.stack([table[plain.bucket_of(distance, table.shape[0], longest)] for distance in range(longest + 1)]))
    block_table = device([pages], torch.int32)
    extras = kernels.AttentionExtras(bias, device(sink) if sink is not None else None, out_scale)
    outputs, position = [], 0
    for count in portions_of:
        count = min(count, n - position)
        if count <= 0:
            break
        rows = slice(position, position + count)
        qkv = np.concatenate([q[rows].reshape(count, -1), k[rows].reshape(count, -1), v[rows].reshape(count, -1)], axis=1)
        positions = device(np.arange(position, position + count), torch.int32)
        slots = device([pages[p // page_size] * page_size + p % page_size for p in range(position, position + count)], torch.int32)
        queries = kernels.qk_norm_store(device(qkv), None, None, 1e-6, positions, slots, 0.0, 1, k_pages, v_pages, heads, kv_heads,
                                        dim, dim, torch.bfloat16, tiled_page_size=page_size)
        wide = torch.zeros((count, heads * dim + 8), dtype=torch.bfloat16, device="cuda")     # the result as columns of a wider buffer
        out = wide[:, 8:]
        requests = device(np.zeros(count), torch.int32)
        if count == 1:
            kernels.paged_attention_decode(queries, k_pages, v_pages, block_table, requests, positions, scale, 0, heads, kv_heads, dim,
                                           splits or kernels.decode_splits(1, kv_heads, position + 1), out=out, extras=extras)
        else:
            tiles = [(0, offset, min(kernels.QUERY_TILE, count - offset), position + offset) for offset in range(0, count, kernels.QUERY_TILE)]
            plan = device(np.asarray(kernels.pair_query_tiles(tiles)).reshape(-1, 5), torch.int32)
            kernels.paged_attention_prefill(queries, k_pages, v_pages, block_table, plan, positions, scale, 0, heads, kv_heads, dim,
                                            out=out, extras=extras)
        assert float(wide[:, :8].abs().max()) == 0.0
        outputs.append(out.float().cpu().numpy().reshape(count, heads, dim))
        position += count
    return np.concatenate(outputs)


def as_bf16(array):
    return torch.as_tensor(array, dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


@pytest.mark.parametrize("heads,kv_heads,dim,n", [(4, 2, 32, 300), (2, 2, 16, 77), (6, 1, 48, 150), (1, 1, 128, 270)])
def test_mfma_attention_with_bias_and_sink(heads, kv_heads, dim, n):
    rng = np.random.default_rng(dim + n)
    q, k, v = (as_bf16(rng.normal(size=shape)) for shape in ((n, heads, dim), (n, kv_heads, dim), (n, kv_heads, dim)))
    table, sink = rng.normal(size=(10, heads)) * 2, rng.normal(size=heads)
    want = plain.bias_sink_attention(q, k, v, 0.2, table, 27, sink) * 1.5
    for portions_of in ([n], [140, 3] + [1] * 20 + [200], [1] * 40 + [2, 129, 1, 1, 1, 500]):
        got = attention_through_mfma(q, k, v, 0.2, table, 27, sink, portions_of, out_scale=1.5)
        assert np.abs(got - want).max() < 0.03 * np.abs(want).max(), portions_of       # weights and results are bfloat16
    got = attention_through_mfma(q, k, v, 0.2, table, 27, sink, [n - 1, 1], splits=3, out_scale=1.5)
    assert np.abs(got - want).max() < 0.03 * np.abs(want).max()
    want = plain.bias_sink_attention(q, k, v, 0.2, None, 0, None)
    assert np.abs(attention_through_mfma(q, k, v, 0.2, None, 0, None, [n]) - want).max() < 0.03 * np.abs(want).max()


def test_mfma_bias_buckets_sink_and_far_keys():
    """The constructed cases of the plain kernel's tests through the MFMA kernels: weights from the bias alone at
    every distance up to beyond the longest, a sink that takes weight, one far key that decides."""
    rows, longest, n = 8, 21, 200
    table = (np.arange(rows)[:, None] * 0.9) * np.array([[1.0, -1.0]])
    q, k = np.zeros((n, 2, 16)), np.zeros((n, 1, 16))
    v = as_bf16(np.random.default_rng(0).normal(size=(n, 1, 16)))
    sink = np.array([0.5, -0.5])
    want = plain.bias_sink_attention(q, k, v, 1.0, table, longest, sink)
    for portions_of in ([n], [150] + [1] * 50, [1] * 30 + [170]):
        got = attention_through_mfma(q, k, v, 1.0, table, longest, sink, portions_of)
        assert np.abs(got - want).max() < 0.02, portions_of
    v = np.ones((n, 1, 16))
    got = attention_through_mfma(q, k, v, 1.0, None, 0, np.array([math.log(3.0), 30.0]), [100] + [1] * 100)
    assert np.abs(got[:, 0, 0] - np.array([(i + 1) / (i + 4) for i in range(n)])).max() < 0.01 and np.abs(got[:, 1]).max() < 1e-9
    for far in (0, 1, 31, 32, 127, 128, 150):
        rng = np.random.default_rng(far)
        q, k, v = as_bf16(rng.normal(size=(n, 1, 16)) * 0.1), as_bf16(rng.normal(size=(n, 1, 16)) * 0.1), as_bf16(rng.normal(size=(n, 1, 16)))
        q[-1, 0] = 0.0
        q[-1, 0, 3] = 6.0
        k[far, 0, 3] = 6.0
        for portions_of in ([n], [n - 1, 1]):
            got = attention_through_mfma(q, k, v, 1.0, None, 0, np.zeros(1), portions_of)
            assert np.abs(got[-1, 0] - v[far, 0]).max() < 0.02, (far, portions_of)


@pytest.mark.parametrize("heads,dim,vdim,rank,tau", [(2, 16, 8, 4, 4.0), (2, 64, 128, 16, 16.0), (3, 16, 8, 5, 4.0), (1, 40, 24, 3, 1.5), (2, 8, 72, 1, 16.0), (1, 130, 5, 2, 1.0)])
def test_linear_attention_walk(heads, dim, vdim, rank, tau):
    """Decays, the walk with carried state and the gate: two requests in one step, then both continued one token at
    a time beside a third that starts, in slots that are not in order."""
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(dim)
    lengths = [83, 9, 4]
    keys, values = heads * dim, heads * vdim
    a2, bias, weight = rng.normal(size=(keys, rank)), rng.normal(size=keys), rng.normal(size=vdim) + 1
    columns = 2 * keys + 2 * values + rank
    rows = {name: rng.normal(size=(length, columns)) for name, length in zip("abc", lengths)}

    def plain_run(proj):
        n = proj.shape[0]
        q = proj[:, :keys].reshape(n, heads, dim) * 0.25
        k = proj[:, keys:2 * keys].reshape(n, heads, dim)
        v = proj[:, 2 * keys:2 * keys + values].reshape(n, heads, vdim)
        gate = proj[:, 2 * keys + values:2 * keys + 2 * values]
        decay = (plain.sigmoid(proj[:, 2 * keys + 2 * values:] @ a2.T + bias) ** (1.0 / tau)).reshape(n, heads, dim)
        o, _ = plain.decayed_state_walk(q, k, v, decay)
        return plain.unit_rms(o, weight, 1e-5).reshape(n, values) * gate * plain.sigmoid(gate) * 1.5

    want = {name: plain_run(proj) for name, proj in rows.items()}
    state = torch.full((6, heads, dim, vdim), 7.0, device="cuda")       # slots hold what the last user left
    slot_of = {"a": 4, "b": 1, "c": 5}
    got = {name: [] for name in rows}
    fed = {name: 0 for name in rows}

    def step(portions_of):
        names = list(portions_of)
        for name in names:
            if fed[name] == 0:
                state[slot_of[name]].zero_()
        proj = np.concatenate([rows[name][fed[name]:fed[name] + portions_of[name]] for name in names])
        cu = np.concatenate([[0], np.cumsum([portions_of[name] for name in names])])
        proj_device = device(proj)
        decay = kernels.gla_decay(proj_device, 2 * keys + 2 * values, device(a2), device(bias), tau)
        slots = device([slot_of[name] for name in names], torch.int32)
        before = state.clone()      # both kernels walk the step: they must leave the same bits
        staged = kernels.gla_scan(proj_device, 0, keys, 2 * keys, decay, before, device(cu, torch.int32), slots, len(names),
                                  heads, dim, vdim, 0.25, long_portions=True)
        o = kernels.gla_scan(proj_device, 0, keys, 2 * keys, decay, state, device(cu, torch.int32), slots, len(names), heads, dim,
                             vdim, 0.25)
        assert torch.equal(o, staged) and torch.equal(state, before)
        out = kernels.gla_gate(o, proj_device, 2 * keys + values, device(weight), 1e-5, heads, vdim, 1.5, torch.float32).cpu().numpy()
        for index, name in enumerate(names):
            got[name].append(out[cu[index]:cu[index + 1]])
            fed[name] += portions_of[name]

    step({"a": 77, "b": 2})
    step({"b": 5, "a": 1})
    step({"a": 1, "c": 4, "b": 1})
    for _ in range(4):
        step({"a": 1})
    step({"b": 1})
    for name in rows:
        result = np.concatenate(got[name])
        assert np.abs(result - want[name][:result.shape[0]]).max() < 3e-5 * max(1.0, np.abs(want[name]).max())
    assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0      # slots of no request were not touched


# ---- the engine ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_whole_decode_and_portions(tmp_path_factory, tmp_path, which, dtype):
    folder, config, weights = model_for(tmp_path_factory, which)
    requests = {"long": tokens_for(1, 150, config["vocab"]), "short": tokens_for(2, 37, config["vocab"]), "one": tokens_for(3, 1, config["vocab"])}
    run_trace(folder, dtype, whole(requests), tmp_path / "whole", max_tokens=256)
    check_against_plain(whole(requests), tmp_path / "whole", requests, config, weights, dtype)
    for rid in ("long", "short"):
        steps = prefill_then_decode(rid, requests[rid], tail=34)       # the decoded tokens cross pages' edges
        run_trace(folder, dtype, steps, tmp_path / f"decode_{rid}", max_tokens=round_up(len(requests[rid]), 64))
        check_against_plain(steps, tmp_path / f"decode_{rid}", {rid: requests[rid]}, config, weights, dtype)
    for sizes in ([2], [3, 16, 1, 2, 31], [64, 2, 17]):
        steps = portions("long", requests["long"], sizes)
        run_trace(folder, dtype, steps, tmp_path / f"portions_{sizes[0]}", max_tokens=192)
        check_against_plain(steps, tmp_path / f"portions_{sizes[0]}", {"long": requests["long"]}, config, weights, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "C", "D"])
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
    """A short prompt, then 140 tokens one by one (steps replayed from captured graphs, state carried in slots, keys
    crossing many pages), two requests at once with unequal lengths."""
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


@pytest.mark.parametrize("which", ["A", "C", "D"])
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


def test_residual_stream_after_every_run(tmp_path_factory, tmp_path):
    """The stream that the replay tool dumps after every layer run (the sum of the copies) is the plain one's."""
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
    assert len(runs) == len(plain.run_order(config)) > len(config["layers"])      # the looped layers count each time
    assert np.abs(got - np.stack(runs)).max() < 1e-4 * np.abs(np.stack(runs)).max()


def test_command_line_and_trace_runner_as_programs(tmp_path_factory, tmp_path, capsys):
    """The generation command line and the trace runner choose the model by its config.json like any other: greedy
    tokens and last logits of the command line, several ways of generating, sampling with a seed, and the trace
    runner as a program fed through a pipe."""
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

    logits_path = tmp_path / "last.f32"
    report = run("--logits-output", str(logits_path))
    assert report["architecture"] == "Siditar" and report["generated_tokens"] == expected
    assert row_errors(np.fromfile(logits_path, dtype="<f4")[None], plain.forward(config, weights, prompt)[-1:]).max() < F32_BOUND
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
