"""Host logic of the Gupitar decoder: its configuration (keys, refusals), the run order with layers that borrow another
layer's cached rows, the model it is built into, and the cache needs of its mixers."""
import json
import os

import numpy as np
import pytest
import torch

import plain_gupitar as plain
from gupitar_tiny import CONFIGS, make_gupitar_folder
from microllm_rocm_amd.cache import CacheManager, CompositeNeed, PagedKVNeed, PagedLatentNeed, StateNeed, flat_needs
from microllm_rocm_amd.config import ConfigError, GupitarConfig, load_config
from microllm_rocm_amd.parts import Model, Runtime


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_folder_round_trip(tmp_path, which):
    folder = make_gupitar_folder(tmp_path, which)
    written = json.load(open(os.path.join(folder, "config.json")))
    assert written["architecture"] == "Gupitar"
    architecture, config = load_config(folder)
    assert architecture.name == "Gupitar" and config == CONFIGS[which]
    spec = architecture.build_spec(config)
    assert [entry.layer for entry in spec.order] == list(range(len(config.layers)))
    assert [entry.reads_cache_of for entry in spec.order] == [layer["mixer"].get("kv_from") for layer in written["layers"]]
    model = Model(spec, Runtime(torch.float32, torch.device("cpu")))
    assert set(model.tensors()) == set(plain.read_safetensors(os.path.join(folder, "model.safetensors")))
    for need, layer in zip(model.cache_needs(), written["layers"]):
        mixer = layer["mixer"]
        if layer["type"] == "rglru":
            assert need == CompositeNeed((StateNeed((mixer["conv"] - 1, mixer["width"])), StateNeed((mixer["width"],))))
        elif "kv_from" in mixer:
            assert need is None
        else:
            assert isinstance(need, PagedLatentNeed) and need.width == mixer["kv_rank"] + mixer["rot_dim"]


def test_cached_rows_are_kept_for_the_widest_window_that_reads_them():
    """Layer 2 of the first model borrows layer 0's rows with a window of 33 where layer 0 itself looks back 17."""
    from microllm_rocm_amd.architectures.gupitar import build_spec
    spec = build_spec(CONFIGS["A"])
    model = Model(spec, Runtime(torch.float32, torch.device("cpu")))
    needs = model.cache_needs()
    assert needs[0] == PagedLatentNeed(48, 33) and needs[4] == PagedLatentNeed(42, 9)
    assert model.blocks[0].mixer.window == 17 and model.blocks[2].mixer.window == 33
    bf16 = Model(spec, Runtime(torch.bfloat16, torch.device("cpu")))       # rows of 48: the paged attention's pages; of 42: plain pages
    assert bf16.cache_needs()[0] == PagedKVNeed(1, 48, 33) and bf16.cache_needs()[4] == PagedLatentNeed(42, 9)
    manager = CacheManager(needs, [entry.reads_cache_of for entry in spec.order], page_size=16, num_pages=32, max_requests=2)
    request = manager.open("r")
    manager.reserve(request, 100)
    manager.commit(request, 100)
    by_window = {group.need.window: request.pages[group.index] for group in manager.groups}
    assert sum(page >= 0 for page in by_window[33]) == 3 and sum(page >= 0 for page in by_window[9]) == 2
    manager.close("r")
    manager.check()


def test_config_refusals():
    good = CONFIGS["A"].to_dict()
    for change, text in (
            (lambda c: c.pop("width"), "width"), (lambda c: c["layers"][0].__setitem__("type", "attention"), "layer type"),
            (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "feed-forward kind"),
            (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 4), "rot.dims"),
            (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "window"),
            (lambda c: c["layers"][1]["mixer"].__setitem__("blocks", 5), "blocks"),
            (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 7), "top"),
            (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 2), "earlier"),
            (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1), "latents"),
            (lambda c: c["layers"][2]["mixer"].__setitem__("kv_rank", 24), "equal"),
            (lambda c: c["layers"][4]["mixer"].__setitem__("scale", "0.25"), "scale"),
            (lambda c: c.__setitem__("vocab", 2.5), "vocab")):
        changed = json.loads(json.dumps(good))
        change(changed)
        with pytest.raises(ConfigError, match=text):
            GupitarConfig.from_dict(changed)


def test_plain_pieces():
    """The plain implementation's own pieces against values worked out by hand."""
    assert abs(plain.gelu_tanh(np.array([1.0]))[0] - 0.8411919906082768) < 1e-12
    assert abs(plain.softplus(np.array([0.0]))[0] - np.log(2.0)) < 1e-12
    turned = plain.rotate_half(np.array([[1.0, 2.0, 3.0, 4.0, 9.0]]), [1], 4, 100.0)      # pairs (0, 2) and (1, 3); the fifth entry stays
    c0, s0, c1, s1 = np.cos(1.0), np.sin(1.0), np.cos(0.1), np.sin(0.1)
    assert np.allclose(turned[0], [1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1, 9.0])
    taps = np.array([[0.5, 2.0, 1.0]])
    assert np.allclose(plain.causal_conv(np.array([[1.0], [10.0], [100.0]]), taps, np.array([0.25]))[:, 0], [1.25, 12.25, 120.75])
    ids, weights = plain.choose_experts(np.array([[0.0, 2.0, 2.0, -1.0]]), 2)
    assert ids.tolist() == [[1, 2]] and np.allclose(weights, plain.sigmoid(np.array([2.0, 2.0])))
    rows = np.array([[1.0, 0.0], [0.0, 1.0], [5.0, 5.0]])
    seen = plain.folded_attention(np.zeros((3, 1, 2)), rows, 2, 2, 1.0)      # equal scores: the mean of the rows in the window
    assert np.allclose(seen[:, 0], [[1.0, 0.0], [0.5, 0.5], [2.5, 3.0]])
