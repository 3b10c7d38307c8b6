"""Host logic of the Siditar decoder: its configuration (keys, the sizes that only tensors give, refusals), the run
order with a looped range, the model it is built into, and a cache manager that serves a mixer with two needs."""
import dataclasses
import json
import os

import pytest
import torch

import plain_siditar as plain
from microllm_rocm_amd.cache import CacheManager, CompositeBinding, CompositeNeed, PagedKeyValueNeed, StateNeed, flat_needs
from microllm_rocm_amd.config import ConfigError, SiditarConfig, load_config
from microllm_rocm_amd.config.siditar import LoopConfig
from microllm_rocm_amd.parts import Model, Runtime
from microllm_rocm_amd.parts.bias_attention import distance_bucket
from siditar_tiny import CONFIGS, make_siditar_folder


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_folder_round_trip(tmp_path, which):
    folder = make_siditar_folder(tmp_path, which)
    written = json.load(open(os.path.join(folder, "config.json")))
    assert written["architecture"] == "Siditar" and "bias_rows" not in json.dumps(written) and "decay_rank" not in json.dumps(written)
    architecture, config = load_config(folder)
    assert architecture.name == "Siditar" and config == CONFIGS[which]       # the two sizes came from the tensors' shapes
    assert list(config.run_order()) == plain.run_order(written)
    spec = architecture.build_spec(config)
    assert [entry.layer for entry in spec.order] == list(config.run_order()) and spec.streams == config.streams
    model = Model(spec, Runtime(torch.float32, torch.device("cpu")))
    names = set(plain.read_safetensors(os.path.join(folder, "model.safetensors")))
    assert set(model.tensors()) == names
    needs = model.cache_needs()
    assert len(needs) == len(spec.order) and all(isinstance(need, CompositeNeed) for need in needs)
    left = config.layers[spec.order[0].layer].mixer.left
    assert flat_needs(needs[0])[0] == PagedKeyValueNeed(left.kv_heads, left.dim, left.vdim)


def test_config_without_weights_needs_the_two_sizes(tmp_path):
    config = CONFIGS["B"]
    config.save(str(tmp_path))
    architecture, read = load_config(str(tmp_path))       # no tensor files yet: the sizes stay open
    assert read.layers[0].mixer.left.bias_rows is None and read.layers[0].mixer.right.decay_rank is None
    with pytest.raises(ConfigError, match="sizes of tensors"):
        architecture.build_spec(read)


def test_config_refusals():
    good = CONFIGS["A"].to_dict()
    for change, text in (
            (lambda c: c.pop("width"), "width"), (lambda c: c.__setitem__("streams", 9), "streams"),
            (lambda c: c["layers"][0].__setitem__("type", "serial"), "layer type"),
            (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "feed-forward kind"),
            (lambda c: c["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3), "multiple"),
            (lambda c: c["loop"].__setitem__("stop", 9), "loop"), (lambda c: c["loop"].__setitem__("times", 0), "loop"),
            (lambda c: c["layers"][1]["mixer"]["right"].__setitem__("tau", "4"), "tau"),
            (lambda c: c.__setitem__("vocab", 2.5), "vocab")):
        changed = json.loads(json.dumps(good))
        change(changed)
        with pytest.raises(ConfigError, match=text):
            SiditarConfig.from_dict(changed)
    assert SiditarConfig.from_dict(good).loop == LoopConfig(0, 2, 3)
    no_loop = json.loads(json.dumps(good))
    del no_loop["loop"], no_loop["streams"]
    plainer = SiditarConfig.from_dict(no_loop)
    assert plainer.loop is None and plainer.streams is None and list(plainer.run_order()) == [0, 1, 2]


def test_run_order_with_a_loop():
    config = CONFIGS["A"]
    assert list(dataclasses.replace(config, loop=LoopConfig(1, 3, 2)).run_order()) == [0, 1, 2, 1, 2]
    assert list(dataclasses.replace(config, loop=LoopConfig(0, 1, 1)).run_order()) == [0, 1, 2]
    assert list(dataclasses.replace(config, loop=LoopConfig(2, 3, 4)).run_order()) == [0, 1, 2, 2, 2, 2]


def test_distance_buckets():
    for rows, longest in ((16, 120), (8, 21), (12, 40), (6, 9), (2, 5), (32, 1000), (64, 4096)):
        buckets = [distance_bucket(distance, rows, longest) for distance in range(longest + 50)]
        assert buckets == [plain.bucket_of(distance, rows, longest) for distance in range(longest + 50)]
        assert buckets[:rows // 2] == list(range(rows // 2)) and all(b == rows - 1 for b in buckets[longest:])
        assert all(later >= earlier for earlier, later in zip(buckets, buckets[1:]))


def test_cache_manager_serves_a_mixer_with_two_needs():
    """Pages for the attention and a slot for the state of every run entry; equal paged needs share a group; a run
    of a looped layer is an entry of its own."""
    first = CompositeNeed((PagedKeyValueNeed(2, 24, 16), StateNeed((3, 16, 8))))
    second = CompositeNeed((PagedKeyValueNeed(1, 20, 40), StateNeed((1, 40, 24))))
    cache = CacheManager([first, second, first, None], [None, None, None, 1], page_size=16, num_pages=8, max_requests=2)
    assert len(cache.groups) == 2 and cache.groups[0].entries == [0, 2] and cache.groups[1].entries == [1]
    bindings = cache.bindings()
    assert all(isinstance(binding, CompositeBinding) for binding in bindings)
    assert bindings[0].parts[0].group == 0 and bindings[1].parts[0].group == 1 and not bindings[3].owned and not bindings[3].parts[1].owned
    assert cache.has_state and cache.state_bytes() == 2 * 4 * (2 * 3 * 16 * 8 + 40 * 24)
    a = cache.open("a")
    cache.reserve(a, 40)
    cache.commit(a, 40)
    assert cache.held_pages() == [3, 3]
    b = cache.open("b")
    with pytest.raises(Exception):
        cache.open("c")                  # two slots
    cache.reserve(b, 70)
    cache.commit(b, 70)
    assert cache.free_pages() == [0, 0]
    cache.close("a")
    c = cache.open("c")
    assert c.slot == a.slot              # the slot that was given back last goes out first
    cache.reserve(c, 48)
    cache.check()
    cache.close("b")
    cache.close("c")
    cache.check()
    assert cache.free_pages() == [8, 8]
