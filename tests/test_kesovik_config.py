"""Kesovik's configuration on the CPU: keys, refusals, the round trip, the model as a list of parts, tensor names and
shapes, the combined cache of a layer with two mixers, and step costs."""
import copy

import pytest

from pulse_infer_amd.cache.manager import CacheManager
from pulse_infer_amd.cache.specs import CombinedSpec, PagedKVSpec, StateSpec
from pulse_infer_amd.config import ConfigError, KesovikConfig, config_from_dict
from pulse_infer_amd.models.causal_lm import expected_tensors
from pulse_infer_amd.models.cost import step_cost

LEFT = {"dim": 32, "heads": 6, "kv_heads": 2, "mask": {"size": 24}, "rot": {"base": 1e4, "dims": 16}, "scale": 0.2,
        "vdim": 16}
RIGHT = {"decay": [0.5, 0.9, 0.99], "dim": 16, "heads": 3, "vdim": 32}
CONFIG = {
    "architecture": "Kesovik", "embedding": {"scale": 2.0}, "logit_softcap": 9.0, "norm": {"eps": 1e-5},
    "postln_alpha": 1.7, "vocab": 307, "width": 96,
    "layers": [
        {"type": "parallel", "mixer": {"left": LEFT, "left_scale": 0.7, "right": RIGHT, "right_scale": 1.3},
         "mlp": {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 5, "identity": 2, "top": 3},
                 "shared": {"ff": 80}}},
        {"type": "lightning", "mixer": {"decay": [0.8, 1.0], "dim": 48, "heads": 2, "vdim": 16},
         "mlp": {"kind": "dense", "ff": 160}},
        {"type": "parallel", "mixer": {"left": LEFT, "left_scale": 1.0, "right": RIGHT, "right_scale": 1.0}, "mlp": None},
    ],
}


def test_round_trip_and_registry():
    cfg = config_from_dict(CONFIG)
    assert isinstance(cfg, KesovikConfig)
    assert cfg.to_dict() == CONFIG
    assert KesovikConfig.from_dict(cfg.to_dict()).to_dict() == CONFIG
    assert (cfg.vocab_size, cfg.width, cfg.postln_alpha, cfg.embedding_scale, cfg.logit_softcap) == (307, 96, 1.7, 2.0, 9.0)


def broken(path, value):
    data = copy.deepcopy(CONFIG)
    at = data
    for key in path[:-1]:
        at = at[key]
    if value is KeyError:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return data


@pytest.mark.parametrize("path,value", [
    (("layers", 0, "type"), "convolution"),
    (("layers", 0, "mlp", "kind"), "sparse"),
    (("layers", 0, "mixer", "left", "kv_heads"), 4),
    (("layers", 0, "mixer", "left", "rot", "dims"), 34),
    (("layers", 0, "mixer", "left", "rot", "dims"), 15),
    (("layers", 0, "mixer", "left", "mask", "size"), 0),
    (("layers", 0, "mixer", "left", "scale"), KeyError),
    (("layers", 0, "mixer", "right", "decay"), [0.5, 0.9]),
    (("layers", 1, "mixer", "decay"), [0.5, 1.5]),
    (("layers", 1, "mixer", "dim"), 300),
    (("layers", 0, "mlp", "router", "top"), 8),
    (("layers", 0, "mlp", "expert"), KeyError),
    (("layers", 1, "mlp", "ff"), 0),
    (("layers",), []),
    (("norm",), KeyError),
    (("vocab",), KeyError),
])
def test_refusals(path, value):
    with pytest.raises(ConfigError):
        KesovikConfig.from_dict(broken(path, value))


def test_the_model_as_parts():
    spec = KesovikConfig.from_dict(CONFIG).model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["side_by_side", "lightning", "side_by_side"]
    assert [layer.ffn.kind if layer.ffn else None for layer in spec.layers] == ["routed_experts", "mlp", None]
    assert all(layer.block.kind == "postnorm" and layer.block.params["alpha"] == 1.7 for layer in spec.layers)
    branches = spec.layers[0].mixer.params["branches"]
    assert [b["kind"] for b in branches] == ["attention_rows", "lightning"] and [b["scale"] for b in branches] == [0.7, 1.3]
    assert branches[0]["params"]["window"] == 24 and branches[0]["params"]["value_dim"] == 16
    assert len(spec.positions) == 1 and next(iter(spec.positions.values())).params["rotary_dim"] == 16
    assert spec.embedding.params["scale"] == 2.0 and spec.head.params["softcap"] == 9.0


def test_a_left_mixer_without_mask_or_rotation():
    """What config.json does not name does not exist: no mask means every earlier token is visible, no rot no rotation."""
    data = broken(("layers", 0, "mixer", "left", "mask"), KeyError)
    del data["layers"][0]["mixer"]["left"]["rot"]
    cfg = KesovikConfig.from_dict(data)
    assert cfg.to_dict() == data
    params = cfg.model_spec().layers[0].mixer.params["branches"][0]["params"]
    assert params["window"] is None and params["position"] is None
    assert not cfg.model_spec().positions


def test_tensor_names_and_shapes():
    names = expected_tensors(KesovikConfig.from_dict(CONFIG).model_spec())
    shape = lambda n: tuple(names[n].shape)
    assert shape("embed") == (307, 96) and shape("head") == (307, 96) and shape("final.norm") == (96,)
    assert shape("l0.mix.left.q") == (192, 96) and shape("l0.mix.left.q.b") == (192,) and shape("l0.mix.left.q.norm") == (192,)
    assert shape("l0.mix.left.k") == (64, 96) and shape("l0.mix.left.k.norm") == (64,) and shape("l0.mix.left.v.b") == (32,)
    assert shape("l0.mix.left.o") == (96, 96) and shape("l0.mix.right.g") == (96, 96) and shape("l0.mix.right.norm") == (96,)
    assert shape("l0.mlp.router") == (7, 96) and shape("l0.mlp.correction") == (7,)
    assert shape("l0.mlp.e4.down") == (96, 48) and "l0.mlp.e5.gate" not in names and shape("l0.mlp.shared.up") == (80, 96)
    assert shape("l1.mix.q") == (96, 96) and shape("l1.mix.v") == (32, 96) and shape("l1.mix.o") == (96, 32)
    assert shape("l1.mlp.up") == (160, 96) and "l1.mlp.gate" not in names
    assert shape("l0.ls1") == (96,) and shape("l0.norm2") == (96,)
    assert "l2.norm2" not in names and "l2.ls2" not in names and shape("l2.norm1") == (96,)


def test_a_layer_with_two_mixers_keeps_pages_and_a_state():
    """The cache manager serves the members of a combined spec like runs' own: equal page specs share a pool, every
    state has an array by slot, and the run is handed a view of each."""
    paged, other = PagedKVSpec(2, 32, 24), PagedKVSpec(2, 32, 7)
    state = StateSpec((3, 16, 32))
    m = CacheManager([CombinedSpec((paged, state)), StateSpec((2, 48, 16)), CombinedSpec((paged, state)),
                      CombinedSpec((other, state)), None], page_size=16, num_pages=8, max_requests=2)
    assert len(m.groups) == 2 and m.groups[0].runs == [(0, 0), (2, 0)] and m.groups[1].runs == [(3, 0)]
    assert sorted(m.state_runs, key=str) == [(0, 1), (2, 1), (3, 1), 1]
    m.add_request("a")
    m.reserve("a", 40)
    assert m.pages_needed("a", 41) == [0, 0] and m.pages_needed("a", 49) == [1, 1]
    m.advance("a", 40)
    assert m.table(1, "a")[:2] == [-1, -1] and m.table(0, "a")[0] == -1 and m.table(0, "a")[1] >= 0
    m.free_request("a")
    m.check()
    with pytest.raises(TypeError):
        CacheManager([CombinedSpec((CombinedSpec((paged,)),))], 16, 8, 2)
    with pytest.raises(TypeError):
        CacheManager([CombinedSpec(())], 16, 8, 2)


def test_step_cost_counts_the_state_and_the_chosen_experts():
    spec = KesovikConfig.from_dict(CONFIG).model_spec()
    one = step_cost(spec, [(100, 1)], 1)
    four = step_cost(spec, [(100, 1)] * 4, 4)
    assert four.cache_bytes == pytest.approx(4 * one.cache_bytes)
    states = 8.0 * (2 * 3 * 16 * 32 + 2 * 48 * 16)
    windows = 2.0 * 2 * 32 * 2 * 24 * 2           # two layers, keys and values of 2 heads stored 32 wide, 24 tokens
    assert one.cache_bytes == pytest.approx(states + windows)
    assert one.weight_bytes < four.weight_bytes     # more rows choose more experts
    prompt = step_cost(spec, [(0, 64)], 1)
    assert prompt.flops > 60 * one.flops * 0.5
