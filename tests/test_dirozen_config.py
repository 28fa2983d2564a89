"""Dirozen's configuration on the CPU: reading config.json's keys, what is refused, the round trip through
``to_dict``, the tensors the model expects and the parts it is described with."""
import copy
import json

import pytest

from pulse_infer_amd.config import ConfigError, DirozenConfig, config_from_dict, load_config
from pulse_infer_amd.models.causal_lm import expected_tensors
from pulse_infer_amd.models.cost import step_cost


def layer(heads, kv_heads, dim, scale, coef, every, ff):
    return {"type": "attention",
            "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "q_temp": {"coef": coef, "every": every},
                      "scale": scale, "vdim": dim},
            "mlp": None if ff is None else {"ff": ff, "kind": "dense"}}


CFG = {"architecture": "Dirozen", "vocab": 301, "width": 96, "norm": {"eps": 1e-5},
       "layers": [layer(6, 2, 32, 0.2, 0.25, 7, 160), layer(4, 4, 16, 0.3, 0.5, 16, None)]}


def test_the_architecture_is_found_by_its_name_and_reads_its_keys(tmp_path):
    cfg = config_from_dict(CFG)
    assert isinstance(cfg, DirozenConfig)
    assert (cfg.vocab_size, cfg.width, cfg.norm_eps, len(cfg.layers)) == (301, 96, 1e-5, 2)
    first, second = cfg.layers
    assert (first.heads, first.kv_heads, first.dim, first.scale, first.temp_coef, first.temp_every, first.ff) == \
        (6, 2, 32, 0.2, 0.25, 7, 160)
    assert second.ff is None
    assert cfg.to_dict() == CFG
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    assert load_config(str(tmp_path)).to_dict() == CFG


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="recurrence"), "mixer"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "feed-forward"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "evenly"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["q_temp"].update(every=0), "positive"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("q_temp"), "q_temp"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "layers"),
    (lambda c: c.pop("width"), "width"),
])
def test_what_the_configuration_refuses(change, word):
    cfg = copy.deepcopy(CFG)
    change(cfg)
    with pytest.raises(ConfigError) as err:
        config_from_dict(cfg)
    assert word in str(err.value)


def test_the_tensors_and_parts_of_the_model():
    cfg = config_from_dict(CFG)
    spec = cfg.model_spec()
    tensors = expected_tensors(spec)
    assert {name: tuple(t.shape) for name, t in tensors.items()} == {
        "embed": (301, 96), "head": (301, 96), "final.norm": (96,),
        "l0.norm1": (96,), "l0.mix.q": (192, 96), "l0.mix.k": (64, 96), "l0.mix.g": (6, 96), "l0.mix.o": (96, 192),
        "l0.mlp.gate": (160, 96), "l0.mlp.up": (160, 96), "l0.mlp.down": (96, 160),
        "l1.norm1": (96,), "l1.mix.q": (64, 96), "l1.mix.k": (64, 96), "l1.mix.g": (4, 96), "l1.mix.o": (96, 64)}
    assert tensors["l0.norm1"].kind == "norm_offset"
    assert [l.block.kind for l in spec.layers] == ["parallel", "parallel"] and spec.layers[1].ffn is None
    mixer = spec.layers[0].mixer.params
    assert mixer["values"] == "keys" and mixer["output_gate"] and not mixer["qk_norm_weights"] and mixer["position"] is None
    assert mixer["query_temperature"] == {"coef": 0.25, "every": 7} and mixer["scale"] == 0.2
    # a step's cost comes from the parts: one token at position 9 reads ten keys and values of every kv head
    one = step_cost(spec, [(9, 1)], wanted=1)
    assert one.cache_bytes == 2 * 10 * 2 * (2 * 32 + 4 * 16)
    weights = sum(t.shape[0] * (t.shape[1] if len(t.shape) > 1 else 1) for n, t in tensors.items() if n != "embed")
    assert one.weight_bytes == 2 * (weights + 96)          # every tensor once, one row of the embedding


def test_max_positions_is_an_option_of_the_engine():
    cfg = config_from_dict(CFG)
    assert cfg.model_spec().max_positions == cfg.max_positions > 100000
    cfg.apply_overrides({"max_positions": 77})
    assert cfg.model_spec().max_positions == 77
    with pytest.raises(ConfigError):
        cfg.apply_overrides({"max_positions": 0})
    assert "max_positions" in DirozenConfig.engine_options
