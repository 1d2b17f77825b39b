"""Tipidra's configuration on the CPU: keys, refusals, round trip, the model as parts, tensor names and shapes, cache
specs and step costs."""
import copy

import pytest

from pulse_infer_amd.config import ConfigError, TipidraConfig, config_from_dict
from pulse_infer_amd.models.causal_lm import expected_tensors

BASE = {
    "architecture": "Tipidra", "vocab": 99, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.5},
    "logit_softcap": 12.0, "streams": 3,
    "layers": [
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.3, "softcap": 25.0,
                                        "rot": {"base": 5000.0, "dims": 8}},
         "mlp": {"kind": "dense", "ff": 80}},
        {"type": "mamba1", "mixer": {"inner": 72, "state": 6, "dt_rank": 5, "conv": 3},
         "mlp": {"kind": "moe", "expert": {"ff": 24, "limit": 1.5}, "router": {"experts": 5, "top": 2}}},
        {"type": "attention", "mixer": {"heads": 2, "dim": 24, "scale": 1.0}, "mlp": None},
    ],
}


def test_keys_become_parts():
    cfg = config_from_dict(BASE)
    assert isinstance(cfg, TipidraConfig) and cfg.streams == 3 and cfg.embedding_scale == 2.5
    spec = cfg.model_spec()
    assert spec.streams == 3 and spec.embedding.params["streams"] == 3 and spec.embedding.params["scale"] == 2.5
    assert [layer.block.kind for layer in spec.layers] == ["hyper"] * 3
    a = spec.layers[0].mixer
    assert a.kind == "attention_rows" and a.params["value_dim"] == 8 and a.params["score_cap"] == 25.0
    assert a.params["qk_norm"] == "head" and a.params["sink"] and a.params["output_gate"] == "channel"
    rope = spec.positions[a.params["position"]]
    assert rope.params == {"theta": 5000.0, "rotary_dim": 8, "head_dim": 16, "pairing": "half"}
    assert spec.layers[0].ffn.kind == "gated_mlp" and spec.layers[0].ffn.params["activation"] == "gelu_tanh"
    m = spec.layers[1].mixer
    assert m.kind == "mamba" and (m.params["inner"], m.params["state"], m.params["dt_rank"], m.params["conv"]) == (72, 6, 5, 3)
    f = spec.layers[1].ffn
    assert f.kind == "routed_experts" and f.params["score"] == "sigmoid" and f.params["renormalize"] is False
    assert f.params["weight_on"] == "input" and f.params["expert_activation"] == "clamped_swish" and f.params["limit"] == 1.5
    last = spec.layers[2]
    assert last.ffn is None and last.mixer.params["num_kv_heads"] == 2 and last.mixer.params["value_dim"] == 24
    assert last.mixer.params["position"] is None and last.mixer.params["score_cap"] == 0.0
    assert spec.final_norm.kind == "layernorm" and spec.head.params["softcap"] == 12.0


def test_tensor_names_and_shapes():
    names = expected_tensors(config_from_dict(BASE).model_spec())
    shape = lambda n: tuple(names[n].shape)
    assert shape("embed") == (99, 48) and shape("head") == (99, 48)
    assert shape("final.norm") == (48,) and shape("final.norm.b") == (48,)
    assert shape("l0.norm1") == (48,) and shape("l0.norm2.b") == (48,)
    assert shape("l0.hc1.in") == (3,) and shape("l0.hc2.out") == (3,) and shape("l1.hc1.mix") == (3, 3)
    assert shape("l0.mix.q") == (96, 48) and shape("l0.mix.k") == (32, 48) and shape("l0.mix.v") == (16, 48)
    assert shape("l0.mix.g") == (48, 48) and shape("l0.mix.o") == (48, 48) and shape("l0.mix.sink") == (6,)
    assert shape("l0.mlp.gate") == (80, 48) and shape("l0.mlp.down") == (48, 80)
    assert shape("l1.mix.in") == (144, 48) and shape("l1.mix.conv") == (72, 3) and shape("l1.mix.conv.b") == (72,)
    assert shape("l1.mix.x") == (17, 72) and shape("l1.mix.dt") == (72, 5) and shape("l1.mix.dt.b") == (72,)
    assert shape("l1.mix.A_log") == (72, 6) and shape("l1.mix.D") == (72,) and shape("l1.mix.o") == (48, 72)
    assert shape("l1.mlp.router") == (5, 48) and shape("l1.mlp.e4.up") == (24, 48) and shape("l1.mlp.e0.down") == (48, 24)
    assert "l2.norm2" not in names and "l2.hc2.in" not in names and "l2.mlp.gate" not in names


def test_round_trip():
    cfg = config_from_dict(BASE)
    again = config_from_dict(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()
    assert again.to_dict()["layers"][2]["mixer"] == {"dim": 24, "heads": 2, "kv_heads": 2, "scale": 1.0, "vdim": 24}


def test_without_the_streams_key_the_residual_is_one_row():
    data = copy.deepcopy(BASE)
    del data["streams"]
    spec = config_from_dict(data).model_spec()
    assert spec.streams == 1 and spec.layers[0].block.params["learned"] is False
    assert not any(".hc" in name for name in expected_tensors(spec))
    assert "streams" not in config_from_dict(data).to_dict()


@pytest.mark.parametrize("change,words", [
    (lambda d: d["layers"][0].update(type="conv"), "no mixer 'conv'"),
    (lambda d: d["layers"][0]["mlp"].update(kind="glu"), "no feed-forward 'glu'"),
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=4), "shared out evenly"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7), "must be even"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=18), "at most dim"),
    (lambda d: d["layers"][1]["mixer"].update(conv=17), "at most 16 taps"),
    (lambda d: d["layers"][1]["mixer"].pop("state"), "'state'"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=6), "cannot be chosen"),
    (lambda d: d["layers"][1]["mlp"]["expert"].update(limit=0.0), "must be positive"),
    (lambda d: d.update(streams=0), "between 1 and"),
    (lambda d: d.update(streams=17), "between 1 and"),
    (lambda d: d.pop("width"), "'width'"),
])
def test_refusals(change, words):
    data = copy.deepcopy(BASE)
    change(data)
    with pytest.raises(ConfigError) as err:
        config_from_dict(data)
    assert words in str(err.value)


def test_cache_specs_and_costs():
    from pulse_infer_amd.cache.specs import PagedKVSpec, StateSpec
    from pulse_infer_amd.models.cost import step_cost
    from pulse_infer_amd.parts.attention_rows import RowPreparedAttention, stored_width
    from pulse_infer_amd.parts.mamba import SelectiveStateSpace

    spec = config_from_dict(BASE).model_spec()
    assert stored_width(16, 8) == 16 and stored_width(24, 24) == 32
    m = spec.layers[1].mixer.params
    cost = SelectiveStateSpace.step_cost(m, [(10, 4), (0, 1)], 2, 2)
    assert cost.cache_bytes == 8.0 * 72 * (6 + 2) * 2 and cost.flops > 0
    a = RowPreparedAttention.step_cost(spec.layers[0].mixer.params, [(10, 4)], 2, 2)
    assert a.cache_bytes == 2.0 * 2 * 16 * 2 * 14
    whole = step_cost(spec, [(0, 7), (30, 1)], 2)
    assert whole.flops > 0 and whole.weight_bytes > 0 and whole.cache_bytes > 0
    assert StateSpec((72, 8), "float32") == StateSpec((72, 8), "float32") and PagedKVSpec(2, 16, None).per_token
