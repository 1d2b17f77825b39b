"""Fosupel's configuration on the CPU: keys, refusals, the round trip, the order of running with its loop, the model
as a list of parts, tensor names and shapes, the cache of its runs (pages of kept first tokens), and step costs."""
import copy

import pytest

from pulse_infer_amd.cache.manager import CacheManager
from pulse_infer_amd.cache.specs import CombinedSpec, PagedKVSpec, StateSpec
from pulse_infer_amd.config import ConfigError, FosupelConfig, config_from_dict
from pulse_infer_amd.models.causal_lm import expected_tensors
from pulse_infer_amd.models.cost import step_cost

LEFT = {"dim": 32, "heads": 6, "kv_heads": 3, "mask": {"keep_first": 3, "size": 24},
        "rot": {"base": 1e4, "dims": 16, "scaling": {"factor": 4.0}}, "scale": 0.2, "vdim": 16}
RIGHT = {"decay": [0.5, 0.9, 0.99], "dim": 16, "heads": 3, "rot": {"base": 500.0, "dims": 8}, "vdim": 32}
LATENT = {"dim": 16, "heads": 3, "kv_rank": 40, "rot": {"base": 1e4, "dims": 8}, "rot_dim": 8, "scale": 0.2, "vdim": 24}
CONFIG = {
    "architecture": "Fosupel", "logit_softcap": 11.0, "loop": {"start": 1, "stop": 3, "times": 3}, "norm": {"eps": 1e-5},
    "residual_mult": 0.7, "vocab": 311, "width": 96,
    "layers": [
        {"type": "latent_attention", "mixer": LATENT, "mlp": {"kind": "dense", "ff": 160}},
        {"type": "parallel", "mixer": {"left": LEFT, "left_scale": 0.7, "right": RIGHT, "right_scale": 1.3},
         "mlp": {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 80}}},
        {"type": "parallel", "mixer": {"left": LEFT, "left_scale": 1.0, "right": RIGHT, "right_scale": 1.0}, "mlp": None},
        {"type": "latent_attention", "mixer": LATENT,
         "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 3, "top": 1}}},
    ],
}


def test_round_trip_and_registry():
    cfg = config_from_dict(CONFIG)
    assert isinstance(cfg, FosupelConfig)
    assert cfg.to_dict() == CONFIG
    assert FosupelConfig.from_dict(cfg.to_dict()).to_dict() == CONFIG
    assert (cfg.vocab_size, cfg.width, cfg.residual_mult, cfg.logit_softcap) == (311, 96, 0.7, 11.0)
    assert (cfg.loop_start, cfg.loop_stop, cfg.loop_times) == (1, 3, 3)


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
    (("layers", 1, "mlp", "kind"), "sparse"),
    (("layers", 1, "mixer", "left", "kv_heads"), 4),
    (("layers", 1, "mixer", "left", "rot", "dims"), 34),
    (("layers", 1, "mixer", "left", "rot", "dims"), 15),
    (("layers", 1, "mixer", "left", "rot", "scaling", "factor"), 0.0),
    (("layers", 1, "mixer", "left", "mask", "size"), 0),
    (("layers", 1, "mixer", "left", "mask", "keep_first"), -1),
    (("layers", 1, "mixer", "left", "scale"), KeyError),
    (("layers", 1, "mixer", "right", "decay"), [0.5, 0.9]),
    (("layers", 1, "mixer", "right", "decay"), [0.5, 0.9, 1.5]),
    (("layers", 1, "mixer", "right", "dim"), 300),
    (("layers", 0, "mixer", "rot_dim"), 6),
    (("layers", 0, "mixer", "kv_rank"), KeyError),
    (("layers", 0, "mixer", "rot"), None),
    (("layers", 1, "mlp", "router", "top"), 8),
    (("layers", 1, "mlp", "expert"), KeyError),
    (("layers", 0, "mlp", "ff"), 0),
    (("loop", "stop"), 5),
    (("loop", "start"), 4),
    (("loop", "times"), 0),
    (("layers",), []),
    (("norm",), KeyError),
    (("vocab",), KeyError),
])
def test_refusals(path, value):
    with pytest.raises(ConfigError):
        FosupelConfig.from_dict(broken(path, value))


def test_the_order_of_running():
    spec = FosupelConfig.from_dict(CONFIG).model_spec()
    assert [(run.layer, run.offset) for run in spec.order] == [
        (0, None), (1, ("loop.step", 0)), (2, None), (1, ("loop.step", 1)), (2, None), (1, ("loop.step", 2)), (2, None),
        (3, None)]
    assert spec.offsets == {"loop.step": 3}
    plain = copy.deepcopy(CONFIG)
    del plain["loop"]
    spec = FosupelConfig.from_dict(plain).model_spec()
    assert [(run.layer, run.offset) for run in spec.order] == [(i, None) for i in range(4)] and not spec.offsets
    assert "loop.step" not in expected_tensors(spec)
    whole = copy.deepcopy(CONFIG)
    whole["loop"] = {"start": 0, "stop": 4, "times": 2}
    spec = FosupelConfig.from_dict(whole).model_spec()
    assert [run.layer for run in spec.order] == [0, 1, 2, 3, 0, 1, 2, 3]
    assert [run.offset for run in spec.order if run.offset] == [("loop.step", 0), ("loop.step", 1)]


def test_the_model_as_parts():
    spec = FosupelConfig.from_dict(CONFIG).model_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["latent_attention", "side_by_side", "side_by_side",
                                                           "latent_attention"]
    assert [layer.ffn.kind if layer.ffn else None for layer in spec.layers] == ["mlp", "routed_experts", None,
                                                                                "routed_experts"]
    assert all(layer.block.kind == "prenorm_scaled" and layer.block.params["residual_scale"] == 0.7 for layer in spec.layers)
    branches = spec.layers[1].mixer.params["branches"]
    assert [b["kind"] for b in branches] == ["attention_rows", "lightning"] and [b["scale"] for b in branches] == [0.7, 1.3]
    left, right = branches[0]["params"], branches[1]["params"]
    assert (left["window"], left["keep_first"], left["value_dim"], left["talk"], left["sink"]) == (24, 3, 16, True, True)
    assert spec.positions[left["position"]].params == {"theta": 1e4, "rotary_dim": 16, "head_dim": 32, "pairing": "half",
                                                       "scaling_factor": 4.0}
    assert (right["key_scale"], right["norm"], right["norm_weight"], right["gate_activation"], right["activation"]) == (
        0.25, "head", False, "silu", "none")
    assert spec.positions[right["position"]].params["pairing"] == "half"
    latent = spec.layers[0].mixer.params
    assert spec.positions[latent["position"]].params["pairing"] == "interleaved"
    assert (latent["latent_dim"], latent["rotary_dim"], latent["output_gate"]) == (40, 8, True)
    routed = spec.layers[1].ffn.params
    assert (routed["renormalize"], routed["shared_gate"], routed["shared_size"]) == (False, True, 80)
    assert spec.layers[3].ffn.params["shared_gate"] is False
    assert spec.layers[0].ffn.params["activation"] == "xielu"
    assert spec.head.params["tied"] and spec.head.params["softcap"] == 11.0


def test_tensor_names_and_shapes():
    names = expected_tensors(FosupelConfig.from_dict(CONFIG).model_spec())
    shape = lambda n: tuple(names[n].shape)
    assert shape("embed") == (311, 96) and shape("loop.step") == (3, 96) and shape("final.norm") == (96,)
    assert shape("l1.mix.left.q") == (192, 96) and shape("l1.mix.left.k") == (96, 96) and shape("l1.mix.left.v") == (48, 96)
    assert shape("l1.mix.left.talk") == (6, 6) and shape("l1.mix.left.sink") == (6,) and shape("l1.mix.left.o") == (96, 96)
    assert shape("l1.mix.right.q") == (48, 96) and shape("l1.mix.right.v") == (96, 96) and shape("l1.mix.right.g") == (96, 96)
    assert "l1.mix.right.norm" not in names
    assert shape("l0.mix.q") == (72, 96) and shape("l0.mix.dkv") == (48, 96) and shape("l0.mix.dkv.norm") == (40,)
    assert shape("l0.mix.uk") == (48, 40) and shape("l0.mix.uv") == (72, 40) and shape("l0.mix.g") == (72, 96)
    assert shape("l0.mix.sink") == (3,) and shape("l0.mix.o") == (96, 72)
    assert shape("l0.mlp.up") == (160, 96) and shape("l0.mlp.act") == (2,)
    assert shape("l1.mlp.router") == (5, 96) and shape("l1.mlp.e4.down") == (96, 48)
    assert shape("l1.mlp.shared.sg") == (1, 96) and shape("l1.mlp.shared.gate") == (80, 96)
    assert "l3.mlp.shared.sg" not in names and "l2.norm2" not in names and "l2.norm1" in names
    assert names["head"].optional


def test_the_cache_keeps_the_pages_of_the_first_tokens():
    """A window group gives back the pages its window has passed, but not those that hold kept first tokens; every
    pass of the loop has a cache of its own."""
    kv = PagedKVSpec(3, 32, 24, 3)
    latent = PagedKVSpec(1, 48, None)
    state = StateSpec((3, 16, 32), "float32")
    runs = [latent, CombinedSpec((kv, state)), CombinedSpec((kv, state)), CombinedSpec((kv, state))]
    cache = CacheManager(runs, page_size=4, num_pages=64, max_requests=2)
    window = next(g for g in cache.groups if g.window == 24)
    assert len(window.runs) == 3
    cache.add_request("a")
    cache.reserve("a", 60)
    cache.advance("a", 60)
    table = window.tables["a"]
    assert table[0] >= 0, "the page of the kept first tokens was given back"
    assert all(p == -1 for p in table[1:9]) and all(p >= 0 for p in table[9:15])   # positions 37 .. 59 are in the window
    whole = next(g for g in cache.groups if g.window is None)
    assert all(p >= 0 for p in whole.tables["a"])
    cache.free_request("a")
    cache.check()
    assert window.pool.num_free == window.pool.num_pages


def test_step_costs():
    cfg = FosupelConfig.from_dict(CONFIG)
    decode = step_cost(cfg.model_spec(), [(100, 1)], 1)
    prompt = step_cost(cfg.model_spec(), [(0, 101)], 1)
    assert 0 < decode.flops < prompt.flops and decode.weight_bytes > 0 and decode.cache_bytes > 0
    longer = step_cost(cfg.model_spec(), [(1000, 1)], 1)
    # only the latent layers read more of a longer context: the windows and the states do not grow
    grown = longer.cache_bytes - decode.cache_bytes
    assert grown == pytest.approx(2 * 2.0 * 48 * 2 * 900)
