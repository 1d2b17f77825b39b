"""Tipidra: a decoder whose layers are listed one by one in config.json, around a residual kept in several streams.

config.json holds ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``logit_softcap``,
``streams`` and ``layers``: for each layer its ``type`` (the mixer), the mixer's sizes and constants (``mixer``) and
its feed-forward (``mlp``, or null for none).  Every size and constant is taken from there.  Tensors: ``embed``,
``l<i>.norm1`` / ``norm2`` (layer norms: weight, and bias with ``.b`` appended), ``l<i>.hc1.*`` / ``hc2.*`` (``in``,
``out``, ``mix``), ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm`` (+ ``.b``), ``head``.

The model: every stream starts as embed[token] * embedding.scale.  Sublayer q of a layer (1 the mixer, 2 the
feed-forward) reads u = sum_s in_q[s] x_s through its layer norm and its result y goes back into all streams at
once, x_t <- sum_s mix_q[s, t] x_s + out_q[t] y.  A configuration without ``streams`` has the plain residual sum.
The logits are head(final.norm(sum_s x_s)), then cap * tanh(. / cap).

Mixers.  ``attention``: grouped query heads (``heads``, ``kv_heads``; keys of ``dim`` and values of ``vdim`` channels),
a rotation of the first ``rot.dims`` channels of every head of q and k in pairs (i, i + dims / 2) by position *
``rot.base``^(-2i / dims), q and k divided head by head by their root mean square, scores (q . k) ``scale`` capped by
``softcap`` tanh(. / ``softcap``), every earlier token visible, a sink per head in the softmax's denominator, the
heads' outputs multiplied element by element by sigmoid(Wg h).  ``mamba1``: a selective state-space mixer
(``inner``, ``state``, ``dt_rank``, ``conv`` taps) with a float32 state per request.

Feed-forwards.  ``dense``: down(gelu_tanh(gate h) * (up h)).  ``moe``: ``router.experts`` experts of width
``expert.ff``; sigmoid scores of router logits formed in float32, the ``router.top`` largest chosen, an expert fed
score * h, results added as they are; an expert is down(g * sigmoid(1.702 g) * (u + 1)) with g = min(gate h,
``expert.limit``) and u = clamp(up h, -limit, limit).

All of that is said to the engine as parameters of registered parts (``model_spec``); there is no model class.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, JsonReader, ModelConfig, require_positive
from ..models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

ARCHITECTURE = "Tipidra"
MIXER_TYPES = ("attention", "mamba1")
MLP_KINDS = ("dense", "moe")
MAX_STREAMS = 16


def _object(value: Any, where: str, what: str) -> Dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"'{where}': key '{what}' must be an object")
    return value


@dataclass
class SinkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float              # 0: config.json names none
    rot_base: float
    rot_dims: int               # 0: config.json names no rotation

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "SinkAttentionSizes":
        r = JsonReader(data, where)
        dim = r.integer("dim")
        base, dims = 1.0, 0
        if r.raw("rot") is not None:
            rot = JsonReader(_object(r.raw("rot"), where, "rot"), f"{where}.rot")
            base, dims = rot.number("base"), rot.integer("dims")
        heads = r.integer("heads")
        return cls(heads=heads, kv_heads=r.integer("kv_heads", heads), dim=dim, vdim=r.integer("vdim", dim),
                   scale=r.number("scale"), softcap=r.number("softcap", 0.0), rot_base=base, rot_dims=dims)

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim)
        if self.heads % self.kv_heads:
            raise ConfigError(f"'{where}': {self.heads} query heads cannot be shared out evenly over {self.kv_heads} "
                              "key/value heads")
        if self.softcap < 0.0:
            raise ConfigError(f"'{where}': softcap ({self.softcap}) must not be negative")
        if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ConfigError(f"'{where}': rot.dims ({self.rot_dims}) must be even and at most dim ({self.dim})")
        if self.rot_dims and not self.rot_base > 0:
            raise ConfigError(f"'{where}': rot.base must be positive")

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return out


@dataclass
class MambaSizes:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "MambaSizes":
        r = JsonReader(data, where)
        return cls(inner=r.integer("inner"), state=r.integer("state"), dt_rank=r.integer("dt_rank"),
                   conv=r.integer("conv"))

    def check(self, where: str) -> None:
        require_positive(where, inner=self.inner, state=self.state, dt_rank=self.dt_rank, conv=self.conv)
        if self.conv > 16:
            raise ConfigError(f"'{where}': the convolution's kernel takes at most 16 taps, conv is {self.conv}")
        if self.state > 256:
            raise ConfigError(f"'{where}': the recurrence's kernel takes at most 256 states a channel, state is {self.state}")

    def to_dict(self) -> Dict[str, Any]:
        return {"conv": self.conv, "dt_rank": self.dt_rank, "inner": self.inner, "state": self.state}


@dataclass
class TipidraMLP:
    kind: str
    ff: int = 0                 # dense: the inner width; moe: an expert's
    experts: int = 0
    top: int = 0
    limit: float = 0.0

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "TipidraMLP":
        r = JsonReader(data, where)
        kind = r.string("kind")
        if kind not in MLP_KINDS:
            raise ConfigError(f"'{where}': there is no feed-forward '{kind}' (known: {', '.join(MLP_KINDS)})")
        if kind == "dense":
            return cls(kind=kind, ff=r.integer("ff"))
        router = JsonReader(_object(r.raw("router"), where, "router"), f"{where}.router")
        expert = JsonReader(_object(r.raw("expert"), where, "expert"), f"{where}.expert")
        return cls(kind=kind, ff=expert.integer("ff"), experts=router.integer("experts"), top=router.integer("top"),
                   limit=expert.number("limit"))

    def check(self, where: str) -> None:
        require_positive(where, ff=self.ff)
        if self.kind == "moe":
            require_positive(where, experts=self.experts, top=self.top)
            if self.top > self.experts:
                raise ConfigError(f"'{where}': {self.top} of {self.experts} experts cannot be chosen")
            if self.top > 64 or self.experts > 1024:
                raise ConfigError(f"'{where}': the router's kernel takes at most 1024 experts and 64 choices")
            if not self.limit > 0.0:
                raise ConfigError(f"'{where}': expert.limit ({self.limit}) must be positive")

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                "router": {"experts": self.experts, "top": self.top}}


@dataclass
class TipidraLayer:
    type: str
    attention: Optional[SinkAttentionSizes] = None
    mamba: Optional[MambaSizes] = None
    mlp: Optional[TipidraMLP] = None

    def to_dict(self) -> Dict[str, Any]:
        mixer = self.attention.to_dict() if self.type == "attention" else self.mamba.to_dict()
        return {"mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass
class TipidraConfig(ModelConfig):
    vocab_size: int
    width: int
    norm_eps: float
    embedding_scale: float = 1.0
    logit_softcap: float = 0.0      # 0: none
    streams: Optional[int] = None   # None: config.json names none, the residual is one row with the plain sum
    layers: List[TipidraLayer] = field(default_factory=list)
    eos_token_ids: List[int] = field(default_factory=list)
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    # An option of the engine, not a key of config.json: the most positions a request may reach.
    max_positions: int = 1 << 20
    architecture: str = ARCHITECTURE

    engine_options = {
        "max_positions": {"type": int, "help": "the most positions a request may reach (the design sets no limit)"}}

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Dict[str, Any], origin: str = "<dict>", generation: Optional[Dict[str, Any]] = None,
                  generation_origin: str = "<dict>") -> "TipidraConfig":
        r = JsonReader(data, origin)
        norm = JsonReader(_object(r.raw("norm"), origin, "norm"), f"{origin}: norm")
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"'{origin}': key 'layers' must be a list with at least one layer")
        scale = 1.0
        if r.raw("embedding") is not None:
            scale = JsonReader(_object(r.raw("embedding"), origin, "embedding"), f"{origin}: embedding").number("scale", 1.0)
        cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"), norm_eps=norm.number("eps"),
                  embedding_scale=scale, logit_softcap=r.number("logit_softcap", 0.0),
                  streams=r.integer("streams", None),
                  layers=[cls._read_layer(entry, f"{origin}: layers[{i}]") for i, entry in enumerate(listed)],
                  eos_token_ids=r.int_or_int_list("eos_token_id"))
        cfg.read_generation_defaults(generation, generation_origin)
        cfg.validate(origin)
        return cfg

    @staticmethod
    def _read_layer(entry: Any, origin: str) -> TipidraLayer:
        if not isinstance(entry, dict):
            raise ConfigError(f"'{origin}' must be an object")
        r = JsonReader(entry, origin)
        kind = r.string("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"'{origin}': there is no mixer '{kind}' (known: {', '.join(MIXER_TYPES)})")
        mixer = _object(r.raw("mixer"), origin, "mixer")
        layer = TipidraLayer(type=kind)
        if kind == "attention":
            layer.attention = SinkAttentionSizes.read(mixer, f"{origin}.mixer")
        else:
            layer.mamba = MambaSizes.read(mixer, f"{origin}.mixer")
        mlp = r.raw("mlp")
        if mlp is not None:
            layer.mlp = TipidraMLP.read(_object(mlp, origin, "mlp"), f"{origin}.mlp")
        return layer

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        require_positive(origin, vocab=self.vocab_size, width=self.width, max_positions=self.max_positions)
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"'{origin}': norm.eps ({self.norm_eps}) must not be negative")
        if self.logit_softcap < 0.0:
            raise ConfigError(f"'{origin}': logit_softcap ({self.logit_softcap}) must not be negative")
        if self.streams is not None and not 1 <= self.streams <= MAX_STREAMS:
            raise ConfigError(f"'{origin}': streams ({self.streams}) must lie between 1 and {MAX_STREAMS}")
        if self.width * 4 > 60 * 1024:
            raise ConfigError(f"'{origin}': the norm's kernel takes rows of at most {60 * 1024 // 4} values")
        if not self.layers:
            raise ConfigError(f"'{origin}': a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"{origin}: layers[{i}]"
            (layer.attention if layer.type == "attention" else layer.mamba).check(f"{where}.mixer")
            if layer.mlp is not None:
                layer.mlp.check(f"{where}.mlp")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architecture": self.architecture,
            "embedding": {"scale": self.embedding_scale},
            "layers": [layer.to_dict() for layer in self.layers],
            "logit_softcap": self.logit_softcap,
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab_size,
            "width": self.width,
        }
        if self.streams is not None:
            out["streams"] = self.streams
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------ the model
    def model_spec(self) -> ModelSpec:
        streams = self.streams if self.streams is not None else 1
        norm = PartSpec("layernorm", {"size": self.width, "eps": self.norm_eps, "tensor": "", "bias_tensor": "b",
                                      "streams": streams})
        block = PartSpec("hyper", {"streams": streams, "learned": self.streams is not None, "mixer_norm": "norm1",
                                   "ffn_norm": "norm2", "mixer_hc": "hc1", "ffn_hc": "hc2"})
        layers = []
        positions: Dict[str, PartSpec] = {}
        for i, layer in enumerate(self.layers):
            if layer.type == "attention":
                a = layer.attention
                rope = None
                if a.rot_dims:
                    rope = f"rope:{a.rot_base!r}:{a.rot_dims}:{a.dim}"
                    positions.setdefault(rope, PartSpec("rope", {"theta": a.rot_base, "rotary_dim": a.rot_dims,
                                                                 "head_dim": a.dim, "pairing": "half"}))
                mixer = PartSpec("attention_rows", {
                    "hidden_size": self.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
                    "value_dim": a.vdim, "qk_norm": "head", "qk_norm_eps": self.norm_eps, "scale": a.scale,
                    "score_cap": a.softcap, "sink": True, "output_gate": "channel", "position": rope, "prefix": "mix"})
            else:
                m = layer.mamba
                mixer = PartSpec("mamba", {"hidden_size": self.width, "inner": m.inner, "state": m.state,
                                           "dt_rank": m.dt_rank, "conv": m.conv, "prefix": "mix"})
            ffn = None
            if layer.mlp is not None and layer.mlp.kind == "dense":
                ffn = PartSpec("gated_mlp", {"hidden_size": self.width, "intermediate_size": layer.mlp.ff,
                                             "activation": "gelu_tanh", "prefix": "mlp",
                                             "names": {"gate": "gate", "up": "up", "down": "down"}})
            elif layer.mlp is not None:
                m = layer.mlp
                ffn = PartSpec("routed_experts", {"hidden_size": self.width, "expert_size": m.ff, "num_experts": m.experts,
                                                  "top": m.top, "score": "sigmoid", "renormalize": False,
                                                  "weight_on": "input", "expert_activation": "clamped_swish",
                                                  "limit": m.limit, "prefix": "mlp"})
            layers.append(LayerSpec(prefix=f"l{i}", mixer=mixer, ffn=ffn, norms={"mixer_norm": norm, "ffn_norm": norm},
                                    block=block))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.width,
            max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "embed",
                                             "scale": self.embedding_scale, "streams": streams}),
            layers=layers,
            order=[RunSpec(layer=i) for i in range(len(layers))],
            final_norm=norm,
            final_norm_prefix="final.norm",
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "head",
                                      "tied": False, "softcap": self.logit_softcap}),
            positions=positions,
            streams=streams,
        )
        spec.validate()
        return spec
