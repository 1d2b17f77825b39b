"""Fosupel: a decoder whose layers are listed one by one in config.json, some of which run several times in a row.

config.json holds ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``logit_softcap``, ``loop``
(``start``, ``stop``, ``times``) and ``layers``: for each layer its ``type`` (the mixer), the mixer's sizes and
constants (``mixer``) and its feed-forward (``mlp``, or null for none).  Every size and constant is taken from there.
Tensors: ``embed``, ``loop.step`` [times, width], ``l<i>.norm1`` / ``norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``; the logits are a product with ``embed``.

The model: x = embed[token]; per layer x <- x + m mixer(norm1(x)), then x <- x + m ff(norm2(x)) with m =
``residual_mult`` and RMSNorms with plain weights.  Layers ``start`` .. ``stop - 1`` run ``times`` times in a row with
the same weights (every pass with a cache and state of its own), and row t of ``loop.step`` is added to x right
before pass t.  logits = embed final.norm(x), then cap * tanh(logits / cap).

Mixers.  ``parallel``: two mixers side by side on the same input, ``left_scale * left + right_scale * right``.  Left:
softmax attention with grouped key/value heads (``heads``, ``kv_heads``, ``dim``, ``vdim``), a rotation of the first
``rot.dims`` channels of every head in pairs (i, i + dims / 2) with every frequency divided by ``rot.scaling.factor``,
``scale`` on the scores, a window of ``mask.size`` tokens below which the first ``mask.keep_first`` tokens stay
visible, a learned sink per head in the softmax's denominator, and the heads' weights mixed by the matrix ``talk``.
Right: linear attention with a constant decay per head (``heads``, ``dim``, ``vdim``, ``decay``), q and k turned
(``rot``), k times dim^(-1/2), every head's output divided by its root mean square, the heads multiplied by
silu(W_g x).  ``latent_attention``: keys and values from one normed latent row a token (``kv_rank``) and one turned key
part (``rot_dim`` channels, adjacent pairs) shared by all heads; sinks; an output gate a channel.

Feed-forwards.  ``dense``: down(xielu(up x)) with two learned numbers.  ``moe``: ``router.experts`` gated experts of
width ``expert.ff``, ``router.top`` a token by softmax score, weighted by the scores as they are; a shared gated expert
(``shared.ff``) for every token, times sigmoid(w_sg . x).

All of that is said to the engine as parameters of registered parts (``model_spec``); there is no model class.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, JsonReader, ModelConfig, require_positive
from ..models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

ARCHITECTURE = "Fosupel"
MIXER_TYPES = ("parallel", "latent_attention")
MLP_KINDS = ("dense", "moe")


def _object(value: Any, where: str, what: str) -> Dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"'{where}': key '{what}' must be an object")
    return value


@dataclass
class Rotation:
    base: float = 1.0
    dims: int = 0               # 0: config.json names no rotation
    factor: float = 1.0         # every frequency is divided by it

    @classmethod
    def read(cls, value: Any, where: str) -> "Rotation":
        if value is None:
            return cls()
        r = JsonReader(_object(value, where, "rot"), f"{where}.rot")
        factor = 1.0
        if r.raw("scaling") is not None:
            factor = JsonReader(_object(r.raw("scaling"), f"{where}.rot", "scaling"), f"{where}.rot.scaling").number("factor", 1.0)
        return cls(base=r.number("base"), dims=r.integer("dims"), factor=factor)

    def check(self, where: str, most: int) -> None:
        if self.dims < 0 or self.dims % 2 or self.dims > most:
            raise ConfigError(f"'{where}': rot.dims ({self.dims}) must be even and at most {most}")
        if self.dims and not (self.base > 0 and self.factor > 0):
            raise ConfigError(f"'{where}': rot.base and rot.scaling.factor must be positive")

    def to_dict(self) -> Optional[Dict[str, Any]]:
        if not self.dims:
            return None
        out: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            out["scaling"] = {"factor": self.factor}
        return out

    def position(self, head_dim: int, pairing: str, positions: Dict[str, PartSpec]) -> Optional[str]:
        """The name under which the model lists this rotation (listed on the way); None without one."""
        if not self.dims:
            return None
        name = f"rope:{self.base!r}:{self.dims}:{self.factor!r}:{pairing}"
        positions.setdefault(name, PartSpec("rope", {"theta": self.base, "rotary_dim": self.dims, "head_dim": max(head_dim, self.dims),
                                                     "pairing": pairing, "scaling_factor": self.factor}))
        return name


@dataclass
class LeftSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    keep_first: int
    rot: Rotation

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "LeftSizes":
        r = JsonReader(data, where)
        dim = r.integer("dim")
        window, keep = None, 0
        if r.raw("mask") is not None:
            mask = JsonReader(_object(r.raw("mask"), where, "mask"), f"{where}.mask")
            window, keep = mask.integer("size"), mask.integer("keep_first", 0)
        return cls(heads=r.integer("heads"), kv_heads=r.integer("kv_heads", r.integer("heads")), dim=dim,
                   vdim=r.integer("vdim", dim), scale=r.number("scale"), window=window, keep_first=keep,
                   rot=Rotation.read(r.raw("rot"), where))

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim)
        if self.window is not None:
            require_positive(where, size=self.window)
        if self.keep_first < 0:
            raise ConfigError(f"'{where}': mask.keep_first ({self.keep_first}) must not be negative")
        if self.heads % self.kv_heads:
            raise ConfigError(f"'{where}': {self.heads} query heads cannot be shared out evenly over {self.kv_heads} "
                              "key/value heads")
        self.rot.check(where, self.dim)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                               "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"keep_first": self.keep_first, "size": self.window}
        if self.rot.dims:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass
class RetentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: List[float]
    rot: Rotation

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "RetentionSizes":
        r = JsonReader(data, where)
        decay = r.raw("decay")
        if not isinstance(decay, list) or not all(isinstance(v, (int, float)) and not isinstance(v, bool) for v in decay):
            raise ConfigError(f"'{where}': key 'decay' must be a list of numbers, one a head")
        dim = r.integer("dim")
        return cls(heads=r.integer("heads"), dim=dim, vdim=r.integer("vdim", dim), decay=[float(v) for v in decay],
                   rot=Rotation.read(r.raw("rot"), where))

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, dim=self.dim, vdim=self.vdim)
        if len(self.decay) != self.heads:
            raise ConfigError(f"'{where}': {len(self.decay)} decays for {self.heads} heads")
        if not all(0.0 <= v <= 1.0 for v in self.decay):
            raise ConfigError(f"'{where}': a decay must lie between 0 and 1")
        if self.dim > 256:
            raise ConfigError(f"'{where}': the state's kernel takes at most 256 key channels a head, dim is {self.dim}")
        self.rot.check(where, self.dim)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}
        if self.rot.dims:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass
class LatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: Rotation

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "LatentSizes":
        r = JsonReader(data, where)
        return cls(heads=r.integer("heads"), dim=r.integer("dim"), rot_dim=r.integer("rot_dim"), vdim=r.integer("vdim"),
                   kv_rank=r.integer("kv_rank"), scale=r.number("scale"), rot=Rotation.read(r.raw("rot"), where))

    def check(self, where: str) -> None:
        require_positive(where, heads=self.heads, dim=self.dim, rot_dim=self.rot_dim, vdim=self.vdim, kv_rank=self.kv_rank)
        self.rot.check(where, self.rot_dim)
        if self.rot.dims != self.rot_dim:
            raise ConfigError(f"'{where}': rot.dims ({self.rot.dims}) must be rot_dim ({self.rot_dim}): the turned part "
                              "is turned as a whole")

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": self.rot.to_dict(),
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass
class FosupelMLP:
    kind: str
    ff: int = 0                 # dense: the inner width; moe: an expert's
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None

    @classmethod
    def read(cls, data: Dict[str, Any], where: str) -> "FosupelMLP":
        r = JsonReader(data, where)
        kind = r.string("kind")
        if kind not in MLP_KINDS:
            raise ConfigError(f"'{where}': there is no feed-forward '{kind}' (known: {', '.join(MLP_KINDS)})")
        if kind == "dense":
            return cls(kind=kind, ff=r.integer("ff"))
        router = JsonReader(_object(r.raw("router"), where, "router"), f"{where}.router")
        expert = JsonReader(_object(r.raw("expert"), where, "expert"), f"{where}.expert")
        shared_ff = None
        if r.raw("shared") is not None:
            shared_ff = JsonReader(_object(r.raw("shared"), where, "shared"), f"{where}.shared").integer("ff")
        return cls(kind=kind, ff=expert.integer("ff"), experts=router.integer("experts"), top=router.integer("top"),
                   shared_ff=shared_ff)

    def check(self, where: str) -> None:
        require_positive(where, ff=self.ff)
        if self.kind == "moe":
            require_positive(where, experts=self.experts, top=self.top)
            if self.top > self.experts:
                raise ConfigError(f"'{where}': {self.top} of {self.experts} experts cannot be chosen")
            if self.shared_ff is not None:
                require_positive(where, shared_ff=self.shared_ff)

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        out: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe",
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass
class FosupelLayer:
    type: str
    left: Optional[LeftSizes] = None
    right: Optional[RetentionSizes] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    latent: Optional[LatentSizes] = None
    mlp: Optional[FosupelMLP] = None

    def to_dict(self) -> Dict[str, Any]:
        if self.type == "parallel":
            mixer = {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                     "right_scale": self.right_scale}
        else:
            mixer = self.latent.to_dict()
        return {"mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass
class FosupelConfig(ModelConfig):
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float = 1.0
    logit_softcap: float = 0.0      # 0: none
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1             # 1 with start == stop: config.json names no loop
    has_loop: bool = False
    layers: List[FosupelLayer] = field(default_factory=list)
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
                  generation_origin: str = "<dict>") -> "FosupelConfig":
        r = JsonReader(data, origin)
        norm = JsonReader(_object(r.raw("norm"), origin, "norm"), f"{origin}: norm")
        listed = r.raw("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError(f"'{origin}': key 'layers' must be a list with at least one layer")
        start = stop = 0
        times, has_loop = 1, False
        if r.raw("loop") is not None:
            loop = JsonReader(_object(r.raw("loop"), origin, "loop"), f"{origin}: loop")
            start, stop, times, has_loop = loop.integer("start"), loop.integer("stop"), loop.integer("times"), True
        cfg = cls(vocab_size=r.integer("vocab"), width=r.integer("width"), norm_eps=norm.number("eps"),
                  residual_mult=r.number("residual_mult", 1.0), logit_softcap=r.number("logit_softcap", 0.0),
                  loop_start=start, loop_stop=stop, loop_times=times, has_loop=has_loop,
                  layers=[cls._read_layer(entry, f"{origin}: layers[{i}]") for i, entry in enumerate(listed)],
                  eos_token_ids=r.int_or_int_list("eos_token_id"))
        cfg.read_generation_defaults(generation, generation_origin)
        cfg.validate(origin)
        return cfg

    @staticmethod
    def _read_layer(entry: Any, origin: str) -> FosupelLayer:
        if not isinstance(entry, dict):
            raise ConfigError(f"'{origin}' must be an object")
        r = JsonReader(entry, origin)
        kind = r.string("type")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"'{origin}': there is no mixer '{kind}' (known: {', '.join(MIXER_TYPES)})")
        mixer = _object(r.raw("mixer"), origin, "mixer")
        layer = FosupelLayer(type=kind)
        if kind == "parallel":
            m = JsonReader(mixer, f"{origin}.mixer")
            layer.left = LeftSizes.read(_object(m.raw("left"), f"{origin}.mixer", "left"), f"{origin}.mixer.left")
            layer.right = RetentionSizes.read(_object(m.raw("right"), f"{origin}.mixer", "right"), f"{origin}.mixer.right")
            layer.left_scale = m.number("left_scale", 1.0)
            layer.right_scale = m.number("right_scale", 1.0)
        else:
            layer.latent = LatentSizes.read(mixer, f"{origin}.mixer")
        mlp = r.raw("mlp")
        if mlp is not None:
            layer.mlp = FosupelMLP.read(_object(mlp, origin, "mlp"), f"{origin}.mlp")
        return layer

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        require_positive(origin, vocab=self.vocab_size, width=self.width, max_positions=self.max_positions)
        if not self.norm_eps >= 0.0:
            raise ConfigError(f"'{origin}': norm.eps ({self.norm_eps}) must not be negative")
        if self.logit_softcap < 0.0:
            raise ConfigError(f"'{origin}': logit_softcap ({self.logit_softcap}) must not be negative")
        if not self.layers:
            raise ConfigError(f"'{origin}': a model needs at least one layer")
        if self.has_loop:
            if not 0 <= self.loop_start <= self.loop_stop <= len(self.layers):
                raise ConfigError(f"'{origin}': loop {self.loop_start} .. {self.loop_stop} does not lie inside the "
                                  f"{len(self.layers)} layers")
            if self.loop_times < 1:
                raise ConfigError(f"'{origin}': loop.times ({self.loop_times}) must be at least 1")
        for i, layer in enumerate(self.layers):
            where = f"{origin}: layers[{i}]"
            if layer.left is not None:
                layer.left.check(f"{where}.mixer.left")
                layer.right.check(f"{where}.mixer.right")
            if layer.latent is not None:
                layer.latent.check(f"{where}.mixer")
            if layer.mlp is not None:
                layer.mlp.check(f"{where}.mlp")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": [layer.to_dict() for layer in self.layers],
            "logit_softcap": self.logit_softcap,
            "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult,
            "vocab": self.vocab_size,
            "width": self.width,
        }
        if self.has_loop:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # ------------------------------------------------------------ the model
    def _mixer(self, layer: FosupelLayer, positions: Dict[str, PartSpec]) -> PartSpec:
        if layer.type == "latent_attention":
            m = layer.latent
            return PartSpec("latent_attention", {
                "hidden_size": self.width, "num_heads": m.heads, "head_dim": m.dim, "rotary_dim": m.rot_dim,
                "value_dim": m.vdim, "latent_dim": m.kv_rank, "scale": m.scale, "norm_eps": self.norm_eps,
                "position": m.rot.position(m.rot_dim, "interleaved", positions), "sink": True, "output_gate": True,
                "prefix": "mix"})
        left, right = layer.left, layer.right
        attention = {"hidden_size": self.width, "num_heads": left.heads, "num_kv_heads": left.kv_heads,
                     "head_dim": left.dim, "value_dim": left.vdim, "scale": left.scale, "window": left.window,
                     "keep_first": left.keep_first, "sink": True, "talk": True,
                     "position": left.rot.position(left.dim, "half", positions), "prefix": "left"}
        retention = {"hidden_size": self.width, "num_heads": right.heads, "head_dim": right.dim, "value_dim": right.vdim,
                     "decay": list(right.decay), "norm_eps": self.norm_eps, "activation": "none",
                     "position": right.rot.position(right.dim, "half", positions), "key_scale": right.dim ** -0.5,
                     "norm": "head", "norm_weight": False, "gate_activation": "silu", "prefix": "right"}
        return PartSpec("side_by_side", {"hidden_size": self.width, "prefix": "mix", "branches": [
            {"kind": "attention_rows", "params": attention, "scale": layer.left_scale},
            {"kind": "lightning", "params": retention, "scale": layer.right_scale}]})

    def _ffn(self, layer: FosupelLayer) -> Optional[PartSpec]:
        m = layer.mlp
        if m is None:
            return None
        if m.kind == "dense":
            return PartSpec("mlp", {"hidden_size": self.width, "intermediate_size": m.ff, "activation": "xielu",
                                    "prefix": "mlp"})
        return PartSpec("routed_experts", {"hidden_size": self.width, "expert_size": m.ff, "num_experts": m.experts,
                                           "top": m.top, "renormalize": False, "shared_size": m.shared_ff,
                                           "shared_gate": m.shared_ff is not None, "prefix": "mlp"})

    def run_order(self) -> List[RunSpec]:
        """The layers in the order of running: those of the loop ``times`` times, every pass marked by its row of
        ``loop.step`` on its first layer."""
        n = len(self.layers)
        if not self.has_loop:
            return [RunSpec(layer=i) for i in range(n)]
        order = [RunSpec(layer=i) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            for i in range(self.loop_start, self.loop_stop):
                order.append(RunSpec(layer=i, offset=("loop.step", t) if i == self.loop_start else None))
        return order + [RunSpec(layer=i) for i in range(self.loop_stop, n)]

    def model_spec(self) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "tensor": ""})
        positions: Dict[str, PartSpec] = {}
        layers = []
        for i, layer in enumerate(self.layers):
            layers.append(LayerSpec(prefix=f"l{i}", mixer=self._mixer(layer, positions), ffn=self._ffn(layer),
                                    norms={"mixer_norm": norm, "ffn_norm": norm},
                                    block=PartSpec("prenorm_scaled", {"mixer_norm": "norm1", "ffn_norm": "norm2",
                                                                      "residual_scale": self.residual_mult})))
        looped = self.has_loop and self.loop_stop > self.loop_start
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.width,
            max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "embed"}),
            layers=layers,
            order=self.run_order(),
            final_norm=norm,
            final_norm_prefix="final.norm",
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.width, "name": "head",
                                      "tied": True, "softcap": self.logit_softcap}),
            positions=positions,
            offsets={"loop.step": self.loop_times} if looped else {},
        )
        spec.validate()
        return spec
