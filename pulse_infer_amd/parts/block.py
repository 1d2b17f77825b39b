"""Arrangements of mixer, feed-forward and norms around the residual stream.

``prenorm``: h <- h + mixer(norm_a(h)); h <- h + ffn(norm_b(h))
(reference: src/model/qwen3/model.cpp:779-923).  The additions are deferred into
the next norm's kernel through ``ResidualStream``.

``prenorm_scaled``: h <- h + m mixer(norm_a(h)); h <- h + m ffn(norm_b(h)) with one multiplier m on both
updates; the feed-forward may be absent.

``parallel``: n = norm(h); h <- h + (mixer(n) + ffn(n)): one norm, whose output both
sublayers read; a layer may have no feed-forward (``LayerSpec.ffn`` None), then
h <- h + mixer(norm(h)).

``postnorm``: h <- norm_a(alpha h + ls_a * mixer(h)); h <- norm_b(alpha h + ls_b * ffn(h)): the
sublayers read the stream itself, the norm comes after the sum, ``alpha`` weighs the
stream in it and ``ls`` are optional factors, one a column, on a sublayer's result.

``hyper``: the residual is S streams x_1 .. x_S.  Sublayer q reads u = sum_s in_q[s] x_s through its norm, and its
result y goes back as x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y, all streams at once from the old ones.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..models.spec import LayerSpec
from ..weights.store import TensorSpec
from ..ops import kernels
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, BuildContext, Part, ResidualStream, StepContext, StreamUpdate,
                   joined, says)


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    NORM_PLACES = ("mixer_norm", "ffn_norm")   # the norms this arrangement has; a layer names a spec for each

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        """All tensors of one layer, by full name."""
        p = layer.block.params
        out: Dict[str, TensorSpec] = {}
        for which in cls.NORM_PLACES:
            norm = layer.norm(which)
            for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
                out[joined(joined(layer.prefix, p[which]), name)] = spec
        for part, registry in ((layer.mixer, MIXERS), (layer.ffn, FEED_FORWARDS)):
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        made = {}
        for which in self.NORM_PLACES:
            norm = layer.norm(which)
            made[which] = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p[which]), build)
        self.mixer_norm, self.ffn_norm = made["mixer_norm"], made["ffn_norm"]
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                     joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        self.act_dtype = build.act_dtype

    def cache_spec(self) -> Optional[Any]:
        return self.mixer.cache_spec()

    def records_cleanly(self) -> bool:
        """Whether a step of this block may be recorded as a graph and replayed: every part of it says so."""
        return all(says(part, "records_cleanly")
                   for part in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm))

    def _input(self, stream: ResidualStream, norm: Any, part: Any, ctx: StepContext) -> Any:
        """norm(h) for ``part``: left to the part's first product where that is possible, else computed here."""
        if getattr(part, "accepts_lazy_input", False):
            lazy = stream.lazy(norm)
            if lazy is not None:
                return lazy
        x = ctx.workspace.buffer("block.normed", ctx.num_tokens, stream.h.shape[1], self.act_dtype)
        return stream.normed(norm, x)

    def entry_norm(self) -> Any:
        """The norm that reads the residual first in this block."""
        return self.mixer_norm

    @staticmethod
    def _scale_of(norm: Any) -> Any:
        return norm.column_scale() if norm is not None and hasattr(norm, "column_scale") else None

    @classmethod
    def _told(cls, norm: Any) -> Dict[str, Any]:
        """What a part that adds into the residual itself is told about the norm that reads the residual next: its
        column factors, and what it adds to them if that is not zero."""
        told = {"next_scale": cls._scale_of(norm)}
        offset = float(getattr(norm, "weight_offset", 0.0) or 0.0) if norm is not None else 0.0
        if offset and told["next_scale"] is not None:
            told["next_offset"] = offset
        return told

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        x = self._input(stream, self.mixer_norm, self.mixer, ctx)
        # a part that says so may add its result into the residual itself and return None (or the new rows' statistics,
        # for which it is told the column factors of the norm that reads the residual next)
        if getattr(self.mixer, "accepts_residual", False):
            stream.push(self.mixer.forward(x, ctx, cache, residual=stream.h, **self._told(self.ffn_norm)))
        else:
            stream.push(self.mixer.forward(x, ctx, cache))
        x = self._input(stream, self.ffn_norm, self.ffn, ctx)
        if getattr(self.ffn, "accepts_residual", False):
            stream.push(self.ffn.forward(x, ctx, residual=stream.h, **self._told(stream.after_block)))
        else:
            stream.push(self.ffn.forward(x, ctx))


@BLOCKS.register("prenorm_scaled")
class ScaledPreNormBlock(PreNormBlock):
    """The pre-norm arrangement with a multiplier on the sublayers' results: h <- h + m * mixer(norm_a(h)), then
    h <- h + m * ffn(norm_b(h)).  Block parameters: ``mixer_norm`` / ``ffn_norm`` (the norms' tensor prefixes below the
    layer's) and ``residual_scale`` = m (default 1).  A layer without a feed-forward ends after the mixer.

    The multiplied update is added inside the kernel of the norm that reads the residual next (a norm that says
    ``takes_scale``), in float32; weights stay what the checkpoint holds.  A feed-forward may hand back two updates."""

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        p = layer.block.params
        out: Dict[str, TensorSpec] = {}
        places = ["mixer_norm"] + (["ffn_norm"] if layer.ffn is not None else [])
        for which in places:
            norm = layer.norm(which)
            for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
                out[joined(joined(layer.prefix, p[which]), name)] = spec
        parts = [(layer.mixer, MIXERS)] + ([(layer.ffn, FEED_FORWARDS)] if layer.ffn is not None else [])
        for part, registry in parts:
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        self.residual_scale = float(p.get("residual_scale", 1.0))
        norm = layer.norm("mixer_norm")
        self.mixer_norm = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p["mixer_norm"]), build)
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = self.ffn_norm = None
        if layer.ffn is not None:
            norm = layer.norm("ffn_norm")
            self.ffn_norm = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p["ffn_norm"]), build)
            self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                         joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        self.act_dtype = build.act_dtype

    def records_cleanly(self) -> bool:
        return all(says(part, "records_cleanly")
                   for part in (self.mixer, self.ffn, self.mixer_norm, self.ffn_norm) if part is not None)

    def _push(self, stream: ResidualStream, update: Any) -> None:
        first, second = update if isinstance(update, tuple) else (update, None)
        stream.push(first, self.residual_scale)
        if second is not None:
            stream.push(second, self.residual_scale)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        x = ctx.workspace.buffer("block.normed", ctx.num_tokens, stream.h.shape[1], self.act_dtype)
        self._push(stream, self.mixer.forward(stream.normed(self.mixer_norm, x), ctx, cache))
        if self.ffn is not None:
            self._push(stream, self.ffn.forward(stream.normed(self.ffn_norm, x), ctx))


@BLOCKS.register("parallel")
class ParallelBlock(PreNormBlock):
    """One norm in front of mixer and feed-forward, which both read its output; their results are added to the
    residual together.  The feed-forward may be absent.  Block parameters: ``norm``: the norm's tensor prefix below
    the layer's.  A mixer that says ``accepts_residual`` is also handed ``leave_stats`` here, and parts that say
    ``accepts_lazy_input`` answer ``takes_lazy_input(x, cache)``."""

    NORM_PLACES = ("norm",)

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        p = layer.block.params
        out: Dict[str, TensorSpec] = {}
        norm = layer.norm("norm")
        for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
            out[joined(joined(layer.prefix, p["norm"]), name)] = spec
        parts = [(layer.mixer, MIXERS)] + ([(layer.ffn, FEED_FORWARDS)] if layer.ffn is not None else [])
        for part, registry in parts:
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        norm = layer.norm("norm")
        self.norm = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p["norm"]), build)
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = None
        if layer.ffn is not None:
            self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                         joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        self.act_dtype = build.act_dtype

    def records_cleanly(self) -> bool:
        return all(says(part, "records_cleanly") for part in (self.mixer, self.ffn, self.norm) if part is not None)

    def entry_norm(self) -> Any:
        return self.norm

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        parts = [part for part in (self.mixer, self.ffn) if part is not None]
        # The norm's output is read twice.  It is left to the parts' first products (rows scaled behind the product)
        # only if every part takes it that way; a part that then cannot after all computes the norm for itself.
        x = None
        if all(getattr(part, "accepts_lazy_input", False) and hasattr(part, "takes_lazy_input") for part in parts):
            x = stream.lazy(self.norm)
            # (a part that computed the norm for itself after the other has changed the residual would norm the wrong
            # rows: so every part is asked beforehand)
            if x is not None and not all(part.takes_lazy_input(x, cache) for part in parts):
                x = None
        if x is None:
            x = stream.normed(self.norm, ctx.workspace.buffer("block.normed", ctx.num_tokens, stream.h.shape[1],
                                                              self.act_dtype))
        # The mixer's update first: the part that adds last is told who reads the residual next, and what it leaves
        # about the new rows then covers both updates.
        last = self.ffn is None
        if getattr(self.mixer, "accepts_residual", False):
            # (told not to leave the new rows' statistics when it is not the last to add: their buffers are the
            # ones the feed-forward's input still lies in)
            told = self._told(stream.after_block) if last else {"leave_stats": False}
            stream.push(self.mixer.forward(x, ctx, cache, residual=stream.h, **told))
        else:
            stream.push(self.mixer.forward(x, ctx, cache))
        if self.ffn is None:
            return
        stream.settle()   # (an update handed back in a workspace buffer must not wait while the next product runs)
        if getattr(self.ffn, "accepts_residual", False):
            stream.push(self.ffn.forward(x, ctx, residual=stream.h, **self._told(stream.after_block)))
        else:
            stream.push(self.ffn.forward(x, ctx))


@BLOCKS.register("postnorm")
class PostNormBlock(Part):
    """The norm after the sum.  Block parameters: ``alpha`` (the stream's weight in the sum, default 1);
    ``mixer_norm`` / ``ffn_norm``: the norms' tensor prefixes below the layer's; ``mixer_scale`` / ``ffn_scale``: names
    of the column factors on the sublayers' results (absent: none).  The norms are RMSNorms with plain weights
    (``LayerSpec.norms`` gives their size and eps).  A layer without a feed-forward ends after the first norm.

    The float32 stream is the normed rows themselves; a copy in the activations' type, which the sublayers'
    products read, comes out of the same kernel (``ResidualStream.copy``).  A feed-forward may return two updates
    (``returns_two``), which the kernel adds both."""

    NORM_PLACES = ("mixer_norm", "ffn_norm")

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        p = layer.block.params
        out: Dict[str, TensorSpec] = {}
        places = [("mixer_norm", "mixer_scale")] + ([("ffn_norm", "ffn_scale")] if layer.ffn is not None else [])
        for which, factors in places:
            norm = layer.norm(which)
            if norm.kind != "rmsnorm" or float(norm.params.get("weight_offset", 0.0)) != 0.0:
                raise ValueError("the postnorm block takes RMSNorms with plain weights")
            for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
                out[joined(joined(layer.prefix, p[which]), name)] = spec
            if p.get(factors):
                out[joined(layer.prefix, p[factors])] = TensorSpec((norm.params["size"],), kind="norm")
        parts = [(layer.mixer, MIXERS)] + ([(layer.ffn, FEED_FORWARDS)] if layer.ffn is not None else [])
        for part, registry in parts:
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        self.alpha = float(p.get("alpha", 1.0))
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = None
        if layer.ffn is not None:
            self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                         joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        places = [("mixer_norm", "mixer_scale")] + ([("ffn_norm", "ffn_scale")] if self.ffn is not None else [])
        self.norms = {}
        for which, factors in places:
            norm = layer.norm(which)
            made = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p[which]), build)
            scale = build.loader.get(joined(layer.prefix, p[factors])) if p.get(factors) else None
            if scale is not None and scale.dtype != made.weight.dtype:
                scale = scale.to(made.weight.dtype)
            self.norms[which] = (made, scale)
        self.act_dtype = build.act_dtype

    def cache_spec(self) -> Optional[Any]:
        return self.mixer.cache_spec()

    def records_cleanly(self) -> bool:
        return all(says(part, "records_cleanly") for part in (self.mixer, self.ffn) if part is not None)

    def _rows(self, stream: ResidualStream, ctx: StepContext) -> torch.Tensor:
        """The stream in the activations' type: itself in a float32 run, else the copy the last norm left (or one made
        now, for the first block behind the embedding)."""
        if self.act_dtype == torch.float32:
            return stream.h
        stream.settle()
        if stream.copy is None:
            stream.copy = ctx.workspace.buffer("block.rows", ctx.num_tokens, stream.h.shape[1], self.act_dtype)
            kernels.round_rows(stream.h, stream.copy)
        return stream.copy

    def _close(self, stream: ResidualStream, ctx: StepContext, which: str, update: Any) -> None:
        norm, scale = self.norms[which]
        first, second = update if isinstance(update, tuple) else (update, None)
        copy = None
        if self.act_dtype != torch.float32:
            copy = ctx.workspace.buffer("block.rows", ctx.num_tokens, stream.h.shape[1], self.act_dtype)
        kernels.scale_add_rmsnorm(stream.h, norm.weight, norm.eps, self.alpha, first, second, scale, copy)
        stream.stats = None
        stream.copy = copy

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        self._close(stream, ctx, "mixer_norm", self.mixer.forward(self._rows(stream, ctx), ctx, cache))
        if self.ffn is not None:
            self._close(stream, ctx, "ffn_norm", self.ffn.forward(self._rows(stream, ctx), ctx))


@BLOCKS.register("hyper")
class HyperConnectionBlock(Part):
    """A pre-norm layer around a residual of several streams (hyper-connections).

    Block parameters: ``streams``; ``mixer_norm`` / ``ffn_norm``: the norms' tensor prefixes below the layer's;
    ``mixer_hc`` / ``ffn_hc``: the prefixes of a sublayer's connection tensors, ``<prefix>.in`` [streams],
    ``<prefix>.out`` [streams] and ``<prefix>.mix`` [streams, streams] (indexed [from, to]); ``learned`` False: there
    are no such tensors, every factor is one and the streams do not mix (with one stream that is the plain residual
    sum x <- x + sublayer(norm(x))).  The norms must say
    ``takes_streams`` (they read the weighted sum of the streams and do a pending update on the way); a layer
    without a feed-forward ends after the mixer.

    The update of the streams is not a launch of its own: it is handed on as a ``StreamUpdate`` and done by the
    kernel of the norm that reads the residual next (this layer's second norm, the next layer's first, the model's
    last).  Connection tensors are kept in float32 whatever their storage type."""

    NORM_PLACES = ("mixer_norm", "ffn_norm")
    CONNECTIONS = (("mixer_norm", "mixer_hc"), ("ffn_norm", "ffn_hc"))

    @classmethod
    def _places(cls, layer: LayerSpec):
        return [pair for pair in cls.CONNECTIONS if pair[0] == "mixer_norm" or layer.ffn is not None]

    @classmethod
    def layer_weight_specs(cls, layer: LayerSpec) -> Dict[str, TensorSpec]:
        p = layer.block.params
        streams = int(p["streams"])
        out: Dict[str, TensorSpec] = {}
        for which, hc in cls._places(layer):
            norm = layer.norm(which)
            for name, spec in NORMS.get(norm.kind).weight_specs(norm.params).items():
                out[joined(joined(layer.prefix, p[which]), name)] = spec
            if not p.get("learned", True):
                continue
            sub = joined(layer.prefix, p[hc])
            out[joined(sub, "in")] = TensorSpec((streams,), kind="linear", fan_in=streams * streams)
            out[joined(sub, "out")] = TensorSpec((streams,), kind="linear", fan_in=2)
            out[joined(sub, "mix")] = TensorSpec((streams, streams), kind="linear", fan_in=streams)
        parts = [(layer.mixer, MIXERS)] + ([(layer.ffn, FEED_FORWARDS)] if layer.ffn is not None else [])
        for part, registry in parts:
            sub = joined(layer.prefix, part.params.get("prefix", ""))
            for name, spec in registry.get(part.kind).weight_specs(part.params).items():
                out[joined(sub, name)] = spec
        return out

    def __init__(self, layer: LayerSpec, build: BuildContext):
        p = layer.block.params
        self.streams = int(p["streams"])
        self.mixer = MIXERS.get(layer.mixer.kind)(layer.mixer.params,
                                                  joined(layer.prefix, layer.mixer.params.get("prefix", "")), build)
        self.ffn = None
        if layer.ffn is not None:
            self.ffn = FEED_FORWARDS.get(layer.ffn.kind)(layer.ffn.params,
                                                         joined(layer.prefix, layer.ffn.params.get("prefix", "")), build)
        self.norms: Dict[str, Any] = {}
        self.connections: Dict[str, Any] = {}
        f32 = lambda name: build.loader.get(name).to(torch.float32).contiguous()
        for which, hc in self._places(layer):
            norm = layer.norm(which)
            made = NORMS.get(norm.kind)(norm.params, joined(layer.prefix, p[which]), build)
            if not getattr(made, "takes_streams", False) or getattr(made, "streams", 1) != self.streams:
                raise ValueError(f"the hyper block needs norms that read {self.streams} streams, '{norm.kind}' does not")
            self.norms[which] = made
            if p.get("learned", True):
                sub = joined(layer.prefix, p[hc])
                self.connections[which] = (f32(joined(sub, "in")), f32(joined(sub, "mix")), f32(joined(sub, "out")))
            else:
                self.connections[which] = (None, torch.eye(self.streams, dtype=torch.float32, device=build.device),
                                           torch.ones(self.streams, dtype=torch.float32, device=build.device))
        self.act_dtype = build.act_dtype

    def cache_spec(self) -> Optional[Any]:
        return self.mixer.cache_spec()

    def records_cleanly(self) -> bool:
        return all(says(part, "records_cleanly") for part in (self.mixer, self.ffn, *self.norms.values())
                   if part is not None)

    def entry_norm(self) -> Any:
        return self.norms["mixer_norm"]

    def _sublayer(self, stream: ResidualStream, ctx: StepContext, which: str, run) -> None:
        norm = self.norms[which]
        w_in, mix, w_out = self.connections[which]
        hidden = stream.h.shape[1] // self.streams
        x = ctx.workspace.buffer("block.normed", ctx.num_tokens, hidden, self.act_dtype)
        norm.apply(stream.h, stream.pending_for(norm), x, stream_weights=w_in)
        y = run(x)
        if isinstance(y, tuple):   # (a feed-forward that hands back two updates)
            first, second = y
            if second is not None:
                raise TypeError("the hyper block takes one result a sublayer")
            y = first
        stream.stats = None
        stream.pending = StreamUpdate(y, mix, w_out)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Any) -> None:
        self._sublayer(stream, ctx, "mixer_norm", lambda x: self.mixer.forward(x, ctx, cache))
        if self.ffn is not None:
            self._sublayer(stream, ctx, "ffn_norm", lambda x: self.ffn.forward(x, ctx))
