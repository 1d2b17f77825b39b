"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * (c + w), float32 inside, one rounding
(reference: src/ops/kernels/cuda/rmsnorm_kernel.cu:97-157; layer: src/layer/rmsnorm.cpp:9-157).

Parameters: ``size``, ``eps``; ``weight_offset`` = c (default 0: the tensor holds the factors themselves; 1: it holds
their distances from one, and the sum is formed in float32 whatever the tensor's storage type); ``tensor``: the
tensor's name below the norm's prefix (default "weight"; "": the prefix itself is the tensor's name)."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import NORMS, BuildContext, LazyNorm, Part, RowStats, StreamUpdate, joined


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        kind = "norm_offset" if float(params.get("weight_offset", 0.0)) == 1.0 else "norm"
        return {params.get("tensor", "weight"): TensorSpec((params["size"],), kind=kind)}

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.weight_offset = float(params.get("weight_offset", 0.0))
        self.weight = build.loader.get(joined(prefix, params.get("tensor", "weight")))

    records_cleanly = True
    takes_parts = True   # delta may be [parts, T, H] float32: the kernel adds the parts in order
    takes_scale = True   # ``apply`` takes a factor on the update

    def apply(self, h: torch.Tensor, delta: Optional[torch.Tensor], out: torch.Tensor,
              rows: Optional[torch.Tensor] = None, delta_scale: float = 1.0) -> torch.Tensor:
        """out = norm(h + delta_scale * delta) * w; h keeps the sum unless rows are gathered."""
        kernels.add_rmsnorm(h, delta, self.weight, self.eps, out, rows=rows, weight_offset=self.weight_offset,
                            delta_scale=delta_scale)
        return out

    def column_scale(self) -> Optional[torch.Tensor]:
        """The factor of every column (plus ``weight_offset``): whoever writes the rows that this norm reads next may
        multiply it in as it writes a rounded copy of them (``RowStats``), and leave the rest of the norm to the
        consumer."""
        return self.weight

    def lazy(self, h: torch.Tensor, stats: RowStats) -> Optional[LazyNorm]:
        """This norm as an input that its consumer finishes: the rows already carry this norm's weight, and dividing
        a row by a number commutes with a linear product."""
        if stats.rounded is None or stats.scaled_by is not self.weight or stats.offset != self.weight_offset:
            return None
        return LazyNorm(stats.rounded, stats.sumsq, self.eps, h, self)


@NORMS.register("layernorm")
class LayerNorm(Part):
    """y = (x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations; float32 inside, one rounding.

    Parameters: ``size``, ``eps``; ``tensor`` / ``bias_tensor``: the tensors' names below the norm's prefix (defaults
    "weight" and "bias"; "": the prefix itself is the tensor's name); ``bias`` False: no bias; ``streams`` (default
    1): the residual it reads holds that many rows a token side by side, and the norm reads their weighted sum
    (``stream_weights`` of ``apply``; None: the plain sum)."""

    records_cleanly = True
    takes_streams = True    # ``apply`` takes a ``StreamUpdate`` as the update and does it on the way

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        out = {params.get("tensor", "weight"): TensorSpec((params["size"],), kind="norm")}
        if params.get("bias", True):
            out[params.get("bias_tensor", "bias")] = TensorSpec((params["size"],), kind="linear", fan_in=100)
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.streams = int(params.get("streams", 1))
        self.weight = build.loader.get(joined(prefix, params.get("tensor", "weight")))
        self.bias = None
        if params.get("bias", True):
            self.bias = build.loader.get(joined(prefix, params.get("bias_tensor", "bias")))
            if self.bias.dtype != self.weight.dtype:
                self.bias = self.bias.to(self.weight.dtype)

    def apply(self, h: torch.Tensor, delta: Any, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
              stream_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
        """out = norm(sum_s weights[s] * h_s) after ``delta`` has gone into h: a ``StreamUpdate`` (done by the same
        kernel; with gathered rows the updated streams are used but not stored: who gathers rows reads the residual
        for the last time), a tensor of h's shape (added first), or None."""
        update = None
        if isinstance(delta, StreamUpdate):
            update = (delta.y, delta.mix, delta.out)
        elif delta is not None:
            kernels.residual_add(h, delta)
        kernels.streams_step(h, self.streams, update=update, in_weight=stream_weights,
                             norm=("layernorm", self.weight, self.bias, self.eps), out=out, rows=rows)
        return out
