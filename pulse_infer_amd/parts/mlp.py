"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases
(reference: src/model/qwen3/model.cpp:893-913; silu: src/ops/kernels/cuda/silu_kernel.cu:82-97).
gate and up are one product with the row-stacked weight; activation and product are one
kernel in float32 with one rounding."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import FEED_FORWARDS, BuildContext, LazyNorm, Part, StepContext, joined
from .linear import Linear


SLAB = 16  # rows of a weight slab of the few-rows product


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, inter = params["hidden_size"], params["intermediate_size"]
        names = cls.tensor_names(params)
        return {
            names["gate"]: TensorSpec((inter, hidden), fan_in=hidden),
            names["up"]: TensorSpec((inter, hidden), fan_in=hidden),
            names["down"]: TensorSpec((hidden, inter), fan_in=inter),
        }

    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        """The tensors' names below the part's prefix; ``params["names"]`` replaces any of the usual ones."""
        return {**cls.NAMES, **params.get("names", {})}

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        if self.activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp has no kernel for activation '{self.activation}' "
                             f"(known: {sorted(kernels.GATE_ACTIVATIONS)})")
        load = build.loader
        names = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        gate, up = load.get(names["gate"]), load.get(names["up"])
        # gate and up rows alternate in slabs of 16 where the sizes allow it, so that one workgroup of the
        # few-rows product holds a gate slab and its up slab and can apply SwiGLU itself (a layout choice)
        self.slab = SLAB if (build.mode == "bfloat16" and gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                             and self.inter % SLAB == 0) else 0
        if self.slab:
            stacked = torch.stack([gate.view(-1, SLAB, self.hidden), up.view(-1, SLAB, self.hidden)], dim=1)
            self.gate_up = Linear(stacked.reshape(2 * self.inter, self.hidden).contiguous(), build.mode)
        else:
            self.gate_up = Linear(load.get_concat([names["gate"], names["up"]]), build.mode)
        del gate, up
        self.down = Linear(load.get(names["down"]), build.mode)
        self.act_dtype = build.act_dtype

    accepts_residual = True
    accepts_lazy_input = True   # the first product may take rows that are not normalised yet and scale its result
    records_cleanly = True

    def takes_lazy_input(self, x: LazyNorm, cache: Any = None) -> bool:
        """Whether ``forward`` would run its first product on rows that are not normalised yet, or compute the norm."""
        return bool(self.slab and self.gate_up.takes_lazy(x))

    def forward(self, x, ctx: StepContext, residual: Optional[torch.Tensor] = None,
                next_scale: Optional[torch.Tensor] = None, next_offset: float = 0.0, leave_stats: bool = True):
        tokens = x.shape[0]
        ws = ctx.workspace
        z = ws.buffer("mlp.act", tokens, self.inter, self.act_dtype)
        if isinstance(x, LazyNorm) and not (self.slab and self.gate_up.takes_lazy(x)):
            x = x.materialize(ws.buffer("mlp.normed", tokens, self.hidden, self.act_dtype))
        gated = True if self.activation == "silu" else self.activation   # what the fused epilogues are told
        if isinstance(x, LazyNorm):
            self.gate_up.forward(x, z, swiglu=gated)
        elif (self.slab and tokens <= kernels.SKINNY_FAST_ROWS and kernels.gemm_skinny_ok(x, self.gate_up.weight)
              and (2 * self.inter) % 32 == 0):
            self.gate_up.forward(x, z, swiglu=gated)
        elif (self.slab and self.gate_up.takes_mid(x) and (2 * self.inter) % 32 == 0
              and kernels.gemm_mid_takes(tokens, 2 * self.inter, self.hidden)):
            self.gate_up.forward(x, z, swiglu=gated)   # 17 to 64 rows: X shared through LDS, SwiGLU in the epilogue
        elif self.slab and self.activation == "silu" and self.gate_up.takes_tiles(x, swiglu=True):
            self.gate_up.forward(x, z, swiglu=True)   # many rows: output tiles on the matrix cores, SwiGLU on the way out
        else:
            gu = ws.buffer("mlp.gate_up", tokens, 2 * self.inter, self.act_dtype)
            self.gate_up.forward(x, gu, own=False)   # (the shapes that come here at 17 to 64 rows are those the library wins)
            kernels.swiglu(gu, z, slab=self.slab, activation=self.activation)
        out = ws.buffer("mlp.out", tokens, self.hidden, self.act_dtype)
        if residual is not None:
            return self.down.add_into(z, residual, out, ws, next_scale, next_offset, leave_stats)
        return self.down.forward(z, out)


@FEED_FORWARDS.register("mlp")
class PlainMLP(Part):
    """down(act(up(x))), no gate and no biases.  Parameters: ``hidden_size``, ``intermediate_size``, ``activation``
    ("relu2": the square of relu, "gelu_tanh", "silu", "xielu": a z^2 + z / 2 for z > 0 and b (exp(z) - 1 - z) + z / 2
    below, a = softplus(p), b = 1/2 + softplus(q) with the two learned numbers p, q in the tensor ``act``), ``names``
    (``up``, ``down``, ``act``)."""

    NAMES = {"up": "up", "down": "down", "act": "act"}
    LEARNED = ("xielu",)    # activations with numbers of their own

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        return {**cls.NAMES, **params.get("names", {})}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, inter = params["hidden_size"], params["intermediate_size"]
        names = cls.tensor_names(params)
        specs = {names["up"]: TensorSpec((inter, hidden), fan_in=hidden),
                 names["down"]: TensorSpec((hidden, inter), fan_in=inter)}
        if params.get("activation", "relu2") in cls.LEARNED:
            specs[names["act"]] = TensorSpec((2,), kind="linear", fan_in=4)
        return specs

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "relu2")
        if self.activation not in kernels.ACTIVATIONS and self.activation not in self.LEARNED:
            raise ValueError(f"mlp has no kernel for activation '{self.activation}' "
                             f"(known: {sorted(list(kernels.ACTIVATIONS) + list(self.LEARNED))})")
        names = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        self.act_numbers = build.loader.get(names["act"]) if self.activation in self.LEARNED else None
        self.up = Linear(build.loader.get(names["up"]), build.mode)
        self.down = Linear(build.loader.get(names["down"]), build.mode)
        self.act_dtype = build.act_dtype

    records_cleanly = True

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        tokens = x.shape[0]
        ws = ctx.workspace
        z = ws.buffer("mlp.act", tokens, self.inter, self.act_dtype)
        self.up.forward(x, z)
        if self.act_numbers is not None:
            kernels.xielu(z, z, self.act_numbers)
        else:
            kernels.activation(z, z, self.activation)
        return self.down.forward(z, ws.buffer("mlp.out", tokens, self.hidden, self.act_dtype))
