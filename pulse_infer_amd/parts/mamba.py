"""A selective state-space mixer (Mamba).

For a token with input h: [x | z] = W_in h (each ``inner`` wide); x <- silu(conv(x)), a causal convolution along
the sequence, one row of ``conv`` taps and a bias per channel, zeros before a sequence's start; [dt | B | C] =
W_x x (``dt_rank``, ``state``, ``state`` wide); dt <- softplus(W_dt dt + dt_bias), one step size a channel;
A = -exp(A_log) [inner, state].  Per channel c and state n, token by token,

    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n          y_c = sum_n S[c, n] C_n + D_c x_c

and the output is W_o (y * silu(z)).  A request keeps S and the last ``conv`` - 1 inputs of the convolution in its
state slot, in float32; both start from zeros with the request.  The four matrix products are ``Linear`` products;
the convolution and the recurrence are one kernel each for prompt portions, decoded tokens and mixed batches alike
(``csrc/mamba.hip``).  Step sizes, decays, exponentials, the state and its sums are float32 in both run modes.

Parameters: ``hidden_size``, ``inner``, ``state``, ``dt_rank``, ``conv`` (taps), ``names`` (tensor names below the
prefix: ``in``, ``conv``, ``conv_bias``, ``x``, ``dt``, ``dt_bias``, ``a_log``, ``d``, ``o``).
"""
from __future__ import annotations

from typing import Any, Dict, List, Tuple

import torch

from ..cache.specs import StateSpec, StateView
from ..ops import kernels
from ..weights.store import TensorSpec
from .base import MIXERS, BuildContext, Part, StepContext, StepCost, joined
from .linear import Linear

MAX_TAPS = 16      # as in csrc/mamba.hip
MAX_STATES = 256


@MIXERS.register("mamba")
class SelectiveStateSpace(Part):
    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
             "a_log": "A_log", "d": "D", "o": "o"}

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        return {**cls.NAMES, **params.get("names", {})}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, inner, n, rank, taps = (params[k] for k in ("hidden_size", "inner", "state", "dt_rank", "conv"))
        names = cls.tensor_names(params)
        return {
            names["in"]: TensorSpec((2 * inner, hidden), fan_in=hidden),
            names["conv"]: TensorSpec((inner, taps), fan_in=taps),
            names["conv_bias"]: TensorSpec((inner,), fan_in=16),
            names["x"]: TensorSpec((rank + 2 * n, inner), fan_in=inner),
            names["dt"]: TensorSpec((inner, rank), fan_in=rank),
            names["dt_bias"]: TensorSpec((inner,), fan_in=1),
            names["a_log"]: TensorSpec((inner, n), fan_in=4),
            names["d"]: TensorSpec((inner,), kind="norm"),
            names["o"]: TensorSpec((hidden, inner), fan_in=inner),
        }

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """The products; the recurrence (about six operations a state element and token, one of them an
        exponential); every request's state read and written once, in float32."""
        cost = super().step_cost(params, entries, weight_bytes, cache_bytes)
        inner, n, taps = params["inner"], params["state"], params["conv"]
        rows = sum(count for _, count in entries)
        cost.flops += rows * inner * (6.0 * n + 2.0 * taps)
        cost.cache_bytes += 8.0 * inner * (n + taps - 1) * len(entries)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.inner = int(params["inner"])
        self.n = int(params["state"])
        self.rank = int(params["dt_rank"])
        self.taps = int(params["conv"])
        if not 1 <= self.taps <= MAX_TAPS:
            raise ValueError(f"the convolution's kernel takes 1 to {MAX_TAPS} taps, got {self.taps}")
        if not 1 <= self.n <= MAX_STATES:
            raise ValueError(f"the recurrence's kernel takes 1 to {MAX_STATES} states a channel, got {self.n}")
        load = build.loader
        names = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        self.w_in = Linear(load.get(names["in"]), build.mode)
        self.w_x = Linear(load.get(names["x"]), build.mode)
        self.w_dt = Linear(load.get(names["dt"]), build.mode)
        self.w_o = Linear(load.get(names["o"]), build.mode)
        self.conv = load.get(names["conv"])
        small = lambda key: load.get(names[key]).to(self.conv.dtype).contiguous()
        self.conv_bias, self.dt_bias, self.d = small("conv_bias"), small("dt_bias"), small("d")
        self.a_log = small("a_log")
        self.act_dtype = build.act_dtype

    records_cleanly = True   # slots, starts and rows are read on the device

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.inner, self.n + self.taps - 1), "float32")

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: StateView) -> torch.Tensor:
        tokens = x.shape[0]
        ws = ctx.workspace
        entries = len(ctx.entries)
        xz = ws.buffer("mamba.xz", tokens, 2 * self.inner, self.act_dtype)
        self.w_in.forward(x, xz)
        xc = ws.buffer("mamba.conv", tokens, self.inner, self.act_dtype)
        kernels.causal_conv(xz, self.conv, self.conv_bias, xc, cache.state, self.n, ctx.positions, ctx.token_entry,
                            ctx.entry_start, ctx.entry_first_row, ctx.entry_slot, entries)
        low = ws.buffer("mamba.low", tokens, self.rank + 2 * self.n, self.act_dtype)
        self.w_x.forward(xc, low)
        dt = ws.buffer("mamba.dt", tokens, self.inner, self.act_dtype)
        self.w_dt.forward(low[:, :self.rank], dt)   # (the first columns of ``low``: rows with a stride)
        y = ws.buffer("mamba.y", tokens, self.inner, self.act_dtype)
        kernels.selective_scan(xc, dt, low, self.rank, self.rank + self.n, xz[:, self.inner:], y, self.dt_bias,
                               self.a_log, self.d, cache.state, ctx.entry_start, ctx.entry_first_row, ctx.entry_slot,
                               entries)
        return self.w_o.forward(y, ws.buffer("mamba.out", tokens, self.hidden, self.act_dtype))
