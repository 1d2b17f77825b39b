"""Linear attention with a constant decay per head ("lightning attention").

For a token with input x: q = act(Wq x), k = act(Wk x) (heads x dim), v = act(Wv x) (heads x vdim), act = silu.
Every head h keeps a state S [dim, vdim] per request, float32, zero at the request's start:

    S <- decay_h S + k v^T          o = S^T q

The heads' outputs of a token, taken together, are divided by their root mean square (eps), multiplied by a weight
and by sigmoid(Wg x), and projected by Wo.  The four input projections are one product with the row-stacked weight;
the recurrence is one kernel for prompts' portions and decoded tokens alike (``csrc/lightning.hip``); norm, gate and
the one rounding are a second kernel.

Parameters: ``hidden_size``, ``num_heads``, ``head_dim``, ``value_dim``, ``decay`` (one number a head), ``norm_eps``,
``activation`` ("silu" or "none"), ``names`` (tensor names below the prefix), ``out_scale`` (a factor on the result).

Variations ("retention" is the combination of all of them): ``position``: a position encoding of the model whose
rotation turns the first channels of every head of q and k (activation "none" only); ``key_scale``: a factor on k,
after the rotation; ``norm``: "all" (default: the heads of a token normed together) or "head" (every head divided by
its own root mean square); ``norm_weight`` (default True; False: the norm has no weight and no tensor);
``gate_activation``: "sigmoid" (default) or "silu".  A rotation and a key factor are applied in float32, by the walk
itself as it fetches q and k (few tokens) or into float32 rows of their own that the walk then reads
(``pulse_rotate_qk_rows``, long portions): nothing behind the projection is rounded before it enters the recurrence.

The part keeps a ``StateSpec`` per run.  It also answers the protocol of a branch of ``side_by_side``:
``inner_width``, ``out_weight()`` and ``forward_inner(x, ctx, cache, out)``.
"""
from __future__ import annotations

from typing import Any, Dict, List, Tuple

import torch

from ..cache.specs import StateSpec, StateView
from ..ops import kernels
from ..weights.store import TensorSpec
from .base import MIXERS, BuildContext, Part, StepContext, StepCost, joined
from .linear import Linear


@MIXERS.register("lightning")
class LightningAttention(Part):
    NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "norm": "norm"}

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        return {**cls.NAMES, **params.get("names", {})}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, heads, d, dv = (params[k] for k in ("hidden_size", "num_heads", "head_dim", "value_dim"))
        n = cls.tensor_names(params)
        specs = {
            n["q"]: TensorSpec((heads * d, hidden), fan_in=hidden),
            n["k"]: TensorSpec((heads * d, hidden), fan_in=hidden),
            n["v"]: TensorSpec((heads * dv, hidden), fan_in=hidden),
            n["gate"]: TensorSpec((heads * dv, hidden), fan_in=hidden),
            n["o"]: TensorSpec((hidden, heads * dv), fan_in=heads * dv),
        }
        if params.get("norm_weight", True):
            specs[n["norm"]] = TensorSpec((heads * dv,), kind="norm")
        return specs

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """The projections, the recurrence (two multiply-adds a state element and token) and every request's state
        read and written once, in float32."""
        cost = super().step_cost(params, entries, weight_bytes, cache_bytes)
        state = params["num_heads"] * params["head_dim"] * params["value_dim"]
        rows = sum(count for _, count in entries)
        cost.flops += 4.0 * state * rows
        cost.cache_bytes += 8.0 * state * len(entries)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.heads = int(params["num_heads"])
        self.d = int(params["head_dim"])
        self.dv = int(params["value_dim"])
        decay = [float(v) for v in params["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"lightning attention of {self.heads} heads got {len(decay)} decays")
        if self.d > 256:
            raise ValueError(f"lightning attention takes at most 256 key channels a head, got {self.d}")
        self.activation = params.get("activation", "silu")
        if self.activation not in ("silu", "none"):
            raise ValueError(f"lightning attention has no kernel for activation '{self.activation}'")
        self.eps = float(params["norm_eps"])
        self.out_scale = float(params.get("out_scale", 1.0))
        self.position = params.get("position")
        self.encodings = build.positions
        if self.position is not None and self.position not in self.encodings:
            raise KeyError(f"lightning attention refers to position encoding '{self.position}', the model defines "
                           f"{sorted(self.encodings)}")
        if self.position is not None and self.activation != "none":
            raise ValueError("lightning attention turns q and k only as they are projected (activation 'none')")
        self.key_scale = float(params.get("key_scale", 1.0))
        self.norm_over = params.get("norm", "all")
        if self.norm_over not in ("all", "head"):
            raise ValueError(f"lightning attention norms 'all' heads together or every 'head', not '{self.norm_over}'")
        self.gate_activation = params.get("gate_activation", "sigmoid")
        if self.gate_activation not in kernels.GATE_FORMS:
            raise ValueError(f"a gate is one of {sorted(kernels.GATE_FORMS)}, not '{self.gate_activation}'")
        self.decay = torch.tensor(decay, dtype=torch.float32, device=build.device)
        load = build.loader
        self.names = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        n = self.names
        self.proj = Linear(load.get_concat([n["q"], n["k"], n["v"], n["gate"]]), build.mode)
        self.norm_weight = load.get(n["norm"]) if params.get("norm_weight", True) else None
        self._o_weight = load.get(n["o"])
        self._o = None
        self.mode = build.mode
        self.act_dtype = build.act_dtype
        self.inner_width = self.heads * self.dv

    records_cleanly = True   # slots, starts and rows are read on the device
    TURN_AHEAD_TOKENS = 256  # steps of at least this many tokens turn q and k in a launch of their own

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.heads, self.d, self.dv), "float32")

    def out_weight(self) -> torch.Tensor:
        """Wo [hidden, inner_width]: what multiplies the rows ``forward_inner`` writes."""
        return self._o_weight

    def forward_inner(self, x: torch.Tensor, ctx: StepContext, cache: StateView, out: torch.Tensor) -> None:
        """The mixer up to its output projection: ``out`` [T, inner_width] (rows may be strided) receives the normed,
        gated heads times ``out_scale``."""
        tokens = x.shape[0]
        ws = ctx.workspace
        hd, hv = self.heads * self.d, self.heads * self.dv
        y = ws.buffer("lightning.proj", tokens, 2 * hd + 2 * hv, self.act_dtype)
        self.proj.forward(x, y)
        o = ws.buffer("lightning.heads", tokens, hv, torch.float32)
        # long portions are walked in pieces that run at the same time (the list depends on the step's shape alone)
        piece_tokens = 64 if tokens < 1024 else 128
        key = f"static:lightning.pieces:{piece_tokens}"
        if key not in ctx.extras:
            flat = kernels.lightning_pieces(ctx.entries, piece_tokens)
            ctx.extras[key] = ctx.to_device(flat) if flat else None
        pieces = ctx.extras[key]
        scratch = None
        walkers = len(ctx.entries)
        if pieces is not None:
            walkers = pieces.numel() // 4
            scratch = ws.buffer("lightning.pieces", walkers, self.heads * self.d * self.dv, torch.float32)
        groups = kernels.lightning_row_groups(walkers, self.heads, self.d, self.dv)
        # A rotation and a key factor, in float32 either way: for few tokens the walk applies them itself as it fetches q
        # and k (a launch less: 47 + 44 -> 49 us for 8 decoded tokens of three layers of 16 heads of 128); long portions,
        # which are walked twice in pieces, get turned float32 rows of their own first (2,048 tokens: 114 + 439 us
        # against 834 with the turn inside both walks).
        turn, rows, scale = None, y, self.key_scale
        if self.position is not None:
            tables = ctx.position_product(self.position, self.encodings)
            turn = (tables.cos, tables.sin, tables.rotary_dim, tables.pairing)
        if tokens >= self.TURN_AHEAD_TOKENS and (turn is not None or scale != 1.0):
            rows = ws.buffer("lightning.rows", tokens, 2 * hd + hv, torch.float32)
            kernels.rotate_qk_rows(y, 0, hd, 2 * hd, rows, self.heads, self.d, self.dv,
                                   turn[0] if turn else None, turn[1] if turn else None, turn[2] if turn else 0,
                                   turn[3] if turn else 0, scale)
            turn, scale = None, 1.0
        kernels.lightning_scan(rows, 0, hd, 2 * hd, o, cache.state, self.decay, ctx.entry_first_row, ctx.entry_start,
                               ctx.entry_slot, self.heads, self.d, self.dv, self.activation, groups, pieces, scratch,
                               turn=turn, key_scale=scale)
        gate = y[:, 2 * hd + hv:]
        if self.norm_over == "all" and self.norm_weight is not None and self.gate_activation == "sigmoid":
            kernels.gated_rmsnorm(o, self.norm_weight, gate, out, self.eps, self.out_scale)
        else:
            kernels.group_norm_gate(o, self.norm_weight, gate, out, self.heads if self.norm_over == "head" else 1,
                                    self.eps, self.out_scale, self.gate_activation)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: StateView) -> torch.Tensor:
        if self._o is None:
            self._o = Linear(self._o_weight, self.mode)
        ws = ctx.workspace
        inner = ws.buffer("lightning.inner", x.shape[0], self.inner_width, self.act_dtype)
        self.forward_inner(x, ctx, cache, inner)
        return self._o.forward(inner, ws.buffer("lightning.out", x.shape[0], self.hidden, self.act_dtype))
