"""A routed feed-forward: every token goes through the few experts its router chooses.

Router: z = Wr x in float32; s = softmax(z) over all router outputs; the ``top`` outputs with the largest
s + correction are chosen; their weights are their s divided by the sum of the chosen s (+ 1e-20).  The first
``num_experts`` outputs are gated feed-forwards, down_e(silu(gate_e x) * (up_e x)), without biases; the last
``num_identity`` outputs are identity experts, whose result is x itself and which have no tensors.  The result is the
weighted sum over the chosen outputs; a shared expert of the same form (``shared_size``, optional) runs for every
token and is added.

Parameters: ``hidden_size``, ``expert_size``, ``num_experts``, ``num_identity``, ``top``, ``correction`` (whether a
correction tensor exists), ``shared_size`` (None: no shared expert), ``names``: ``router``, ``correction``,
``expert`` (a pattern with ``{e}``), ``gate`` / ``up`` / ``down`` (below an expert's or the shared expert's prefix),
``shared``; ``score``: "softmax" (default) or "sigmoid" (s = sigmoid(z), every output by itself); ``renormalize``
(default True; False: the weights are the chosen scores as they are); ``weight_on``: "output" (default) or "input" (an
expert is fed weight * x, and the experts' results are added as they are); ``expert_activation``: "silu" (default) or
"clamped_swish" with ``limit``: g = min(gate x, limit), u = clamp(up x, -limit, limit), down(g * sigmoid(1.702 g) *
(u + 1)); ``shared_gate`` (default False): the shared expert's result is multiplied by sigmoid(w_sg . x), one number a
token, with w_sg the tensor ``shared_gate`` [1, hidden] below the shared expert's prefix (the product then goes into
the routed float32 sum and the part hands back one update).

The experts' weights are stacked at load time ([experts, rows, columns]).  ``forward`` returns the routed part
(float32) and the shared expert's part as two updates that the block adds.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from ..ops import kernels
from ..weights.store import TensorSpec
from .base import FEED_FORWARDS, BuildContext, Part, StepContext, StepCost, joined
from .mlp import GatedMLP


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(Part):
    NAMES = {"router": "router", "correction": "correction", "expert": "e{e}", "gate": "gate", "up": "up",
             "down": "down", "shared": "shared", "shared_gate": "sg"}

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        return {**cls.NAMES, **params.get("names", {})}

    @classmethod
    def _shared_params(cls, params: Dict[str, Any]) -> Optional[Dict[str, Any]]:
        if params.get("shared_size") is None:
            return None
        n = cls.tensor_names(params)
        return {"hidden_size": params["hidden_size"], "intermediate_size": params["shared_size"], "activation": "silu",
                "names": {"gate": n["gate"], "up": n["up"], "down": n["down"]}}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, ff, experts = params["hidden_size"], params["expert_size"], params["num_experts"]
        outputs = experts + params.get("num_identity", 0)
        n = cls.tensor_names(params)
        specs = {n["router"]: TensorSpec((outputs, hidden), fan_in=hidden)}
        if params.get("correction", False):
            specs[n["correction"]] = TensorSpec((outputs,), kind="linear", fan_in=100 * outputs)
        for e in range(experts):
            sub = n["expert"].format(e=e)
            specs[joined(sub, n["gate"])] = TensorSpec((ff, hidden), fan_in=hidden)
            specs[joined(sub, n["up"])] = TensorSpec((ff, hidden), fan_in=hidden)
            specs[joined(sub, n["down"])] = TensorSpec((hidden, ff), fan_in=ff)
        shared = cls._shared_params(params)
        if shared is not None:
            for name, spec in GatedMLP.weight_specs(shared).items():
                specs[joined(n["shared"], name)] = spec
            if params.get("shared_gate", False):
                specs[joined(n["shared"], n["shared_gate"])] = TensorSpec((1, hidden), fan_in=hidden)
        return specs

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries: List[Tuple[int, int]], weight_bytes: int,
                  cache_bytes: int) -> StepCost:
        """Router and shared expert for every row; of the routed experts what the rows choose: ``top`` experts a row
        in arithmetic (less the identity experts' share), and at most all experts' weights once."""
        hidden, ff, experts = params["hidden_size"], params["expert_size"], params["num_experts"]
        outputs = experts + params.get("num_identity", 0)
        rows = sum(count for _, count in entries)
        real = params["top"] * experts / float(outputs)
        cost = StepCost(flops=2.0 * rows * outputs * hidden + 6.0 * rows * real * hidden * ff,
                        weight_bytes=float(outputs * hidden * weight_bytes)
                        + 3.0 * hidden * ff * weight_bytes * min(experts, rows * real))
        shared = cls._shared_params(params)
        if shared is not None:
            cost = cost + GatedMLP.step_cost(shared, entries, weight_bytes, cache_bytes)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.ff = int(params["expert_size"])
        self.experts = int(params["num_experts"])
        self.identity = int(params.get("num_identity", 0))
        self.top = int(params["top"])
        outputs = self.experts + self.identity
        if not 0 < self.top <= outputs:
            raise ValueError(f"a router with {outputs} outputs cannot choose {self.top}")
        if self.experts <= 0:
            raise ValueError("routed_experts needs at least one expert with weights")
        load = build.loader
        n = self.tensor_names(params)
        self.router = load.get(joined(prefix, n["router"]))
        self.correction = load.get(joined(prefix, n["correction"])) if params.get("correction", False) else None
        if self.correction is not None and self.correction.dtype != self.router.dtype:
            self.correction = self.correction.to(self.router.dtype)
        stack = lambda which: torch.stack([load.get(joined(joined(prefix, n["expert"].format(e=e)), n[which]))
                                           for e in range(self.experts)], dim=0).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        shared = self._shared_params(params)
        self.shared = GatedMLP(shared, joined(prefix, n["shared"]), build) if shared is not None else None
        self.shared_gate = None
        if self.shared is not None and params.get("shared_gate", False):
            self.shared_gate = load.get(joined(joined(prefix, n["shared"]), n["shared_gate"])).reshape(-1).contiguous()
        self.score = params.get("score", "softmax")
        if self.score not in kernels.ROUTER_SCORES:
            raise ValueError(f"a router scores by {sorted(kernels.ROUTER_SCORES)}, not '{self.score}'")
        self.renormalize = bool(params.get("renormalize", True))
        weight_on = params.get("weight_on", "output")
        if weight_on not in ("output", "input"):
            raise ValueError(f"an expert's weight goes on its 'output' or its 'input', not '{weight_on}'")
        self.weight_on_input = weight_on == "input"
        if self.weight_on_input and self.identity:
            raise ValueError("identity experts take their weight on the output")
        self.expert_activation = params.get("expert_activation", "silu")
        if self.expert_activation not in kernels.EXPERT_ACTIVATIONS:
            raise ValueError(f"experts know the activations {sorted(kernels.EXPERT_ACTIVATIONS)}, not "
                             f"'{self.expert_activation}'")
        self.limit = float(params.get("limit", 0.0))
        if self.expert_activation == "clamped_swish" and not self.limit > 0.0:
            raise ValueError("the clamped activation needs a positive limit")
        self.act_dtype = build.act_dtype
        self.device = build.device

    records_cleanly = True   # choices stay on the device; the launches do not depend on them
    returns_two = True       # forward gives (routed update, shared update or None)

    def forward(self, x: torch.Tensor, ctx: StepContext):
        tokens = x.shape[0]
        ws = ctx.workspace
        idx = ws.buffer("moe.idx", tokens, self.top, torch.int32)
        weight = ws.buffer("moe.weight", tokens, self.top, torch.float32)
        kernels.moe_router(x, self.router, self.correction, self.top, idx, weight, score=self.score,
                           renormalize=self.renormalize)   # logits in float32 inside
        act = ws.buffer("moe.act", tokens * self.top, self.ff, self.act_dtype)
        routed = ws.buffer("moe.out", tokens, self.hidden, torch.float32)
        if kernels.moe_grouped_takes(x, self.w_gate, self.w_down):
            # bfloat16: the pairs grouped by expert on the device, every expert's rows on the matrix cores; tiles of
            # 128 rows once an expert gets about that many
            pairs = tokens * self.top
            rows = kernels.MOE_TILE_ROWS[1] if pairs >= 64 * self.experts else kernels.MOE_TILE_ROWS[0]
            y = ws.buffer("moe.y", pairs, self.hidden, torch.float32)
            ints = ws.buffer("moe.ints", 2 * pairs + 3 * kernels.moe_max_tiles(pairs, self.experts, rows) + 1, 1, torch.int32)
            kernels.moe_grouped(x, self.w_gate, self.w_up, self.w_down, idx, weight, act, y, routed, ints.view(-1), rows,
                                weight_on_input=self.weight_on_input, activation=self.expert_activation,
                                limit=self.limit)
        else:
            kernels.moe_gate_up(x, self.w_gate, self.w_up, idx, act, in_weight=weight if self.weight_on_input else None,
                                activation=self.expert_activation, limit=self.limit)
            kernels.moe_down(x, act, self.w_down, idx, None if self.weight_on_input else weight, routed)
        shared = self.shared.forward(x, ctx) if self.shared is not None else None
        if shared is not None and self.shared_gate is not None:
            kernels.token_gate_add(x, self.shared_gate, shared, routed)
            shared = None
        return routed, shared
