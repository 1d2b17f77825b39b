"""Attention over a paged cache whose inputs are prepared a row at a time: biases on the projections, a norm of q
and of k over a token's WHOLE projection (all heads together, a weight per channel of the projection), keys and values
of different widths.  Window, grouped key/value heads, rotation on the first channels of every head and the scale are
those of ``attention``; so are the attention kernels, which this part inherits.

Parameters beyond those of ``attention``: ``value_dim`` (default ``head_dim``); ``bias`` (q, k and v have biases,
named by ``names`` as ``q_bias`` ...); ``qk_norm``: "projection", "head" (every head of q and k divided by its own root
mean square, no weights; the same before or after the rotation, which keeps a head's sum of squares) or False;
``qk_norm_eps``; ``out_scale`` (a factor on the result; it is multiplied into the values as they are stored, in
float32 before their one rounding); ``output_gate``: "channel": the heads' outputs are multiplied element by element
by sigmoid(Wg x), Wg [heads * value_dim, hidden] (tensor ``gate``), whose rows ride behind q, k and v in the stacked
projection and whose sigmoid the attention kernels apply as they store; ``score_cap`` and ``sink`` as for
``attention``; ``keep_first`` (with a window): a request's first ``keep_first`` tokens stay visible below the window,
at their true positions; ``talk``: the heads' attention weights are mixed before they meet the values, weight_h <-
sum_g T[h, g] weight_g with T the tensor ``talk`` [heads, heads] (a sink's share is not mixed); head h applies its
mixed weights to the values of its own kv head.  Both run on ``pulse_attn_wide`` (bfloat16, the matrix cores) or the
generic attention kernel: with ``talk`` either leaves every head's weights applied to the values of every kv head, in
float32, and ``pulse_head_mix`` forms the sums.

Keys and values are stored with one width D = max(head_dim, value_dim) rounded up to a multiple of 16, the missing
channels as zeros: zero key channels add nothing to a score, and zero value channels come out as zeros, which meet
zero columns of the output weight.  The attention kernels then see ordinary heads of D channels.

It answers the protocol of a branch of ``side_by_side`` (``inner_width``, ``out_weight()``, ``forward_inner``).
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..cache.manager import PagedKVSpec
from ..ops import kernels
from ..weights.store import TensorSpec
from .attention import PagedAttention
from .base import MIXERS, BuildContext, PagedCacheView, Part, StepContext, StepCost, joined
from .linear import Linear


def stored_width(d: int, dv: int) -> int:
    return (max(d, dv) + 15) // 16 * 16


@MIXERS.register("attention_rows")
class RowPreparedAttention(PagedAttention):
    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
             "q_norm": "q.norm", "k_norm": "k.norm", "gate": "g", "sink": "sink", "talk": "talk"}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, nq, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        dv = params.get("value_dim", d)
        n = cls.tensor_names(params)
        specs = {
            n["q"]: TensorSpec((nq * d, hidden), fan_in=hidden),
            n["k"]: TensorSpec((nkv * d, hidden), fan_in=hidden),
            n["v"]: TensorSpec((nkv * dv, hidden), fan_in=hidden),
            n["o"]: TensorSpec((hidden, nq * dv), fan_in=nq * dv),
        }
        if params.get("bias", False):
            specs[n["q_bias"]] = TensorSpec((nq * d,), fan_in=hidden)
            specs[n["k_bias"]] = TensorSpec((nkv * d,), fan_in=hidden)
            specs[n["v_bias"]] = TensorSpec((nkv * dv,), fan_in=hidden)
        if params.get("qk_norm", False) == "projection":
            specs[n["q_norm"]] = TensorSpec((nq * d,), kind="norm")
            specs[n["k_norm"]] = TensorSpec((nkv * d,), kind="norm")
        if params.get("output_gate", False):
            specs[n["gate"]] = TensorSpec((nq * dv, hidden), fan_in=hidden)
        if params.get("sink", False):
            specs[n["sink"]] = TensorSpec((nq,), kind="linear", fan_in=4)
        if params.get("talk", False):
            specs[n["talk"]] = TensorSpec((nq, nq), kind="linear", fan_in=nq)
        return specs

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries, weight_bytes: int, cache_bytes: int) -> StepCost:
        """The projections; scores over head_dim channels and weighted values over value_dim channels for every key a
        token sees; every request's visible keys and values read once, as wide as they are stored."""
        cost = Part.step_cost.__func__(cls, params, entries, weight_bytes, cache_bytes)
        nq, nkv, d, window = params["num_heads"], params["num_kv_heads"], params["head_dim"], params.get("window")
        dv = params.get("value_dim", d)
        first = int(params.get("keep_first", 0) or 0) if window else 0
        fan = nkv if params.get("talk", False) else 1     # every head's weights meet the values of every kv head
        for start, count in entries:
            seen = 0
            for p in range(start, start + count):
                seen += min(p + 1, window + first) if window else p + 1
            cost.flops += 2.0 * nq * (d + dv * fan) * seen
            context = start + count
            kept = min(context, window + first + count - 1) if window else context
            cost.cache_bytes += 2.0 * nkv * stored_width(d, dv) * cache_bytes * kept
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.qk_dim = int(params["head_dim"])
        self.v_dim = int(params.get("value_dim", self.qk_dim))
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} key/value heads")
        self.d = stored_width(self.qk_dim, self.v_dim)     # what the cache and the attention kernels see
        self.scale = float(params["scale"])
        self.window = params.get("window")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"an attention window must be positive, got {self.window}")
        norm = params.get("qk_norm", False)
        if norm not in (False, None, "projection", "head"):
            raise ValueError(f"attention_rows norms q and k over the 'projection', by 'head' or not at all, got {norm!r}")
        self.row_norm = norm == "projection"
        self.head_norm = norm == "head"
        gate = params.get("output_gate", False)
        if gate not in (False, None, "channel"):
            raise ValueError(f"attention_rows has an output gate by 'channel' or none, got {gate!r}")
        self.channel_gate = gate == "channel"
        self.keep_first = int(params.get("keep_first", 0) or 0)
        if self.keep_first < 0:
            raise ValueError(f"the number of kept first tokens must not be negative, got {self.keep_first}")
        if self.window is None:
            self.keep_first = 0
        self.talks = bool(params.get("talk", False))
        if self.talks and self.channel_gate:
            raise ValueError("attention_rows has no kernel for mixed heads with an output gate")
        self._read_score_form(params)
        self.eps = float(params.get("qk_norm_eps", 0.0))
        self.out_scale = float(params.get("out_scale", 1.0))
        self.position = params.get("position")
        self.encodings = build.positions
        if self.position is not None and self.position not in self.encodings:
            raise KeyError(f"attention refers to position encoding '{self.position}', the model defines "
                           f"{sorted(self.encodings)}")
        load = build.loader
        n = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        self.qkv = Linear(load.get_concat([n["q"], n["k"], n["v"]] + ([n["gate"]] if self.channel_gate else [])),
                          build.mode)
        self.kv_cols = self.nq * self.qk_dim + self.nkv * (self.qk_dim + self.v_dim)   # where the gate's columns start
        self.gate_width = self.v_dim if self.channel_gate else 0
        self.sink = self._load_sink(load, n["sink"]) if params.get("sink", False) else None
        self.talk = load.get(n["talk"]) if self.talks else None
        self.biases = tuple(load.get(n[k]) for k in ("q_bias", "k_bias", "v_bias")) if params.get("bias", False) else None
        self.norm_weights = (load.get(n["q_norm"]), load.get(n["k_norm"])) if self.row_norm else None
        o = load.get(n["o"])
        if self.d != self.v_dim:   # zero columns where the stored heads hold zero value channels
            wide = o.new_zeros(self.hidden, self.nq, self.d)
            wide[:, :, :self.v_dim] = o.view(self.hidden, self.nq, self.v_dim)
            o = wide.view(self.hidden, self.nq * self.d).contiguous()
        self._o_weight = o
        self._o = None
        self.mode = build.mode
        self.inner_width = self.nq * self.d
        self.act_dtype = build.act_dtype
        self.options = build.options
        # what the inherited kernel choice asks about (none of it applies here)
        self.qk_norm = self.plain_norm = self.values_are_keys = self.output_gate = False
        self.q_temperature = None
        self.q_w = self.k_w = None

    accepts_residual = False
    accepts_lazy_input = False
    records_cleanly = True

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.nkv, self.d, int(self.window) if self.window is not None else None, self.keep_first)

    def uses_matrix_cores(self, q: torch.Tensor, cache: PagedCacheView) -> bool:
        # (kept first tokens and mixed heads are the generic kernel's)
        return not (self.keep_first or self.talks) and super().uses_matrix_cores(q, cache)

    def out_weight(self) -> torch.Tensor:
        return self._o_weight

    def forward_inner(self, x: torch.Tensor, ctx: StepContext, cache: PagedCacheView, out: torch.Tensor) -> None:
        tokens = x.shape[0]
        ws = ctx.workspace
        write = cache.writable
        rows = None if (write or self.channel_gate) else self.nq * self.qk_dim
        cols = self.qkv.out_features if rows is None else rows
        qkv = ws.buffer("attention_rows.qkv", tokens, cols, self.act_dtype)
        self.qkv.forward(x, qkv, rows=rows)
        tables = ctx.position_product(self.position, self.encodings) if self.position is not None else None
        table = ctx.block_tables[cache.group]
        q = ws.buffer("attention_rows.q", tokens, self.nq * self.d, self.act_dtype)
        kernels.qkv_rows(qkv, q, self.nq, self.nkv, self.qk_dim, self.v_dim, self.d, self.biases, self.norm_weights,
                         self.eps, tables.cos if tables is not None else None,
                         tables.sin if tables is not None else None, tables.rotary_dim if tables is not None else 0,
                         tables.pairing if tables is not None else 0, cache.keys, cache.values, ctx.positions,
                         ctx.token_entry, table, write_kv=write, value_scale=self.out_scale,
                         norm="head" if self.head_norm else self.row_norm)
        gate = qkv[:, self.kv_cols:self.kv_cols + self.nq * self.v_dim] if self.channel_gate else None
        if not (self.keep_first or self.talks):
            self.attend(q, out, ctx, cache, table, gate=gate)
            return
        window = int(self.window) if self.window is not None else 0
        wide = (self.options.get("attention", "auto") != "generic" and gate is None
                and kernels.attn_wide_takes(q, cache.keys, self.d))
        if not self.talks and not wide:
            kernels.attn_generic(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                 ctx.token_entry, table, self.scale, window, gate=gate, gate_width=self.gate_width,
                                 sink=self.sink, softcap=self.score_cap, keep_first=self.keep_first)
            return
        # float32 rows first: with mixed heads every head's weights on every kv head's values, then the sums over heads
        # that the mixing matrix asks for; without, the rows as they are (the branch's factor is in the stored values)
        width = self.nq * self.d * (self.nkv if self.talks else 1)
        each = ws.buffer("attention_rows.each", tokens, width, torch.float32)
        if wide:
            items, hp, row_tiles = self._wide_items(ctx)
            wv = self.nkv * self.d if self.talks else self.d
            keys = min(ctx.max_context, window + self.keep_first + 32) if window else ctx.max_context
            splits = kernels.attn_wide_splits(items.numel() // 4, (wv + 255) // 256, keys) if row_tiles == 1 else 1
            part = part_ml = None
            if splits > 1:
                part = ws.buffer("attn_wide.part", tokens * self.nq * splits, wv, torch.float32)
                part_ml = ws.buffer("attn_wide.part_ml", tokens * self.nq * splits, 2, torch.float32)
            kernels.attn_wide(q, each, self.nq, self.nkv, self.d, wv, self.talks, cache.keys, cache.values, ctx.positions,
                              ctx.token_entry, table, items, hp, self.scale, window, self.keep_first, self.sink,
                              self.score_cap, row_tiles, splits, part, part_ml)
        else:
            kernels.attn_generic(q, each, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                 ctx.token_entry, table, self.scale, window, sink=self.sink, softcap=self.score_cap,
                                 keep_first=self.keep_first, all_values=True)
        if self.talks:
            kernels.head_mix(each, self.talk, out, self.nq, self.nkv, self.d, self.v_dim, self.d)
        else:
            kernels.head_mix(each, self._identity(each.device), out, self.nq, 1, self.d, self.v_dim, self.d)

    def _wide_items(self, ctx: StepContext):
        """The work list of ``attn_wide`` for this step (it depends on the step's shape alone; every layer with these
        head counts shares it)."""
        key = f"static:attention_rows.wide_items:{self.nq}:{self.nkv}"
        if key not in ctx.extras:
            row_tiles = kernels.attn_wide_row_tiles(ctx.num_tokens)
            flat, hp = kernels.attn_wide_items(ctx.entries, self.nq, self.nkv, row_tiles)
            ctx.extras[key] = (ctx.to_device(flat), hp, row_tiles)
        return ctx.extras[key]

    def _identity(self, device) -> torch.Tensor:
        if getattr(self, "_eye", None) is None:
            self._eye = torch.eye(self.nq, dtype=torch.float32, device=device)
        return self._eye

    def decodes_from_raw(self, ctx, cache, qkv, tables) -> bool:
        return False

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: PagedCacheView) -> torch.Tensor:
        if self._o is None:
            self._o = Linear(self._o_weight, self.mode)
        ws = ctx.workspace
        inner = ws.buffer("attention_rows.inner", x.shape[0], self.inner_width, self.act_dtype)
        self.forward_inner(x, ctx, cache, inner)
        return self._o.forward(inner, ws.buffer("attention_rows.out", x.shape[0], self.hidden, self.act_dtype))
