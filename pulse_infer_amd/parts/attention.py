"""Causal attention over a paged cache, with grouped key/value heads, optional
per-head RMSNorm of q and k, an optional window and a pluggable position encoding.

Order of operations per token (reference: src/model/qwen3/model.cpp:784-876):
q, k, v = x Wq^T, x Wk^T, x Wv^T; q, k <- RMSNorm over head_dim (one weight for
all heads); q, k <- rotation at the token's position; k, v written to the
cache; o = softmax(q K^T * scale) V over keys lo..position of the same request;
output = o Wo^T.  Query head h reads kv head h // (num_heads // num_kv_heads).
A window w gives lo = max(0, position - w + 1); without one lo = 0.

The three projections are one product with the row-stacked weight (a layout
choice); norm, rotation and the cache write are one kernel; the attention
kernel is chosen by size and storage type.

Variations, all parameters of the part:

* ``values = "keys"``: there is no value projection; a token's values are its keys as projected, before the norm
  (the cache then holds the normed keys and the raw ones);
* ``qk_norm_weights = False``: the per-head norm of q and k has no weights (x / sqrt(mean(x^2) + eps) alone);
* ``query_temperature = {"coef": c, "every": n}``: after the norm q is multiplied by
  1 + c * ln(floor((position + 1) / n) + 1), in float32;
* ``output_gate = True``: head h's output is multiplied by sigmoid(g_h), g = x Wg^T with Wg [heads, hidden] (one
  number a token and head), before the output projection; Wg's rows ride behind the other projections in the
  stacked weight, and the attention kernels apply the gate as they store their result;
* ``score_cap = c``: a scaled score s becomes c * tanh(s / c) before the softmax;
* ``sink = True``: a learned number per query head (tensor ``sink`` [heads]) whose exponential is one more term of
  the softmax's denominator; it has no key and no value;
* ``names``: the tensors' names below the part's prefix.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..cache.manager import PagedKVSpec
from ..ops import attention_mfma, kernels
from ..weights.store import TensorSpec
from .base import MIXERS, BuildContext, LazyNorm, PagedCacheView, Part, StepContext, StepCost, joined
from .linear import Linear


@MIXERS.register("attention")
class PagedAttention(Part):
    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, nq, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads", "head_dim"))
        names = cls.tensor_names(params)
        specs = {
            names["q"]: TensorSpec((nq * d, hidden), fan_in=hidden),
            names["k"]: TensorSpec((nkv * d, hidden), fan_in=hidden),
            names["o"]: TensorSpec((hidden, nq * d), fan_in=nq * d),
        }
        if params.get("values", "projection") == "projection":
            specs[names["v"]] = TensorSpec((nkv * d, hidden), fan_in=hidden)
        if params.get("output_gate", False):
            specs[names["gate"]] = TensorSpec((nq, hidden), fan_in=hidden)
        if params.get("qk_norm", False) and params.get("qk_norm_weights", True):
            specs[names["q_norm"]] = TensorSpec((d,), kind="norm")
            specs[names["k_norm"]] = TensorSpec((d,), kind="norm")
        if params.get("sink", False):
            specs[names["sink"]] = TensorSpec((nq,), kind="linear", fan_in=4)
        return specs

    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "gate": "g_proj.weight", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "sink": "sink"}
    GATE_PAD = 16   # the gate's rows of the stacked weight are filled up with zero rows to a multiple of this, so that
                    # the projection output's rows keep the alignment the kernels' 16-byte accesses need

    @classmethod
    def tensor_names(cls, params: Dict[str, Any]) -> Dict[str, str]:
        """The tensors' names below the part's prefix; ``params["names"]`` replaces any of the usual ones."""
        return {**cls.NAMES, **params.get("names", {})}

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries, weight_bytes: int, cache_bytes: int) -> StepCost:
        """The projections, plus scores and weighted values over the keys each token sees (2 x 2 x heads x head size
        a key), plus the keys and values of every request's visible context read once."""
        cost = super().step_cost(params, entries, weight_bytes, cache_bytes)
        nq, nkv, d, window = params["num_heads"], params["num_kv_heads"], params["head_dim"], params.get("window")
        for start, count in entries:
            seen = 0
            for p in range(start, start + count):
                seen += min(p + 1, window) if window else p + 1
            cost.flops += 4.0 * nq * d * seen
            context = start + count
            cost.cache_bytes += 2.0 * nkv * d * cache_bytes * (min(context, window + count - 1) if window else context)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = int(params["num_kv_heads"])
        self.d = int(params["head_dim"])
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} key/value heads")
        self.scale = float(params["scale"])
        self.window = params.get("window")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"an attention window must be positive, got {self.window}")
        self.qk_norm = bool(params.get("qk_norm", False))
        self.plain_norm = self.qk_norm and not params.get("qk_norm_weights", True)
        self.eps = float(params.get("qk_norm_eps", 0.0))
        values = params.get("values", "projection")
        if values not in ("projection", "keys"):
            raise ValueError(f"attention values must be 'projection' or 'keys', got '{values}'")
        self.values_are_keys = values == "keys"
        temperature = params.get("query_temperature")
        self.q_temperature = None
        if temperature is not None:
            self.q_temperature = (float(temperature["coef"]), int(temperature["every"]))
            if self.q_temperature[1] <= 0:
                raise ValueError(f"query_temperature.every must be positive, got {self.q_temperature[1]}")
        self.output_gate = bool(params.get("output_gate", False))
        self._read_score_form(params)
        self.position = params.get("position")
        self.encodings = build.positions
        if self.position is not None and self.position not in self.encodings:
            raise KeyError(f"attention refers to position encoding '{self.position}', the model defines "
                           f"{sorted(self.encodings)}")
        load = build.loader
        names = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        stacked = [names["q"], names["k"]] + ([] if self.values_are_keys else [names["v"]])
        # columns of the projection output: q heads, k heads, v heads (unless the values are the keys), gate
        self.v_head0 = self.nq if self.values_are_keys else self.nq + self.nkv
        self.kv_cols = (self.nq + self.nkv * (1 if self.values_are_keys else 2)) * self.d
        self.gate_rows = 0
        if self.output_gate:
            weight = load.get_concat(stacked + [names["gate"]])
            self.gate_rows = (self.nq + self.GATE_PAD - 1) // self.GATE_PAD * self.GATE_PAD
            if self.gate_rows > self.nq:
                weight = torch.cat([weight, weight.new_zeros(self.gate_rows - self.nq, self.hidden)], dim=0).contiguous()
            self.qkv = Linear(weight, build.mode)
        else:
            self.qkv = Linear(load.get_concat(stacked), build.mode)
        self.o = Linear(load.get(names["o"]), build.mode)
        weighted = self.qk_norm and not self.plain_norm
        self.q_w = load.get(names["q_norm"]) if weighted else None
        self.k_w = load.get(names["k_norm"]) if weighted else None
        self.sink = self._load_sink(load, names["sink"]) if params.get("sink", False) else None
        self.act_dtype = build.act_dtype
        self.options = build.options

    gate_width = 0     # > 0: the output gate has a logit for each of that many channels of a head (a subclass's)
    score_cap = 0.0
    sink = None

    def _read_score_form(self, params: Dict[str, Any]) -> None:
        self.score_cap = float(params.get("score_cap") or 0.0)
        if self.score_cap < 0.0:
            raise ValueError(f"a score cap must be positive, got {self.score_cap}")

    @staticmethod
    def _load_sink(load: Any, name: str) -> torch.Tensor:
        """The sinks as float32 [heads], whatever the checkpoint's storage type."""
        return load.get(name).to(torch.float32).contiguous()

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(self.nkv, self.d, int(self.window) if self.window is not None else None)

    accepts_residual = True
    accepts_lazy_input = True   # the first product may take rows that are not normalised yet and scale its result
    records_cleanly = True      # positions, tables and work lists are read on the device

    def forward(self, x, ctx: StepContext, cache: PagedCacheView, residual: Optional[torch.Tensor] = None,
                next_scale: Optional[torch.Tensor] = None, next_offset: float = 0.0, leave_stats: bool = True):
        tokens = x.shape[0]
        ws = ctx.workspace
        write = cache.writable
        q_cols = self.nq * self.d
        # a run that reads another run's cache needs its queries only (and all rows if a gate rides behind the keys)
        rows = None if (write or self.output_gate) else q_cols
        cols = self.qkv.out_features if rows is None else rows
        qkv = ws.buffer("attention.qkv", tokens, cols, self.act_dtype)
        if isinstance(x, LazyNorm) and not self.qkv.takes_lazy(x, rows=rows):
            x = x.materialize(ws.buffer("attention.normed", tokens, self.hidden, self.act_dtype))
        self.qkv.forward(x, qkv, rows=rows)
        gate = qkv[:, self.kv_cols:self.kv_cols + self.nq] if self.output_gate else None
        tables = ctx.position_product(self.position, self.encodings) if self.position is not None else None
        table = ctx.block_tables[cache.group]
        attn = ws.buffer("attention.out", tokens, q_cols, self.act_dtype)
        if self.decodes_from_raw(ctx, cache, qkv, tables):
            # decoded tokens only: the attention kernel prepares q and each token's own key itself
            self.attend(qkv, attn, ctx, cache, table, raw=(tables, write), gate=gate)
        else:
            kernels.qk_rope_kv(
                qkv, self.nq, self.nkv, self.d, self.q_w, self.k_w, self.eps,
                tables.cos if tables is not None else None, tables.sin if tables is not None else None,
                tables.rotary_dim if tables is not None else 0, tables.pairing if tables is not None else 0,
                cache.keys, cache.values, ctx.positions, ctx.token_entry, table, write_kv=write,
                plain_norm=self.plain_norm, v_head0=self.v_head0, q_temperature=self.q_temperature)
            self.attend(qkv, attn, ctx, cache, table, gate=gate)
        out = ws.buffer("attention.proj", tokens, self.hidden, self.act_dtype)
        if residual is not None:
            return self.o.add_into(attn, residual, out, ws, next_scale, next_offset, leave_stats)
        return self.o.forward(attn, out)

    def takes_lazy_input(self, x: LazyNorm, cache: PagedCacheView) -> bool:
        """Whether ``forward`` would run its first product on rows that are not normalised yet, or compute the norm."""
        rows = None if (cache.writable or self.output_gate) else self.nq * self.d
        return self.qkv.takes_lazy(x, rows=rows)

    def uses_matrix_cores(self, q: torch.Tensor, cache: PagedCacheView) -> bool:
        return (self.options.get("attention", "auto") != "generic"
                and attention_mfma.supported(self.d, cache.page_size, q.dtype, cache.keys.dtype))

    def decodes_from_raw(self, ctx: StepContext, cache: PagedCacheView, qkv: torch.Tensor, tables: Any) -> bool:
        """Whether this step's attention can start from the raw projection output: every entry is one decoded
        token, the matrix-core kernel takes the sizes, and norm weights and rotation are of the kinds it prepares."""
        if self.options.get("decode_from_raw", True) is False or not self.uses_matrix_cores(qkv, cache):
            return False
        if self.score_cap or self.sink is not None:
            return False
        if "static:attention.single_tokens" not in ctx.extras:
            ctx.extras["static:attention.single_tokens"] = all(e.count == 1 for e in ctx.entries)
        if not ctx.extras["static:attention.single_tokens"]:
            return False
        if any(w is not None and w.dtype != torch.bfloat16 for w in (self.q_w, self.k_w)):
            return False
        if tables is None:
            return True
        return (tables.cos.dtype == torch.float32 and tables.cos.is_contiguous() and tables.sin.is_contiguous()
                and attention_mfma.decode_takes(self.d, tables.rotary_dim, tables.pairing))

    def attend(self, q: torch.Tensor, out: torch.Tensor, ctx: StepContext, cache: PagedCacheView,
               table: torch.Tensor, raw: Optional[tuple] = None, gate: Optional[torch.Tensor] = None) -> None:
        """out = attention of the step's tokens over the cache.  ``raw = (rotation tables, write)``: q is the raw
        projection output of decoded tokens, which the kernel prepares itself (see ``decodes_from_raw``).  ``gate``
        [T, heads]: the logits of the output gate, applied by whichever kernel stores the result."""
        window = int(self.window) if self.window is not None else 0
        if not self.uses_matrix_cores(q, cache):
            kernels.attn_generic(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                 ctx.token_entry, table, self.scale, window, gate=gate, gate_width=self.gate_width,
                                 sink=self.sink, softcap=self.score_cap)
            return
        group = self.nq // self.nkv
        per = attention_mfma.tokens_per_item(group)
        portion = attention_mfma.portion_tokens(group, self.d)
        key = f"static:attention.items:{per}:{portion}"
        if key not in ctx.extras:  # depends only on the step's shape; the same lists serve every layer
            short, long = attention_mfma.split_entries(ctx.entries)
            dev = lambda flat: ctx.to_device(flat) if flat else None
            ctx.extras[key] = (
                dev(attention_mfma.build_items(short, per)),
                dev(attention_mfma.build_items(long, portion)),
                max((e.start + e.count for _, e in short), default=0))
        short_items, long_items, short_context = ctx.extras[key]
        if long_items is not None:
            skey = f"static:attention.portion_splits:{portion}:{window}:{self.nkv}:{group}:{self.d}"
            if skey not in ctx.extras:
                ctx.extras[skey] = attention_mfma.choose_prefill_splits(
                    attention_mfma.split_entries(ctx.entries)[1], portion, self.nkv, group, self.d, window)
            split_size, n_splits = ctx.extras[skey]
            part_o = part_ml = None
            if n_splits > 1:
                rows = ctx.num_tokens * self.nq * n_splits
                part_o = ctx.workspace.buffer("attention.portion_part_o", rows, self.d, torch.float32)
                part_ml = ctx.workspace.buffer("attention.portion_part_ml", rows, 2, torch.float32)
            attention_mfma.attn_prefill(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                        table, long_items, self.scale, window, split_size, n_splits, part_o, part_ml,
                                        gate=gate, gate_width=self.gate_width, sink=self.sink, softcap=self.score_cap)
        if short_items is not None:
            # a recorded step passes its context bucket as max_context: its splits must cover that
            max_context = ctx.max_context if long_items is None else short_context
            n_items = short_items.numel() // attention_mfma.ITEM_INTS
            split_size, n_splits = attention_mfma.choose_splits(n_items, self.nkv, group, max_context)
            plan = None
            if ctx.uneven and long_items is None and not window:
                # contexts that differ much: every request's keys cut by its own length, the workgroups in an order
                # that starts the longest walks first (the plan is made on the device, once a step for all layers)
                planned = min(attention_mfma.PLAN_SPLITS, 1024 // n_items)
                if planned > 1 and attention_mfma.plan_fits(n_items, planned):
                    n_splits = planned
                    split_size = max(32, ((max_context + n_splits - 1) // n_splits + 31) // 32 * 32)
                    slots, first = attention_mfma.plan_slots(self.nkv, group)
                    pkey = f"attention.plan:{per}:{n_splits}:{slots}:{first}"
                    if pkey not in ctx.extras:
                        made = ctx.workspace.buffer(f"attention.plan:{n_splits}:{slots}:{first}",
                                                    attention_mfma.plan_ints(n_items, n_splits), 1, torch.int32)
                        attention_mfma.attn_plan(short_items if raw is None else None, ctx.positions, n_splits, slots,
                                                 first, made, self.d)
                        ctx.extras[pkey] = made
                    plan = ctx.extras[pkey]
            part_o = part_ml = None
            if n_splits > 1:
                rows = ctx.num_tokens * self.nq * n_splits
                part_o = ctx.workspace.buffer("attention.part_o", rows, self.d, torch.float32)
                part_ml = ctx.workspace.buffer("attention.part_ml", rows, 2, torch.float32)
            if raw is not None:
                tables, write = raw
                # (no list of items: the step's tokens are its requests' in order, each with its row of the table)
                attention_mfma.attn_decode(
                    q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions, table, None,
                    self.scale, window, split_size, n_splits, max_context, part_o, part_ml, self.q_w, self.k_w,
                    self.eps, tables.cos if tables is not None else None, tables.sin if tables is not None else None,
                    tables.rotary_dim if tables is not None else 0, tables.pairing if tables is not None else 0,
                    new_key=write, live_context=ctx.live_context if plan is None else None, plan=plan, gate=gate,
                    plain_norm=self.plain_norm, v_head0=self.v_head0, q_temperature=self.q_temperature)
                return
            attention_mfma.attn_mfma(q, out, self.nq, self.nkv, self.d, cache.keys, cache.values, ctx.positions,
                                     table, short_items, self.scale, window, split_size, n_splits,
                                     max_context, part_o, part_ml,
                                     live_context=ctx.live_context if plan is None else None, plan=plan, gate=gate,
                                     gate_width=self.gate_width, sink=self.sink, softcap=self.score_cap)
