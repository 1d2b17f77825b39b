"""Attention whose keys and values come from one latent row a token ("latent attention").

For a token with input x: q = Wq x, laid out head by head as [dim plain | rot_dim turned]; [c_raw | k_rot] = Wd x with
``latent_dim`` + ``rotary_dim`` rows; c = c_raw / rms(c_raw) * w (the latent row) and k_rot, turned by the token's
position, are all that is cached.  Head h's key is [W_uk,h c | k_rot] (the turned part is shared by all heads), its
value W_uv,h c; scores are (q . key) * scale over all earlier tokens, softmax with an optional sink per head; the
heads' results, side by side, are multiplied element by element by sigmoid(Wg x) (optional) and projected by Wo.

Scores and weighted sums are linear in c, so the part works in the latent space and paged attention kernels serve it
as they are (those of ``attention`` where they are compiled for rows this wide, else ``pulse_attn_wide``, else the
generic one): one kv head whose stored key is [c | k_rot] and whose stored value is c, query head
h = [W_uk,h^T q_plain,h | q_rot,h], and W_uv,h applied to the weighted sum of latent rows afterwards.  Keys and values
are stored ``stored`` = latent_dim + rotary_dim (rounded up to 16) channels wide, the rest zeros.

Parameters: ``hidden_size``, ``num_heads``, ``head_dim`` (plain channels of a head), ``rotary_dim``, ``value_dim``,
``latent_dim``, ``scale``, ``norm_eps``, ``position`` (a rotary encoding of ``rotary_dim`` channels), ``sink``,
``output_gate`` (True: by channel), ``names``, ``out_scale``.

Kernels: ``pulse_latent_rows`` (norm of the latent row, turns, page write), ``pulse_heads_product`` (bfloat16: both
products a head on the matrix cores) or ``pulse_latent_absorb`` / ``pulse_latent_expand`` (queries into the latent
space, values out of it with the gate), and the attention kernels between them.  It answers the
protocol of a branch of ``side_by_side``.
"""
from __future__ import annotations

from typing import Any, Dict

import torch

from ..cache.manager import PagedKVSpec
from ..ops import kernels
from ..weights.store import TensorSpec
from .attention import PagedAttention
from .base import MIXERS, BuildContext, PagedCacheView, Part, StepContext, StepCost, joined
from .linear import Linear


def latent_stored_width(rank: int, rot: int) -> int:
    return (rank + rot + 15) // 16 * 16


@MIXERS.register("latent_attention")
class LatentAttention(PagedAttention):
    NAMES = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "gate": "g", "sink": "sink",
             "o": "o"}

    @classmethod
    def weight_specs(cls, params: Dict[str, Any]) -> Dict[str, TensorSpec]:
        hidden, heads, d, rot, dv, rank = (params[k] for k in ("hidden_size", "num_heads", "head_dim", "rotary_dim",
                                                               "value_dim", "latent_dim"))
        n = cls.tensor_names(params)
        specs = {
            n["q"]: TensorSpec((heads * (d + rot), hidden), fan_in=hidden),
            n["down"]: TensorSpec((rank + rot, hidden), fan_in=hidden),
            n["down_norm"]: TensorSpec((rank,), kind="norm"),
            n["up_k"]: TensorSpec((heads * d, rank), fan_in=rank),
            n["up_v"]: TensorSpec((heads * dv, rank), fan_in=rank),
            n["o"]: TensorSpec((hidden, heads * dv), fan_in=heads * dv),
        }
        if params.get("output_gate", False):
            specs[n["gate"]] = TensorSpec((heads * dv, hidden), fan_in=hidden)
        if params.get("sink", False):
            specs[n["sink"]] = TensorSpec((heads,), kind="linear", fan_in=4)
        return specs

    @classmethod
    def step_cost(cls, params: Dict[str, Any], entries, weight_bytes: int, cache_bytes: int) -> StepCost:
        """The projections (the two up projections a head and row); scores and weighted sums in the latent space over
        every earlier token; every request's stored rows read once."""
        cost = Part.step_cost.__func__(cls, params, entries, weight_bytes, cache_bytes)
        heads, rot, rank = params["num_heads"], params["rotary_dim"], params["latent_dim"]
        stored = latent_stored_width(rank, rot)
        for start, count in entries:
            seen = sum(p + 1 for p in range(start, start + count))
            cost.flops += 2.0 * heads * (2 * rank + rot) * seen
            cost.cache_bytes += 2.0 * stored * cache_bytes * (start + count)
        return cost

    def __init__(self, params: Dict[str, Any], prefix: str, build: BuildContext):
        self.hidden = int(params["hidden_size"])
        self.nq = int(params["num_heads"])
        self.nkv = 1
        self.plain_dim = int(params["head_dim"])
        self.rot_dim = int(params["rotary_dim"])
        self.v_dim = int(params["value_dim"])
        self.rank = int(params["latent_dim"])
        if min(self.nq, self.plain_dim, self.rot_dim, self.v_dim, self.rank) <= 0 or self.rot_dim % 2:
            raise ValueError("latent attention needs positive sizes and an even rotary_dim")
        self.d = latent_stored_width(self.rank, self.rot_dim)    # what the cache and the attention kernels see
        self.scale = float(params["scale"])
        self.window = None
        self.eps = float(params["norm_eps"])
        self.out_scale = float(params.get("out_scale", 1.0))
        self._read_score_form(params)
        self.position = params.get("position")
        self.encodings = build.positions
        if self.position is None or self.position not in self.encodings:
            raise KeyError(f"latent attention needs a position encoding of the model, got '{self.position}' "
                           f"(the model defines {sorted(self.encodings)})")
        load = build.loader
        n = {k: joined(prefix, v) for k, v in self.tensor_names(params).items()}
        self.gated = bool(params.get("output_gate", False))
        self.proj = Linear(load.get_concat([n["q"], n["down"]] + ([n["gate"]] if self.gated else [])), build.mode)
        self.q_cols = self.nq * (self.plain_dim + self.rot_dim)
        self.gate_col0 = self.q_cols + self.rank + self.rot_dim
        self.norm_weight = load.get(n["down_norm"])
        self.w_uk = load.get(n["up_k"])
        self.w_uv = load.get(n["up_v"])
        # for the matrix cores: a head's rows side by side ([heads, out, in]); w_uk transposed once, so that both
        # products walk their inner dimension along a row (a layout choice, not new maths)
        self.w_uk_t = self.w_uv_h = None
        if build.mode == "bfloat16" and self.w_uk.dtype == torch.bfloat16 and self.plain_dim % 8 == 0 and self.rank % 8 == 0:
            self.w_uk_t = self.w_uk.view(self.nq, self.plain_dim, self.rank).transpose(1, 2).contiguous()
            self.w_uv_h = self.w_uv.view(self.nq, self.v_dim, self.rank)
        self.sink = self._load_sink(load, n["sink"]) if params.get("sink", False) else None
        self._o_weight = load.get(n["o"])
        self._o = None
        self.mode = build.mode
        self.inner_width = self.nq * self.v_dim
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
        return PagedKVSpec(1, self.d, None)

    def out_weight(self) -> torch.Tensor:
        return self._o_weight

    def decodes_from_raw(self, ctx, cache, qkv, tables) -> bool:
        return False

    def forward_inner(self, x: torch.Tensor, ctx: StepContext, cache: PagedCacheView, out: torch.Tensor) -> None:
        tokens = x.shape[0]
        ws = ctx.workspace
        y = ws.buffer("latent.proj", tokens, self.proj.out_features, self.act_dtype)
        self.proj.forward(x, y)
        tables = ctx.position_product(self.position, self.encodings)
        if tables.rotary_dim != self.rot_dim:
            raise ValueError(f"latent attention turns {self.rot_dim} channels, its position encoding {tables.rotary_dim}")
        table = ctx.block_tables[cache.group]
        q = ws.buffer("latent.q", tokens, self.nq * self.d, self.act_dtype)
        kernels.latent_rows(y, 0, self.q_cols, q, self.norm_weight, tables.cos, tables.sin, tables.pairing, cache.keys,
                            cache.values, ctx.positions, ctx.token_entry, table, self.nq, self.plain_dim, self.rot_dim,
                            self.rank, self.d, self.eps, write=cache.writable)
        q_head = self.plain_dim + self.rot_dim
        if self.w_uk_t is not None and kernels.heads_product_takes(y, self.w_uk_t, q, q_head):
            kernels.heads_product(y, q_head, self.w_uk_t, None, q, self.d)
        else:
            kernels.latent_absorb(y, 0, q_head, self.w_uk, q, self.d, self.nq, self.plain_dim, self.rank)
        # the weighted latent rows: from the matrix-core kernels of ``attention`` where they are compiled for rows this
        # wide (the activations' type), else in float32 from the matrix-core kernel for wide values or the generic one
        if self.uses_matrix_cores(q, cache):
            o = ws.buffer("latent.rows", tokens, self.nq * self.d, self.act_dtype)
            self.attend(q, o, ctx, cache, table)
        elif self.options.get("attention", "auto") != "generic" and kernels.attn_wide_takes(q, cache.keys, self.d):
            o = ws.buffer("latent.rows", tokens, self.nq * self.d, torch.float32)
            key = f"static:latent.wide_items:{self.nq}"
            if key not in ctx.extras:
                row_tiles = kernels.attn_wide_row_tiles(ctx.num_tokens)
                flat, hp = kernels.attn_wide_items(ctx.entries, self.nq, 1, row_tiles)
                ctx.extras[key] = (ctx.to_device(flat), hp, row_tiles)
            items, hp, row_tiles = ctx.extras[key]
            wv = (self.rank + 15) // 16 * 16
            splits = kernels.attn_wide_splits(items.numel() // 4, (wv + 255) // 256, ctx.max_context) if row_tiles == 1 else 1
            part = part_ml = None
            if splits > 1:
                part = ws.buffer("attn_wide.part", tokens * self.nq * splits, self.d, torch.float32)
                part_ml = ws.buffer("attn_wide.part_ml", tokens * self.nq * splits, 2, torch.float32)
            kernels.attn_wide(q, o, self.nq, 1, self.d, wv, False, cache.keys, cache.values, ctx.positions,
                              ctx.token_entry, table, items, hp, self.scale, 0, 0, self.sink, self.score_cap, row_tiles,
                              splits, part, part_ml)
        else:
            o = ws.buffer("latent.rows", tokens, self.nq * self.d, torch.float32)
            kernels.attn_generic(q, o, self.nq, 1, self.d, cache.keys, cache.values, ctx.positions, ctx.token_entry,
                                 table, self.scale, 0, sink=self.sink, softcap=self.score_cap)
        gate = y[:, self.gate_col0:self.gate_col0 + self.nq * self.v_dim] if self.gated else None
        if self.w_uv_h is not None and kernels.heads_product_takes(o, self.w_uv_h, out, self.d):
            kernels.heads_product(o, self.d, self.w_uv_h, gate, out, self.v_dim, self.out_scale)
        else:
            kernels.latent_expand(o, self.d, self.w_uv, gate, out, self.nq, self.v_dim, self.rank, self.out_scale)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: PagedCacheView) -> torch.Tensor:
        if self._o is None:
            self._o = Linear(self._o_weight, self.mode)
        ws = ctx.workspace
        inner = ws.buffer("latent.inner", x.shape[0], self.inner_width, self.act_dtype)
        self.forward_inner(x, ctx, cache, inner)
        return self._o.forward(inner, ws.buffer("latent.out", x.shape[0], self.hidden, self.act_dtype))
