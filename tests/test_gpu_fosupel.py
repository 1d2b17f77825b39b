"""Fosupel on the GPU against the plain implementation (tests/plain/fosupel_plain.py), in 32-bit and in bfloat16.

Small configurations of their own and seeded random weights: one whose layers all differ (keys wider than values and
the other way round, grouped and ungrouped heads, rotations on a part of a head, on all of it and none, windows of 7
and 24 tokens with 3 and no kept first tokens, a layer without a feed-forward, routers with and without a shared
expert, a decay of exactly one, a loop of three passes), one whose constants are one and whose sizes coincide (no
loop), and one at widths where the serving kernels run.  Each mechanism alone at its kernels, with inputs made so that
a fault shows (a stored key that takes all the weight just inside and just outside the window, at the last kept
first token and the first one not kept, at a page's border; pages and states filled with NaN before use); then whole
prompts, token-by-token decoding, portions down to two tokens, mixed batches with pages and slots used again, a
prompt far beyond the windows, long decoding, greedy generation through the scheduler, the command line and the trace
replay program.
"""
import json
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, token_ids
from plain import fosupel_plain as P
from test_gpu_model import SPLIT_TOL, close, mixed_trace, pages_were_used_again, run_alone, run_mixed

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def rot(base, dims, factor=None):
    out = {"base": base, "dims": dims}
    if factor is not None:
        out["scaling"] = {"factor": factor}
    return out


def left(heads, kv_heads, dim, vdim, window, keep, turn, scale):
    out = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if window is not None:
        out["mask"] = {"keep_first": keep, "size": window}
    if turn is not None:
        out["rot"] = turn
    return out


def right(heads, dim, vdim, decay, turn):
    out = {"decay": decay, "dim": dim, "heads": heads, "vdim": vdim}
    if turn is not None:
        out["rot"] = turn
    return out


def parallel(l, r, left_scale, right_scale):
    return "parallel", {"left": l, "left_scale": left_scale, "right": r, "right_scale": right_scale}


def latent(heads, dim, rot_dim, vdim, rank, base, scale):
    return "latent_attention", {"dim": dim, "heads": heads, "kv_rank": rank, "rot": rot(base, rot_dim), "rot_dim": rot_dim,
                                "scale": scale, "vdim": vdim}


def moe(experts, top, ff, shared):
    out = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def layer(mixer, mlp):
    return {"mixer": mixer[1], "mlp": mlp, "type": mixer[0]}


def config(vocab, width, eps, mult, softcap, loop, layers):
    out = {"architecture": "Fosupel", "layers": layers, "logit_softcap": softcap, "norm": {"eps": eps},
           "residual_mult": mult, "vocab": vocab, "width": width}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# every layer another shape; layers 1 and 2 run three times
MIXED = config(311, 96, 1e-5, 0.7, 11.0, (1, 3, 3), [
    layer(latent(3, 16, 8, 24, 40, 1e4, 0.2), dense(160)),
    layer(parallel(left(6, 3, 32, 16, 24, 3, rot(1e4, 16, 4.0), 0.2), right(3, 16, 32, [0.5, 0.9, 0.99], rot(500.0, 8)),
                   0.7, 1.3), moe(5, 2, 48, 80)),
    layer(parallel(left(4, 4, 16, 48, 7, 0, rot(300.0, 16), 0.4), right(1, 32, 64, [1.0], None), 1.2, 0.6), None),
    layer(latent(2, 32, 16, 16, 24, 5e3, 0.15), moe(3, 1, 64, None)),
])
# constants that are one, sizes that coincide, no loop, a window no prompt of the tests reaches, no kept tokens
EQUAL = config(515, 128, 1e-6, 1.0, 30.0, None, [
    layer(parallel(left(2, 2, 64, 64, 1000, 0, rot(1e4, 64), 0.125), right(2, 64, 64, [0.9, 0.9], rot(1e4, 64)), 1.0, 1.0),
          dense(128)),
    layer(latent(2, 64, 64, 64, 64, 1e4, 0.1), moe(2, 1, 128, 128)),
])
# widths of a real model's layers; both layers run twice (decays near one: a head that forgets fast sums few terms, and
# its output, which is divided by its own size, is then small by chance at many positions)
WIDE = config(300, 1024, 1e-6, 0.5, 20.0, (0, 2, 2), [
    layer(parallel(left(8, 2, 128, 128, 64, 4, rot(1e6, 64, 2.0), 0.09), right(4, 128, 128, [0.97, 0.99, 0.995, 0.999], rot(1e6, 32)),
                   0.9, 1.1), moe(4, 2, 256, 512)),
    layer(latent(8, 64, 32, 64, 256, 1e5, 0.1), dense(2048)),
])
CONFIGS = {"mixed": MIXED, "equal": EQUAL, "wide": WIDE}
CLOSE_CALL = 0.015     # (a looped layer's router sees what three passes' roundings left)
# Against float64.  The bfloat16 bound is twice that of the other designs' tests: the loop makes eight layer runs of
# four layers at a width of 96, and every run's roundings reach the logits (the float32 bound is the usual one).
TOL = {"float32": 3e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import FosupelConfig
    from pulse_infer_amd.weights import write_model_folder

    out = {}
    for seed, (name, cfg) in enumerate(CONFIGS.items()):
        out[name] = write_model_folder(FosupelConfig.from_dict(cfg), str(tmp_path_factory.mktemp(name)), seed=270 + seed)
    return out


@pytest.fixture(scope="module")
def plain(folders):
    models = {name: P.PlainFosupel.from_folder(folder) for name, folder in folders.items()}
    memo = {}

    def logits(name, ids):
        key = (name, tuple(ids))
        if key not in memo:
            memo[key] = models[name].logits(list(ids))
        return memo[key]

    def router_calls(name, ids):
        """Positions at which a router's choice hangs on less than CLOSE_CALL: bfloat16 may choose otherwise there."""
        key = ("calls", name, tuple(ids))
        if key not in memo:
            memo[key] = set((models[name].router_margins(list(ids)) < CLOSE_CALL).nonzero().flatten().tolist())
        return memo[key]

    def fragile(name, ids):
        """Positions whose logits hang on cancellations (see ``fragile_positions``): left out of every comparison."""
        key = ("fragile", name, tuple(ids))
        if key not in memo:
            memo[key] = models[name].fragile_positions(list(ids))
        return memo[key]

    def close_calls(name, ids):   # noqa: F811  (the two sets travel together: Calls carries the second)
        return Calls(router_calls(name, ids), fragile(name, ids))

    logits.models = models
    logits.close_calls = close_calls
    return logits


class Calls(set):
    """A router's close calls (bfloat16 only), with the fragile positions (any arithmetic) beside them."""

    def __init__(self, calls, fragile):
        super().__init__(calls)
        self.fragile = set(fragile)


def agree(got, want, dtype, what, calls=(), first=0, tol=TOL, by_median=False):
    """``close``, without the fragile positions; in bfloat16 another choice of a router at one position reaches all
    later ones through the states, so the positions before the first close call are compared one by one and of the rest
    the median error."""
    fragile = getattr(calls, "fragile", set())
    if fragile:
        keep = [i for i in range(want.shape[0]) if i + first not in fragile]
        assert len(keep) >= 0.7 * want.shape[0] or want.shape[0] < 10, f"{what}: too many fragile positions to say anything"
        if not keep:
            return
        # (positions are renumbered: close calls move down past the rows that were dropped)
        moved = {sum(1 for k in keep if k + first < c) + first for c in calls}
        got, want, calls = got[keep], want[keep], moved
    if dtype == "bfloat16" and by_median:
        # random configurations multiply bfloat16's roundings by whatever their constants are (a multiplier above one
        # over three passes, say): the median position within the bound, no position beyond three times it
        rows = (got.double().cpu() - want.double().cpu()).abs().max(dim=1).values
        bound = tol[dtype] * max(1.0, float(want.abs().max()))
        cut = max(0, min(calls) - first) if calls else rows.shape[0]
        assert torch.isfinite(rows).all(), what
        assert float(rows.median()) <= bound, f"{what}: median error {float(rows.median()):.3e} exceeds {bound:.3e}"
        assert cut == 0 or float(rows[:cut].max()) <= 3.0 * bound, f"{what}: max error {float(rows[:cut].max()):.3e}"
        return
    if dtype == "bfloat16" and calls:
        cut = max(0, min(calls) - first)
        if cut:
            close(got[:cut], want[:cut], dtype, what + " (before the first close call)", tol)
        if cut < want.shape[0]:
            rest = (got[cut:].double().cpu() - want[cut:].double().cpu()).abs().max(dim=1).values
            assert torch.isfinite(rest).all(), what
            assert float(rest.median()) <= tol[dtype] * max(1.0, float(want.abs().max())), \
                f"{what}: median error {float(rest.median()):.3e}"
        return
    close(got, want, dtype, what, tol)


@pytest.fixture(scope="module")
def runners(folders):
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model

    made = {}

    def get(name, dtype, page=16, tokens=512):
        key = (name, dtype, page, tokens)
        if key not in made:
            _, model = load_model(folders[name], mode=dtype)
            made[key] = ModelRunner(model, page_size=page, num_pages=tokens // page, max_requests=4)
        return made[key]

    return get


# ------------------------------------------------------------------------------------------- mechanisms alone
def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32) * scale


def stored(x, dtype):
    dev = x.to(dtype).to(DEV)
    return dev, dev.cpu().to(F64)


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def ints(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def paged(lens, nkv, d, bs, dtype, seed):
    """Pages filled with NaN (nothing stale may reach an output) and a shuffled block table."""
    pages_per = [(n + bs - 1) // bs for n in lens]
    total = sum(pages_per) + 2
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    kc = torch.full((total, nkv, bs, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((total, nkv, d, bs), float("nan"), dtype=dtype, device=DEV)
    table = torch.full((len(lens), max(pages_per)), -1, dtype=torch.int32)
    at = 0
    for r, n in enumerate(pages_per):
        table[r, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    return kc, vc, table


TALK_CASES = [
    dict(nq=6, nkv=3, d=32, dv=16, bs=16, window=24, keep=3, lens=[150, 1, 64, 65, 27, 28, 300], portion=70),
    dict(nq=4, nkv=4, d=16, dv=16, bs=16, window=7, keep=0, lens=[90, 33, 7, 8], portion=40),
    dict(nq=8, nkv=2, d=128, dv=128, bs=32, window=64, keep=33, lens=[257, 100, 98], portion=2),
    dict(nq=2, nkv=1, d=48, dv=48, bs=4, window=5, keep=9, lens=[45, 15, 14, 6], portion=11),
    dict(nq=12, nkv=6, d=128, dv=128, bs=16, window=40, keep=2, lens=[70, 45], portion=3),   # 768 value channels a head
]
NEEDLES = [None, "window_in", "window_out", "first_in", "first_out"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", TALK_CASES)
@pytest.mark.parametrize("needle", NEEDLES)
def test_kept_first_tokens_window_sinks_and_mixed_heads(case, dtype, needle):
    """A portion of request 0 beside single (decoded) tokens of the others, over shuffled pages: every head's weights
    (window, kept first tokens, sink) on every kv head's values, then the sums that the mixing matrix asks for.  With a
    needle one stored key of every request is 40 times its last query: at the window's far edge, one beyond it, the last
    kept first token, or the first one not kept; seen or unseen, it decides the last token's output."""
    from pulse_infer_amd.ops import kernels

    nq, nkv, d, dv, bs, window, keep, lens, portion = (case[x] for x in ("nq", "nkv", "d", "dv", "bs", "window", "keep",
                                                                         "lens", "portion"))
    scale, share = 0.3, nq // nkv
    kc, vc, table = paged(lens, nkv, d, bs, dtype, seed=5)
    sink = rnd(nq, seed=1, scale=1.5)
    mix, mix_ref = stored(rnd(nq, nq, seed=2, scale=0.5), dtype)
    keys = [stored(rnd(n, nkv, d, seed=20 + r), dtype)[1] for r, n in enumerate(lens)]
    values = [stored(rnd(n, nkv, d, seed=40 + r), dtype)[1] for r, n in enumerate(lens)]
    queries = [stored(rnd(n, nq, d, seed=60 + r), dtype) for r, n in enumerate(lens)]
    for r, n in enumerate(lens):
        where = {"window_in": n - window, "window_out": n - window - 1, "first_in": keep - 1, "first_out": keep}.get(needle)
        if where is not None and 0 <= where < n - 1:
            for g in range(nkv):
                keys[r][where, g] = (40.0 * queries[r][1][n - 1, g * share]).to(dtype).to(F64)
        for j in range(n):
            page, slot = int(table[r, j // bs]), j % bs
            kc[page, :, slot, :] = keys[r][j].to(dtype).to(DEV)
            vc[page, :, :, slot] = values[r][j].to(dtype).to(DEV)
    positions = list(range(lens[0] - portion, lens[0])) + [n - 1 for n in lens[1:]]
    entry = [0] * portion + list(range(1, len(lens)))
    q = torch.cat([queries[0][0][lens[0] - portion:]] + [queries[r][0][n - 1:] for r, n in enumerate(lens) if r])
    q = q.reshape(len(positions), nq * d).contiguous()
    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count
    step_entries = [E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)]
    paths = ["generic"] + (["wide", "wide4", "wide in splits"] if kernels.attn_wide_takes(q, kc, d) else [])
    assert dtype != torch.bfloat16 or bs % 16 or d % 16 or "wide" in paths
    for path in paths:
        row_tiles = 4 if path == "wide4" else 1
        splits = 3 if path == "wide in splits" else 1
        scratch = {}
        if splits > 1:   # (filled with NaN: every sum that is merged must have been written)
            scratch = dict(n_splits=splits,
                           part=torch.full((len(positions) * nq * splits, nkv * d), float("nan"), device=DEV),
                           part_ml=torch.full((len(positions) * nq * splits, 2), float("nan"), device=DEV))
        each = torch.full((len(positions), nq * nkv * d), float("nan"), dtype=torch.float32, device=DEV)
        if path == "generic":
            kernels.attn_generic(q, each, nq, nkv, d, kc, vc, ints(positions), ints(entry), table.to(DEV), scale, window,
                                 sink=sink.to(DEV), keep_first=keep, all_values=True)
        else:
            flat, hp = kernels.attn_wide_items(step_entries, nq, nkv, row_tiles)
            kernels.attn_wide(q, each, nq, nkv, d, nkv * d, True, kc, vc, ints(positions), ints(entry), table.to(DEV),
                              ints(flat), hp, scale, window, keep, sink.to(DEV), row_tiles=row_tiles, **scratch)
        out = torch.full((len(positions), nq * d), float("nan"), dtype=dtype, device=DEV)
        kernels.head_mix(each, mix, out, nq, nkv, d, dv, d, 0.8)
        got = out.cpu().to(F64).view(-1, nq, d)
        assert float(got[..., dv:].abs().sum()) == 0.0
        row = 0
        for r, n in enumerate(lens):
            rows = portion if r == 0 else 1
            scores = torch.stack([queries[r][1][:, h] @ keys[r][:, h // share].T for h in range(nq)]) * scale
            a = P.weights_with_sink(scores, P.visible(n, window, keep), sink.to(F64))
            a = torch.einsum("hg,gij->hij", mix_ref, a)
            want = 0.8 * torch.stack([a[h] @ values[r][:, h // share, :dv] for h in range(nq)], dim=1)[n - rows:]
            assert torch.allclose(got[row:row + rows, :, :dv], want, **tol(dtype)), \
                (path, r, float((got[row:row + rows, :, :dv] - want).abs().max()))
            row += rows
        if path != "generic":   # a head's own values alone, as the part asks for them without mixed heads
            own = torch.full((len(positions), nq * d), float("nan"), dtype=torch.float32, device=DEV)
            kernels.attn_wide(q, own, nq, nkv, d, d, False, kc, vc, ints(positions), ints(entry), table.to(DEV),
                              ints(flat), hp, scale, window, keep, sink.to(DEV), row_tiles=row_tiles, **scratch)
            got, row = own.cpu().to(F64).view(-1, nq, d), 0
            for r, n in enumerate(lens):
                rows = portion if r == 0 else 1
                scores = torch.stack([queries[r][1][:, h] @ keys[r][:, h // share].T for h in range(nq)]) * scale
                a = P.weights_with_sink(scores, P.visible(n, window, keep), sink.to(F64))
                want = torch.stack([a[h] @ values[r][:, h // share] for h in range(nq)], dim=1)[n - rows:]
                assert torch.allclose(got[row:row + rows], want, **tol(dtype)), ("wide, own values", r)
                row += rows
    # kept first tokens alone (no mixing), in the storage type of q
    plain_out = torch.full((len(positions), nq * d), float("nan"), dtype=dtype, device=DEV)
    kernels.attn_generic(q, plain_out, nq, nkv, d, kc, vc, ints(positions), ints(entry), table.to(DEV), scale, window,
                         sink=sink.to(DEV), keep_first=keep)
    got, row = plain_out.cpu().to(F64).view(-1, nq, d), 0
    for r, n in enumerate(lens):
        rows = portion if r == 0 else 1
        scores = torch.stack([queries[r][1][:, h] @ keys[r][:, h // share].T for h in range(nq)]) * scale
        a = P.weights_with_sink(scores, P.visible(n, window, keep), sink.to(F64))
        want = torch.stack([a[h] @ values[r][:, h // share] for h in range(nq)], dim=1)[n - rows:]
        assert torch.allclose(got[row:row + rows], want, **tol(dtype)), r
        row += rows


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,dv,dims,pairing", [(3, 16, 32, 8, "half"), (1, 32, 64, 0, "half"), (4, 128, 128, 32, "half"),
                                                      (2, 20, 10, 20, "adjacent"), (2, 64, 64, 64, "half")])
def test_turned_rows_the_walk_and_the_gated_head_norm(dtype, heads, d, dv, dims, pairing):
    """Retention from its projections on: q and k turned at positions of their own, k scaled, the state walk (a
    portion that continues a state, a fresh prompt in a slot that holds NaN, a single token), every head divided by its
    own root mean square and multiplied by silu of the gate."""
    from pulse_infer_amd.ops import kernels

    decay, base, eps = [0.5, 1.0, 0.97, 0.999][:heads], 700.0, 1e-5
    counts, starts, slot_of = [37, 20, 1], [12, 0, 300], [3, 0, 4]
    hd, hv = heads * d, heads * dv
    state0 = torch.full((5, heads, d, dv), float("nan"), dtype=torch.float32, device=DEV)
    state1 = state0.clone()
    wants, rows_of = [], []
    for r, (n, s0) in enumerate(zip(counts, starts)):
        total = s0 + n
        y, ref = stored(rnd(total, 2 * hd + 2 * hv, seed=r), dtype)
        positions = list(range(total))
        q, k = ref[:, :hd].view(total, heads, d), ref[:, hd:2 * hd].view(total, heads, d)
        if dims:
            q, k = P.turn(q, positions, base, dims, pairing), P.turn(k, positions, base, dims, pairing)
        o = P.unit_rms(P.retention_walk(q, k * d ** -0.5, ref[:, 2 * hd:2 * hd + hv].view(total, heads, dv), decay), eps)
        wants.append((o.reshape(total, hv) * P.silu(ref[:, 2 * hd + hv:]) * 1.3)[s0:])
        rows_of.append(y)
    inv = base ** (-2.0 * torch.arange(max(dims, 2) // 2, dtype=F64) / max(dims, 2))

    def run(rows, positions, first_row, start, slots, state=None, fused=False):
        state = state0 if state is None else state
        tokens = rows.shape[0]
        cos = sin = None
        if dims:
            angle = torch.tensor(positions, dtype=F64).view(-1, 1) * inv.view(1, -1)
            cos, sin = torch.cos(angle).float().to(DEV).contiguous(), torch.sin(angle).float().to(DEV).contiguous()
        o = torch.full((tokens, hv), float("nan"), dtype=torch.float32, device=DEV)
        groups = kernels.lightning_row_groups(len(start), heads, d, dv)
        if fused:    # the walk turns and scales as it fetches
            kernels.lightning_scan(rows, 0, hd, 2 * hd, o, state, torch.tensor(decay, device=DEV), ints(first_row),
                                   ints(start), ints(slots), heads, d, dv, "none", groups,
                                   turn=(cos, sin, dims, 1 if pairing == "half" else 0), key_scale=d ** -0.5)
        else:        # turned float32 rows of their own first
            wide = torch.full((tokens, 2 * hd + hv), float("nan"), dtype=torch.float32, device=DEV)
            kernels.rotate_qk_rows(rows, 0, hd, 2 * hd, wide, heads, d, dv, cos, sin, dims, 1 if pairing == "half" else 0,
                                   d ** -0.5)
            kernels.lightning_scan(wide, 0, hd, 2 * hd, o, state, torch.tensor(decay, device=DEV), ints(first_row),
                                   ints(start), ints(slots), heads, d, dv, "none", groups)
        out = torch.full((tokens, hv), float("nan"), dtype=dtype, device=DEV)
        kernels.group_norm_gate(o, None, rows[:, 2 * hd + hv:], out, heads, eps, 1.3, "silu")
        return out.cpu().to(F64)

    # what came before this step: the first and the third request's earlier tokens
    step = torch.cat([rows_of[r][starts[r]:] for r in range(3)]).contiguous()
    positions = [p for r in range(3) for p in range(starts[r], starts[r] + counts[r])]
    first_row = [0, counts[0], counts[0] + counts[1], sum(counts)]
    for state, fused in ((state0, False), (state1, True)):
        for r in (0, 2):
            run(rows_of[r][:starts[r]].contiguous(), list(range(starts[r])), [0, starts[r]], [0], [slot_of[r]], state, fused)
        got = run(step, positions, first_row, starts, slot_of, state, fused)
        assert torch.allclose(got, torch.cat(wants), **tol(dtype)), (fused, float((got - torch.cat(wants)).abs().max()))
    assert torch.allclose(state0[[0, 3, 4]], state1[[0, 3, 4]], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,d,dr,dv,rank,bs", [(3, 16, 8, 24, 40, 16), (2, 32, 16, 16, 24, 4), (4, 64, 32, 64, 128, 16),
                                                    (1, 8, 2, 5, 13, 16), (8, 64, 64, 128, 512, 16), (24, 16, 8, 8, 40, 16)])
def test_latent_attention_from_its_projections_on(dtype, heads, d, dr, dv, rank, bs):
    """The latent row normed and stored with the turned key part, the queries taken into the latent space, attention
    over one kv head with sinks, the values taken out again and gated: a portion of request 0 beside single tokens,
    against the plain mixer whose projections are made the identity."""
    from pulse_infer_amd.ops import attention_mfma as M
    from pulse_infer_amd.ops import kernels
    from pulse_infer_amd.parts.latent import latent_stored_width

    lens, portion = [75, 1, 33, 16, 17], 30
    eps, scale, base = 1e-5, 0.2, 3e3
    q_cols, down, inner = heads * (d + dr), rank + dr, heads * dv
    width = q_cols + down + inner
    D = latent_stored_width(rank, dr)
    kc, vc, table = paged(lens, 1, D, bs, dtype, seed=9)
    norm_w, norm_ref = stored(1.0 + rnd(rank, seed=3, scale=0.1), dtype)
    w_uk, uk_ref = stored(rnd(heads * d, rank, seed=4, scale=rank ** -0.5), dtype)
    w_uv, uv_ref = stored(rnd(heads * dv, rank, seed=5, scale=rank ** -0.5), dtype)
    sink = rnd(heads, seed=6)
    eye = torch.eye(width, dtype=F64)
    weights = {"m.q": eye[:q_cols], "m.dkv": eye[q_cols:q_cols + down], "m.g": eye[q_cols + down:], "m.dkv.norm": norm_ref,
               "m.uk": uk_ref, "m.uv": uv_ref, "m.sink": sink.to(F64), "m.o": torch.eye(inner, dtype=F64)}
    sizes = {"heads": heads, "dim": d, "rot_dim": dr, "vdim": dv, "kv_rank": rank, "scale": scale, "rot": {"base": base, "dims": dr}}
    inv = base ** (-2.0 * torch.arange(dr // 2, dtype=F64) / dr)
    rows_of, wants = [], []
    for r, n in enumerate(lens):
        y, ref = stored(rnd(n, width, seed=30 + r), dtype)
        rows_of.append(y)
        wants.append(P.latent_attention(ref, weights, "m", sizes, list(range(n)), eps))

    def prepare(rows, positions, entry):
        angle = torch.tensor(positions, dtype=F64).view(-1, 1) * inv.view(1, -1)
        cos, sin = torch.cos(angle).float().to(DEV).contiguous(), torch.sin(angle).float().to(DEV).contiguous()
        q = torch.full((rows.shape[0], heads * D), float("nan"), dtype=dtype, device=DEV)
        kernels.latent_rows(rows, 0, q_cols, q, norm_w, cos, sin, 0, kc, vc, ints(positions), ints(entry), table.to(DEV),
                            heads, d, dr, rank, D, eps)
        kernels.latent_absorb(rows, 0, d + dr, w_uk, q, D, heads, d, rank)
        return q

    fed = [lens[0] - portion] + [n - 1 for n in lens[1:]]
    for r, n in enumerate(fed):
        if n:
            prepare(rows_of[r][:n].contiguous(), list(range(n)), [r] * n)
    positions = list(range(fed[0], lens[0])) + [n - 1 for n in lens[1:]]
    entry = [0] * portion + list(range(1, len(lens)))
    step = torch.cat([rows_of[0][fed[0]:]] + [rows_of[r][n - 1:] for r, n in enumerate(lens) if r]).contiguous()
    q = prepare(step, positions, entry)
    assert not torch.isnan(q.float()).any()
    want = torch.cat([wants[0][fed[0]:]] + [wants[r][n - 1:] for r, n in enumerate(lens) if r])
    gate = step[:, q_cols + down:]
    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count
    paths = [torch.float32] + ([dtype] if M.supported(D, bs, dtype, dtype) else [])
    paths += ["wide", "wide4"] if kernels.attn_wide_takes(q, kc, D) else []
    for kind in paths:
        o = torch.full((len(positions), heads * D), float("nan"), dtype=torch.float32 if kind in ("wide", "wide4") else kind, device=DEV)
        if kind == torch.float32:
            kernels.attn_generic(q, o, heads, 1, D, kc, vc, ints(positions), ints(entry), table.to(DEV), scale, 0,
                                 sink=sink.to(DEV))
        elif kind in ("wide", "wide4"):
            row_tiles = 4 if kind == "wide4" else 1
            flat, hp = kernels.attn_wide_items([E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)], heads, 1,
                                               row_tiles)
            kernels.attn_wide(q, o, heads, 1, D, (rank + 15) // 16 * 16, False, kc, vc, ints(positions), ints(entry),
                              table.to(DEV), ints(flat), hp, scale, 0, 0, sink.to(DEV), row_tiles=row_tiles)
        else:
            numbered = list(enumerate([E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)]))
            items = ints(M.build_items(numbered, M.tokens_per_item(heads)))
            split = (max(lens) + 31) // 32 * 32
            M.attn_mfma(q, o, heads, 1, D, kc, vc, ints(positions), table.to(DEV), items, scale, 0, split, 1, max(lens),
                        None, None, sink=sink.to(DEV))
        out = torch.full((len(positions), inner), float("nan"), dtype=dtype, device=DEV)
        kernels.latent_expand(o, D, w_uv, gate, out, heads, dv, rank)
        assert torch.allclose(out.cpu().to(F64), want, **tol(dtype)), (kind, float((out.cpu().to(F64) - want).abs().max()))
        # the same two products a head on the matrix cores
        w_uv_h = w_uv.view(heads, dv, rank)
        if kernels.heads_product_takes(o, w_uv_h, out, D) and d % 8 == 0 and rank % 8 == 0:
            again = torch.full((len(positions), inner), float("nan"), dtype=dtype, device=DEV)
            kernels.heads_product(o, D, w_uv_h, gate, again, dv)
            assert torch.allclose(again.cpu().to(F64), want, **tol(dtype)), (kind, "heads_product")
            w_uk_t = w_uk.view(heads, d, rank).transpose(1, 2).contiguous()
            q2 = q.clone()
            q2.view(-1, heads, D)[:, :, :rank] = float("nan")
            kernels.heads_product(step, d + dr, w_uk_t, None, q2, D)
            assert torch.allclose(q2.float(), q.float(), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_small_kernels_of_the_layer(dtype):
    """xIELU on both sides of zero, the shared expert's gate of one number a token, a factor on the update inside the
    norm and in the plain sum, and a row added to every token."""
    from pulse_infer_amd.ops import kernels

    z, zref = stored(rnd(37, 100, seed=1, scale=2.0), dtype)
    pq, pqref = stored(torch.tensor([0.3, -0.7]), dtype)
    out = torch.empty_like(z)
    kernels.xielu(z, out, pq)
    assert torch.allclose(out.cpu().to(F64), P.xielu(zref, pqref), **tol(dtype))

    x, xref = stored(rnd(19, 96, seed=2), dtype)
    w, wref = stored(rnd(96, seed=3, scale=0.2), dtype)
    y, yref = stored(rnd(19, 96, seed=4), dtype)
    acc = rnd(19, 96, seed=5).to(DEV)
    want = acc.cpu().to(F64) + torch.sigmoid(xref @ wref).view(-1, 1) * yref
    kernels.token_gate_add(x, w, y, acc)
    assert torch.allclose(acc.cpu().to(F64), want, atol=2e-5, rtol=2e-5)

    for hidden in (96, 1000, 4096):
        h = rnd(9, hidden, seed=6).to(DEV)
        d, dref = stored(rnd(9, hidden, seed=7), dtype)
        nw, nwref = stored(1.0 + rnd(hidden, seed=8, scale=0.1), dtype)
        normed = torch.empty(9, hidden, dtype=dtype, device=DEV)
        want_h = h.cpu().to(F64) + 0.7 * dref
        kernels.add_rmsnorm(h, d, nw, 1e-5, normed, delta_scale=0.7)
        assert torch.allclose(h.cpu().to(F64), want_h, atol=1e-5, rtol=1e-5)
        assert torch.allclose(normed.cpu().to(F64), P.unit_rms(want_h, 1e-5) * nwref, **tol(dtype))
        kernels.residual_add(h, d, 0.3)
        want_h = want_h + 0.3 * dref
        row, rowref = stored(rnd(hidden, seed=9), dtype)
        kernels.residual_add_row(h, row)
        assert torch.allclose(h.cpu().to(F64), want_h + rowref, atol=1e-5, rtol=1e-5)


# ------------------------------------------------------------------------------------------------ whole models
LENGTH = {"mixed": 150, "equal": 130, "wide": 90}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("mixed", 4), ("equal", 16), ("equal", 64), ("wide", 16)])
def test_whole_tail_and_portions(runners, plain, name, page, dtype):
    ids = token_ids(CONFIGS[name]["vocab"], LENGTH[name], seed=3)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, page)
    n = len(ids)
    whole = run_alone(runner, ids, [n])
    agree(whole, want, dtype, f"{name} whole", calls)
    tail = run_alone(runner, ids, [n - 40] + [1] * 40)               # prefill against token-by-token decoding
    agree(tail, want, dtype, f"{name} tail", calls)
    agree(tail, whole, dtype, f"{name} tail against whole", calls, tol=SPLIT_TOL)
    for cuts in ([2, 3, 31, 2, 17, n - 57, 2], [1, 1, 1, 31, n - 34], [n - 2, 2], [7] * (n // 7) + [n % 7 or 7][:n % 7 > 0]):
        cuts = [c for c in cuts if c]
        portions = run_alone(runner, ids, cuts)
        agree(portions, want, dtype, f"{name} portions {cuts}", calls)
        agree(portions, whole, dtype, f"{name} portions against whole", calls, tol=SPLIT_TOL)
    first = run_alone(runner, ids[:3], [1, 1, 1])                     # the first tokens of a sequence
    agree(first, want[:3], dtype, f"{name} first tokens", calls)


@pytest.mark.parametrize("name", ["mixed", "equal"])
def test_the_stream_after_every_layer(runners, plain, name):
    from pulse_infer_amd.engine.runner import StepEntry

    ids = token_ids(CONFIGS[name]["vocab"], 37, seed=8)
    runner = runners(name, "float32")
    model, seen = runner.model, []
    originals = [b.forward for b in model.blocks]

    def watched(forward):
        def run(stream, ctx, cache):
            forward(stream, ctx, cache)
            stream.settle()
            seen.append(stream.h.clone())
        return run

    try:
        for block, forward in zip(model.blocks, originals):
            block.forward = watched(forward)
        runner.add_request("layers")
        runner.reserve("layers", len(ids))
        runner.step([StepEntry("layers", ids, [])])
    finally:
        for block, forward in zip(model.blocks, originals):
            block.forward = forward
        runner.free_request("layers")
    want = plain.models[name].residuals(ids)
    assert len(seen) == len(want) == len(model.spec.order)
    for i, (got, ref) in enumerate(zip(seen, want)):
        close(got, ref, "float32", f"{name} after layer run {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("equal", 16), ("equal", 32), ("wide", 16)])
def test_mixed_batches_with_pages_and_slots_used_again(runners, plain, name, page, dtype):
    """Up to four live requests over a pool of 256 tokens and four slots, portions of some beside single tokens of
    others: every request's logits are what it gets alone, whoever held its pages and its state's slot before."""
    ids, steps = mixed_trace(CONFIGS[name]["vocab"], seed=6, sizes=(2, 3, 5, 8, 13, 21, 34))
    runner = runners(name, dtype, page, tokens=256)
    got, pages_seen, most_live = run_mixed(runner, steps)
    assert most_live == 4 and pages_were_used_again(pages_seen)
    for k, mine in got.items():
        agree(mine, plain(name, ids[k]), dtype, f"{name} mixed request {k}", plain.close_calls(name, ids[k]))


def test_slots_and_pages_are_used_again_by_requests_of_other_lengths(runners, plain):
    from pulse_infer_amd.engine.runner import StepEntry

    name = "mixed"
    runner = runners(name, "float32", 16, tokens=160)
    for storage in runner.cache.state.values():       # whatever a slot held before must not show
        storage.fill_(float("nan"))
    lengths = [70, 3, 64, 17, 1, 80, 33, 16, 65, 48]
    for i in range(0, len(lengths), 2):
        pair = {f"q{i + j}": token_ids(CONFIGS[name]["vocab"], n, seed=40 + i + j) for j, n in enumerate(lengths[i:i + 2])}
        for rid, ids in pair.items():
            runner.add_request(rid)
            runner.reserve(rid, len(ids))
        logits = runner.step([StepEntry(rid, ids, [len(ids) - 1]) for rid, ids in pair.items()])
        for row, (rid, ids) in enumerate(pair.items()):
            close(logits[row:row + 1], plain(name, ids)[-1:], "float32", f"request {rid} of {len(ids)} tokens")
            runner.free_request(rid)
        runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_far_beyond_the_windows(runners, plain, dtype):
    """400 tokens through windows of 7 and 24 (pages below the windows go back to the pool while the request runs; the
    page of the kept first tokens stays), through a state that keeps everything (a decay of one) and through latent
    attention that sees all of them: whole, and with the last 60 tokens decoded."""
    name = "mixed"
    ids = token_ids(CONFIGS[name]["vocab"], 400, seed=21)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, 16, tokens=512)
    agree(run_alone(runner, ids, [400]), want, dtype, "whole", calls)
    agree(run_alone(runner, ids, [150, 190] + [1] * 60), want, dtype, "decoded tail", calls)


# ------------------------------------------------------------------------------------ seeded random configurations
def random_config(rng):
    """Layers drawn one by one, in any order: head sizes that are no multiples of 16, keys wider or narrower than values,
    any grouping of heads (more than 16 a kv head too), windows from one token on and none, kept tokens beyond the
    window, rotations on a part of a head, on all of it and none, with and without scaled frequencies, latent rows that
    are no multiples of 8, routers that choose all their experts, layers without a feed-forward, loops over any stretch
    of the layers (also none, and a single pass)."""
    width = rng.choice([64, 96, 160, 256])
    layers = []
    for _ in range(rng.choice([1, 2, 3])):
        if rng.random() < 0.6:
            groups, share = rng.choice([1, 2, 3]), rng.choice([1, 2, 3, 4, 18])
            dim = rng.choice([16, 24, 32, 48, 64])
            dims = rng.choice([x for x in (0, 2, 8, 16, 24, dim) if x <= dim])
            window = rng.choice([1, 5, 16, 33, 100, None])
            l = left(groups * share, groups, dim, rng.choice([8, 16, 40, 48, 64]), window, rng.choice([0, 1, 4, 20]),
                     rot(rng.choice([100.0, 1e4, 5e5]), dims, rng.choice([None, 1.0, 8.0])) if dims else None,
                     rng.choice([0.1, dim ** -0.5, 0.5]))
            heads, rdim = rng.choice([1, 2, 3, 5]), rng.choice([16, 24, 32, 64])
            rdims = rng.choice([x for x in (0, 4, 16, rdim) if x <= rdim])
            r = right(heads, rdim, rng.choice([16, 20, 32, 72]), [rng.choice([0.9, 0.97, 0.99, 1.0]) for _ in range(heads)],
                      rot(rng.choice([100.0, 1e4]), rdims) if rdims else None)
            mixer = parallel(l, r, rng.choice([0.5, 1.0, 1.5]), rng.choice([0.7, 1.0]))
        else:
            mixer = latent(rng.choice([1, 2, 4, 20]), rng.choice([8, 16, 24, 40]), rng.choice([2, 8, 16, 32]),
                           rng.choice([8, 16, 20, 48]), rng.choice([12, 24, 32, 64, 100]), rng.choice([1e3, 1e4, 1e6]),
                           rng.choice([0.1, 0.2]))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = dense(rng.choice([32, 100, 256]))
        else:
            experts = rng.choice([1, 2, 4, 9])
            mlp = moe(experts, rng.randint(1, min(4, experts)), rng.choice([32, 40, 64, 100]), rng.choice([None, 48, 128]))
        layers.append(layer(mixer, mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers))
        loop = (start, rng.randint(start, len(layers)), rng.choice([1, 2, 3]))
    return config(rng.choice([257, 300, 1000]), width, rng.choice([1e-6, 1e-5]), rng.choice([0.3, 1.0, 1.4]),
                  rng.choice([0.0, 5.0, 50.0]), loop, layers)


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(tmp_path, seed):
    """Whole, with the last 20 tokens one by one, and in portions of 2 to 70 tokens, in 32-bit and in bfloat16."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    import random

    from pulse_infer_amd.config import FosupelConfig
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    rng = random.Random(9000 + seed)
    cfg = random_config(rng)
    length = rng.choice([90, 150])
    folder = write_model_folder(FosupelConfig.from_dict(cfg), str(tmp_path / "m"), seed=seed)
    oracle = P.PlainFosupel.from_folder(folder)
    ids = token_ids(cfg["vocab"], length, seed=seed)
    want = oracle.logits(ids)
    calls = Calls(set((oracle.router_margins(ids) < CLOSE_CALL).nonzero().flatten().tolist()), oracle.fragile_positions(ids))
    what = f"{cfg} length {length}"
    for dtype in ("float32", "bfloat16"):
        _, model = load_model(folder, mode=dtype)
        runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=4)
        whole = run_alone(runner, ids, [length])
        agree(whole, want, dtype, f"whole: {what}", calls, by_median=True)
        tail = run_alone(runner, ids, [length - 20] + [1] * 20)
        agree(tail, want, dtype, f"tail: {what}", calls, by_median=True)
        cuts, left_over, sizes = [], length, [40, 2, 17, 3, 70, 5, 19]
        while left_over:
            n = min(sizes[len(cuts) % len(sizes)], left_over)
            cuts.append(n)
            left_over -= n
        portions = run_alone(runner, ids, cuts)
        agree(portions, want, dtype, f"portions {cuts}: {what}", calls, by_median=True)
        # however the prompt is cut: the same logits (in 32-bit only the fragile positions are left out; in bfloat16
        # another cut may also tip a router's close call)
        left_out = Calls(set(), calls.fragile) if dtype == "float32" else calls
        agree(tail, whole, dtype, f"tail against whole: {what}", left_out, by_median=True)
        agree(portions, whole, dtype, f"portions against whole: {what}", left_out, by_median=True)
        del runner, model
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_long_decoding_of_three_requests(runners, plain, name, dtype):
    """Three requests of unequal prompts decode 100 tokens together, over page borders and out of every window."""
    from pulse_infer_amd.engine.runner import StepEntry

    vocab, new = CONFIGS[name]["vocab"], 100
    runner = runners(name, dtype, 16, tokens=704)
    prompt = {"d0": 1, "d1": 30, "d2": 47}
    ids = {k: token_ids(vocab, n + new, seed=60 + i) for i, (k, n) in enumerate(prompt.items())}
    got = {k: [] for k in ids}
    for k in ids:
        runner.add_request(k)
        runner.reserve(k, prompt[k])
    first = runner.step([StepEntry(k, ids[k][:prompt[k]], [prompt[k] - 1]) for k in ids])
    for row, k in enumerate(ids):
        got[k].append(first[row:row + 1])
    for step in range(new):
        for k in ids:
            runner.reserve(k, prompt[k] + step + 1)
        logits = runner.step([StepEntry(k, [ids[k][prompt[k] + step]], [0]) for k in ids])
        for row, k in enumerate(ids):
            got[k].append(logits[row:row + 1])
    for k in ids:
        runner.free_request(k)
        agree(torch.cat(got[k]), plain(name, ids[k])[prompt[k] - 1:], dtype, f"{name} decoding request {k}",
              plain.close_calls(name, ids[k]), first=prompt[k] - 1)


# --------------------------------------------------------------------------- generation through the scheduler
@pytest.mark.parametrize("name", ["mixed", "equal"])
def test_greedy_generation_through_the_engine(folders, plain, name):
    """In 32-bit the greedy choice does not depend on the batch: requests generated together, in small portions and
    with a pool so tight that some are preempted and recomputed (their states start again from zero), give what
    each gives alone and what the plain implementation chooses."""
    from pulse_infer_amd import LLM

    vocab, new, page = CONFIGS[name]["vocab"], 12, 16
    prompts = [token_ids(vocab, n, seed=80 + i) for i, n in enumerate((1, 5, 18, 40, 77))]
    make = lambda **kw: LLM.from_pretrained(folders[name], dtype="float32", page_size=page, **kw)
    alone = [make(max_batch_size=1, chunk_size=256, num_pages=32).generate([p], max_new_tokens=new, ignore_eos=True)[0]
             for p in prompts]
    assert alone == [plain.models[name].greedy(p, new) for p in prompts]
    roomy = make(max_batch_size=4, chunk_size=16, num_pages=64, max_num_batched_tokens=24)
    assert roomy.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    need = max((len(p) + new + page - 1) // page for p in prompts)
    tight = make(max_batch_size=4, chunk_size=16, num_pages=need + 2)
    assert tight.generate(prompts, max_new_tokens=new, ignore_eos=True) == alone
    tight.engine.runner.cache.check()


def test_bfloat16_generation_stays_within_rounding_of_the_plain_choice(folders, plain):
    """Every token that the bfloat16 engine chooses is, for the plain implementation, within rounding of the best one
    (where the position is not fragile and no router's choice at it is a close call)."""
    from pulse_infer_amd import LLM

    name, new = "wide", 10
    prompts = [token_ids(CONFIGS[name]["vocab"], n, seed=90 + i) for i, n in enumerate((3, 21))]
    llm = LLM.from_pretrained(folders[name], dtype="bfloat16", max_batch_size=2, chunk_size=8, page_size=16, num_pages=32)
    judged = 0
    for prompt, out in zip(prompts, llm.generate(prompts, max_new_tokens=new, ignore_eos=True)):
        assert len(out) == new
        for t, token in enumerate(out):
            ids = prompt + out[:t]
            calls = plain.close_calls(name, ids)
            if len(ids) - 1 in calls or len(ids) - 1 in calls.fragile:
                continue
            row = plain(name, ids)[-1]
            assert float(row[token]) >= float(row.max()) - TOL["bfloat16"] * float(row.abs().max())
            judged += 1
    assert judged >= new


def test_the_command_line_generates(folders, plain):
    name = "equal"
    prompt = token_ids(CONFIGS[name]["vocab"], 9, seed=99)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "pulse_infer"), folders[name], "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--greedy",
                          "--ignore-eos", "--max-positions", "64"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    out = json.loads(run.stdout.strip().splitlines()[0])
    assert out["output_ids"] == plain.models[name].greedy(prompt, 6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(folders, plain, tmp_path, dtype):
    import numpy as np

    name = "mixed"
    vocab = CONFIGS[name]["vocab"]
    a, b = token_ids(vocab, 70, seed=1), token_ids(vocab, 21, seed=2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:69], "want": []}, {"id": "b", "tokens": b[:20], "want": [19]}],
         "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[20:], "want": [0]}, {"id": "a", "tokens": a[69:], "want": [0]}],
         "end": ["a", "b"]},
    ]
    out = tmp_path / f"out_{dtype}"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype,
                          "--out", str(out), "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = plain(name, a), plain(name, b)
    read = lambda i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab).copy())
    judged = 0
    for step, rows in ((0, [(a, la, 0), (a, la, 49)]), (1, [(b, lb, 19)]), (2, [(b, lb, 20), (a, la, 69)])):
        got = read(step)
        assert got.shape[0] == len(rows) and torch.isfinite(got).all()
        for i, (ids, want, at) in enumerate(rows):
            calls = plain.close_calls(name, ids)
            if at in calls.fragile or (dtype == "bfloat16" and at in calls):
                continue
            close(got[i:i + 1], want[at:at + 1], dtype, f"step {step} row {i}", TOL)
            judged += 1
    assert judged >= (3 if dtype == "float32" else 1)
