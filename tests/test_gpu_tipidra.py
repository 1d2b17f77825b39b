"""Tipidra on the GPU against the plain implementation (tests/plain/tipidra_plain.py), in 32-bit and in bfloat16.

Small configurations of their own and seeded random weights: one whose layers all differ (keys wider than values and
the other way round, grouped and ungrouped heads, a rotation on part of a head, on all of it and none, with and
without a score cap, state sizes that are no powers of two, two to four taps, a layer without a feed-forward,
routers that choose one, two and three experts), one whose constants are one and whose sizes coincide (one stream),
one without the streams' key, and one at widths where the serving kernels run.  Each mechanism alone at its kernel,
with inputs made so that a fault shows (a far key that takes all the weight, a sink that takes it all, states and
pages filled with NaN before use); then whole prompts, token-by-token decoding, portions down to two tokens, mixed
batches with pages and slots used again, long decoding through recorded steps, greedy generation through the
scheduler, the command line and the trace replay program.
"""
import json
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT, token_ids
from plain import tipidra_plain as P
from test_gpu_model import SPLIT_TOL, TOL, close, mixed_trace, pages_were_used_again, run_alone, run_mixed

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def attention(heads, kv_heads, dim, vdim, scale, softcap=None, rot=None):
    out = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if softcap:
        out["softcap"] = softcap
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    return "attention", out


def mamba(inner, state, dt_rank, conv):
    return "mamba1", {"conv": conv, "dt_rank": dt_rank, "inner": inner, "state": state}


def moe(experts, top, ff, limit):
    return {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "top": top}}


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def layer(mixer, mlp):
    return {"mixer": mixer[1], "mlp": mlp, "type": mixer[0]}


def config(vocab, width, eps, embed_scale, softcap, streams, layers):
    out = {"architecture": "Tipidra", "embedding": {"scale": embed_scale}, "layers": layers, "logit_softcap": softcap,
           "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if streams is not None:
        out["streams"] = streams
    return out


# every layer another shape
MIXED = config(307, 96, 1e-5, 3.0, 9.0, 3, [
    layer(mamba(80, 5, 3, 2), moe(5, 2, 48, 0.7)),
    layer(attention(6, 2, 32, 16, 0.2, 20.0, (1e4, 16)), dense(160)),
    layer(attention(4, 4, 16, 48, 0.4, None, (500.0, 16)), None),
    layer(mamba(128, 24, 8, 3), dense(64)),
    layer(attention(3, 1, 48, 48, 0.1, 5.0, None), moe(3, 3, 40, 2.0)),
    layer(mamba(48, 16, 16, 4), None),
])
# constants that are one, sizes that coincide, one stream
EQUAL = config(515, 128, 1e-6, 1.0, 30.0, 1, [
    layer(attention(2, 2, 64, 64, 1.0, 1.0, (1e4, 64)), dense(128)),
    layer(mamba(128, 16, 16, 4), moe(2, 1, 128, 1.0)),
    layer(attention(2, 2, 64, 64, 1.0, 1.0, (1e4, 64)), moe(2, 1, 128, 1.0)),
])
# no streams' key: the plain residual sum
PLAIN_SUM = config(211, 64, 1e-5, 2.0, 0.0, None, [
    layer(attention(4, 2, 16, 32, 0.25, 10.0, (1e4, 8)), dense(96)),
    layer(mamba(96, 8, 4, 4), moe(4, 2, 32, 1.5)),
])
# widths of a real model's layers (inner sizes that are multiples of 1,024, heads of 128 in groups of four)
WIDE = config(300, 1024, 1e-6, 8.0, 20.0, 2, [
    layer(attention(8, 2, 128, 128, 0.09, 30.0, (1e6, 64)), moe(4, 2, 256, 1.0)),
    layer(mamba(2048, 16, 64, 4), dense(2048)),
    layer(attention(8, 2, 128, 64, 0.09, 50.0, (1e4, 128)), dense(1024)),
])
CONFIGS = {"mixed": MIXED, "equal": EQUAL, "plain_sum": PLAIN_SUM, "wide": WIDE}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.config import TipidraConfig
    from pulse_infer_amd.weights import write_model_folder

    out = {}
    for seed, (name, cfg) in enumerate(CONFIGS.items()):
        out[name] = write_model_folder(TipidraConfig.from_dict(cfg), str(tmp_path_factory.mktemp(name)), seed=270 + seed)
    return out


@pytest.fixture(scope="module")
def plain(folders):
    models = {name: P.PlainTipidra.from_folder(folder) for name, folder in folders.items()}
    memo = {}

    def logits(name, ids):
        key = (name, tuple(ids))
        if key not in memo:
            memo[key] = models[name].logits(list(ids))
        return memo[key]

    def close_calls(name, ids):
        """Positions at which a router's choice hangs on less than CLOSE_CALL: bfloat16 may choose otherwise there."""
        key = ("calls", name, tuple(ids))
        if key not in memo:
            memo[key] = set((models[name].router_margins(list(ids)) < CLOSE_CALL).nonzero().flatten().tolist())
        return memo[key]

    logits.models = models
    logits.close_calls = close_calls
    return logits


CLOSE_CALL = 0.004
# bfloat16 against the plain implementation: the streams' mixing matrices and factors multiply what every rounding of
# an activation leaves (random ones of the tests more than trained ones would), so the bound is twice that of the
# other designs' tests; the 32-bit bound, which is what pins schedules, pages and slots, is theirs
OWN_TOL = {"float32": TOL["float32"], "bfloat16": 2 * TOL["bfloat16"]}


def agree(got, want, dtype, what, calls=(), first=0, tol=OWN_TOL):
    """``close``; in bfloat16 another choice of a router at one position reaches all later ones through the states
    of the recurrent layers, so the positions before the first close call (``calls``, positions in the sequence; row 0
    of ``got`` is position ``first``) are compared one by one, and of the rest the median error."""
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("streams,hidden", [(1, 96), (2, 1000), (4, 320), (3, 4096), (16, 64)])
def test_streams_their_update_and_the_layer_norm(dtype, streams, hidden):
    """The weighted sum of the streams through the layer norm; the update of all streams at once from the old ones
    (alone, and inside the norm's kernel); gathered rows; a plain sum where no factors are given."""
    from pulse_infer_amd.ops import kernels

    tokens, eps = 7, 1e-5
    x0 = rnd(tokens, streams, hidden, seed=1, scale=3.0)
    w, wref = stored(1.0 + rnd(hidden, seed=2, scale=0.1), dtype)
    b, bref = stored(rnd(hidden, seed=3, scale=0.1), dtype)
    y, yref = stored(rnd(tokens, hidden, seed=4), dtype)
    w_in, mix, w_out = rnd(streams, seed=5), rnd(streams, streams, seed=6, scale=0.7), rnd(streams, seed=7)
    ref = x0.to(F64).permute(1, 0, 2)                                   # [S, T, H]
    u = torch.einsum("s,stw->tw", w_in.to(F64), ref)
    x = x0.reshape(tokens, streams * hidden).to(DEV).contiguous()
    out = torch.full((tokens, hidden), float("nan"), dtype=dtype, device=DEV)
    kernels.streams_step(x, streams, in_weight=w_in.to(DEV), norm=("layernorm", w, b, eps), out=out)
    assert torch.allclose(out.cpu().to(F64), P.layer_norm(u, wref, bref, eps), **tol(dtype))
    assert torch.equal(x.cpu(), x0.reshape(tokens, -1))
    rows = [5, 0, 5, 2]
    some = torch.full((len(rows), hidden), float("nan"), dtype=dtype, device=DEV)
    kernels.streams_step(x, streams, norm=("layernorm", w, b, eps), out=some, rows=ints(rows))
    assert torch.allclose(some.cpu().to(F64), P.layer_norm(ref.sum(0), wref, bref, eps)[rows], **tol(dtype))
    new = torch.einsum("st,sxw->txw", mix.to(F64), ref) + w_out.to(F64).view(-1, 1, 1) * yref
    fused = x.clone()
    kernels.streams_step(fused, streams, update=(y, mix.to(DEV), w_out.to(DEV)), in_weight=w_in.to(DEV),
                         norm=("layernorm", w, b, eps), out=out)
    kernels.streams_step(x, streams, update=(y, mix.to(DEV), w_out.to(DEV)))
    assert torch.equal(fused, x)
    assert torch.allclose(x.cpu().to(F64).view(tokens, streams, hidden).permute(1, 0, 2), new, atol=1e-5, rtol=1e-5)
    u2 = torch.einsum("s,stw->tw", w_in.to(F64), new)
    assert torch.allclose(out.cpu().to(F64), P.layer_norm(u2, wref, bref, eps), **tol(dtype))
    # gathered rows with an update (a row asked for twice): the new streams are used and the residual is left alone
    before = x.clone()
    kernels.streams_step(x, streams, update=(y, mix.to(DEV), w_out.to(DEV)), norm=("layernorm", w, b, eps), out=some,
                         rows=ints(rows))
    assert torch.equal(x, before)
    again = torch.einsum("st,sxw->txw", mix.to(F64), new) + w_out.to(F64).view(-1, 1, 1) * yref
    assert torch.allclose(some.cpu().to(F64), P.layer_norm(again.sum(0), wref, bref, eps)[rows], **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inner,state,taps", [(80, 5, 2), (128, 16, 4), (48, 24, 3), (200, 32, 4), (33, 70, 1),
                                              (64, 1, 4), (72, 2, 4), (40, 3, 2), (2048, 16, 4), (24, 256, 3)])
def test_the_convolution_and_the_recurrence(dtype, inner, state, taps):
    """Three requests in one step (a portion of 37 tokens that continues a state, a fresh prompt of 20 in a slot that
    holds NaN, a single decoded token), then the same requests a few tokens further (fewer than the taps for one of
    them): outputs, states and the convolution's tails are the plain walk's."""
    from pulse_infer_amd.ops import kernels

    slots = 5
    counts, starts, slot_of = [37, 20, 1], [12, 0, 300], [3, 0, 4]
    more = [2, 1, 5]
    w_conv, cref = stored(rnd(inner, taps, seed=1, scale=0.5), dtype)
    b_conv, cbref = stored(rnd(inner, seed=2, scale=0.2), dtype)
    dt_bias, dbref = stored(rnd(inner, seed=3), dtype)
    a_log, aref = stored(rnd(inner, state, seed=4, scale=0.5), dtype)
    d_skip, dref = stored(1.0 + rnd(inner, seed=5, scale=0.1), dtype)
    row = state + taps - 1
    dev_state = torch.full((slots, inner, row), float("nan"), dtype=torch.float32, device=DEV)
    ref_state, ref_tail, fed = {}, {}, {}
    for r, (s, slot) in enumerate(zip(starts, slot_of)):
        if s > 0:
            ref_state[r] = rnd(inner, state, seed=20 + r).to(F64)
            ref_tail[r] = rnd(taps - 1, inner, seed=30 + r).to(dtype).to(F64)
            dev_state[slot, :, :state] = ref_state[r].float().to(DEV)
            dev_state[slot, :, state:] = ref_tail[r].T.float().to(DEV)
        else:
            ref_state[r], ref_tail[r] = None, None
        fed[r] = s
    for round_, step_counts in enumerate((counts, more)):
        total = sum(step_counts)
        xin, xref = stored(rnd(total, 2 * inner, seed=40 + round_), dtype)        # [x | z] rows
        dt_raw, dtref = stored(rnd(total, inner, seed=50 + round_), dtype)
        bc, bcref = stored(rnd(total, 3 + 2 * state, seed=60 + round_), dtype)    # three columns of something else first
        first_row = [0]
        for c in step_counts:
            first_row.append(first_row[-1] + c)
        positions = [fed[r] + i for r, c in enumerate(step_counts) for i in range(c)]
        entry = [r for r, c in enumerate(step_counts) for _ in range(c)]
        conv_out = torch.full((total, inner), float("nan"), dtype=dtype, device=DEV)
        kernels.causal_conv(xin, w_conv, b_conv, conv_out, dev_state, state, ints(positions), ints(entry),
                            ints([fed[r] for r in range(3)]), ints(first_row), ints(slot_of), 3)
        y = torch.full((total, inner), float("nan"), dtype=dtype, device=DEV)
        kernels.selective_scan(conv_out, dt_raw, bc, 3, 3 + state, xin[:, inner:], y, dt_bias, a_log, d_skip, dev_state,
                               ints([fed[r] for r in range(3)]), ints(first_row), ints(slot_of), 3)
        for r, c in enumerate(step_counts):
            lo, hi = first_row[r], first_row[r + 1]
            x_r = xref[lo:hi, :inner]
            want_conv = P.silu(P.causal_taps(x_r, cref, cbref, before=ref_tail[r] if taps > 1 else None))
            got_conv = conv_out[lo:hi].cpu().to(F64)
            assert torch.allclose(got_conv, want_conv, **tol(dtype)), (round_, r)
            dt = P.softplus(dtref[lo:hi] + dbref)
            want_y, ref_state[r] = P.selective_scan(got_conv, dt, -torch.exp(aref), bcref[lo:hi, 3:3 + state],
                                                    bcref[lo:hi, 3 + state:], dref, ref_state[r])
            want_y = want_y * P.silu(xref[lo:hi, inner:])
            assert torch.allclose(y[lo:hi].cpu().to(F64), want_y, **tol(dtype)), (round_, r)
            before = torch.zeros(taps - 1, inner, dtype=F64) if ref_tail[r] is None else ref_tail[r]
            ref_tail[r] = torch.cat([before, x_r])[-(taps - 1):] if taps > 1 else before
            got_state = dev_state[slot_of[r]].cpu().to(F64)
            assert torch.allclose(got_state[:, :state], ref_state[r], atol=1e-4, rtol=1e-4), (round_, r)
            assert torch.equal(got_state[:, state:], ref_tail[r].T), (round_, r)
            fed[r] += c


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


ATTENTION_CASES = [
    dict(nq=6, nkv=2, d=32, dv=16, bs=16, rot=16, cap=20.0, lens=[150, 1, 64, 65, 33], portion=70),
    dict(nq=4, nkv=4, d=16, dv=48, bs=16, rot=16, cap=0.0, lens=[90, 33, 17], portion=40),
    dict(nq=8, nkv=2, d=128, dv=128, bs=32, rot=64, cap=30.0, lens=[300, 100], portion=129),
    dict(nq=8, nkv=2, d=64, dv=32, bs=16, rot=0, cap=40.0, lens=[700, 260, 17], portion=300),
    dict(nq=3, nkv=1, d=48, dv=96, bs=16, rot=48, cap=8.0, lens=[200, 41, 40, 5], portion=2),
    dict(nq=2, nkv=1, d=20, dv=10, bs=4, rot=10, cap=3.0, lens=[45, 9], portion=11),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTENTION_CASES)
@pytest.mark.parametrize("needle", [None, 2, "border", "near", "sink"])
def test_capped_scores_sinks_and_the_gate_over_prepared_rows(case, dtype, needle):
    """The rotation in halves on part of a head, q and k divided head by head by their root mean square, keys and
    values of different widths in pages of one width, the cap on the scores, the sink in the denominator and the gate
    a channel: a portion of request 0 beside single tokens of the others, through every attention kernel, with one
    split and with several.  With a needle, one stored key (at position 2, at a page's last slot far back, or next
    to the query) is replaced by many times the last query of every request, so that it takes all the weight that
    the cap lets it take; with "sink" one head's sink is so large that its output vanishes."""
    from pulse_infer_amd.parts.attention_rows import stored_width
    from pulse_infer_amd.ops import attention_mfma as M
    from pulse_infer_amd.ops import kernels

    nq, nkv, d, dv, bs, rot, cap, lens, portion = (case[x] for x in ("nq", "nkv", "d", "dv", "bs", "rot", "cap", "lens",
                                                                      "portion"))
    eps, scale, share, base = 1e-5, 0.3, nq // nkv, 1e4
    D = stored_width(d, dv)
    kc, vc, table = paged(lens, nkv, D, bs, dtype, seed=3)
    cols = nq * d + nkv * (d + dv) + nq * dv
    gate0 = nq * d + nkv * (d + dv)
    sink = rnd(nq, seed=77)
    if needle == "sink":
        sink[0] = 60.0
    rows_of, keys, values, queries, gates = [], [], [], [], []
    for r, n in enumerate(lens):
        rows, ref = stored(rnd(n, cols, seed=10 + r), dtype)
        rows_of.append(rows)
        q, k = ref[:, :nq * d].view(n, nq, d), ref[:, nq * d:nq * d + nkv * d].view(n, nkv, d)
        if rot:
            q, k = P.rotate_halves(q, list(range(n)), base, rot), P.rotate_halves(k, list(range(n)), base, rot)
        queries.append(P.unit_rms(q, eps))
        keys.append(P.unit_rms(k, eps))
        values.append(ref[:, nq * d + nkv * d:gate0].view(n, nkv, dv))
        gates.append(ref[:, gate0:].view(n, nq, dv))
    inv = base ** (-2.0 * torch.arange(max(rot, 2) // 2, dtype=F64) / max(rot, 2))

    def prepare(rows, positions, entry):
        cos = sin = None
        if rot:
            angle = torch.tensor(positions, dtype=F64).view(-1, 1) * inv.view(1, -1)
            cos, sin = torch.cos(angle).float().to(DEV).contiguous(), torch.sin(angle).float().to(DEV).contiguous()
        q = torch.full((rows.shape[0], nq * D), float("nan"), dtype=dtype, device=DEV)
        kernels.qkv_rows(rows, q, nq, nkv, d, dv, D, None, None, eps, cos, sin, rot, 1, kc, vc, ints(positions),
                         ints(entry), table.to(DEV), norm="head")
        return q

    fed = [lens[0] - portion] + [n - 1 for n in lens[1:]]
    for r, n in enumerate(fed):
        if n:
            prepare(rows_of[r][:n].contiguous(), list(range(n)), [r] * n)
    positions = list(range(fed[0], lens[0])) + [n - 1 for n in lens[1:]]
    entry = [0] * portion + list(range(1, len(lens)))
    step = torch.cat([rows_of[0][fed[0]:]] + [rows_of[r][n - 1:] for r, n in enumerate(lens) if r]).contiguous()
    q = prepare(step, positions, entry)
    got_q = q.cpu().to(F64).view(-1, nq, D)
    want_q = torch.cat([queries[0][fed[0]:]] + [queries[r][n - 1:] for r, n in enumerate(lens) if r])
    stored_keys = [k.clone() for k in keys]
    planted_at = {}
    if needle is None:
        assert torch.allclose(got_q[..., :d], want_q, **tol(dtype))
        assert float(got_q[..., d:].abs().sum()) == 0.0
        for r, n in enumerate(lens):
            for j in (0, n // 2, n - 1):
                page, slot = int(table[r, j // bs]), j % bs
                assert torch.allclose(kc[page, :, slot, :d].cpu().to(F64), keys[r][j], **tol(dtype))
                assert torch.allclose(vc[page, :, :dv, slot].cpu().to(F64), values[r][j], **tol(dtype))
                assert float(kc[page, :, slot, d:].float().abs().sum()) == 0.0
                assert float(vc[page, :, dv:, slot].float().abs().sum()) == 0.0
    elif needle != "sink":
        for r, n in enumerate(lens):
            j = {2: 2, "border": bs - 1, "near": n - 2}[needle]
            if not 0 <= j < n - 1:
                continue
            page, slot = int(table[r, j // bs]), j % bs
            for g in range(nkv):
                planted = (60.0 * queries[r][n - 1, g * share]).to(dtype)
                kc[page, g, slot, :d] = planted.to(DEV)
                stored_keys[r][j, g] = planted.to(F64)
            planted_at[r] = j
    out = torch.zeros(len(positions), nq * D, dtype=dtype, device=DEV)
    pos_t, ent_t = ints(positions), ints(entry)
    used_q = got_q[..., :d]
    gate_rows = step[:, gate0:]
    used_gate = gate_rows.cpu().to(F64).view(-1, nq, dv)
    want = torch.zeros(len(positions), nq, dv, dtype=F64)
    for t, (p, e) in enumerate(zip(positions, entry)):
        k_e = stored_keys[e][:p + 1].to(dtype).to(F64)
        v_e = values[e][:p + 1].to(dtype).to(F64)
        for h in range(nq):
            g = h // share
            s = P.capped((k_e[:, g] @ used_q[t, h]) * scale, cap)
            top = torch.maximum(s.max(), sink[h].to(F64))
            e_s = torch.exp(s - top)
            w = e_s / (e_s.sum() + torch.exp(sink[h].to(F64) - top))
            want[t, h] = (w.view(-1, 1) * v_e[:, g]).sum(0) * torch.sigmoid(used_gate[t, h])
    if planted_at and cap == 0.0:
        # without a cap the needle decides the last token's output of the group's first head
        for r, j in planted_at.items():
            t = portion - 1 if r == 0 else portion + r - 1
            ref = values[r][j, 0].to(dtype).to(F64) * torch.sigmoid(used_gate[t, 0])
            assert torch.allclose(want[t, 0], ref, atol=1e-2, rtol=1e-2)
    if needle == "sink":
        assert float(want[:, 0].abs().max()) < 1e-6 and float(want[:, 1:].abs().max()) > 1e-3
    sink_dev = sink.to(DEV)
    extra = dict(gate=gate_rows, gate_width=dv, sink=sink_dev, softcap=cap)
    paths = ["generic"]
    if M.supported(D, bs, dtype, dtype):
        paths += ["matrix", "matrix in splits"]

    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count

    for path in paths:
        out.zero_()
        if path == "generic":
            kernels.attn_generic(q, out, nq, nkv, D, kc, vc, pos_t, ent_t, table.to(DEV), scale, 0, **extra)
        else:
            splits = 1 if path == "matrix" else 3
            numbered = list(enumerate([E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)]))
            small = numbered
            rows = len(positions) * nq * splits
            part_o = torch.full((rows, D), float("nan"), dtype=torch.float32, device=DEV) if splits > 1 else None
            part_ml = torch.full((rows, 2), float("nan"), dtype=torch.float32, device=DEV) if splits > 1 else None
            if portion >= M.PORTION_MIN_TOKENS:
                small = numbered[1:]
                big = ints(M.build_items(numbered[:1], M.portion_tokens(share, D)))
                cut = splits if D in M.PREFILL_SPLIT_HEAD_DIMS else 1
                size = (lens[0] + cut * 64 - 1) // (cut * 64) * 64 if cut > 1 else 0
                M.attn_prefill(q, out, nq, nkv, D, kc, vc, pos_t, table.to(DEV), big, scale, 0, size, cut,
                               part_o if cut > 1 else None, part_ml if cut > 1 else None, **extra)
            items = ints(M.build_items(small, M.tokens_per_item(share)))
            split = (max(lens) + splits * 32 - 1) // (splits * 32) * 32
            M.attn_mfma(q, out, nq, nkv, D, kc, vc, pos_t, table.to(DEV), items, scale, 0, split, splits, max(lens),
                        part_o, part_ml, **extra)
        got = out.cpu().to(F64).view(-1, nq, D)
        assert torch.allclose(got[..., :dv], want, **tol(dtype)), (path, float((got[..., :dv] - want).abs().max()))
        assert float(got[..., dv:].abs().sum()) == 0.0, path


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,ff,hidden,limit", [(5, 2, 48, 96, 0.7), (3, 3, 40, 80, 2.0), (12, 1, 64, 192, 1.0),
                                                         (4, 2, 256, 1024, 1.0)])
def test_sigmoid_router_and_experts_fed_their_weighted_input(dtype, experts, top, ff, hidden, limit):
    """Scores are sigmoids of float32 router logits and stay as they are; an expert is fed score * x; the clamped
    activation: through the kernels of few tokens and, in bfloat16, through the grouped products of both tile heights."""
    from pulse_infer_amd.ops import kernels

    tokens = 150
    x, xref = stored(rnd(tokens, hidden, seed=1), dtype)
    w = {}
    router, w["mlp.router"] = stored(rnd(experts, hidden, seed=2, scale=hidden ** -0.5 * 2), dtype)
    gates, ups, downs = [], [], []
    for e in range(experts):
        for name, shape, keep in (("gate", (ff, hidden), gates), ("up", (ff, hidden), ups), ("down", (hidden, ff), downs)):
            dev, w[f"mlp.e{e}.{name}"] = stored(rnd(*shape, seed=10 + 3 * e + len(keep) % 3, scale=shape[1] ** -0.5 * 1.5), dtype)
            keep.append(dev)
    w_gate, w_up, w_down = torch.stack(gates).contiguous(), torch.stack(ups).contiguous(), torch.stack(downs).contiguous()
    idx = torch.zeros(tokens, top, dtype=torch.int32, device=DEV)
    weight = torch.zeros(tokens, top, dtype=torch.float32, device=DEV)
    kernels.moe_router(x, router, None, top, idx, weight, score="sigmoid", renormalize=False)
    scores = P.router_scores(xref, w, "mlp")
    ranked = torch.sort(scores, dim=-1, descending=True)
    clear = (ranked.values[:, top - 1] - ranked.values[:, top] > 1e-3) if top < experts else torch.ones(tokens, dtype=torch.bool)
    assert int(clear.sum()) > tokens // 2
    got_sets = torch.sort(idx.cpu().long(), dim=-1).values
    want_sets = torch.sort(ranked.indices[:, :top], dim=-1).values
    assert torch.equal(got_sets[clear], want_sets[clear])
    assert torch.allclose(weight.cpu().to(F64), torch.gather(scores, 1, idx.cpu().long()), atol=1e-5, rtol=1e-5)
    want = torch.zeros(tokens, hidden, dtype=F64)
    for t in range(tokens):
        for k in range(top):
            e = int(idx[t, k])
            want[t] += P.clamped_expert((float(weight[t, k]) * xref[t]).view(1, -1), w, f"mlp.e{e}", limit)[0]
    loose = dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=4e-2, rtol=4e-2)
    act = torch.full((tokens * top, ff), float("nan"), dtype=dtype, device=DEV)
    out = torch.full((tokens, hidden), float("nan"), dtype=torch.float32, device=DEV)
    kernels.moe_gate_up(x, w_gate, w_up, idx, act, in_weight=weight, activation="clamped_swish", limit=limit)
    kernels.moe_down(x, act, w_down, idx, None, out)
    assert torch.allclose(out.cpu().to(F64), want, **loose), float((out.cpu().to(F64) - want).abs().max())
    if kernels.moe_grouped_takes(x, w_gate, w_down):
        for rows in kernels.MOE_TILE_ROWS:
            pairs = tokens * top
            y = torch.full((pairs, hidden), float("nan"), dtype=torch.float32, device=DEV)
            scratch = torch.zeros(2 * pairs + 3 * kernels.moe_max_tiles(pairs, experts, rows) + 1, dtype=torch.int32, device=DEV)
            act.fill_(float("nan"))
            out.fill_(float("nan"))
            kernels.moe_grouped(x, w_gate, w_up, w_down, idx, weight, act, y, out, scratch, rows, weight_on_input=True,
                                activation="clamped_swish", limit=limit)
            assert torch.allclose(out.cpu().to(F64), want, **loose), (rows, float((out.cpu().to(F64) - want).abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_gate_with_the_tanh_form_of_gelu(dtype):
    from pulse_infer_amd.ops import kernels

    gu, ref = stored(rnd(9, 2 * 88, seed=5, scale=2.0), dtype)
    out = torch.empty(9, 88, dtype=dtype, device=DEV)
    kernels.swiglu(gu, out, activation="gelu_tanh")
    assert torch.allclose(out.cpu().to(F64), P.gelu_tanh(ref[:, :88]) * ref[:, 88:], **tol(dtype))


# ------------------------------------------------------------------------------------------------ whole models
LENGTH = {"mixed": 150, "equal": 130, "plain_sum": 120, "wide": 90}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("mixed", 4), ("equal", 16), ("equal", 64), ("plain_sum", 16),
                                       ("wide", 16)])
def test_whole_tail_and_portions(runners, plain, name, page, dtype):
    ids = token_ids(CONFIGS[name]["vocab"], LENGTH[name], seed=3)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, page)
    n = len(ids)
    whole = run_alone(runner, ids, [n])
    agree(whole, want, dtype, f"{name} whole", calls)
    tail = run_alone(runner, ids, [n - 40] + [1] * 40)               # prefill against token-by-token decoding
    agree(tail, want, dtype, f"{name} tail", calls)
    if not (dtype == "bfloat16" and calls):
        close(tail, whole, dtype, f"{name} tail against whole", tol=SPLIT_TOL)
    for cuts in ([2, 3, 31, 2, 17, n - 57, 2], [1, 1, 1, 31, n - 34], [n - 2, 2], [7] * (n // 7) + [n % 7 or 7][:n % 7 > 0]):
        cuts = [c for c in cuts if c]
        portions = run_alone(runner, ids, cuts)
        agree(portions, want, dtype, f"{name} portions {cuts}", calls)
        if not (dtype == "bfloat16" and calls):
            close(portions, whole, dtype, f"{name} portions against whole", tol=SPLIT_TOL)
    first = run_alone(runner, ids[:3], [1, 1, 1])                     # the first tokens of a sequence
    agree(first, want[:3], dtype, f"{name} first tokens", calls)


@pytest.mark.parametrize("name", ["mixed", "equal", "plain_sum"])
def test_the_residual_after_every_layer(runners, plain, name):
    from pulse_infer_amd.engine.runner import StepEntry

    ids = token_ids(CONFIGS[name]["vocab"], 37, seed=8)
    runner = runners(name, "float32")
    model, seen = runner.model, []
    originals = [b.forward for b in model.blocks]
    streams = model.spec.streams

    def watched(forward):
        def run(stream, ctx, cache):
            forward(stream, ctx, cache)
            stream.settle()
            seen.append(stream.h.view(len(ids), streams, -1).sum(dim=1))
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
    assert len(seen) == len(want)
    for i, (got, ref) in enumerate(zip(seen, want)):
        close(got, ref, "float32", f"{name} after layer {i}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("mixed", 16), ("equal", 16), ("equal", 32), ("plain_sum", 16), ("wide", 16)])
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
def test_a_long_prompt(runners, plain, dtype):
    """700 tokens, whole (the keys walked in splits) and with the last 60 tokens decoded."""
    name = "plain_sum"
    ids = token_ids(CONFIGS[name]["vocab"], 700, seed=21)
    want, calls = plain(name, ids), plain.close_calls(name, ids)
    runner = runners(name, dtype, 16, tokens=704)
    agree(run_alone(runner, ids, [700]), want, dtype, "whole", calls)
    agree(run_alone(runner, ids, [250, 390] + [1] * 60), want, dtype, "decoded tail", calls)


# ------------------------------------------------------------------------------------ seeded random configurations
def random_config(rng):
    """Layers drawn one by one from shapes the kernels' own tests cover: head sizes that are multiples of 16 and
    some that are not, keys wider and narrower than values, rotations on a part of a head and none, states from 1 to
    40 values a channel, routers that choose one of seven and all of three, any number of streams or none."""
    pick = lambda *values: values[int(rng.randint(len(values)))]
    width = pick(64, 72, 96, 160)
    layers = []
    for _ in range(int(rng.randint(2, 5))):
        if rng.rand() < 0.55:
            kv = pick(1, 2, 4)
            dim = pick(16, 24, 32, 64)
            rot = pick(None, (1e4, dim), (777.0, dim // 2 // 2 * 2))
            # (scores of unit q and k reach dim * scale: scales far above dim ** -0.5 make the softmax hang on single
            # keys, and bfloat16's rounding of q and k then moves whole weights)
            mixer = attention(kv * pick(1, 2, 3), kv, dim, pick(8, 16, 40, 64), float(pick(0.5, 1.0, 2.0)) * dim ** -0.5,
                              pick(None, 4.0, 50.0), rot if rot is None or rot[1] else None)
        else:
            mixer = mamba(pick(40, 64, 100, 136), pick(1, 4, 16, 40), pick(1, 6, 16), pick(1, 2, 4))
        kind = rng.rand()
        if kind < 0.25:
            mlp = None
        elif kind < 0.6:
            mlp = dense(pick(40, 60, 64, 128))
        else:
            experts = pick(3, 7)
            mlp = moe(experts, pick(1, 2, experts) if experts == 3 else pick(1, 2), pick(24, 40), float(pick(0.5, 1.0, 3.0)))
        layers.append(layer(mixer, mlp))
    if not any(entry["type"] == "attention" for entry in layers):
        layers.append(layer(attention(2, 1, 16, 16, 0.25, 10.0, (1e4, 8)), dense(64)))
    return config(int(pick(97, 256, 301)), width, float(pick(1e-5, 1e-6)), float(pick(1.0, 4.0)), float(pick(0.0, 12.0)),
                  pick(None, 1, 2, 4, 6), layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    import numpy as np
    from pulse_infer_amd.config import TipidraConfig
    from pulse_infer_amd.engine.runner import ModelRunner
    from pulse_infer_amd.models.factory import load_model
    from pulse_infer_amd.weights import write_model_folder

    cfg = random_config(np.random.RandomState(500 + seed))
    print("configuration", json.dumps(cfg), flush=True)
    folder = write_model_folder(TipidraConfig.from_dict(cfg), str(tmp_path / "m"), seed=600 + seed)
    oracle = P.PlainTipidra.from_folder(folder)
    ids = token_ids(cfg["vocab"], 83, seed=seed)
    want = oracle.logits(ids)
    calls = set((oracle.router_margins(ids) < CLOSE_CALL).nonzero().flatten().tolist())
    for dtype in ("float32", "bfloat16"):
        _, model = load_model(folder, mode=dtype)
        runner = ModelRunner(model, page_size=16, num_pages=8, max_requests=2)
        for cuts in ([83], [60] + [1] * 23, [2, 30, 2, 40, 9]):
            agree(run_alone(runner, ids, cuts), want, dtype, f"seed {seed} {dtype} portions {cuts}", calls)
        del runner, model
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------------ long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_long_decoding_of_three_requests(runners, plain, name, dtype):
    """Three requests of unequal prompts decode 100 tokens together, over page borders; in bfloat16 the steps are
    recorded and replayed."""
    from pulse_infer_amd.engine.runner import StepEntry

    vocab, new = CONFIGS[name]["vocab"], 100
    runner = runners(name, dtype, 16, tokens=704)
    prompt = {"d0": 1, "d1": 30, "d2": 47}
    ids = {k: token_ids(vocab, n + new, seed=60 + i) for i, (k, n) in enumerate(prompt.items())}
    replays = runner.graph_replays
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
    if dtype == "bfloat16" and runner.model.recordable(list(range(3))):
        assert runner.graph_replays > replays, "no decoding step was replayed from a recording"


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
    from pulse_infer_amd import LLM

    name, new = "wide", 10
    prompts = [token_ids(CONFIGS[name]["vocab"], n, seed=90 + i) for i, n in enumerate((3, 21))]
    llm = LLM.from_pretrained(folders[name], dtype="bfloat16", max_batch_size=2, chunk_size=8, page_size=16, num_pages=32)
    for prompt, out in zip(prompts, llm.generate(prompts, max_new_tokens=new, ignore_eos=True)):
        assert len(out) == new
        for t, token in enumerate(out):
            row = plain(name, prompt + out[:t])[-1]
            assert float(row[token]) >= float(row.max()) - 3e-2 * float(row.abs().max())


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

    name = "plain_sum"
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
    close(read(0), la[[0, 49]], dtype, "step 0")
    close(read(1), lb[[19]], dtype, "step 1")
    close(read(2), torch.stack([lb[20], la[69]]), dtype, "step 2")
