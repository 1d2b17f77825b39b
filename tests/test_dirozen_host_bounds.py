"""The host side of whole steps on the CPU, with every HIP entry point replaced by a function that verifies its operands.

Seeded random Dirozen configurations (the sweep of tests/test_gpu_dirozen.py: head sizes the matrix-core kernels take
and two they do not, widths that are no multiple of 16, one query head, up to four cache groups) run whole prompts,
token-by-token decoding, portions and mixed batches through ``ModelRunner.step`` (eagerly: no recording without a
GPU); the vendor library's products run on the CPU, and in place of each kernel a function checks that what the
entry point is told to read and write lies inside the tensors it was handed: rows times strides against the
buffers' ends, gate and raw-value columns inside the projection output, scratch for the splits, items inside the
step's rows and the block table, positions inside the table's width.  No numbers are compared here.
"""
import ctypes
import random

import numpy as np
import pytest
import torch

from conftest import token_ids
from test_gpu_dirozen import random_config
from test_gpu_model import mixed_trace


class Ptr(ctypes.c_void_p):
    pass


def _ptr(t):
    p = Ptr(t.data_ptr() if t is not None else 0)
    p.tensor = t
    return p


def room(p):
    """Elements from the pointer to the end of its tensor's storage."""
    t = p.tensor
    if t is None:
        return 0
    storage = t.untyped_storage()
    return (storage.nbytes() - (t.data_ptr() - storage.data_ptr())) // t.element_size()


def val(a):
    return a.value if hasattr(a, "value") else a


def check(name, args):
    def need(cond, what):
        assert cond, f"{name}: {what}"

    if name == "pulse_qk_rope_kv":
        (qkv, _, stride, _, _, _, _, _, _, _, _, kc, vc, _, pos, ent, bt, width, tokens, nq, nkv, d, page, pages, write,
         _, vh0, _, _, _) = args
        tokens, stride, nq, nkv, d, vh0, page, width = (val(x) for x in (tokens, stride, nq, nkv, d, vh0, page, width))
        cols = max(nq + nkv, vh0 + nkv) * d if val(write) else nq * d
        need(room(qkv) >= (tokens - 1) * stride + cols, "the projection output is too short")
        need(room(pos) >= tokens, "positions")
        if val(write):
            need(min(room(kc), room(vc)) >= val(pages) * nkv * page * d, "cache")
            need(int(ent.tensor[:tokens].max()) < bt.tensor.shape[0] and bt.tensor.shape[1] == width, "table")
            need(int(pos.tensor[:tokens].max()) // page < width, "a position beyond the table")
    elif name == "pulse_attn_generic_ex":
        (q, qs, out, os_, _, _, _, _, pos, ent, bt, width, tokens, nq, _, d, page, _, _, _, gate, gs, _, _, _, _, _, _,
         _) = args
        tokens, nq, d = val(tokens), val(nq), val(d)
        need(room(q) >= (tokens - 1) * val(qs) + nq * d and room(out) >= (tokens - 1) * val(os_) + nq * d, "q / out")
        need(gate.tensor is None or room(gate) >= (tokens - 1) * val(gs) + nq, "gate")
        need(int(ent.tensor[:tokens].max()) < bt.tensor.shape[0] and bt.tensor.shape[1] == val(width), "table")
    elif name in ("pulse_attn_mfma", "pulse_attn_decode", "pulse_attn_prefill"):
        q, qs, out, os_, kc = args[0], val(args[1]), args[2], val(args[3]), args[4]
        bt, width, items, n_items, tokens, nq, nkv = args[7], val(args[8]), args[9], val(args[10]), val(args[11]), \
            val(args[12]), val(args[13])
        n_splits = val(args[19])
        part_o, part_ml = (args[21], args[22]) if name != "pulse_attn_prefill" else (args[20], args[21])
        extras = args[-2]
        d = kc.tensor.shape[-1]
        need(room(q) >= (tokens - 1) * qs + nq * d and room(out) >= (tokens - 1) * os_ + nq * d, "q / out")
        need(qs % 8 == 0 and q.tensor.data_ptr() % 16 == 0, "alignment of q")
        if n_splits > 1:
            need(room(part_o) >= tokens * nq * n_splits * d and room(part_ml) >= tokens * nq * n_splits * 2, "scratch")
        if extras is not None:
            e = extras._obj
            if e.gate:
                base = q.tensor.untyped_storage()
                first = (e.gate - base.data_ptr()) // 2
                need(first >= 0 and first + (tokens - 1) * e.gate_stride + nq <= base.nbytes() // 2, "gate")
            if name == "pulse_attn_decode":
                v0 = e.v_head0 if e.v_head0 >= 0 else nq + nkv
                need(room(q) >= (tokens - 1) * qs + (v0 + nkv) * d, "raw values")
        if items.tensor is not None:
            it = items.tensor.view(-1, 4)
            need(it.shape[0] == n_items and int((it[:, 0] + it[:, 1]).max()) <= tokens
                 and int(it[:, 2].max()) < bt.tensor.shape[0], "items")
        else:
            need(bt.tensor.shape[0] >= tokens, "a table row for every token")
        need(bt.tensor.shape[1] == width, "table width")
    elif name == "pulse_gemm_skinny_fused":
        (a, ldx, w, ldw, c, ldc, m, n, k, _, swiglu, _, ssq, sparts, _, sout, cout, ldcopy, cscale, _, _) = args
        m, n, k = val(m), val(n), val(k)
        need(room(a) >= (m - 1) * val(ldx) + k and room(w) >= (n - 1) * val(ldw) + k, "operands")
        need(room(c) >= (m - 1) * val(ldc) + (n // 2 if val(swiglu) else n), "out")
        need(ssq.tensor is None or room(ssq) >= m * val(sparts), "sums of squares in")
        need(sout.tensor is None or room(sout) >= m * ((n + 15) // 16), "sums of squares out")
        need(cout.tensor is None or room(cout) >= (m - 1) * val(ldcopy) + n, "copy")
        need(cscale.tensor is None or room(cscale) >= n, "copy scale")
    elif name == "pulse_add_rmsnorm":
        (h, delta, _, parts, part_stride, rows, w, _, y, _, n_out, hidden, _, _, _, _, _) = args
        n_out, hidden = val(n_out), val(hidden)
        last = int(rows.tensor.max()) + 1 if rows.tensor is not None else n_out
        need(room(w) >= hidden and room(y) >= n_out * hidden and room(h) >= last * hidden, "w / y / h")
        need(delta.tensor is None or room(delta) >= (val(parts) - 1) * val(part_stride) + last * hidden, "update")
    elif name == "pulse_gemm_f32":
        (a, _, w, _, c, _, m, n, k, lda, ldw, ldc, _) = args
        m, n, k = val(m), val(n), val(k)
        need(room(a) >= (m - 1) * val(lda) + k and room(w) >= (n - 1) * val(ldw) + k and room(c) >= (m - 1) * val(ldc) + n,
             "operands")
    elif name in ("pulse_gemm_mid", "pulse_gemm_rows"):
        a, ldx, w, ldw, c, ldc, m, n, k = args[:9]
        m, n, k = val(m), val(n), val(k)
        need(room(a) >= (m - 1) * val(ldx) + k and room(w) >= (n - 1) * val(ldw) + k, "operands")
        if name == "pulse_gemm_mid":
            splits, swiglu = val(args[11]), val(args[10])
            need(room(c) >= (splits - 1) * m * val(ldc) + (m - 1) * val(ldc) + (n // 2 if swiglu else n), "out")
        else:
            need(room(c) >= (m - 1) * val(ldc) + n, "out")
    elif name == "pulse_swiglu":
        gu, out, _, tokens, inter, _, _, _ = args
        need(room(gu) >= val(tokens) * 2 * val(inter) and room(out) >= val(tokens) * val(inter), "operands")
    elif name == "pulse_embed_gather":
        ids, _, _, out, tokens, hidden, _, _, _, _ = args
        need(room(out) >= val(tokens) * val(hidden) and room(ids) >= val(tokens), "operands")
    elif name == "pulse_residual_add":
        h, delta, _, parts, n, _, _ = args
        need(room(h) >= val(n) and room(delta) >= val(parts) * val(n), "operands")
    elif name != "pulse_attn_plan":
        raise AssertionError(f"an entry point that nothing verifies: {name}")


@pytest.fixture
def checked_kernels(monkeypatch):
    """Every entry point becomes the function that verifies its operands; pointers remember their tensors; library products run on the CPU."""
    from pulse_infer_amd.engine import runner as runner_module
    from pulse_infer_amd.ops import attention_mfma, kernels

    seen = []
    for module in (kernels, attention_mfma):
        monkeypatch.setattr(module, "_ptr", _ptr)
        monkeypatch.setattr(module, "_gpu", lambda *a, **k: None)
        monkeypatch.setattr(module, "_stream", lambda: ctypes.c_void_p(0))
    monkeypatch.setattr(kernels, "call", lambda name, *args, label="": (seen.append(name), check(name, args)))
    monkeypatch.setattr(attention_mfma, "call_in", lambda lib, name, *args, label="": (seen.append(name), check(name, args)))
    takes = type("Variant", (), {"pulse_attn_decode_takes": staticmethod(lambda rotary_dim, pairing: 1)})
    monkeypatch.setattr(attention_mfma, "load_variant", lambda source, defines: takes())
    plain_mm = torch.mm

    def mm(a, b, out_dtype=None, out=None):
        product = plain_mm(a.float(), b.float())
        return product if out is None else out.copy_(product)

    monkeypatch.setattr(torch, "mm", mm)

    class Staging:
        def __init__(self, device, depth=4):
            pass

        def upload(self, data):
            return torch.from_numpy(np.asarray(data, dtype=np.int32).copy())

        def upload_values(self, values):
            return self.upload(values)

    monkeypatch.setattr(runner_module, "_Staging", Staging)
    return seen


@pytest.mark.parametrize("seed", range(10))
def test_every_entry_point_stays_inside_its_tensors(checked_kernels, seed):
    from pulse_infer_amd.config import DirozenConfig
    from pulse_infer_amd.engine.runner import ModelRunner, StepEntry
    from pulse_infer_amd.models.causal_lm import expected_tensors
    from pulse_infer_amd.models.factory import build_model
    from pulse_infer_amd.weights.random_init import RandomSource

    rng = random.Random(3000 + seed)
    cfg = random_config(rng)
    page, length = rng.choice([16, 32, 64]), 70
    typed = DirozenConfig.from_dict(cfg)
    ids = token_ids(cfg["vocab"], length, seed=seed)
    _, steps = mixed_trace(cfg["vocab"], seed=seed)
    for dtype in ("float32", "bfloat16"):
        source = RandomSource(expected_tensors(typed.model_spec()), seed, 0.02, torch.bfloat16, device="cpu")
        model = build_model(typed, source, mode=dtype, device="cpu")
        runner = ModelRunner(model, page_size=page, num_pages=256 // page, max_requests=4, use_graphs=False)
        for cuts in ([length], [length - 5] + [1] * 5, [40, 2, 17, 11]):
            runner.add_request("r")
            at = 0
            for n in cuts:
                runner.reserve("r", at + n)
                runner.step([StepEntry("r", ids[at:at + n], list(range(n)))])
                at += n
            runner.free_request("r")
        for step in steps:
            entries = []
            for e in step["entries"]:
                if not runner.cache.has_request(e["id"]):
                    runner.add_request(e["id"])
                runner.reserve(e["id"], runner.cache.computed(e["id"]) + len(e["tokens"]))
                entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
            runner.step(entries)
            for k in step["end"]:
                runner.free_request(k)
        runner.cache.check()
    assert {"pulse_qk_rope_kv", "pulse_add_rmsnorm", "pulse_embed_gather"} <= set(checked_kernels)
