"""A plain, slow Fosupel decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.
It shares no code with ``pulse_infer_amd``: it reads a model folder with ``json`` and the ``safetensors`` package
(or takes a dictionary of tensors) and is written from the design's equations.  Tests compare the engine with it.

Notation: x [T, W] the stream, p the position of a token (from 0 in each sequence), W_foo a weight stored [out, in].
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Dict, List, Optional

import torch

DT = torch.float64


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z / 2; else (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    a, b = softplus(pq[0]), 0.5 + softplus(pq[1])
    pos = a * z * z + 0.5 * z
    neg = b * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def turn(x: torch.Tensor, positions: List[int], base: float, dims: int, pairing: str, divide: float = 1.0) -> torch.Tensor:
    """The first ``dims`` channels of every head turned by p * base^(-2i/dims) / divide; x [T, heads, d].
    ``pairing`` "half": channel i with i + dims/2; "adjacent": 2i with 2i+1."""
    out = x.clone()
    pos = torch.tensor(positions, dtype=DT).view(-1, 1, 1)
    i = torch.arange(dims // 2, dtype=DT)
    angle = pos * (base ** (-2.0 * i / dims) / divide).view(1, 1, -1)
    c, s = torch.cos(angle), torch.sin(angle)
    if pairing == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def visible(t: int, size: Optional[int], keep_first: int) -> torch.Tensor:
    """[T, T] bool: i sees j if j <= i and (i - j < size or j < keep_first); no size: every j <= i."""
    i = torch.arange(t).view(-1, 1)
    j = torch.arange(t).view(1, -1)
    near = (i - j < size) if size is not None else torch.ones(t, t, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def weights_with_sink(scores: torch.Tensor, mask: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """Softmax over the visible keys of scores [H, T, T] whose denominator holds exp(sink_h) once more."""
    s = scores.masked_fill(~mask.unsqueeze(0), float("-inf"))
    top = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.view(-1, 1, 1))
    e = torch.exp(s - top)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.view(-1, 1, 1) - top)
    return e / den


def talking_window_attention(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any],
                             positions: List[int]) -> torch.Tensor:
    """Grouped softmax attention with a rotation of half-paired channels, a window that keeps the first tokens, a sink
    and the heads' weights mixed by a matrix before they meet the values."""
    t, heads, groups, d, dv = x.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[p + ".q"].T).view(t, heads, d)
    k = (x @ w[p + ".k"].T).view(t, groups, d)
    v = (x @ w[p + ".v"].T).view(t, groups, dv)
    rot = m.get("rot")
    if rot:
        divide = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = turn(q, positions, rot["base"], rot["dims"], "half", divide)
        k = turn(k, positions, rot["base"], rot["dims"], "half", divide)
    per = heads // groups
    scores = torch.stack([q[:, h] @ k[:, h // per].T for h in range(heads)]) * m["scale"]
    mask = m.get("mask") or {}
    a = weights_with_sink(scores, visible(t, mask.get("size"), mask.get("keep_first", 0)),
                          w[p + ".sink"] if p + ".sink" in w else None)
    if p + ".talk" in w:
        a = torch.einsum("hg,gij->hij", w[p + ".talk"], a)
    o = torch.stack([a[h] @ v[:, h // per] for h in range(heads)], dim=1)
    return o.reshape(t, heads * dv) @ w[p + ".o"].T


def retention_walk(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: List[float]) -> torch.Tensor:
    """Per head, token by token: S <- decay_h S + k_t v_t^T, o_t = S^T q_t, S zero at the start."""
    t, heads, d = q.shape
    dv = v.shape[2]
    out = torch.zeros(t, heads, dv, dtype=DT)
    for h in range(heads):
        s = torch.zeros(d, dv, dtype=DT)
        for i in range(t):
            s = decay[h] * s + torch.outer(k[i, h], v[i, h])
            out[i, h] = s.T @ q[i, h]
    return out


def retention(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], positions: List[int],
              eps: float, sizes: Optional[list] = None) -> torch.Tensor:
    """``sizes`` collects the root mean square of every head's output before it is divided by it, [T, heads]."""
    t, heads, d, dv = x.shape[0], m["heads"], m["dim"], m["vdim"]
    q = (x @ w[p + ".q"].T).view(t, heads, d)
    k = (x @ w[p + ".k"].T).view(t, heads, d)
    v = (x @ w[p + ".v"].T).view(t, heads, dv)
    rot = m.get("rot")
    if rot:
        q = turn(q, positions, rot["base"], rot["dims"], "half")
        k = turn(k, positions, rot["base"], rot["dims"], "half")
    k = k * d ** -0.5
    o = retention_walk(q, k, v, m["decay"])
    if sizes is not None:
        sizes.append((o * o).mean(dim=-1).sqrt())
    o = unit_rms(o, eps)
    return (o.reshape(t, heads * dv) * silu(x @ w[p + ".g"].T)) @ w[p + ".o"].T


def parallel_mixer(x, w, p, m, positions, eps, sizes=None):
    return (m["left_scale"] * talking_window_attention(x, w, p + ".left", m["left"], positions)
            + m["right_scale"] * retention(x, w, p + ".right", m["right"], positions, eps, sizes))


def latent_attention(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], positions: List[int],
                     eps: float) -> torch.Tensor:
    """Keys and values come from one normed latent row a token; one turned key part is shared by all heads."""
    t, heads, d, dr, dv, rank = x.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (x @ w[p + ".q"].T).view(t, heads, d + dr)
    down = x @ w[p + ".dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[p + ".dkv.norm"]
    rot = m["rot"]
    k_turned = turn(down[:, rank:].view(t, 1, dr), positions, rot["base"], dr, "adjacent")[:, 0]
    q_turned = turn(q[:, :, d:], positions, rot["base"], dr, "adjacent")
    k_plain = (c @ w[p + ".uk"].T).view(t, heads, d)
    v = (c @ w[p + ".uv"].T).view(t, heads, dv)
    scores = torch.stack([q[:, h, :d] @ k_plain[:, h].T + q_turned[:, h] @ k_turned.T for h in range(heads)]) * m["scale"]
    a = weights_with_sink(scores, visible(t, None, 0), w[p + ".sink"] if p + ".sink" in w else None)
    o = torch.stack([a[h] @ v[:, h] for h in range(heads)], dim=1).reshape(t, heads * dv)
    return (o * torch.sigmoid(x @ w[p + ".g"].T)) @ w[p + ".o"].T


def gated_expert(x, w, p):
    return (silu(x @ w[p + ".gate"].T) * (x @ w[p + ".up"].T)) @ w[p + ".down"].T


def router_scores(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return torch.softmax(x @ w[p + ".router"].T, dim=-1)


def feed_forward(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any]) -> torch.Tensor:
    if m["kind"] == "dense":
        return xielu(x @ w[p + ".up"].T, w[p + ".act"]) @ w[p + ".down"].T
    s = router_scores(x, w, p)
    chosen = torch.topk(s, m["router"]["top"], dim=-1).indices
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in chosen[t].tolist():
            out[t] += s[t, e] * gated_expert(x[t:t + 1], w, f"{p}.e{e}")[0]
    if m.get("shared"):
        out = out + torch.sigmoid(x @ w[p + ".shared.sg"].T) * gated_expert(x, w, p + ".shared")
    return out


def router_margins(cfg: Dict[str, Any], w: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """Per position the smallest gap, over all routed layer runs, between the last chosen score and the first one left
    out (inf for a model without routers): where it is tiny a bfloat16 run may choose differently."""
    gaps: List[torch.Tensor] = []
    forward(cfg, w, tokens, margins=gaps)
    if not gaps:
        return torch.full((len(tokens),), float("inf"), dtype=DT)
    return torch.stack(gaps).min(dim=0).values


def layer_order(cfg: Dict[str, Any]) -> List[tuple]:
    """(layer, number of the pass if it is the first layer of a pass of the loop, else None) in the order of running."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        out += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return out + [(i, None) for i in range(loop["stop"], n)]


def fragile_positions(cfg: Dict[str, Any], w: Dict[str, torch.Tensor], tokens: List[int], above: float = 4.0) -> set:
    """Positions whose logits hang on cancellations: where these same equations evaluated in float32 stray from their
    float64 values ``above`` times further than at the median position.  (A retention head's output is divided by its
    own root mean square; where that output is small by chance, the division multiplies whatever rounding left in it,
    in any arithmetic, and no bound that holds elsewhere says anything there.)"""
    global DT
    exact = forward(cfg, w, tokens)
    DT = torch.float32
    try:
        rough = forward(cfg, w, tokens).to(torch.float64)
    finally:
        DT = torch.float64
    err = (rough - exact).abs().max(dim=1).values
    return set((err > above * err.median()).nonzero().flatten().tolist())


def forward(cfg: Dict[str, Any], w: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None,
            margins: Optional[list] = None, sizes: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; ``residuals`` collects the stream after every layer run."""
    w = {k: v.to(DT) for k, v in w.items()}
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens)]
    for i, step in layer_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}"
        if step is not None:
            x = x + w["loop.step"][step]
        n = unit_rms(x, eps) * w[p + ".norm1"]
        if layer["type"] == "parallel":
            x = x + mult * parallel_mixer(n, w, p + ".mix", layer["mixer"], positions, eps, sizes)
        elif layer["type"] == "latent_attention":
            x = x + mult * latent_attention(n, w, p + ".mix", layer["mixer"], positions, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            n = unit_rms(x, eps) * w[p + ".norm2"]
            if margins is not None and layer["mlp"]["kind"] == "moe":
                s = torch.sort(router_scores(n, w, p + ".mlp"), dim=-1, descending=True).values
                top = layer["mlp"]["router"]["top"]
                margins.append(s[:, top - 1] - s[:, top] if s.shape[1] > top else torch.full((len(tokens),), float("inf"), dtype=DT))
            x = x + mult * feed_forward(n, w, p + ".mlp", layer["mlp"])
        if residuals is not None:
            residuals.append(x.clone())
    z = (unit_rms(x, eps) * w["final.norm"]) @ w["embed"].T
    cap = cfg.get("logit_softcap", 0.0)
    return cap * torch.tanh(z / cap) if cap else z


def load_folder(path: str):
    from safetensors.torch import load_file

    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    w: Dict[str, torch.Tensor] = {}
    for name in sorted(os.listdir(path)):
        if name.endswith(".safetensors"):
            w.update(load_file(os.path.join(path, name)))
    return cfg, w


class PlainFosupel:
    """The functions above behind the few calls the tests make."""

    def __init__(self, cfg: Dict[str, Any], weights: Dict[str, torch.Tensor]):
        self.cfg = cfg
        self.w = {k: v.to(DT) for k, v in weights.items()}

    @classmethod
    def from_folder(cls, path: str) -> "PlainFosupel":
        return cls(*load_folder(path))

    def logits(self, ids: List[int]) -> torch.Tensor:
        return forward(self.cfg, self.w, list(ids))

    def residuals(self, ids: List[int]) -> List[torch.Tensor]:
        out: List[torch.Tensor] = []
        forward(self.cfg, self.w, list(ids), residuals=out)
        return out

    def router_margins(self, ids: List[int]) -> torch.Tensor:
        return router_margins(self.cfg, self.w, list(ids))

    def fragile_positions(self, ids: List[int]) -> set:
        return fragile_positions(self.cfg, self.w, list(ids))

    def greedy(self, prompt: List[int], new: int) -> List[int]:
        ids, out = list(prompt), []
        for _ in range(new):
            token = int(self.logits(ids)[-1].argmax())
            out.append(token)
            ids.append(token)
        return out
