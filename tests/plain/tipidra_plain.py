"""A plain, slow Tipidra decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.
It shares no code with ``pulse_infer_amd``: it reads a model folder with ``json`` and the ``safetensors`` package
(or takes a dictionary of tensors) and is written from the design's equations.  Tests compare the engine with it.

Notation: X [S, T, W] the streams (S copies of the residual), p the position of a token (from 0 in each sequence),
W_foo a weight stored [out, in].
"""
from __future__ import annotations

import json
import math
import os
from typing import Any, Dict, List, Optional

import torch

DT = torch.float64


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w + b over the last axis; var is the mean squared deviation."""
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * w + b


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_halves(x: torch.Tensor, positions: List[int], base: float, dims: int) -> torch.Tensor:
    """Channel i < dims / 2 of every head is paired with channel i + dims / 2 and the pair turned by
    p * base^(-2i/dims); channels from dims on pass.  x [T, heads, d]."""
    out = x.clone()
    half = dims // 2
    pos = torch.tensor(positions, dtype=DT).view(-1, 1, 1)
    i = torch.arange(half, dtype=DT)
    angle = pos * (base ** (-2.0 * i / dims)).view(1, 1, -1)
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * torch.cos(angle) - v * torch.sin(angle)
    out[..., half:dims] = v * torch.cos(angle) + u * torch.sin(angle)
    return out


def capped(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap) if cap else z


def sink_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: float,
                           sink: Optional[torch.Tensor]) -> torch.Tensor:
    """Grouped causal attention of a whole sequence.  The score (q . k) scale is capped by cap tanh(. / cap); the
    softmax's denominator holds exp(sink_h) once more, for which there is no value.
    q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]."""
    t, heads, _ = q.shape
    share = heads // k.shape[1]
    out = torch.zeros(t, heads, v.shape[2], dtype=DT)
    for h in range(heads):
        g = h // share
        s = capped((q[:, h] @ k[:, g].T) * scale, cap)
        for i in range(t):
            row = s[i, : i + 1]
            top = row.max() if sink is None else torch.maximum(row.max(), sink[h])
            e = torch.exp(row - top)
            denom = e.sum() + (torch.exp(sink[h] - top) if sink is not None else 0.0)
            out[i, h] = (e / denom) @ v[: i + 1, g]
    return out


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any], eps: float,
                    positions: Optional[List[int]] = None) -> torch.Tensor:
    t = h.shape[0]
    heads, groups, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    positions = list(range(t)) if positions is None else positions
    q = (h @ w[p + ".q"].T).view(t, heads, d)
    k = (h @ w[p + ".k"].T).view(t, groups, d)
    v = (h @ w[p + ".v"].T).view(t, groups, dv)
    rot = m.get("rot")
    if rot:
        q = rotate_halves(q, positions, float(rot["base"]), int(rot["dims"]))
        k = rotate_halves(k, positions, float(rot["base"]), int(rot["dims"]))
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    sink = w.get(p + ".sink")
    o = sink_softmax_attention(q, k, v, float(m["scale"]), float(m.get("softcap") or 0.0), sink)
    o = o.reshape(t, heads * dv) * torch.sigmoid(h @ w[p + ".g"].T)
    return o @ w[p + ".o"].T


def causal_taps(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor,
                before: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[t, c] = bias[c] + sum_j taps[c, j] x[t - (K - 1) + j, c]; inputs before the start are zero (or ``before``,
    the K - 1 inputs that came last)."""
    t, c = x.shape
    k = taps.shape[1]
    pad = torch.zeros(k - 1, c, dtype=DT) if before is None else before
    full = torch.cat([pad, x], dim=0)
    y = torch.zeros(t, c, dtype=DT)
    for j in range(k):
        y += full[j:j + t] * taps[:, j]
    return y + bias


def selective_scan(x: torch.Tensor, dt: torch.Tensor, a: torch.Tensor, b: torch.Tensor, c: torch.Tensor,
                   d: torch.Tensor, state: Optional[torch.Tensor] = None):
    """S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n; y_c = sum_n S[c, n] C_n + D_c x_c, token by token.
    x, dt [T, C]; a [C, N]; b, c [T, N]; returns (y [T, C], the last state)."""
    t, ch = x.shape
    s = torch.zeros(ch, a.shape[1], dtype=DT) if state is None else state.clone()
    y = torch.zeros(t, ch, dtype=DT)
    for i in range(t):
        s = torch.exp(dt[i].view(-1, 1) * a) * s + (dt[i] * x[i]).view(-1, 1) * b[i].view(1, -1)
        y[i] = s @ c[i] + d * x[i]
    return y, s


def mamba1_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any]) -> torch.Tensor:
    inner, rank, n = m["inner"], m["dt_rank"], m["state"]
    xz = h @ w[p + ".in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_taps(x, w[p + ".conv"], w[p + ".conv.b"]))
    low = x @ w[p + ".x"].T
    dt = softplus(low[:, :rank] @ w[p + ".dt"].T + w[p + ".dt.b"])
    y, _ = selective_scan(x, dt, -torch.exp(w[p + ".A_log"]), low[:, rank:rank + n], low[:, rank + n:rank + 2 * n],
                          w[p + ".D"])
    return (y * silu(z)) @ w[p + ".o"].T


def dense_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def clamped_expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w[p + ".gate"].T, max=limit)
    u = torch.clamp(h @ w[p + ".up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + ".down"].T


def router_scores(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return torch.sigmoid(h @ w[p + ".router"].T)


def routed_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: Dict[str, Any]) -> torch.Tensor:
    """Each token goes to the ``top`` experts with the largest sigmoid scores; an expert is fed score * h and the
    experts' results are added as they are."""
    s = router_scores(h, w, p)
    top = int(m["router"]["top"])
    limit = float(m["expert"]["limit"])
    out = torch.zeros_like(h)
    chosen = torch.topk(s, top, dim=-1).indices
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += clamped_expert((s[t, e] * h[t]).view(1, -1), w, f"{p}.e{e}", limit)[0]
    return out


def read_model(folder: str):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as fh:
        for name in fh.keys():
            tensors[name] = fh.get_tensor(name)
    return config, tensors


class PlainTipidra:
    def __init__(self, config: Dict[str, Any], tensors: Dict[str, torch.Tensor]):
        self.config = config
        self.w = {k: v.to(DT) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])
        self.streams = config.get("streams")

    @classmethod
    def from_folder(cls, folder: str) -> "PlainTipidra":
        return cls(*read_model(folder))

    def mixer(self, i: int, h: torch.Tensor) -> torch.Tensor:
        entry = self.config["layers"][i]
        if entry["type"] == "attention":
            return attention_mixer(h, self.w, f"l{i}.mix", entry["mixer"], self.eps)
        if entry["type"] == "mamba1":
            return mamba1_mixer(h, self.w, f"l{i}.mix", entry["mixer"])
        raise ValueError(entry["type"])

    def feed_forward(self, i: int, h: torch.Tensor) -> torch.Tensor:
        m = self.config["layers"][i]["mlp"]
        if m["kind"] == "dense":
            return dense_feed_forward(h, self.w, f"l{i}.mlp")
        return routed_feed_forward(h, self.w, f"l{i}.mlp", m)

    def sublayer(self, i: int, q: int, x: torch.Tensor) -> torch.Tensor:
        """Sublayer q (1: mixer, 2: feed-forward) of layer i around the streams x [S, T, W] (or the one residual
        [T, W] of a model without streams)."""
        w, p = self.w, f"l{i}."
        run = (lambda n: self.mixer(i, n)) if q == 1 else (lambda n: self.feed_forward(i, n))
        norm = lambda u: layer_norm(u, w[f"{p}norm{q}"], w[f"{p}norm{q}.b"], self.eps)
        if self.streams is None:
            return x + run(norm(x))
        u = torch.einsum("s,stw->tw", w[f"{p}hc{q}.in"], x)
        y = run(norm(u))
        return torch.einsum("st,sxw->txw", w[f"{p}hc{q}.mix"], x) + w[f"{p}hc{q}.out"].view(-1, 1, 1) * y

    def layer(self, i: int, x: torch.Tensor) -> torch.Tensor:
        x = self.sublayer(i, 1, x)
        if self.config["layers"][i]["mlp"] is not None:
            x = self.sublayer(i, 2, x)
        return x

    def start(self, ids: List[int]) -> torch.Tensor:
        x = self.w["embed"][torch.tensor(ids, dtype=torch.long)] * float(self.config["embedding"]["scale"])
        return x if self.streams is None else x.unsqueeze(0).repeat(int(self.streams), 1, 1)

    def joined(self, x: torch.Tensor) -> torch.Tensor:
        return x if self.streams is None else x.sum(dim=0)

    def residuals(self, ids: List[int]) -> List[torch.Tensor]:
        """The residual (the sum of the streams) after every layer."""
        x = self.start(ids)
        out = []
        for i in range(len(self.config["layers"])):
            x = self.layer(i, x)
            out.append(self.joined(x))
        return out

    def router_margins(self, ids: List[int]) -> torch.Tensor:
        """Per position, the smallest distance over the routed layers between the last chosen score and the best one
        not chosen: where it is tiny, an implementation in reduced precision may rightly choose otherwise."""
        x = self.start(ids)
        least = torch.full((len(ids),), float("inf"), dtype=DT)
        for i, entry in enumerate(self.config["layers"]):
            x = self.sublayer(i, 1, x)
            m = entry["mlp"]
            if m is None:
                continue
            if m["kind"] == "moe":
                p = f"l{i}."
                u = x if self.streams is None else torch.einsum("s,stw->tw", self.w[p + "hc2.in"], x)
                s = router_scores(layer_norm(u, self.w[p + "norm2"], self.w[p + "norm2.b"], self.eps), self.w, p + "mlp")
                top = int(m["router"]["top"])
                if top < s.shape[1]:
                    ranked = torch.sort(s, dim=-1, descending=True).values
                    least = torch.minimum(least, ranked[:, top - 1] - ranked[:, top])
            x = self.sublayer(i, 2, x)
        return least

    def logits(self, ids: List[int]) -> torch.Tensor:
        x = self.residuals(ids)[-1]
        z = layer_norm(x, self.w["final.norm"], self.w["final.norm.b"], self.eps) @ self.w["head"].T
        return capped(z, float(self.config.get("logit_softcap") or 0.0))

    def greedy(self, prompt: List[int], steps: int) -> List[int]:
        ids, out = list(prompt), []
        for _ in range(steps):
            nxt = int(torch.argmax(self.logits(ids)[-1]))
            out.append(nxt)
            ids.append(nxt)
        return out
