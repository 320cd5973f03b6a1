"""A plain float64 implementation of the Rupatar design, one function per mechanism, written from its equations.

Whole sequences, no cache, no batching, nothing shared with the package: the tests compare the engine with this.
``config`` is the checkpoint's config.json as a dict, ``tensors`` maps checkpoint names to arrays.

Notation: a sequence of n tokens, width W; linear weights are [out, in].
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

F64 = torch.float64


def _w(tensors, name) -> torch.Tensor:
    return tensors[name].to(F64)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """The vector in ``groups`` equal consecutive parts, each over its own root mean square, the whole times w."""
    n, W = x.shape
    return unit_rms(x.view(n, groups, W // groups), eps).reshape(n, W) * w


def rotate_pairs(x: torch.Tensor, dims: int, base: float, factor: float) -> torch.Tensor:
    """x [n, heads, d]: dimensions (2i, 2i + 1), i < dims / 2, of the token at position p turn by the angle
    p * base^(-2i / dims) / factor; the other dimensions pass."""
    n = x.shape[0]
    out = x.clone()
    if dims == 0:
        return out
    i = torch.arange(dims // 2, dtype=F64)
    freq = torch.pow(torch.tensor(base, dtype=F64), -2.0 * i / dims) / factor
    ang = torch.arange(n, dtype=F64)[:, None] * freq[None, :]          # [n, dims / 2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def visible(i: int, size: Optional[int], pool: Optional[int]) -> Tuple[List[int], List[int]]:
    """(token positions, pooled block numbers) that the query at position i sees."""
    if not size:
        return list(range(i + 1)), []
    toks = [j for j in range(i + 1) if i - j < size]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def attention(h: torch.Tensor, tensors, pre: str, m: dict, eps: float, v_first: Optional[torch.Tensor],
              round_cache=None):
    """The windowed attention mixer with pooled far blocks.  Returns (output [n, W], this layer's cached values).
    ``round_cache``: a function applied to keys and values as a cache would hold them (identity by default)."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ _w(tensors, pre + "q").T + _w(tensors, pre + "q.b")).view(n, H, D)
    k = (h @ _w(tensors, pre + "k").T + _w(tensors, pre + "k.b")).view(n, G, D)
    v = (h @ _w(tensors, pre + "v").T + _w(tensors, pre + "v.b")).view(n, G, V)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    q = unit_rms(rotate_pairs(q, dims, float(rot.get("base", 10000.0)), factor), eps)
    k = unit_rms(rotate_pairs(k, dims, float(rot.get("base", 10000.0)), factor), eps)
    if m.get("v_mix") and v_first is not None:
        lam = _w(tensors, pre + "vmix").reshape(())
        v = (1.0 - lam) * v + lam * v_first
    if round_cache is not None:
        k, v = round_cache(k), round_cache(v)
    mask = m.get("mask") or {}
    size, pool = mask.get("size"), mask.get("pool")
    out = torch.zeros(n, H, V, dtype=F64)
    for i in range(n):
        toks, blocks = visible(i, size, pool)
        ks = [k[j] for j in toks] + [k[b * pool:(b + 1) * pool].mean(0) for b in blocks]
        vs = [v[j] for j in toks] + [v[b * pool:(b + 1) * pool].mean(0) for b in blocks]
        K, Vv = torch.stack(ks), torch.stack(vs)                       # [keys, G, .]
        for hd in range(H):
            g = hd // (H // G)
            s = (K[:, g] @ q[i, hd]) * m["scale"]
            mx = torch.clamp(s.max(), min=0.0)
            e = torch.exp(s - mx)
            p = e / (torch.exp(-mx) + e.sum())                         # one more unit in the denominator
            out[i, hd] = p @ Vv[:, g]
    gate = sigmoid(h @ _w(tensors, pre + "g").T)
    y = (out.reshape(n, H * V) * gate) @ _w(tensors, pre + "o").T + _w(tensors, pre + "o.b")
    return y, v


def hgrn2(h: torch.Tensor, tensors, pre: str, m: dict, eps: float) -> torch.Tensor:
    """Gated linear recurrence whose forget gate also sets what is written."""
    n = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    z = h @ _w(tensors, pre + "q").T
    q = (z * sigmoid(z)).view(n, H, D)
    v = (h @ _w(tensors, pre + "v").T).view(n, H, V)
    low = _w(tensors, pre + "lower")
    f = (low + (1.0 - low) * sigmoid(h @ _w(tensors, pre + "f").T + _w(tensors, pre + "f.b"))).view(n, H, D)
    S = torch.zeros(H, D, V, dtype=F64)
    o = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps) * _w(tensors, pre + "norm")
    return o.reshape(n, H * V) @ _w(tensors, pre + "o").T


def mlstm(h: torch.Tensor, tensors, pre: str, m: dict, eps: float) -> torch.Tensor:
    """Matrix memory with exponential input gate, kept in range by a running maximum that starts at 0."""
    n = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ _w(tensors, pre + "q").T).view(n, H, D) / math.sqrt(D)
    k = (h @ _w(tensors, pre + "k").T).view(n, H, D)
    v = (h @ _w(tensors, pre + "v").T).view(n, H, V)
    ig = cap * torch.tanh((h @ _w(tensors, pre + "i").T + _w(tensors, pre + "i.b")) / cap)
    fr = cap * torch.tanh((h @ _w(tensors, pre + "f").T + _w(tensors, pre + "f.b")) / cap)
    fg = -torch.log1p(torch.exp(-fr))                                  # log sigmoid
    S = torch.zeros(H, D, V, dtype=F64)
    nn = torch.zeros(H, D, dtype=F64)
    mm = torch.zeros(H, dtype=F64)
    o = torch.zeros(n, H, V, dtype=F64)
    for t in range(n):
        m_new = torch.maximum(fg[t] + mm, ig[t])
        a = torch.exp(fg[t] + mm - m_new)
        b = torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        nn = a[:, None] * nn + b[:, None] * k[t]
        mm = m_new
        den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        o[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
    y = unit_rms(o, eps).reshape(n, H * V) * _w(tensors, pre + "norm") * sigmoid(h @ _w(tensors, pre + "g").T)
    return y @ _w(tensors, pre + "o").T


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def expert(x, tensors, pre: str):
    return gelu_erf(x @ _w(tensors, pre + "up").T) @ _w(tensors, pre + "down").T


def moe(h: torch.Tensor, tensors, pre: str, f: dict) -> torch.Tensor:
    """Sigmoid router; the chosen experts' scores scale the experts' inputs; a shared expert for every token."""
    E, top = f["router"]["experts"], f["router"]["top"]
    s = sigmoid(h @ _w(tensors, pre + "router").T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.argsort(s[t], descending=True, stable=True)[:top].tolist():
            out[t] += expert(s[t, e] * h[t], tensors, f"{pre}e{e}.")
    if f.get("shared"):
        out = out + expert(h, tensors, pre + "shared.")
    return out


def forward(tokens: List[int], tensors: Dict[str, torch.Tensor], config: dict, round_cache=None):
    """(logits [n, vocab], [residual stream after every layer]) in float64."""
    eps, groups = float(config["norm"]["eps"]), int(config["norm"].get("groups", 1))
    x = _w(tensors, "embed")[torch.tensor(tokens)] * float((config.get("embedding") or {}).get("scale", 1.0))
    v_first = None
    after = []
    for i, L in enumerate(config["layers"]):
        pre = f"l{i}."
        h = group_norm(x, _w(tensors, pre + "norm1"), groups, eps)
        if L["type"] == "attention":
            y, v = attention(h, tensors, pre + "mix.", L["mixer"], eps, v_first, round_cache)
            if L["mixer"].get("v_mix") and v_first is None:
                v_first = v
        elif L["type"] == "hgrn2":
            y = hgrn2(h, tensors, pre + "mix.", L["mixer"], eps)
        elif L["type"] == "mlstm":
            y = mlstm(h, tensors, pre + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        x = x + y
        if L.get("mlp"):
            x = x + moe(group_norm(x, _w(tensors, pre + "norm2"), groups, eps), tensors, pre + "mlp.", L["mlp"])
        after.append(x.clone())
    hf = group_norm(x, _w(tensors, "final.norm"), groups, eps)
    return hf @ _w(tensors, "head").T, after


def greedy(prompt: List[int], tensors, config: dict, n: int) -> List[int]:
    """n tokens of greedy continuation (the whole sequence is recomputed for every token)."""
    toks, out = list(prompt), []
    for _ in range(n):
        logits, _ = forward(toks, tensors, config)
        out.append(int(torch.argmax(logits[-1])))
        toks.append(out[-1])
    return out
