"""Plain, slow float64 implementation of the Putulorn design: one function per mechanism, whole sequences only (no
cache, no state carried between calls, no batching), written from the design's equations.  It is the oracle of
tests/test_putulorn*.py and shares no code with the framework's model, ops or kernels.

Inputs: the configuration in its config.json form (a dict) and a dict name -> tensor with the checkpoint's names.
"""

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def block_norm(x, w, eps):
    """Norm of a block: weight stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def tanh_gelu(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def wkv_mixer(P, pre, mc, eps, h):
    """Recurrent mixer over one whole sequence h [T, width]."""
    T, width = h.shape
    H, D = mc["heads"], mc["dim"]
    before = torch.cat([torch.zeros(1, width, dtype=F64), h[:-1]])

    def lerp(s):
        return h + (before - h) * P[pre + "mu." + s]

    r = lerp("r") @ P[pre + "r"].T
    k = lerp("k") @ P[pre + "k"].T
    v = lerp("v") @ P[pre + "v"].T
    gate = lerp("g") @ P[pre + "g"].T
    gate = gate * torch.sigmoid(gate)
    decay = torch.exp(-torch.exp(torch.tanh(lerp("w") @ P[pre + "w1"].T) @ P[pre + "w2"].T + P[pre + "w0"]))
    bonus = P[pre + "u"].reshape(H, D)
    y = torch.zeros(T, H * D, dtype=F64)
    for hd in range(H):
        cols = slice(hd * D, (hd + 1) * D)
        S = torch.zeros(D, D, dtype=F64)
        for t in range(T):
            outer = k[t, cols].reshape(D, 1) * v[t, cols].reshape(1, D)
            o = (S + bonus[hd].reshape(D, 1) * outer).T @ r[t, cols]
            S = decay[t, cols].reshape(D, 1) * S + outer
            y[t, cols] = unit_rms(o, eps)
    return (y * P[pre + "norm"] * gate) @ P[pre + "o"].T


def rotate(x, positions, dims, base):
    """Rotate-half rotary embedding on the first `dims` entries of the last axis; x [T, ..., n]."""
    if dims == 0:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = positions.to(F64).reshape(-1, *([1] * (x.dim() - 1))) * freq
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang), x[..., dims:]], -1)


def latent_attention_mixer(P, pre, mc, eps, h):
    T = h.shape[0]
    H, Dn, R, V, C = mc["heads"], mc["dim"], mc["rot_dim"], mc["vdim"], mc["kv_rank"]
    rot = mc.get("rot") or {}
    dims, base = rot.get("dims", R), rot.get("base", 10000.0)
    window = (mc.get("mask") or {}).get("size")
    scale = mc.get("scale", 1.0 / math.sqrt(Dn + R))
    positions = torch.arange(T)
    q = (h @ P[pre + "q"].T).reshape(T, H, Dn + R)
    q_plain, q_rot = q[..., :Dn], rotate(q[..., Dn:], positions, dims, base)
    down = h @ P[pre + "dkv"].T
    latent = unit_rms(down[:, :C], eps) * P[pre + "dkv.norm"]
    k_rot = rotate(down[:, C:], positions, dims, base)                    # one per token, all heads
    k_plain = (latent @ P[pre + "uk"].T).reshape(T, H, Dn)
    val = (latent @ P[pre + "uv"].T).reshape(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for i in range(T):
        first = 0 if not window else max(0, i - window + 1)
        for hd in range(H):
            s = (k_plain[first:i + 1, hd] @ q_plain[i, hd] + k_rot[first:i + 1] @ q_rot[i, hd]) * scale
            out[i, hd] = torch.softmax(s, 0) @ val[first:i + 1, hd]
    return out.reshape(T, H * V) @ P[pre + "o"].T


def expert_ff(P, pre, limit, h):
    g = h @ P[pre + "gate"].T
    u = h @ P[pre + "up"].T
    if limit:
        g = torch.clamp(g, max=limit)
        u = torch.clamp(u, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ P[pre + "down"].T


def dense_ff(P, pre, h):
    return (tanh_gelu(h @ P[pre + "gate"].T) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def expert_mixture(P, pre, fc, h):
    rc = fc["router"]
    score = torch.softmax(h @ P[pre + "router"].T, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = sorted(range(rc["experts"]), key=lambda e: (-float(score[t, e]), e))[:rc["top"]]
        total = sum(score[t, e] for e in chosen) + 1e-20
        for e in chosen:
            out[t] += score[t, e] / total * rc.get("scale", 1.0) * \
                expert_ff(P, f"{pre}e{e}.", fc["expert"].get("limit"), h[t:t + 1])[0]
    if fc.get("shared"):
        sh = expert_ff(P, pre + "shared.", fc["shared"].get("limit"), h)
        if pre + "shared.sg" in P:
            sh = sh * torch.sigmoid(h @ P[pre + "shared.sg"].reshape(-1, 1))
        out = out + sh
    return out


def layer_order(cfg):
    """[(layer, loop pass at whose start the layer stands, or None)]"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, tensors, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence; `streams` (a list) receives the residual stream after every layer run."""
    P = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    m = cfg.get("residual_mult", 1.0)
    x = P["embed"][torch.tensor(tokens)]
    for i, t in layer_order(cfg):
        L = cfg["layers"][i]
        if t is not None:
            x = x + P["loop.step"][t]
        mixer = wkv_mixer if L["type"] == "wkv" else latent_attention_mixer
        x = x + m * mixer(P, f"l{i}.mix.", L["mixer"], eps, block_norm(x, P[f"l{i}.norm1"], eps))
        if L.get("mlp"):
            h = block_norm(x, P[f"l{i}.norm2"], eps)
            x = x + m * (dense_ff(P, f"l{i}.mlp.", h) if L["mlp"]["kind"] == "dense"
                         else expert_mixture(P, f"l{i}.mlp.", L["mlp"], h))
        if streams is not None:
            streams.append(x.clone())
    return block_norm(x, P["final.norm"], eps) @ P["head"].T


def greedy(cfg, tensors, tokens, n):
    """n greedy tokens after `tokens`, each from a full forward of the sequence so far."""
    seq = list(tokens)
    for _ in range(n):
        seq.append(int(forward(cfg, tensors, seq)[-1].argmax()))
    return seq[len(tokens):]
