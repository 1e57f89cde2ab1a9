"""Slow float64 oracle of the Lituvik decoder, written from its equations: one function per mechanism, whole sequences
at once, plain loops over tokens, heads and keys. It shares no code with the framework (no ops, no engine, no model
class); it reads the checkpoint layout (tensor names) and the config dictionary only.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(x, W, name):
    """Dynamic tanh: a norm without statistics."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def yarn_frequencies(dims, base, sc):
    """Per pair i < dims / 2: the angle step per position, and the common magnitude of cos and sin."""
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(v, pos, freqs, mag):
    """v [..., dims] at position pos; pair (i, i + dims / 2)."""
    half = len(freqs)
    out = v.clone()
    for i in range(half):
        a = pos * freqs[i]
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, w = v[..., i], v[..., i + half]
        out[..., i] = u * c - w * s
        out[..., i + half] = w * c + u * s
    return out


def latent_attention(h, W, p, m, eps):
    """Attention whose keys and values are expanded from one low-rank latent per token plus one rotated key part that
    all heads share; sliding window; softmax."""
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    freqs, mag = yarn_frequencies(dr, float(rot.get("base", 10000.0)), rot.get("scaling"))
    win = int((m.get("mask") or {}).get("size") or 0)
    q = (h @ W[p + "q"].T).reshape(T, H, dn + dr)
    low = h @ W[p + "dkv"].T
    c = rms_div(low[:, :R], eps) * W[p + "dkv.norm"]
    kr = torch.stack([rotate(low[t, R:], t, freqs, mag) for t in range(T)])
    kn = (c @ W[p + "uk"].T).reshape(T, H, dn)
    v = (c @ W[p + "uv"].T).reshape(T, H, dv)
    heads = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        first = max(0, i - win + 1) if win > 0 else 0
        for hh in range(H):
            qn, qr = q[i, hh, :dn], rotate(q[i, hh, dn:], i, freqs, mag)
            s = torch.stack([(qn @ kn[j, hh] + qr @ kr[j]) * m["scale"] for j in range(first, i + 1)])
            a = torch.softmax(s, 0)
            heads[i, hh] = (a[:, None] * v[first:i + 1, hh]).sum(0)
    return heads.reshape(T, H * dv) @ W[p + "o"].T


def lightning(h, W, p, m, eps):
    """Linear attention with one constant decay per head, a whole-row norm and a sigmoid gate."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).reshape(T, H, dk)
    k = silu(h @ W[p + "k"].T).reshape(T, H, dk)
    v = silu(h @ W[p + "v"].T).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = float(m["decay"][hh]) * S + k[t, hh][:, None] * v[t, hh][None, :]
            out[t, hh] = S.T @ q[t, hh]
    y = rms_div(out.reshape(T, H * dv), eps) * W[p + "norm"]
    return (y * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column = the current token), zeros before the start."""
    T, C = x.shape
    K = w.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=F64), x])
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for i in range(K):
            y[t] += pad[t + i] * w[:, i]
    return y + b


def selective_scan(h, W, p, m):
    """State-space layer with one decay per channel AND state element, all driven by the input."""
    T = h.shape[0]
    I, N, rk = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[p + "in"].T
    x = silu(causal_conv(xz[:, :I], W[p + "conv"], W[p + "conv.b"]))
    z = xz[:, I:]
    low = x @ W[p + "x"].T
    dt = softplus(low[:, :rk] @ W[p + "dt"].T + W[p + "dt.b"])        # [T, I]
    B, C = low[:, rk:rk + N], low[:, rk + N:]
    A = -torch.exp(W[p + "A_log"])                                      # [I, N]
    S = torch.zeros(I, N, dtype=F64)
    y = torch.zeros(T, I, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + W[p + "D"] * x[t]
    return (y * silu(z)) @ W[p + "o"].T


def dense_ff(h, W, p):
    return (torch.relu(h @ W[p + "up"].T) ** 2) @ W[p + "down"].T


def gated_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, ml):
    """-> (chosen ids [T, top], weights [T, top]); ids >= experts are identity experts."""
    top = ml["router"]["top"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + W[p + "correction"]
    ids = torch.topk(choice, top, dim=-1).indices
    w = torch.gather(s, 1, ids)
    return ids, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, ml):
    E = ml["router"]["experts"]
    ids, w = route(h, W, p, ml)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            y = gated_expert(h[t:t + 1], W, p + f"e{e}.")[0] if e < E else h[t]
            out[t] += w[t, j] * y
    if ml.get("shared"):
        out = out + gated_expert(h, W, p + "shared.")
    return out


def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {}
    times = int(lp.get("times", 0))
    if not times:
        return [(i, 0) for i in range(n)]
    a, b = int(lp["start"]), int(lp["stop"])
    return [(i, 0) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)] + \
        [(i, 0) for i in range(b, n)]


def forward(cfg, W, tokens, residuals=None):
    """Logits [T, vocab] of one sequence (float64). W: checkpoint tensors as float64."""
    eps = float(cfg["norm"]["eps"])
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    lp = cfg.get("loop") or {}
    for i, t in layer_runs(cfg):
        if t > 0 and i == int(lp["start"]):
            x = x + x0
        l = cfg["layers"][i]
        p = f"l{i}."
        h = dyt(x, W, p + "norm1")
        if l["type"] == "latent_attention":
            x = x + latent_attention(h, W, p + "mix.", l["mixer"], eps)
        elif l["type"] == "lightning":
            x = x + lightning(h, W, p + "mix.", l["mixer"], eps)
        elif l["type"] == "mamba1":
            x = x + selective_scan(h, W, p + "mix.", l["mixer"])
        else:
            raise ValueError(l["type"])
        ml = l.get("mlp")
        if ml is not None:
            h = dyt(x, W, p + "norm2")
            x = x + (dense_ff(h, W, p + "mlp.") if ml["kind"] == "dense" else moe_ff(h, W, p + "mlp.", ml))
        if residuals is not None:
            residuals.append(x.clone())
    logits = dyt(x, W, "final.norm") @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
