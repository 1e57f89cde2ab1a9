"""A plain, slow float64 implementation of the Vipolix decoder, written from its equations: one function per mechanism,
whole sequences at a time, no cache, no batching. It shares no code with the serving path and is what the tests compare
the framework against.

Notation: x is the residual stream [T, D]; W[name] are the checkpoint tensors (linear weights [out, in], applied as
W x); positions count from 0.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64
UNIT_EPS = 1e-6          # inside the root of the delta rule's unit key
ROUTE_EPS = 1e-20        # added to the sum of the chosen router scores
DECAY_RATE = math.exp(-0.5)
GATE_SLOPE = 1.702       # slope of the sigmoid in the experts' activation


def t64(t) -> torch.Tensor:
    return torch.as_tensor(t).to(F64)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def centred_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1 + w)


def token_shift(h, mu):
    """h_t + (h_(t-1) - h_t) * mu, with the rows as they were before the replacement; zeros before the first."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def gla_mixer(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    H, dk, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = h.shape[0]
    q = (h @ W[p + "q"].T * dk ** -0.5).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, H, dk)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=F64)
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = unit_rms(o, eps) * W[p + "norm"]
    g = h @ W[p + "g"].T
    return (o.reshape(T, H * dv) * (g * torch.sigmoid(g))) @ W[p + "o"].T


def short_conv(u, w):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j); u [T, C], w [C, taps]."""
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u])
    return sum(pad[j:j + u.shape[0]] * w[:, j] for j in range(taps))


def rotate_pairs(x, dims: int, base: float):
    """x [T, H, d]: channels (2i, 2i + 1), i < dims / 2, turned by position * base^(-2i / dims)."""
    if not dims:
        return x
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=F64)
    ang = torch.arange(T, dtype=F64)[:, None] * base ** (-2 * i / dims)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def chunk_sink_attention(h, W, p: str, m: dict):
    """GQA over the keys of the query's own chunk of positions, softmax with one added to the denominator."""
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    proj = {}
    for n in "qkv":
        y = h @ W[p + n].T + W[p + n + ".b"]
        proj[n] = short_conv(y, W[p + n + ".conv"]) if (p + n + ".conv") in W else y
    rot = m.get("rot") or {}
    q = rotate_pairs(proj["q"].view(T, H, dk), int(rot.get("dims") or 0), float(rot.get("base") or 1.0))
    k = rotate_pairs(proj["k"].view(T, G, dk), int(rot.get("dims") or 0), float(rot.get("base") or 1.0))
    v = proj["v"].view(T, G, dv)
    size = int((m.get("mask") or {}).get("size") or 0)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            lo = (i // size) * size if size else 0
            s = (k[lo:i + 1, g] @ q[i, hd]) * float(m["scale"]) * W[p + "temp"][hd]
            e = torch.exp(s)
            out[i, hd] = (e / (1 + e.sum())) @ v[lo:i + 1, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def delta_mixer(h, W, p: str, m: dict, eps: float):
    """Generalised delta rule: a decay per key channel and a removal along the unit key."""
    H, d = m["heads"], m["dim"]
    T = h.shape[0]
    r = (h @ W[p + "r"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, d)
    w = torch.exp(-DECAY_RATE * torch.sigmoid(torch.tanh(h @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).view(T, H, d)
    a = torch.sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + UNIT_EPS)
    S = torch.zeros(H, d, d, dtype=F64)
    o = torch.zeros(T, H, d, dtype=F64)
    for t in range(T):
        uS = torch.einsum("hk,hkv->hv", u[t], S)
        S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, r[t])
    o = unit_rms(o, eps).reshape(T, H * d) * W[p + "norm"]
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel_mixer(h, W, p: str, m: dict, eps: float):
    return float(m["left_scale"]) * chunk_sink_attention(h, W, p + "left.", m["left"]) + \
        float(m["right_scale"]) * delta_mixer(h, W, p + "right.", m["right"], eps)


def clamped_expert(h, W, p: str, limit: float):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(GATE_SLOPE * g) * (u + 1)) @ W[p + "down"].T


def route(h, W, p: str, r: dict):
    """-> chosen expert ids [T, top] and their weights."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ W[p + "router"].T)
    choice = s + W[p + "correction"]
    gr = r.get("groups") or {}
    n, keep = int(gr.get("count") or 1), int(gr.get("keep") or 1)
    if n > 1 and keep < n:
        per = choice.view(-1, n, E // n)
        score = per.topk(min(2, E // n), -1).values.sum(-1)
        best = score.topk(keep, -1).indices
        allowed = torch.zeros_like(score, dtype=torch.bool).scatter_(1, best, True)
        choice = torch.where(allowed[:, :, None].expand_as(per).reshape(-1, E), choice,
                             torch.full_like(choice, -math.inf))
    ids = choice.topk(top, -1).indices
    wts = s.gather(1, ids)
    wts = wts / (wts.sum(-1, keepdim=True) + ROUTE_EPS) * float(r.get("scale", 1.0))
    return ids, wts


def moe(h, W, p: str, ml: dict, all_experts: bool = False):
    r = ml["router"]
    ids, wts = route(h, W, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(r["top"]):
            e = int(ids[t, j])
            out[t] += wts[t, j] * clamped_expert(h[t:t + 1], W, p + f"e{e}.", float(ml["expert"]["limit"]))[0]
    if ml.get("shared"):
        sh = clamped_expert(h, W, p + "shared.", float(ml["shared"]["limit"]))
        out = out + sh * torch.sigmoid(h @ W[p + "shared.sg"].T)
    return out


def token_side(x, tokens, W, i: int, dim: int, eps: float):
    """The layer's own slice of a second embedding, gated by the stream, projected, normed and added."""
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e) @ W[f"l{i}.side.proj"].T
    return x + unit_rms(y, eps) * W[f"l{i}.side.norm"]


def forward(cfg: dict, sd: Dict[str, torch.Tensor], tokens: List[int], residuals: Optional[list] = None):
    """Logits [T, vocab] of one sequence; `residuals` collects the stream after every layer."""
    W = {k: t64(v) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    side = int((cfg.get("token_side") or {}).get("dim") or 0)
    x = W["embed"][tok]
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = centred_norm(x, W[p + "norm1"], eps)
        h = token_shift(h, W[p + "shift"])
        if l["type"] == "gla":
            x = x + gla_mixer(h, W, p + "mix.", l["mixer"], eps)
        else:
            x = x + parallel_mixer(h, W, p + "mix.", l["mixer"], eps)
        if l.get("mlp") is not None:
            x = x + moe(centred_norm(x, W[p + "norm2"], eps), W, p + "mlp.", l["mlp"])
        if side:
            x = token_side(x, tok, W, i, side, eps)
        if residuals is not None:
            residuals.append(x.clone())
    return centred_norm(x, W["final.norm"], eps) @ W["head"].T
