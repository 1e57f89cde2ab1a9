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
    """RMS norm with a zero-centred weight (applied as 1 + w)."""
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
    """GQA over the keys of the query's own chunk of positions, softmax whose denominator carries an extra 1."""
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


# ------------------------------------------------------------------------------------------------ made-up checkpoints
def gla(heads=2, dim=8, vdim=12, tau=6.0):
    return dict(type="gla", mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau))


def par(heads=4, kv_heads=2, dim=8, vdim=12, conv=3, chunk=11, rot=4, base=100.0, scale=0.4, rheads=2, rdim=8,
        left_scale=0.7, right_scale=1.3):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, scale=scale, mask=dict(size=chunk),
                rot=dict(base=base, dims=rot))
    return dict(type="parallel", mixer=dict(left=left, right=dict(heads=rheads, dim=rdim), left_scale=left_scale,
                                            right_scale=right_scale))


def moe_ff(layer, ff=16, experts=6, top=2, groups=3, keep=2, scale=1.4, limit=1.5, shared=24, shared_limit=2.5):
    ml = dict(kind="moe", expert=dict(ff=ff, limit=limit),
              router=dict(experts=experts, top=top, scale=scale, groups=dict(count=groups, keep=keep)))
    if shared:
        ml["shared"] = dict(ff=shared, limit=shared_limit)
    return dict(layer, mlp=ml)


def no_ff(layer):
    return dict(layer, mlp=None)


def make_config(layers, width=32, vocab=96, side=6, eps=1e-5):
    cfg = dict(architecture="Vipolix", layers=list(layers), norm=dict(eps=eps), vocab=vocab, width=width)
    if side:
        cfg["token_side"] = dict(dim=side)
    return cfg


def random_checkpoint(cfg, seed, slow_decay=False, low_rank=5):
    """bf16-representable random tensors with the checkpoint's names, sized so that every mechanism matters: biases,
    temperatures, corrections and norm weights well away from their neutral values."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).bfloat16().float()  # noqa: E731
    un = lambda *s, lo=0.0, hi=1.0: (torch.rand(*s, generator=g) * (hi - lo) + lo).bfloat16().float()  # noqa: E731
    lin = lambda o, i, gain=1.0: rn(o, i, std=gain * i ** -0.5)  # noqa: E731
    sd = {"embed": rn(V, D), "head": lin(V, D, 2.0), "final.norm": rn(D, std=0.3)}
    sdim = int((cfg.get("token_side") or {}).get("dim") or 0)
    if sdim:
        sd["side.embed"] = rn(V, len(cfg["layers"]) * sdim)
    for i, l in enumerate(cfg["layers"]):
        p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        sd[p + "norm1"], sd[p + "shift"] = rn(D, std=0.3), un(D, lo=-0.2, hi=0.9)
        if l["type"] == "gla":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            sd[x + "q"], sd[x + "k"], sd[x + "v"] = lin(H * dk, D, 2.0), lin(H * dk, D), lin(H * dv, D)
            sd[x + "g"], sd[x + "o"] = lin(H * dv, D, 1.5), lin(D, H * dv)
            sd[x + "norm"] = 1 + rn(dv, std=0.3)
            sd[x + "a1"], sd[x + "a2"] = lin(low_rank, D), lin(H * dk, low_rank, 2.0)
            sd[x + "a2.b"] = un(H * dk, lo=5.0, hi=8.0) if slow_decay else un(H * dk, lo=-1.0, hi=4.0)
        else:
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            xl, xr = x + "left.", x + "right."
            for n, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                sd[xl + n], sd[xl + n + ".b"] = lin(rows, D, 1.0 if n == "v" else 2.0), rn(rows, std=0.3)
                if a.get("conv"):
                    sd[xl + n + ".conv"] = rn(rows, a["conv"], std=0.4)
                    sd[xl + n + ".conv"][:, -1] += 1.0
            sd[xl + "temp"], sd[xl + "o"] = un(H, lo=0.5, hi=1.6), lin(D, H * dv)
            Hr, d = r["heads"], r["dim"]
            for n in ("r", "k", "v", "g", "a"):
                sd[xr + n] = lin(Hr * d, D, 1.5)
            sd[xr + "a.b"] = rn(Hr * d, std=0.7)
            sd[xr + "w1"], sd[xr + "w2"] = lin(low_rank, D, 1.5), lin(Hr * d, low_rank, 2.0)
            sd[xr + "w0"] = un(Hr * d, lo=-9.0, hi=-6.0) if slow_decay else un(Hr * d, lo=-3.0, hi=2.0)
            sd[xr + "norm"], sd[xr + "o"] = 1 + rn(Hr * d, std=0.3), lin(D, Hr * d)
        ml = l.get("mlp")
        if ml is not None:
            sd[p + "norm2"] = rn(D, std=0.3)
            q, r = p + "mlp.", ml["router"]
            for e in list(range(r["experts"])) + (["shared"] if ml.get("shared") else []):
                pre = q + (f"e{e}." if e != "shared" else "shared.")
                F_ = ml["shared"]["ff"] if e == "shared" else ml["expert"]["ff"]
                sd[pre + "gate"], sd[pre + "up"], sd[pre + "down"] = lin(F_, D, 2.0), lin(F_, D, 2.0), lin(D, F_)
            sd[q + "router"], sd[q + "correction"] = lin(r["experts"], D, 2.0), rn(r["experts"], std=0.3)
            if ml.get("shared"):
                sd[q + "shared.sg"] = lin(1, D, 2.0)
        if sdim:
            sd[p + "side.gate"], sd[p + "side.proj"] = lin(sdim, D, 1.5), lin(D, sdim)
            sd[p + "side.norm"] = rn(D, std=0.5)
    return {k: v.bfloat16().float() for k, v in sd.items()}


def router_margin(cfg, sd, tokens):
    """Smallest gap, over all positions and routed layers, between the choice scores that decide the chosen set: the
    last chosen and the first rejected expert, and the last kept and the first dropped group."""
    W = {k: t64(v) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    sdim = int((cfg.get("token_side") or {}).get("dim") or 0)
    x = W["embed"][tok]
    gap = math.inf
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = token_shift(centred_norm(x, W[p + "norm1"], eps), W[p + "shift"])
        x = x + (gla_mixer(h, W, p + "mix.", l["mixer"], eps) if l["type"] == "gla" else
                 parallel_mixer(h, W, p + "mix.", l["mixer"], eps))
        ml = l.get("mlp")
        if ml is not None:
            h = centred_norm(x, W[p + "norm2"], eps)
            r = ml["router"]
            E, top = r["experts"], r["top"]
            c = torch.sigmoid(h @ W[p + "mlp.router"].T) + W[p + "mlp.correction"]
            gr = r.get("groups") or {}
            n, keep = int(gr.get("count") or 1), int(gr.get("keep") or 1)
            if n > 1 and keep < n:
                per = c.view(-1, n, E // n)
                gs = per.topk(min(2, E // n), -1).values.sum(-1).sort(-1, descending=True).values
                gap = min(gap, float((gs[:, keep - 1] - gs[:, keep]).min()))
                ok = torch.zeros_like(gs, dtype=torch.bool).scatter_(
                    1, per.topk(min(2, E // n), -1).values.sum(-1).topk(keep, -1).indices, True)
                c = torch.where(ok[:, :, None].expand_as(per).reshape(-1, E), c, torch.full_like(c, -math.inf))
            if top < E:
                cs = c.sort(-1, descending=True).values
                d = cs[:, top - 1] - cs[:, top]
                gap = min(gap, float(d[torch.isfinite(d)].min()) if torch.isfinite(d).any() else math.inf)
            x = x + moe(h, W, p + "mlp.", ml)
        if sdim:
            x = token_side(x, tok, W, i, sdim, eps)
    return gap
