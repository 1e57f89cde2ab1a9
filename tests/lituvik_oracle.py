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
    freqs, mag = yarn_frequencies(int(rot.get("dims", dr)), float(rot.get("base", 10000.0)), rot.get("scaling"))
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
            s = (kn[first:i + 1, hh] @ qn + kr[first:i + 1] @ qr) * m["scale"]
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


def route(h, W, p, ml, gaps=None):
    """-> (chosen ids [T, top], weights [T, top]); ids >= experts are identity experts."""
    top = ml["router"]["top"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + W[p + "correction"]
    ids = torch.topk(choice, top, dim=-1).indices
    if gaps is not None and top < choice.shape[1]:
        srt = torch.sort(choice, -1, descending=True).values
        gaps.append(float((srt[:, top - 1] - srt[:, top]).min()))
    w = torch.gather(s, 1, ids)
    return ids, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, ml, gaps=None):
    E = ml["router"]["experts"]
    ids, w = route(h, W, p, ml, gaps)
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


def forward(cfg, W, tokens, residuals=None, gaps=None):
    """Logits [T, vocab] of one sequence (float64). W: checkpoint tensors (any float type; used as float64)."""
    W = {k: v.to(F64) for k, v in W.items()}
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
            x = x + (dense_ff(h, W, p + "mlp.") if ml["kind"] == "dense" else moe_ff(h, W, p + "mlp.", ml, gaps))
        if residuals is not None:
            residuals.append(x.clone())
    logits = dyt(x, W, "final.norm") @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


# ------------------------------------------------------------------------------------------ made-up models for tests
def att(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=10, scale=0.4, window=9, base=50.0, scaling=(3.0, 24, 4.0, 1.0),
        dims=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim if dims is None else dims))
    if window:
        m["mask"] = dict(size=window)
    if scaling:
        m["rot"]["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    return dict(type="latent_attention", mixer=m)


def lin(heads=3, dim=8, vdim=12, decay=(0.5, 0.9, 0.99)):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def ssm(inner=40, state=6, dt_rank=5, conv=3):
    return dict(type="mamba1", mixer=dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv))


def dense(layer, ff=48):
    return dict(layer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def moe(layer, ff=24, experts=5, identity=2, top=3, shared=20):
    ml = dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, identity=identity, top=top))
    if shared:
        ml["shared"] = dict(ff=shared)
    return dict(layer, mlp=ml)


def make_config(layers, width=32, vocab=97, eps=1e-5, loop=None, softcap=12.0):
    c = dict(architecture="Lituvik", vocab=vocab, width=width, norm=dict(eps=eps), layers=list(layers))
    if loop:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    if softcap:
        c["logit_softcap"] = softcap
    return c


def random_checkpoint(cfg, seed, slow_decay=False):
    """Random weights under the checkpoint's tensor names, rounded to bfloat16 (what a stored checkpoint holds), with
    magnitudes that make every mechanism matter: norm biases, sizeable rotated parts, corrections that change the
    choice of experts, decays from fast to slow."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def rn(*s, std=1.0):
        return (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()

    def un(*s, lo=0.0, hi=1.0):
        return (torch.rand(*s, generator=g) * (hi - lo) + lo).to(torch.bfloat16).float()

    def mat(o, i, gain=1.0):
        return rn(o, i, std=gain * i ** -0.5)

    W = {"embed": rn(cfg["vocab"], D), "head": mat(cfg["vocab"], D, 3.0)}

    def norm(name):
        W[name], W[name + ".b"] = un(D, lo=0.5, hi=1.5), rn(D, std=0.2)
        W[name + ".alpha"] = un(1, lo=0.4, hi=0.9).reshape(())

    def gated(p, F_):
        W[p + "gate"], W[p + "up"], W[p + "down"] = mat(F_, D, 2.0), mat(F_, D, 1.5), mat(D, F_)

    norm("final.norm")
    for i, l in enumerate(cfg["layers"]):
        p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        norm(p + "norm1")
        if l["type"] == "latent_attention":
            H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[x + "q"], W[x + "dkv"] = mat(H * (dn + dr), D, 2.0), mat(R + dr, D, 2.0)
            W[x + "dkv.norm"] = un(R, lo=0.5, hi=1.5)
            W[x + "uk"], W[x + "uv"] = mat(H * dn, R, 1.5), mat(H * dv, R)
            W[x + "o"] = mat(D, H * dv)
        elif l["type"] == "lightning":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            W[x + "q"], W[x + "k"], W[x + "v"] = mat(H * dk, D, 1.5), mat(H * dk, D, 1.5), mat(H * dv, D, 1.5)
            W[x + "g"], W[x + "o"] = mat(H * dv, D, 2.0), mat(D, H * dv)
            W[x + "norm"] = un(H * dv, lo=0.5, hi=1.5)
        else:
            I, N, rk, K = m["inner"], m["state"], m["dt_rank"], m["conv"]
            W[x + "in"] = mat(2 * I, D)
            W[x + "conv"], W[x + "conv.b"] = rn(I, K, std=0.6), rn(I, std=0.2)
            W[x + "x"] = mat(rk + 2 * N, I)
            W[x + "dt"] = mat(I, rk)
            W[x + "dt.b"] = un(I, lo=-7.0, hi=-5.0) if slow_decay else un(I, lo=-3.0, hi=0.5)
            W[x + "A_log"] = un(I, N, lo=-2.0, hi=-1.0) if slow_decay else un(I, N, lo=-1.5, hi=0.7)
            W[x + "D"] = rn(I)
            W[x + "o"] = mat(D, I)
        ml = l.get("mlp")
        if ml is None:
            continue
        norm(p + "norm2")
        if ml["kind"] == "dense":
            W[p + "mlp.up"], W[p + "mlp.down"] = mat(ml["ff"], D, 1.5), mat(D, ml["ff"])
        else:
            r = ml["router"]
            n = r["experts"] + r.get("identity", 0)
            for e in range(r["experts"]):
                gated(p + f"mlp.e{e}.", ml["expert"]["ff"])
            W[p + "mlp.router"] = mat(n, D, 3.0)
            W[p + "mlp.correction"] = rn(n, std=0.15)
            if ml.get("shared"):
                gated(p + "mlp.shared.", ml["shared"]["ff"])
    return W


def router_margin(cfg, W, tokens):
    """Smallest gap between the last chosen and the first not chosen corrected router score over all layers and
    positions (a test with a near-tie would rest on rounding)."""
    gaps = []
    forward(cfg, W, tokens, gaps=gaps)
    return min(gaps) if gaps else 1.0
