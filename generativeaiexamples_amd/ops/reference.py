"""Plain-PyTorch fp32 reference implementations of every native op.

These define the semantics the HIP kernels are tested against (tests compare the
gfx950 kernels with these on random inputs) and they are the execution path for
CPU tensors (BASELINE config 1, the CPU plumbing config, and the CPU test tier).
Layouts are identical to the native ones:

* paged K cache  ``[num_blocks, Hkv, 16, D]``
* paged V^T cache ``[num_blocks, Hkv, D, 16]``
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

BLOCK = 16


def rms_norm(x, w, eps, residual=None):
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


def layer_norm(x, w, b, eps, residual=None):
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    y = F.layer_norm(x.float(), (x.shape[-1],), w.float(), None if b is None else b.float(), eps)
    return y.to(x.dtype)


def linear(x, w, bias=None, residual=None, act=None, out_dtype=None):
    """y = act(x @ w^T + bias) + residual; act in {None, 'gelu', 'relu', 'quick_gelu', 'swiglu'}.

    'swiglu' expects w interleaved per 16 rows [gate16 | up16 | ...] (see
    ``interleave_gate_up``) and returns width N/2.
    """
    y = x.float() @ w.float().t()
    if bias is not None:
        y = y + bias.float()
    if act == "gelu":
        y = F.gelu(y)
    elif act == "relu":
        y = F.relu(y)
    elif act == "quick_gelu":
        y = y * torch.sigmoid(1.702 * y)
    elif act == "gelu_tanh":
        y = F.gelu(y, approximate="tanh")
    elif act in ("swiglu", "geglu"):
        n = y.shape[-1]
        y4 = y.reshape(*y.shape[:-1], n // 32, 2, 16)
        g = F.silu(y4[..., 0, :]) if act == "swiglu" else F.gelu(y4[..., 0, :], approximate="tanh")
        y = (g * y4[..., 1, :]).reshape(*y.shape[:-1], n // 2)
    if residual is not None:
        y = y + residual.float()
    return y.to(out_dtype or x.dtype)


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """[I, K] gate and up -> [2I, K] with rows interleaved per 16 (the fused SwiGLU GEMM layout)."""
    I, K = gate.shape
    assert I % 16 == 0
    return torch.stack([gate.reshape(I // 16, 16, K), up.reshape(I // 16, 16, K)], 1).reshape(2 * I, K)


def rope_cos_sin(max_pos: int, head_dim: int, theta: float = 500000.0, scaling: dict | None = None,
                 device=None) -> torch.Tensor:
    """fp32 table [max_pos, D] = [cos(D/2) | sin(D/2)], neox rotate-half convention.

    ``scaling`` implements the Llama-3.1 frequency-dependent rope scaling
    ({"factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings"}).
    """
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if scaling:
        factor = scaling.get("factor", 8.0)
        lf, hf = scaling.get("low_freq_factor", 1.0), scaling.get("high_freq_factor", 4.0)
        old = scaling.get("original_max_position_embeddings", 8192)
        low_wl, high_wl = old / lf, old / hf
        wl = 2 * math.pi / inv
        smooth = (old / wl - lf) / (hf - lf)
        scaled = torch.where(wl > low_wl, inv / factor, inv)
        mid = (wl <= low_wl) & (wl >= high_wl)
        inv = torch.where(mid, (1 - smooth) * inv / factor + smooth * inv, scaled)
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv)
    return torch.cat([f.cos(), f.sin()], -1).float().to(device)


def _to_cache(x, cache, scale):
    """Values -> cache dtype; fp8 caches hold x / scale saturated to the e4m3fn range (like the kernel)."""
    if cache.dtype == torch.float8_e4m3fn:
        return (x.float() / scale).clamp(-448.0, 448.0).to(cache.dtype)
    return x.to(cache.dtype)


def _from_cache(x, scale):
    return x.float() * scale if x.dtype == torch.float8_e4m3fn else x.float()


def rope_kv_write(qkv, positions, cos_sin, slots, q_out, k_cache, v_cache, Hq, Hkv, D, rope=True, k_scale=1.0,
                  v_scale=1.0):
    T = qkv.shape[0]
    x = qkv.view(T, Hq + 2 * Hkv, D).float()
    q, k, v = x[:, :Hq], x[:, Hq:Hq + Hkv], x[:, Hq + Hkv:]
    if rope:
        cs = cos_sin[positions.long()]
        c, s = cs[:, None, : D // 2], cs[:, None, D // 2:]

        def rot(t):
            t = t.to(qkv.dtype).float()  # kernel rounds inputs to bf16 first (they already are)
            a, b = t[..., : D // 2], t[..., D // 2:]
            return torch.cat([a * c - b * s, b * c + a * s], -1)

        q, k = rot(q), rot(k)
    q_out.copy_(q.to(q_out.dtype).reshape(q_out.shape))
    valid = slots >= 0
    if valid.any():
        sl = slots[valid].long()
        blk, off = sl // BLOCK, sl % BLOCK
        # the kernel rounds k (after RoPE) and v to bf16 before an fp8 conversion
        k_cache[blk, :, off, :] = _to_cache(k[valid].to(qkv.dtype), k_cache, k_scale)
        v_cache[blk, :, :, off] = _to_cache(v[valid].to(qkv.dtype), v_cache, v_scale)


def gather_kv(k_cache, v_cache, block_table, n):
    """-> K [n, Hkv, D], V [n, Hkv, D] for the first n tokens of a sequence."""
    nb = (n + BLOCK - 1) // BLOCK
    blocks = block_table[:nb].long()
    k = k_cache[blocks].permute(0, 2, 1, 3).reshape(nb * BLOCK, k_cache.shape[1], k_cache.shape[3])[:n]
    v = v_cache[blocks].permute(0, 3, 1, 2).reshape(nb * BLOCK, v_cache.shape[1], v_cache.shape[2])[:n]
    return k, v


def attention_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale, causal=True, return_lse=False,
                      k_scale=1.0, v_scale=1.0):
    """q [Tq, Hq, D]; per sequence b the queries are the last q_len positions of ctx_lens[b] keys.
    return_lse: also return the fp32 [Tq, Hq] natural-log softmax normalisers (-1e30 for empty rows)."""
    out = torch.empty_like(q)
    lse = torch.full(q.shape[:2], -1e30, dtype=torch.float32, device=q.device)
    Hq = q.shape[1]
    Hkv = k_cache.shape[1]
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        n = int(ctx_lens[b])
        k, v = gather_kv(k_cache, v_cache, block_tables[b], n)
        k = _from_cache(k, k_scale).repeat_interleave(Hq // Hkv, dim=1)
        v = _from_cache(v, v_scale).repeat_interleave(Hq // Hkv, dim=1)
        qq = q[s:e].float()
        att = torch.einsum("qhd,khd->hqk", qq, k) * scale
        if causal:
            qpos = torch.arange(n - (e - s), n, device=q.device)
            mask = torch.arange(n, device=q.device)[None, :] > qpos[:, None]
            att = att.masked_fill(mask[None], float("-inf"))
        p = att.softmax(-1)
        out[s:e] = torch.einsum("hqk,khd->qhd", p, v).to(q.dtype)
        lse[s:e] = torch.logsumexp(att, -1).transpose(0, 1)
    return (out, lse) if return_lse else out


def attention_decode(q, k_cache, v_cache, block_tables, ctx_lens, scale, k_scale=1.0, v_scale=1.0):
    """q [B, Hq, D], one token per sequence attending to its ctx_lens[b] cached keys."""
    B = q.shape[0]
    cu = torch.arange(B + 1, dtype=torch.int32)
    return attention_prefill(q, k_cache, v_cache, block_tables, cu, ctx_lens, scale, causal=True, k_scale=k_scale,
                             v_scale=v_scale)


def attention_dense(q, k, v, cu_seqlens, scale, causal):
    """Contiguous varlen attention (encoders): q/k/v [T, H, D] (k/v may have fewer heads)."""
    out = torch.empty_like(q)
    cu = cu_seqlens.tolist()
    rep = q.shape[1] // k.shape[1]
    for b in range(len(cu) - 1):
        s, e = cu[b], cu[b + 1]
        qq, kk, vv = q[s:e].float(), k[s:e].float(), v[s:e].float()
        kk, vv = kk.repeat_interleave(rep, 1), vv.repeat_interleave(rep, 1)
        att = torch.einsum("qhd,khd->hqk", qq, kk) * scale
        if causal:
            n = e - s
            att = att.masked_fill(torch.ones(n, n, dtype=torch.bool, device=q.device).triu(1)[None], float("-inf"))
        out[s:e] = torch.einsum("hqk,khd->qhd", att.softmax(-1), vv).to(q.dtype)
    return out


def sample(logits, temperature, top_p, top_k, seeds, step, generator=None):
    """Reference sampler (distributionally equivalent to the kernel, not bit-identical)."""
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int32, device=logits.device)
    for i in range(B):
        x = logits[i].float()
        T = float(temperature[i])
        if T <= 0:
            out[i] = int(torch.argmax(x))
            continue
        x = x / T
        k = int(top_k[i])
        if 0 < k < V:
            kth = torch.topk(x, k).values[-1]
            x = x.masked_fill(x < kth, float("-inf"))
        p = float(top_p[i])
        if p < 1.0:
            probs = x.softmax(-1)
            sp, si = probs.sort(descending=True)
            cum = sp.cumsum(0)
            keep = (cum - sp) < p
            thr = sp[keep].min()
            x = x.masked_fill(probs < thr, float("-inf"))
        g = torch.Generator(device="cpu")
        g.manual_seed((int(seeds[i]) * 1000003 + int(step)) & 0x7FFFFFFFFFFFFFFF)
        probs = x.softmax(-1).cpu()
        out[i] = int(torch.multinomial(probs, 1, generator=g))
    return out


def token_mask(logits, rows, mask):
    V = logits.shape[1]
    bits = (mask.long().unsqueeze(-1) >> torch.arange(32, device=mask.device)) & 1  # [R, W, 32]
    allowed = bits.reshape(mask.shape[0], -1)[:, :V].bool()
    for r, row in enumerate(rows.tolist()):
        logits[row] = torch.where(allowed[r], logits[row], torch.full_like(logits[row], float("-inf")))
    return logits


def apply_penalties(logits, tok_ids, tok_cnt, n, freq, pres, rep):
    for b in range(logits.shape[0]):
        m = int(n[b])
        ids, cnt = tok_ids[b, :m].long(), tok_cnt[b, :m].float()
        v = logits[b, ids]
        r = float(rep[b])
        if r != 1.0:
            v = torch.where(v > 0, v / r, v * r)
        v = v - float(freq[b]) * cnt - (cnt > 0).float() * float(pres[b])
        logits[b, ids] = v
    return logits


def sim_topk(Q, X, bias, n_rows, k):
    s = Q.float() @ X[:n_rows].float().t() + bias[:n_rows].float()
    k = min(k, n_rows)
    v, i = torch.topk(s, k, dim=-1)
    return v, i


def moe_route(logits, k, renorm=True):
    p = logits.float().softmax(-1)
    w, ids = torch.topk(p, k, dim=-1)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return ids.int(), w


def moe_gemm(A, a_rows, W, offs, rows_total, swiglu):
    E, N, K = W.shape
    outw = N // 2 if swiglu else N
    C = torch.empty(rows_total, outw, dtype=A.dtype)
    o = offs.tolist()
    for e in range(E):
        s, t = o[e], o[e + 1]
        if t == s:
            continue
        rows = a_rows[s:t].long() if a_rows is not None else torch.arange(s, t)
        C[s:t] = linear(A[rows], W[e], act="swiglu" if swiglu else None)
    return C


def moe_combine(Y, pos, w, residual=None, residual_gate=None):
    y = Y[pos.long()].float()
    y = (y * w.float()[..., None]).sum(1) if w is not None else y.sum(1)
    if residual is not None:
        r = residual.float()
        y = y + (r * torch.sigmoid(residual_gate.float().reshape(-1, 1)) if residual_gate is not None else r)
    return y.to(Y.dtype)


def gemv(x, W, gamma=None, eps=1e-5, epi="plain", res=None, swi=None, ks=1):
    """Small-batch decode GEMV oracle (gemv.hip): optional RMSNorm of x (rounded to bf16), fp32 product, epilogue.
    ``swi``: the input is bf16(silu(g) * u) of an fp32 [M, 2K] [gate16 | up16] interleave (x unused); ``part``: the
    fp32 row sums of ``ks`` equal K parts, [ks, M, N]."""
    if swi is not None:
        g = swi.float().view(swi.shape[0], -1, 2, 16)
        xf = (torch.nn.functional.silu(g[:, :, 0]) * g[:, :, 1]).reshape(swi.shape[0], -1).to(torch.bfloat16).float()
    else:
        xf = x.float()
    if gamma is not None:
        xf = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * gamma.float()).to(torch.bfloat16).float()
    if epi == "part":
        kp = xf.shape[1] // ks
        return torch.stack([xf[:, h * kp:(h + 1) * kp] @ W.float()[:, h * kp:(h + 1) * kp].t() for h in range(ks)])
    y = xf @ W.float().t()
    if epi == "f32":
        return y
    if epi == "residual":
        res.copy_((y.to(torch.bfloat16).float() + res.float()).to(res.dtype))
        return res
    if epi == "swiglu":
        g = y.view(y.shape[0], -1, 2, 16)
        return (torch.nn.functional.silu(g[:, :, 0]) * g[:, :, 1]).reshape(y.shape[0], -1).to(torch.bfloat16)
    return y.to(torch.bfloat16)


def ep_dispatch_plan(ids, world, e_local):
    """(offs [W+1], pos [T, k], a_pairs [T*k]): the pairs stably sorted by destination rank id // e_local."""
    T, k = ids.shape
    dest = (ids.reshape(-1).long() // e_local).clamp(0, world - 1)
    order = torch.argsort(dest, stable=True)
    counts = torch.bincount(dest, minlength=world)
    offs = torch.zeros(world + 1, dtype=torch.int32, device=ids.device)
    offs[1:] = counts.cumsum(0).to(torch.int32)
    pos = torch.empty(T * k, dtype=torch.int32, device=ids.device)
    pos[order] = torch.arange(T * k, dtype=torch.int32, device=ids.device)
    return offs, pos.view(T, k), order.to(torch.int32)


def ep_pack(x, ids, offs, a_pairs, world, C, e_local):
    """Send slabs [W*C, D] + local expert ids [W*C] (padding rows: sentinel e_local, zero rows)."""
    k, D = ids.shape[1], x.shape[1]
    send = torch.zeros(world * C, D, dtype=x.dtype, device=x.device)
    eid = torch.full((world * C,), e_local, dtype=torch.int32, device=x.device)
    o, flat = offs.tolist(), ids.reshape(-1).long()
    for d in range(world):
        n = min(o[d + 1] - o[d], C)
        if n > 0:
            pairs = a_pairs[o[d]:o[d] + n].long()
            send[d * C:d * C + n] = x[pairs // k]
            eid[d * C:d * C + n] = (flat[pairs] - d * e_local).to(torch.int32)
    return send, eid


def ep_combine(back, ids, pos, offs, w, residual, e_local, C):
    T, k = ids.shape
    flat = ids.reshape(-1).long()
    dest = flat // e_local
    r = pos.reshape(-1).long() - offs.long()[dest]
    keep = r < C
    rows = back[(dest * C + r.clamp(max=C - 1))].float() * (w.reshape(-1).float() * keep.float())[:, None]
    y = rows.view(T, k, -1).sum(1)
    if residual is not None:
        y = y + residual.float()
    return y.to(back.dtype)


def embedding(ids, table, vstart=0, vend=None):
    vend = table.shape[0] + vstart if vend is None else vend
    ids = ids.long()
    ok = (ids >= vstart) & (ids < vend)
    out = table[(ids - vstart).clamp(0, table.shape[0] - 1)]
    return out * ok[:, None].to(out.dtype)


def decode_advance(toks, ids, pos, ctx, slots, bt, n_valid, block):
    n = int(n_valid.reshape(-1)[0])
    p = pos[:n].long() + 1
    ids[:n] = toks[:n].to(ids.dtype)
    pos[:n] = p.to(pos.dtype)
    ctx[:n] = (p + 1).to(ctx.dtype)
    rows = torch.arange(n, device=bt.device)
    slots[:n] = (bt[rows, p // block].long() * block + p % block).to(slots.dtype)


def pool(h, cu_seqlens, mode="mean", normalize=True):
    cu = cu_seqlens.tolist()
    outs = []
    for b in range(len(cu) - 1):
        s, e = cu[b], cu[b + 1]
        x = h[s:e].float()
        if mode == "mean":
            v = x.mean(0)
        elif mode == "cls":
            v = x[0]
        else:
            v = x[-1]
        outs.append(v)
    o = torch.stack(outs) if outs else h.new_zeros(0, h.shape[-1], dtype=torch.float32)
    if normalize:
        o = F.normalize(o, dim=-1, eps=1e-12)
    return o


def silu_mul(x):
    i = x.shape[-1] // 2
    return (F.silu(x[..., :i].float()) * x[..., i:].float()).to(x.dtype)


def gelu(x):
    return F.gelu(x.float()).to(x.dtype)


def gelu_tanh(x):
    return F.gelu(x.float(), approximate="tanh").to(x.dtype)


def geglu_interleaved(x):
    n = x.shape[-1]
    x4 = x.float().reshape(*x.shape[:-1], n // 32, 2, 16)
    return (F.gelu(x4[..., 0, :], approximate="tanh") * x4[..., 1, :]).reshape(*x.shape[:-1], n // 2).to(x.dtype)


# ---------------------------------------------------------------------------------------------- fp8
FP8_MAX = 448.0


def quant_rows_fp8(x: torch.Tensor):
    """Per-row dynamic e4m3fn quantisation: (q [.., K] float8_e4m3fn, scale [rows] fp32 = amax/448)."""
    xf = x.float().reshape(-1, x.shape[-1])
    s = xf.abs().amax(-1).clamp_min(1e-12) / FP8_MAX
    # x * (1 / s) in fp32, as the kernel (a reciprocal multiply, not a division per element)
    q = (xf * (1.0 / s)[:, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(x.shape), s


def linear_fp8(xq, sx, wq, sw, bias=None, residual=None, act=None, out_dtype=torch.bfloat16):
    """fp32 reference of the fp8 GEMM: dequantise both operands, then ``linear``."""
    x = xq.float().reshape(-1, xq.shape[-1]) * sx.reshape(-1, 1)
    w = wq.float() * sw.reshape(-1, 1)
    y = linear(x, w, bias, None if residual is None else residual.reshape(x.shape[0], -1), act, torch.float32)
    return y.reshape(*xq.shape[:-1], y.shape[-1]).to(out_dtype)


# ---------------------------------------------------------------------------------------------- vision
def patchify(img: torch.Tensor, P: int, mean: torch.Tensor, inv_std: torch.Tensor, Kp: int) -> torch.Tensor:
    """[B, C, H, W] fp32 -> normalised patches [B * gh * gw, Kp] bf16, (c, ky, kx) order, zero padded."""
    B, C, H, W = img.shape
    x = (img.float() - mean[:C].view(1, C, 1, 1)) * inv_std[:C].view(1, C, 1, 1)
    x = x.reshape(B, C, H // P, P, W // P, P).permute(0, 2, 4, 1, 3, 5).reshape(B * (H // P) * (W // P), C * P * P)
    out = torch.zeros(x.shape[0], Kp, dtype=torch.bfloat16)
    out[:, : C * P * P] = x.to(torch.bfloat16)
    return out


def vit_embed(patches: torch.Tensor, cls: torch.Tensor, pos: torch.Tensor, B: int) -> torch.Tensor:
    D = cls.numel()
    p = patches.float().reshape(B, -1, D)
    x = torch.cat([cls.float().view(1, 1, D).expand(B, 1, D), p], 1) + pos.float()[: p.shape[1] + 1]
    return x.reshape(-1, D).to(torch.bfloat16)


# ---------------------------------------------------------------------------------------------
# sequence mixers with a 32-bit residual / state (window attention, WKV, channel-decay delta rule)
# ---------------------------------------------------------------------------------------------
def _seqs(cu, slots):
    c = [int(x) for x in cu.tolist()]
    return [(c[i], c[i + 1], int(s)) for i, s in enumerate(slots.tolist())]


def add_rmsnorm_f32(res, delta, mult, w, eps, out_dtype):
    """res (fp32, in place) += mult * delta; returns rms-normalised res * w (w None: res itself) as out_dtype."""
    if delta is not None:
        res.add_(delta.float(), alpha=float(mult))
    if out_dtype is None:
        return None
    if w is None:
        return res.to(out_dtype)
    return (res * torch.rsqrt(res.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def poly_norm(z, coef, eps):
    x = z.float()
    n = lambda t: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)  # noqa: E731
    a, b, c, e = [float(v) for v in coef.tolist()]
    return (a * n(x) + b * n(x * x) + c * n(x * x * x) + e).to(z.dtype)


def head_norm_gate(o, gate, nw, act, eps, out_dtype):
    T, H, DV = o.shape
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    y = y * (nw.float().view(H, DV) if nw.numel() == H * DV else nw.float())
    g = gate.float().reshape(T, H, DV)
    y = y * (F.silu(g) if act == 0 else torch.sigmoid(g))
    return y.reshape(T, H * DV).to(out_dtype)


def embed_scale_f32(ids, table, scale):
    return table[ids.long().clamp(0, table.shape[0] - 1)].float() * float(scale)


def qknorm_kv_write(q, k, v, wq, wk, slots, k_cache, v_cache, H, G, DK, DV, eps):
    T = q.shape[0]
    n = lambda t, w: t.float() * torch.rsqrt(t.float().pow(2).mean(-1, keepdim=True) + eps) * w.float()  # noqa: E731
    qn = n(q, wq).to(q.dtype)
    kn = n(k, wk).to(k_cache.dtype).view(T, G, DK)
    s = slots[:T].long()
    k_cache[s // BLOCK, :, s % BLOCK] = kn
    v_cache[s // BLOCK, :, :, s % BLOCK] = v.reshape(T, G, DV).to(v_cache.dtype)
    return qn


def window_attention(q, k_cache, v_cache, block_tables, cu_q, ctx, H, G, DK, DV, scale, softcap, window, r1, r2, gate):
    T = q.numel() // (H * DK)
    q3 = q.float().view(T, H, DK)
    out = torch.zeros(T, H, DV)
    cu = [int(x) for x in cu_q.tolist()]
    for s, n in enumerate(ctx.tolist()):
        b, e = cu[s], cu[s + 1]
        if e <= b:
            continue
        n = int(n)
        pages = block_tables[s, : (n + BLOCK - 1) // BLOCK].long()
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(G, -1, DK)[:, :n]          # [G, n, DK]
        V = v_cache[pages].float().permute(1, 0, 3, 2).reshape(G, -1, DV)[:, :n]          # [G, n, DV]
        pos = torch.arange(n - (e - b), n)
        dist = pos[:, None] - torch.arange(n)[None, :]
        vis = (dist >= 0) & ((dist < window) if window > 0 else True)
        for h in range(H):
            sc = (q3[b:e, h] @ K[h // (H // G)].t()) * scale
            if softcap > 0:
                sc = softcap * torch.tanh(sc / softcap)
            if r1 is not None:
                sc = sc - float(r1[h]) * torch.log1p(float(r2[h]) * dist.clamp(min=0).float())
            sc = sc.masked_fill(~vis, float("-inf"))
            out[b:e, h] = torch.softmax(sc, -1) @ V[h // (H // G)]
    out = out.reshape(T, H * DV)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


def token_shift_mix(h, mu, shift_state, cu, slots):
    x = h.float()
    prev = torch.empty_like(x)
    prev[1:] = x[:-1]
    for b, e, s in _seqs(cu, slots):
        if e > b:
            prev[b] = shift_state[s]
    return (x[None] + (prev - x)[None] * mu.float()[:, None]).to(h.dtype)


def state_tail_write(x, state, cu, slots):
    NR = state.shape[1]
    if NR == 0:
        return
    for b, e, s in _seqs(cu, slots):
        if e > b:
            state[s] = torch.cat([state[s], x[b:e].float()])[-NR:]


def conv_silu(x, w, state, cu, slots):
    K = w.shape[1]
    y = torch.empty(x.shape, dtype=torch.float32)
    for b, e, s in _seqs(cu, slots):
        if e > b:
            xs = torch.cat([state[s], x[b:e].float()])
            y[b:e] = (xs.unfold(0, K, 1) * w.float()).sum(-1)
    return F.silu(y)


def wkv_scan(r, k, v, wpre, w0, u, state, cu, slots):
    H, D = state.shape[1], state.shape[2]
    T = r.shape[0]
    r3, k3, v3 = (t.float().reshape(T, H, D) for t in (r, k, v))
    w = torch.exp(-torch.exp(wpre.float().reshape(T, H, D) + w0.float().reshape(H, D)))
    uu = u.float().reshape(H, D)
    out = torch.empty(T, H, D)
    for b, e, s in _seqs(cu, slots):
        S = state[s]
        for t in range(b, e):
            kv = k3[t][:, :, None] * v3[t][:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S + uu[:, :, None] * kv, r3[t])
            S = w[t][:, :, None] * S + kv
        if e > b:
            state[s] = S
    return out


def delta_prep(qkv, a, b, A_log, dt_bias, H, G, DK):
    T = qkv.shape[0]
    l2 = lambda t: t * torch.rsqrt(t.pow(2).sum(-1, keepdim=True) + 1e-6)  # noqa: E731
    qn = l2(qkv[:, : G * DK].float().reshape(T, G, DK)) * DK ** -0.5
    kn = l2(qkv[:, G * DK: 2 * G * DK].float().reshape(T, G, DK))
    sp = F.softplus(a.float() + dt_bias.float().reshape(1, -1)).reshape(T, H, DK)
    decay = torch.exp(-torch.exp(A_log.float())[None, :, None] * sp)
    return qn, kn, decay, torch.sigmoid(b.float())


def delta_scan(q, k, v, decay, beta, state, cu, slots, G):
    H, DK, DV = state.shape[1:]
    T = v.shape[0]
    rep = H // G
    q3 = q.reshape(T, G, DK).repeat_interleave(rep, 1)
    k3 = k.reshape(T, G, DK).repeat_interleave(rep, 1)
    v3 = v.float().reshape(T, H, DV)
    out = torch.empty(T, H, DV)
    for b, e, s in _seqs(cu, slots):
        S = state[s]
        for t in range(b, e):
            S = decay[t][:, :, None] * S
            u = beta[t][:, None] * (v3[t] - torch.einsum("hkv,hk->hv", S, k3[t]))
            S = S + k3[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S, q3[t])
        if e > b:
            state[s] = S
    return out


# ---------------------------------------------------------------------------------------------
# post-norm gated residual, per-head q/k norm with a query temperature, sigmoid attention, gated linear recurrence,
# state-space scan, sigmoid router with input-side expert weights
# ---------------------------------------------------------------------------------------------
def embed_pos_f32(ids, table, scale, positions, pos_table):
    x = embed_scale_f32(ids, table, scale)
    return x + pos_table[positions.long().clamp(0, pos_table.shape[0] - 1)].float()


def gated_norm_add_f32(res, y, gate, wpost, eps, wnext, out_dtype):
    """res (fp32, in place) += rmsnorm(y * sigmoid(gate)) * wpost; returns rmsnorm(res) * wnext (wnext None: res) as
    out_dtype, or None when out_dtype is None."""
    g = y.float() * torch.sigmoid(gate.float()) if gate is not None else y.float()
    res.add_(g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps) * wpost.float())
    return add_rmsnorm_f32(res, None, 1.0, wnext, eps, out_dtype)


def headnorm_kv_write(q, k, v, wq, wk, slots, k_cache, v_cache, H, G, DK, DV, eps, positions, temp_coef, temp_every):
    T = q.shape[0]
    n = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()  # noqa: E731
    qn = n(q.float().reshape(T, H, DK), wq)
    if temp_coef:
        p = positions[:T].long()
        qn = qn * (1.0 + float(temp_coef) * torch.log(((p + 1) // int(temp_every) + 1).float()))[:, None, None]
    kn = n(k.float().reshape(T, G, DK), wk).to(k_cache.dtype)
    s = slots[:T].long()
    k_cache[s // BLOCK, :, s % BLOCK] = kn
    v_cache[s // BLOCK, :, :, s % BLOCK] = v.reshape(T, G, DV).to(v_cache.dtype)
    return qn.reshape(T, H * DK).to(q.dtype)


def sigmoid_attention(q, k_cache, v_cache, block_tables, cu_q, ctx, H, G, DK, DV, scale, bias, window, out_scale=1.0):
    """o_i = sum_j sigmoid(scale q_i . k_j + bias_h) v_j over the visible keys (no normalisation over keys)."""
    T = q.numel() // (H * DK)
    q3 = q.float().view(T, H, DK)
    out = torch.zeros(T, H, DV)
    cu = [int(x) for x in cu_q.tolist()]
    for s, n in enumerate(ctx.tolist()):
        b, e = cu[s], cu[s + 1]
        if e <= b:
            continue
        n = int(n)
        pages = block_tables[s, : (n + BLOCK - 1) // BLOCK].long()
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(G, -1, DK)[:, :n]
        V = v_cache[pages].float().permute(1, 0, 3, 2).reshape(G, -1, DV)[:, :n]
        pos = torch.arange(n - (e - b), n)
        dist = pos[:, None] - torch.arange(n)[None, :]
        vis = (dist >= 0) & ((dist < window) if window > 0 else True)
        for h in range(H):
            sc = (q3[b:e, h] @ K[h // (H // G)].t()) * scale + (float(bias[h]) if bias is not None else 0.0)
            out[b:e, h] = (torch.sigmoid(sc) * vis) @ V[h // (H // G)]
    return (out.reshape(T, H * DV) * float(out_scale)).to(q.dtype)


def conv_bias_act(x, w, state, cu, slots, bias, act):
    K = w.shape[1]
    y = torch.empty(x.shape, dtype=torch.float32)
    for b, e, s in _seqs(cu, slots):
        if e > b:
            xs = torch.cat([state[s], x[b:e].float()])
            y[b:e] = (xs.unfold(0, K, 1) * w.float()).sum(-1)
    if bias is not None:
        y = y + bias.float()
    return F.silu(y) if act else y


def rglru_gates(u, wa_t, ba, wi_t, bi, lam, c):
    """Block-diagonal gates of a real-gated linear recurrent unit. u [T, W] fp32; wa_t / wi_t [nb, in, out];
    returns (a, b): a = exp(-c r softplus(lam)), b = sqrt(1 - a^2) i u with r, i = sigmoid(block(u) + bias)."""
    T, W = u.shape
    nb, bs = wa_t.shape[0], wa_t.shape[1]
    ub = u.float().reshape(T, nb, bs).transpose(0, 1)                      # [nb, T, bs]
    r = torch.sigmoid(torch.bmm(ub, wa_t.float()).transpose(0, 1).reshape(T, W) + ba.float().reshape(-1))
    i = torch.sigmoid(torch.bmm(ub, wi_t.float()).transpose(0, 1).reshape(T, W) + bi.float().reshape(-1))
    a = torch.exp(-float(c) * r * F.softplus(lam.float()))
    return a, torch.sqrt(1.0 - a * a) * i * u.float()


def rglru_scan(a, b, y, state, cu, slots, out_dtype, act=None, out_scale=1.0):
    """S_t = a_t S_(t-1) + b_t per channel; returns S_t * y_t. state [slots, W] fp32 in place."""
    out = torch.empty(a.shape, dtype=torch.float32)
    for lo, hi, s in _seqs(cu, slots):
        S = state[s]
        for t in range(lo, hi):
            S = a[t] * S + b[t]
            out[t] = S
        if hi > lo:
            state[s] = S
    yy = F.gelu(y.float(), approximate="tanh") if act == "gelu_tanh" else y.float()
    return (out * yy * float(out_scale)).to(out_dtype)


def ssd_scan(x, B, C, dt, dt_bias, A_log, D, state, cu, slots, G):
    """State-space scan with one decay per head: S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T,
    y_t = S_t^T C_t + D x_t; dt_t = softplus(dt + dt_bias). state [slots, H, N, DV] fp32 in place."""
    H, N, DV = state.shape[1:]
    T = x.shape[0]
    rep = H // G
    x3 = x.float().reshape(T, H, DV)
    B3 = B.float().reshape(T, G, N).repeat_interleave(rep, 1)
    C3 = C.float().reshape(T, G, N).repeat_interleave(rep, 1)
    dts = F.softplus(dt.float() + dt_bias.float().reshape(1, -1))          # [T, H]
    dec = torch.exp(-torch.exp(A_log.float())[None] * dts)
    out = torch.empty(T, H, DV)
    for lo, hi, s in _seqs(cu, slots):
        S = state[s]
        for t in range(lo, hi):
            S = dec[t][:, None, None] * S + (dts[t][:, None] * B3[t])[:, :, None] * x3[t][:, None, :]
            out[t] = torch.einsum("hnv,hn->hv", S, C3[t]) + D.float()[:, None] * x3[t]
        if hi > lo:
            state[s] = S
    return out


def gate_group_norm(y, z, w, groups, eps, out_dtype):
    """(y * silu(z)) RMS-normalised in `groups` equal parts of the last dim, times w."""
    T, C = y.shape
    g = (y.float() * F.silu(z.float())).reshape(T, groups, C // groups)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    return (g.reshape(T, C) * w.float()).to(out_dtype)


def moe_route_sigmoid(logits, k):
    s = torch.sigmoid(logits.float())
    w, ids = torch.topk(s, k, dim=-1)
    return ids.int(), w


def moe_scale_rows(h, pos, w):
    """Expert-sorted copies of the token rows, each times its routing weight: out[pos[t, j]] = w[t, j] * h[t]."""
    T, k = pos.shape
    out = torch.empty(T * k, h.shape[1], dtype=h.dtype)
    out[pos.reshape(-1).long()] = (h.float()[:, None, :] * w.float()[:, :, None]).reshape(T * k, -1).to(h.dtype)
    return out


def moe_gemm_act(A, a_rows, W, offs, rows_total, act):
    E, N, K = W.shape
    C = torch.empty(rows_total, N, dtype=A.dtype)
    o = offs.tolist()
    for e in range(E):
        if o[e + 1] > o[e]:
            rows = A[a_rows[o[e]:o[e + 1]].long()] if a_rows is not None else A[o[e]:o[e + 1]]
            y = rows.float() @ W[e].float().t()
            if act == "relu2":
                y = torch.relu(y) ** 2
            C[o[e]:o[e + 1]] = y.to(A.dtype)
    return C


# ---------------------------------------------------------------------------------------------
# statistics-free tanh norm, latent (low-rank) key / value cache with a partly rotated key, constant-decay linear
# attention, selective state-space scan, biased top-k routing with identity experts
# ---------------------------------------------------------------------------------------------
def add_dyt_f32(res, delta, extra, alpha, w, b, out_dtype):
    """res (fp32, in place) += delta (+ extra); returns tanh(alpha res) * w + b as out_dtype (None: nothing)."""
    if delta is not None:
        res.add_(delta.float())
    if extra is not None:
        res.add_(extra.float())
    if out_dtype is None:
        return None
    return (torch.tanh(float(alpha) * res) * w.float() + b.float()).to(out_dtype)


def act_mul(a, b, act, out_dtype, cap=0.0):
    """act(a) (* b): "silu", "relu2" (squared ReLU), "tanh_cap" (cap tanh(a / cap)), "gelu_tanh", or "clamp_glu" (the
    clamped gated activation of a, b with limit cap), in fp32."""
    x = a.float()
    if act == "clamp_glu":
        return clamp_glu(x, b, cap).to(out_dtype)
    if act == "gelu_tanh":
        y = F.gelu(x, approximate="tanh")
    elif act == "silu":
        y = F.silu(x)
    elif act == "relu2":
        y = torch.relu(x) ** 2
    else:
        y = float(cap) * torch.tanh(x / float(cap))
    if b is not None:
        y = y * b.float()
    return y.to(out_dtype)


def yarn_inv_freq(dims, base, scaling=None):
    """(fp32 [dims / 2] angle steps per position, magnitude of cos / sin) of a rotation over `dims` channels with the
    pairs (i, i + dims / 2); scaling {factor, original, fast, slow}: wavelengths longer than original / slow are
    stretched by factor, shorter than original / fast kept, a linear ramp over the pair index between them."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling:
        import math

        fac, orig = float(scaling["factor"]), float(scaling["original"])
        at = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))  # noqa: E731
        lo = max(math.floor(at(float(scaling["fast"]))), 0)
        hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / fac * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(fac) + 1.0
    return f.to(torch.float32), float(mag)


def _rot_half(x, pos, inv_freq, mag):
    """x [T, ..., dims] fp32, pos [T]; pair (i, i + dims / 2) turned by pos * inv_freq[i], cos / sin times mag."""
    half = inv_freq.numel()
    a = pos.float().reshape(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    c, s = torch.cos(a) * mag, torch.sin(a) * mag
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def latent_kv_write(q, dkv, norm_w, inv_freq, mag, positions, slots, q_cat, k_cache, v_cache, H, DN, DR, R, eps):
    """One low-rank latent per token as the only cache row: c = rmsnorm(dkv[:, :R]) * norm_w, kr = rot(dkv[:, R:]).
    K page row = [c | kr] (one kv head, key size R + DR), V^T page = c. The rotated part of every query head
    (q [T, H, DN + DR], last DR channels) goes to q_cat[:, h, R:]."""
    T = q.shape[0]
    pos = positions[:T]
    x = dkv.float()
    c = x[:, :R]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = _rot_half(x[:, R:R + DR], pos, inv_freq, mag)
    s = slots[:T].long()
    k_cache[s // BLOCK, 0, s % BLOCK] = torch.cat([c, kr], -1).to(k_cache.dtype)
    v_cache[s // BLOCK, 0, :, s % BLOCK] = c.to(v_cache.dtype)
    qr = _rot_half(q.float().reshape(T, H, DN + DR)[:, :, DN:], pos, inv_freq, mag)
    q_cat.view(T, H, R + DR)[:, :, R:] = qr.to(q_cat.dtype)


def linear_attention_scan(q, k, v, decay, state, cu, slots):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; q / k [T, H * DK], v [T, H * DV] fp32; state
    [slots, H, DK, DV] fp32 in place -> fp32 [T, H, DV]."""
    H, DK, DV = state.shape[1:]
    T = q.shape[0]
    q3, k3, v3 = q.float().reshape(T, H, DK), k.float().reshape(T, H, DK), v.float().reshape(T, H, DV)
    d = decay.float().reshape(H, 1, 1)
    out = torch.empty(T, H, DV)
    for lo, hi, s in _seqs(cu, slots):
        S = state[s]
        for t in range(lo, hi):
            S = d * S + k3[t][:, :, None] * v3[t][:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S, q3[t])
        if hi > lo:
            state[s] = S
    return out


def selective_scan(x, dt, dt_bias, A, B, C, D, z, state, cu, slots, out_dtype):
    """Selective state-space scan: per channel c and state n, S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,
    y_c = sum_n S[c, n] C_n + D_c x_c, times silu(z_c); dt = softplus(dt + dt_bias). x [T, I] fp32, dt [T, I],
    B / C [T, N], A [I, N] (negative), state [slots, I, N] fp32 in place -> [T, I] in out_dtype."""
    T, I = x.shape
    xs = x.float()
    dts = F.softplus(dt.float() + dt_bias.float().reshape(1, -1))
    Bf, Cf, Af = B.float(), C.float(), A.float()
    y = torch.empty(T, I)
    for lo, hi, s in _seqs(cu, slots):
        S = state[s]
        for t in range(lo, hi):
            S = torch.exp(dts[t][:, None] * Af) * S + (dts[t] * xs[t])[:, None] * Bf[t][None, :]
            y[t] = S @ Cf[t] + D.float() * xs[t]
        if hi > lo:
            state[s] = S
    return (y * F.silu(z.float())).to(out_dtype)


def moe_route_biased(logits, k, bias, eps):
    """softmax scores s; the k experts with the largest s + bias are chosen; weights s / (sum of the chosen s + eps)."""
    s = torch.softmax(logits.float(), -1)
    ids = torch.topk(s + bias.float(), k, dim=-1).indices
    w = torch.gather(s, 1, ids)
    return ids.int(), w / (w.sum(-1, keepdim=True) + eps)


def moe_combine_identity(Y, pos, w, residual, ids, n_real, h):
    """moe_combine where an expert id >= n_real is an identity expert: its output is the token's own input row."""
    T, k = pos.shape
    rows = Y.float()[pos.reshape(-1).long().clamp(0, max(Y.shape[0] - 1, 0))].reshape(T, k, -1) if Y.shape[0] else \
        torch.zeros(T, k, h.shape[1])
    ident = (ids >= n_real)[:, :, None]
    rows = torch.where(ident, h.float()[:, None, :].expand_as(rows), rows)
    out = (rows * w.float()[:, :, None]).sum(1)
    if residual is not None:
        out = out + residual.float()
    return out.to(h.dtype)


# ---------------------------------------------------------------------------------------------
# pair-interleaved partial rotation, chunk-local attention with a sink and per-head temperatures, diagonal-plus-rank-one
# linear recurrences (gated linear attention, generalised delta rule), group-limited sigmoid routing, clamped gated
# experts
# ---------------------------------------------------------------------------------------------
GLU_SLOPE = 1.702      # slope of the sigmoid in the clamped gated activation


def rotary_kv_write(q, k, v, positions, slots, k_cache, v_cache, H, G, DK, DV, rot_dims, base):
    """Rotation of the channel pairs (2i, 2i + 1), i < rot_dims / 2, of every q and k head by position * base^(-2i /
    rot_dims) (channels past rot_dims pass unchanged); k and v into their cache slots; returns q [T, H * DK]."""
    T = q.shape[0]
    pos = positions[:T].to(torch.float64)

    def rot(x):
        x = x.float()
        if not rot_dims:
            return x
        i = torch.arange(rot_dims // 2, dtype=torch.float64)
        ang = pos[:, None] * float(base) ** (-2.0 * i / rot_dims)
        c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
        a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
        y = x.clone()
        y[..., 0:rot_dims:2] = a * c - b * s
        y[..., 1:rot_dims:2] = b * c + a * s
        return y

    s = slots[:T].long()
    k_cache[s // BLOCK, :, s % BLOCK] = rot(k.reshape(T, G, DK)).to(k_cache.dtype)
    v_cache[s // BLOCK, :, :, s % BLOCK] = v.reshape(T, G, DV).to(v_cache.dtype)
    return rot(q.reshape(T, H, DK)).reshape(T, H * DK).to(k_cache.dtype)


def masked_attention(q, k_cache, v_cache, block_tables, cu_q, ctx, H, G, DK, DV, scale, window, chunk, head_scale, sink,
                     out_scale):
    """Softmax attention over the visible keys j <= i: the last `window` ones (window > 0), those of the query's own
    chunk of positions floor(i / chunk) = floor(j / chunk) (chunk > 0), or all. head_scale [H] multiplies the scores of
    a head; sink (a score, or None) adds exp(sink) to the softmax denominator without adding a value."""
    T = q.numel() // (H * DK)
    q3 = q.float().view(T, H, DK)
    out = torch.zeros(T, H, DV)
    cu = [int(x) for x in cu_q.tolist()]
    for s, n in enumerate(ctx.tolist()):
        b, e = cu[s], cu[s + 1]
        if e <= b:
            continue
        n = int(n)
        pages = block_tables[s, : (n + BLOCK - 1) // BLOCK].long()
        K = k_cache[pages].float().permute(1, 0, 2, 3).reshape(G, -1, DK)[:, :n]
        V = v_cache[pages].float().permute(1, 0, 3, 2).reshape(G, -1, DV)[:, :n]
        pos = torch.arange(n - (e - b), n)
        key = torch.arange(n)
        vis = key[None, :] <= pos[:, None]
        if window > 0:
            vis = vis & (pos[:, None] - key[None, :] < window)
        if chunk > 0:
            vis = vis & (torch.div(pos, chunk, rounding_mode="floor")[:, None] ==
                         torch.div(key, chunk, rounding_mode="floor")[None, :])
        for h in range(H):
            sc = (q3[b:e, h] @ K[h // (H // G)].t()) * (scale * (float(head_scale[h]) if head_scale is not None else 1.0))
            sc = sc.masked_fill(~vis, float("-inf"))
            m = sc.max(-1, keepdim=True).values
            if sink is not None:
                m = m.clamp(min=float(sink))
            p = torch.exp(sc - m)
            den = p.sum(-1, keepdim=True)
            if sink is not None:
                den = den + torch.exp(float(sink) - m)
            out[b:e, h] = (p / den) @ V[h // (H // G)]
    return (out.reshape(T, H * DV) * float(out_scale)).to(q.dtype)


def decay_gate(z, bias, kind, param):
    """fp32 gates of a recurrence from their logits z (+ bias): "sigmoid" -> sigmoid(x); "sigmoid_root" ->
    sigmoid(x)^(1 / param); "exp_sigmoid" -> exp(-param * sigmoid(x))."""
    x = z.float() + (bias.float().reshape(1, -1) if bias is not None else 0.0)
    if kind == "sigmoid":
        return torch.sigmoid(x)
    if kind == "sigmoid_root":
        return torch.exp(F.logsigmoid(x) / float(param))
    return torch.exp(-float(param) * torch.sigmoid(x))


def unit_key_removal(k, a, a_bias, H, DK, eps):
    """Per head the unit key u = k / sqrt(sum(k^2) + eps) and the removal vector sigmoid(a + a_bias) * u (both fp32
    [T, H * DK])."""
    T = k.shape[0]
    k3 = k.float().reshape(T, H, DK)
    u = k3 * torch.rsqrt(k3.pow(2).sum(-1, keepdim=True) + eps)
    rate = torch.sigmoid(a.float() + (a_bias.float().reshape(1, -1) if a_bias is not None else 0.0)).reshape(T, H, DK)
    return (rate * u).reshape(T, H * DK), u.reshape(T, H * DK)


def dplr_scan(q, k, v, decay, av, bv, state, cu, slots, q_scale):
    """S_t = diag(decay_t) S_(t-1) - av_t (bv_t^T S_(t-1)) + k_t v_t^T, o_t = q_scale * S_t^T q_t (av / bv None: no
    removal term). q / k / decay / av / bv [T, H * DK], v [T, H * DV]; state [slots, H, DK, DV] fp32 in place."""
    H, DK, DV = state.shape[1:]
    T = q.shape[0]
    r3 = lambda t: t.float().reshape(T, H, -1)  # noqa: E731
    q3, k3, v3, w3 = r3(q), r3(k), r3(v), r3(decay)
    a3, b3 = (r3(av), r3(bv)) if av is not None else (None, None)
    out = torch.empty(T, H, DV)
    for lo, hi, s in _seqs(cu, slots):
        S = state[s]
        for t in range(lo, hi):
            new = w3[t][:, :, None] * S + k3[t][:, :, None] * v3[t][:, None, :]
            if a3 is not None:
                new = new - a3[t][:, :, None] * torch.einsum("hk,hkv->hv", b3[t], S)[:, None, :]
            S = new
            out[t] = torch.einsum("hkv,hk->hv", S, q3[t]) * float(q_scale)
        if hi > lo:
            state[s] = S
    return out


def moe_route_grouped(logits, k, bias, eps, groups, keep, scale, group_top=2):
    """Sigmoid scores s; choice scores s + bias; the expert list is cut into `groups` contiguous parts of
    equal size, each ranked by its group_top best choice scores added up, and the choice is confined to the `keep` best parts; weights
    s / (sum of the chosen s + eps) * scale."""
    s = torch.sigmoid(logits.float())
    c = s + bias.float() if bias is not None else s.clone()
    T, E = c.shape
    if groups > 1 and keep < groups:
        per = c.view(T, groups, E // groups)
        gs = per.topk(min(group_top, E // groups), -1).values.sum(-1)
        best = gs.topk(keep, -1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        c = torch.where(ok[:, :, None].expand_as(per).reshape(T, E), c, torch.full_like(c, float("-inf")))
    ids = torch.topk(c, k, dim=-1).indices
    w = torch.gather(s, 1, ids)
    return ids.int(), w / (w.sum(-1, keepdim=True) + eps) * float(scale)


def clamp_glu(g, u, limit):
    g = g.float().clamp(max=float(limit))
    u = u.float().clamp(-float(limit), float(limit))
    return g * torch.sigmoid(GLU_SLOPE * g) * (u + 1.0)


def moe_gemm_clamp_glu(A, a_rows, W, offs, rows_total, limit):
    """Grouped GEMM whose rows of W are interleaved [gate16 | up16] blocks, with the clamped gated activation."""
    E, N, K = W.shape
    C = torch.empty(rows_total, N // 2, dtype=A.dtype)
    o = offs.tolist()
    for e in range(E):
        if o[e + 1] > o[e]:
            rows = A[a_rows[o[e]:o[e + 1]].long()] if a_rows is not None else A[o[e]:o[e + 1]]
            y = (rows.float() @ W[e].float().t()).view(rows.shape[0], N // 32, 2, 16)
            C[o[e]:o[e + 1]] = clamp_glu(y[:, :, 0], y[:, :, 1], limit).reshape(rows.shape[0], N // 2).to(A.dtype)
    return C
