// Sliding-window paged attention with a tanh score cap and a logarithmic distance penalty, in fp32 arithmetic.
//
//   s_ij = cap * tanh(scale * (q_i . k_j) / cap) - r1_h * ln(1 + r2_h * (i - j)),   0 <= i - j < window
//   o_i  = softmax_j(s_ij) V
//
// optionally times sigmoid(gate_i) element by element (an output gate read from the same projection as q, k, v).
// (cap <= 0: no cap; r1 = nullptr: no distance term; window <= 0: plain causal.) Positions enter only through the
// distance term and the window: there is no rotation. K / V live in the engine's paged cache (16-token pages,
// K [page, G, 16, DK], V^T [page, G, DV, 16]) in bf16 or fp32; scores, softmax weights and the P.V sums are fp32.
// Head sizes are run-time values (DK != DV allowed, DV <= 512).
//
// Sigmoid mode (template SIG): no softmax - a visible key weighs sigmoid(scale * (q_i . k_j) + bias_h) and the weights
// are not normalised over the keys: o_i = out_scale * sum_j sigmoid(.) v_j. Same paging, tiling and key walk; the
// running maximum, the rescaling of the accumulators and the final division drop out.
//
// Chunk mode (chunk > 0): a key is visible only inside the query's own chunk of positions, floor(j / chunk) ==
// floor(i / chunk), counted from position 0 of the sequence. hscale (per head) multiplies the scores of a head. A sink
// (has_sink) is a virtual key of score `sink` without a value: the softmax denominator gains exp(sink). out_scale
// multiplies the output in both modes.
//
// rotary_kv_write: rotation of the channel pairs (2i, 2i + 1), i < ROT / 2, of every q and k head by position *
// base^(-2i / ROT) (the rest of a head passes unchanged), then q -> q_out and k, v -> their cache slots. The angle is
// formed and reduced to (-pi, pi] in fp64, sine and cosine are libm sincosf of the reduced angle.
//
// headnorm_kv_write: RMS norm of every q head and every k head over its own DK channels (one weight vector of size DK
// shared by the heads), optionally times a query temperature 1 + coef * ln(floor((p + 1) / every) + 1) of the token's
// position p, then q -> q_out and k, v -> their cache slots; one wave64 per head.
//
// qknorm_kv_write: RMS norm over the WHOLE q projection (all heads at once) and over the whole k projection, each
// with its own weight vector, then q -> q_out and k, v -> their cache slots: one pass over the token's rows.
//
// latent_kv_write: the cache write of latent attention. A token's cache row is ONE low-rank latent c = rmsnorm(first R
// channels of the down projection) * w plus DR rotated key channels shared by all heads: K page row [c | kr] (one kv
// head, key size R + DR), V^T page c. The rotated DR channels of every query head go to the tail of that head's row of
// q_cat (whose first R channels hold the query folded through the key expansion), so window_attention scores against
// the cached row directly. Rotation over the first ROT of the DR channels (the rest pass unchanged): channel i pairs
// with i + ROT / 2, angle = position * inv_freq[i] (fp32, libm sincosf), cos and sin times one magnitude.
//
// window_attention, row kernel: one wave64 per (token, head) (a sequence is (cu_q[s], ctx[s]); the query at row t has
// position ctx - q_len + (t - cu_q)). Keys are walked in page-aligned blocks of 64: lane j scores key j (q broadcast
// from LDS, the K row read with 16-byte loads), an online softmax keeps (m, l) per wave, then lane c accumulates output
// channel c over the block, reading its 16 V^T values of every page with 16-byte loads. It serves decoded tokens, short
// portions, fp32 activations and head sizes off the MFMA grid; bf16 prompt portions run on the query-tiled matrix-core
// kernel further down.
#include "gai_common.h"
#include "gai_kernels.h"

using namespace gai;

namespace {

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const bf16* __restrict__ k, int DK) {
  float a = 0.f;
  if ((DK & 7) == 0) {
    for (int i = 0; i < DK; i += 8) {
      const bf16x8 v = load8(k + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) a = fmaf(qs[i + j], (float)v[j], a);
    }
  } else {
    for (int i = 0; i < DK; ++i) a = fmaf(qs[i], (float)k[i], a);
  }
  return a;
}

__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const float* __restrict__ k, int DK) {
  float a = 0.f;
  if ((DK & 3) == 0) {
    for (int i = 0; i < DK; i += 4) {
      const float4 v = *reinterpret_cast<const float4*>(k + i);
      a = fmaf(qs[i], v.x, a);
      a = fmaf(qs[i + 1], v.y, a);
      a = fmaf(qs[i + 2], v.z, a);
      a = fmaf(qs[i + 3], v.w, a);
    }
  } else {
    for (int i = 0; i < DK; ++i) a = fmaf(qs[i], k[i], a);
  }
  return a;
}

// sum_j p[j] * v[j] over the 16 tokens of one V^T page row
__device__ __forceinline__ float pv16(const float* __restrict__ p, const bf16* __restrict__ v) {
  const bf16x8 a = load8(v), b = load8(v + 8);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s = fmaf(p[j], (float)a[j], s);
#pragma unroll
  for (int j = 0; j < 8; ++j) s = fmaf(p[8 + j], (float)b[j], s);
  return s;
}

__device__ __forceinline__ float pv16(const float* __restrict__ p, const float* __restrict__ v) {
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 a = *reinterpret_cast<const float4*>(v + 4 * q);
    s = fmaf(p[4 * q], a.x, s);
    s = fmaf(p[4 * q + 1], a.y, s);
    s = fmaf(p[4 * q + 2], a.z, s);
    s = fmaf(p[4 * q + 3], a.w, s);
  }
  return s;
}

template <typename TA>
__global__ __launch_bounds__(256) void qknorm_kv_write_kernel(const TA* __restrict__ q, int ldq, const TA* __restrict__ k,
                                                              int ldk, const TA* __restrict__ v, int ldv,
                                                              const float* __restrict__ wq, const float* __restrict__ wk,
                                                              const int* __restrict__ slots, TA* __restrict__ q_out,
                                                              TA* __restrict__ k_cache, TA* __restrict__ v_cache, int H,
                                                              int G, int DK, int DV, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const TA* qr = q + (size_t)t * ldq;
  const TA* kr = k + (size_t)t * ldk;
  const TA* vr = v + (size_t)t * ldv;
  const int NQ = H * DK, NK = G * DK, NV = G * DV;
  float sq = 0.f, sk = 0.f;
  for (int i = tid; i < NQ; i += 256) {
    const float x = (float)qr[i];
    sq += x * x;
  }
  for (int i = tid; i < NK; i += 256) {
    const float x = (float)kr[i];
    sk += x * x;
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float iq = 1.0f / sqrtf(sq / NQ + eps), ik = 1.0f / sqrtf(sk / NK + eps);
  TA* qo = q_out + (size_t)t * NQ;
  for (int i = tid; i < NQ; i += 256) qo[i] = (TA)((float)qr[i] * iq * wq[i]);
  const int slot = slots[t];
  const size_t page = slot >> 4;
  const int off = slot & 15;
  for (int i = tid; i < NK; i += 256) {
    const int g = i / DK, d = i - g * DK;
    k_cache[((page * G + g) * 16 + off) * DK + d] = (TA)((float)kr[i] * ik * wk[i]);
  }
  for (int i = tid; i < NV; i += 256) {
    const int g = i / DV, c = i - g * DV;
    v_cache[((page * G + g) * DV + c) * 16 + off] = vr[i];
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void headnorm_kv_write_kernel(const TA* __restrict__ q, int ldq, const TA* __restrict__ k,
                                                                int ldk, const TA* __restrict__ v, int ldv,
                                                                const float* __restrict__ wq, const float* __restrict__ wk,
                                                                const int* __restrict__ slots,
                                                                const int* __restrict__ positions, TA* __restrict__ q_out,
                                                                TA* __restrict__ k_cache, TA* __restrict__ v_cache, int H,
                                                                int G, int DK, int DV, float eps, float temp_coef,
                                                                int temp_every) {
  const int t = blockIdx.x, wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int slot = slots[t];
  const size_t page = slot >> 4;
  const int off = slot & 15;
  float temp = 1.0f;
  if (positions) temp = 1.0f + temp_coef * logf((float)((positions[t] + 1) / temp_every + 1));
  for (int hh = wid; hh < H + G; hh += 4) {  // q heads, then k heads: wave-uniform
    const bool isq = hh < H;
    const int g = isq ? hh : hh - H;
    const TA* src = isq ? q + (size_t)t * ldq + (size_t)g * DK : k + (size_t)t * ldk + (size_t)g * DK;
    float ss = 0.f;
    for (int i = lane; i < DK; i += 64) {
      const float x = (float)src[i];
      ss += x * x;
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / DK + eps);
    if (isq) {
      TA* qo = q_out + ((size_t)t * H + g) * DK;
      for (int i = lane; i < DK; i += 64) qo[i] = (TA)((float)src[i] * inv * wq[i] * temp);
    } else {
      TA* ko = k_cache + ((page * G + g) * 16 + off) * DK;
      for (int i = lane; i < DK; i += 64) ko[i] = (TA)((float)src[i] * inv * wk[i]);
    }
  }
  const int NV = G * DV;
  const TA* vr = v + (size_t)t * ldv;
  for (int i = threadIdx.x; i < NV; i += 256) {
    const int g = i / DV, c = i - g * DV;
    v_cache[((page * G + g) * DV + c) * 16 + off] = vr[i];
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const TA* __restrict__ q, int ldq, const TA* __restrict__ dkv,
                                                              int ldk, const float* __restrict__ nw,
                                                              const float* __restrict__ inv_freq, float mag,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ slots, TA* __restrict__ q_cat,
                                                              TA* __restrict__ k_cache, TA* __restrict__ v_cache, int H,
                                                              int DN, int DR, int R, float eps, int ROT) {
  extern __shared__ float cs[];  // cos[ROT / 2] | sin[ROT / 2]
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x, half = ROT >> 1;
  const TA* lr = dkv + (size_t)t * ldk;
  const float pos = (float)positions[t];
  for (int i = tid; i < half; i += 256) {
    float sn, c;
    sincosf(pos * inv_freq[i], &sn, &c);
    cs[i] = c * mag;
    cs[half + i] = sn * mag;
  }
  float ss = 0.f;
  for (int i = tid; i < R; i += 256) {
    const float x = (float)lr[i];
    ss += x * x;
  }
  ss = block_sum(ss, scratch);  // also orders the cos / sin table before its readers
  __syncthreads();
  const float inv = 1.0f / sqrtf(ss / R + eps);
  const int slot = slots[t];
  const size_t page = slot >> 4;
  const int off = slot & 15, DK = R + DR;
  TA* kr = k_cache + (page * 16 + off) * DK;
  for (int i = tid; i < R; i += 256) {
    const TA c = (TA)((float)lr[i] * inv * nw[i]);
    kr[i] = c;
    v_cache[(page * R + i) * 16 + off] = c;
  }
  for (int i = tid; i < half; i += 256) {
    const float u = (float)lr[R + i], v = (float)lr[R + half + i], c = cs[i], sn = cs[half + i];
    kr[R + i] = (TA)(u * c - v * sn);
    kr[R + half + i] = (TA)(v * c + u * sn);
  }
  const int rest = DR - ROT;  // channels past the rotated ones pass unchanged
  for (int i = tid; i < rest; i += 256) kr[R + ROT + i] = lr[R + ROT + i];
  for (int x = tid; x < H * rest; x += 256) {
    const int h = x / rest, i = x - h * rest;
    q_cat[((size_t)t * H + h) * DK + R + ROT + i] = q[(size_t)t * ldq + (size_t)h * (DN + DR) + DN + ROT + i];
  }
  for (int x = tid; x < H * half; x += 256) {
    const int h = x / half, i = x - h * half;
    const TA* qr = q + (size_t)t * ldq + (size_t)h * (DN + DR) + DN;
    TA* qo = q_cat + ((size_t)t * H + h) * DK + R;
    const float u = (float)qr[i], v = (float)qr[half + i], c = cs[i], sn = cs[half + i];
    qo[i] = (TA)(u * c - v * sn);
    qo[half + i] = (TA)(v * c + u * sn);
  }
}

template <typename TI, typename TA>
__global__ __launch_bounds__(256) void rotary_kv_write_kernel(const TI* __restrict__ q, int ldq, const TI* __restrict__ k,
                                                              int ldk, const TI* __restrict__ v, int ldv,
                                                              const int* __restrict__ positions,
                                                              const int* __restrict__ slots, TA* __restrict__ q_out,
                                                              TA* __restrict__ k_cache, TA* __restrict__ v_cache, int H,
                                                              int G, int DK, int DV, int ROT, float base) {
  extern __shared__ float cs[];  // cos[ROT / 2] | sin[ROT / 2]
  const int t = blockIdx.x, tid = threadIdx.x, half = ROT >> 1;
  const double pos = (double)positions[t], l2b = log2((double)base);
  for (int i = tid; i < half; i += 256) {
    const double a = pos * exp2(-(double)(2 * i) / (double)ROT * l2b);
    const double r = a - 6.283185307179586476925 * rint(a * 0.15915494309189533577);
    float sn, c;
    sincosf((float)r, &sn, &c);
    cs[i] = c;
    cs[half + i] = sn;
  }
  __syncthreads();
  const int slot = slots[t];
  const size_t page = slot >> 4;
  const int off = slot & 15, hp = DK >> 1;  // pairs of a head; an odd last channel is handled with the rest
  const TI* qr = q + (size_t)t * ldq;
  const TI* kr = k + (size_t)t * ldk;
  TA* qo = q_out + (size_t)t * H * DK;
  for (int x = tid; x < (H + G) * hp; x += 256) {
    const int hh = x / hp, i = x - hh * hp;
    const bool isq = hh < H;
    const int g = isq ? hh : hh - H;
    const TI* src = (isq ? qr : kr) + (size_t)g * DK + 2 * i;
    TA* dst = isq ? qo + (size_t)g * DK + 2 * i : k_cache + ((page * G + g) * 16 + off) * DK + 2 * i;
    const float u = (float)src[0], w = (float)src[1];
    if (i < half) {
      const float c = cs[i], sn = cs[half + i];
      dst[0] = (TA)(u * c - w * sn);
      dst[1] = (TA)(w * c + u * sn);
    } else {
      dst[0] = (TA)u;
      dst[1] = (TA)w;
    }
  }
  if (DK & 1) {
    for (int hh = tid; hh < H + G; hh += 256) {
      const bool isq = hh < H;
      const int g = isq ? hh : hh - H;
      const TI xv = ((isq ? qr : kr) + (size_t)g * DK)[DK - 1];
      if (isq) qo[(size_t)g * DK + DK - 1] = (TA)(float)xv;
      else k_cache[((page * G + g) * 16 + off) * DK + DK - 1] = (TA)(float)xv;
    }
  }
  const int NV = G * DV;
  const TI* vr = v + (size_t)t * ldv;
  for (int i = tid; i < NV; i += 256) {
    const int g = i / DV, c = i - g * DV;
    v_cache[((page * G + g) * DV + c) * 16 + off] = (TA)(float)vr[i];
  }
}

constexpr int kMaxVChunks = 8;  // DV <= 512

template <typename TA, bool SIG>
__global__ __launch_bounds__(256) void window_attention_kernel(
    const TA* __restrict__ q, const TA* __restrict__ k_cache, const TA* __restrict__ v_cache,
    const int* __restrict__ block_tables, int maxb, const int* __restrict__ cu_q, const int* __restrict__ ctx, int S,
    TA* __restrict__ out, int ldo, int TH, int H, int G, int DK, int DV, float scale, float softcap, int window,
    const float* __restrict__ r1, const float* __restrict__ r2, const TA* __restrict__ gate, int ldg, int skip_len,
    const float* __restrict__ sig_bias, float out_scale, int nsplit, float* __restrict__ part, int chunk,
    const float* __restrict__ hscale, int has_sink, float sink) {
  extern __shared__ float lds[];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int th = blockIdx.x * 4 + wid;
  if (th >= TH) return;  // wave-uniform; no workgroup barrier below
  float* qs = lds + wid * (DK + 64);
  float* ps = qs + DK;
  const int t = th / H, h = th - t * H, g = h / (H / G);
  int lo = 0, hi = S;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int s = lo, c0 = cu_q[s];
  if (cu_q[s + 1] - c0 >= skip_len) return;  // long portions run on the matrix-core kernel
  const int pos = ctx[s] - (cu_q[s + 1] - c0) + (t - c0);
  int first = window > 0 ? max(0, pos - window + 1) : 0;
  if (chunk > 0) first = max(first, pos / chunk * chunk);
  if (hscale) scale *= hscale[h];
  const TA* qr = q + (size_t)th * DK;
  for (int i = lane; i < DK; i += 64) qs[i] = (float)qr[i];
  __builtin_amdgcn_wave_barrier();
  const float b1 = r1 ? r1[h] : 0.f, b2 = r1 ? r2[h] : 0.f;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const float pb = (SIG && sig_bias) ? sig_bias[h] : 0.f;
  const int* bt = block_tables + (size_t)s * maxb;
  float m = -INFINITY, l = 0.f, acc[kMaxVChunks];
#pragma unroll
  for (int n = 0; n < kMaxVChunks; ++n) acc[n] = 0.f;
  // decode steps: the key blocks of a row are dealt out to nsplit waves (blockIdx.y). Sigmoid mode: their unnormalised
  // partial sums are added up by sigmoid_split_reduce_kernel (no softmax state to merge); softmax mode: every split
  // leaves (sums, running maximum, denominator) and softmax_split_reduce_kernel merges them
  int kb0 = first & ~15, kb1 = pos;
  if (nsplit > 1) {
    const int nblk = (pos - kb0) / 64 + 1, per = (nblk + nsplit - 1) / nsplit;
    kb0 += (int)blockIdx.y * per * 64;
    kb1 = min(pos, kb0 + per * 64 - 1);
  }
  for (int kb = kb0; kb <= kb1; kb += 64) {
    const int p = kb + lane;
    const bool valid = p >= first && p <= pos;
    float sc = -INFINITY;
    if (valid) {
      const size_t page = bt[p >> 4];
      sc = dot_row(qs, k_cache + ((page * G + g) * 16 + (p & 15)) * DK, DK) * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc * inv_cap);
      if (r1) sc -= b1 * log1pf(b2 * (float)(pos - p));
    }
    float pe;
    if (SIG) {
      pe = valid ? 1.0f / (1.0f + expf(-(sc + pb))) : 0.f;
    } else {
      const float m_new = fmaxf(m, wave_max(sc));
      pe = valid ? expf(sc - m_new) : 0.f;
      const float alpha = expf(m - m_new);
      l = l * alpha + wave_sum(pe);
      m = m_new;
#pragma unroll
      for (int n = 0; n < kMaxVChunks; ++n) acc[n] *= alpha;
    }
    __builtin_amdgcn_wave_barrier();  // the previous block's reads of ps are done
    ps[lane] = pe;
    __builtin_amdgcn_wave_barrier();
    for (int pg = 0; pg < 4; ++pg) {
      const int pp = kb + 16 * pg;
      if (pp > pos) break;
      if (pp + 15 < first) continue;
      const size_t page = bt[pp >> 4];
#pragma unroll
      for (int n = 0; n < kMaxVChunks; ++n) {
        const int c = lane + 64 * n;
        if (c < DV) acc[n] += pv16(ps + 16 * pg, v_cache + ((page * G + g) * DV + c) * 16);
      }
    }
  }
  if (nsplit > 1) {
    float* po = part + ((size_t)blockIdx.y * TH + th) * (SIG ? DV : DV + 2);
#pragma unroll
    for (int n = 0; n < kMaxVChunks; ++n) {
      const int c = lane + 64 * n;
      if (c < DV) po[c] = acc[n];
    }
    if (!SIG && lane == 0) {
      po[DV] = m;
      po[DV + 1] = l;
    }
    return;
  }
  float inv_l = out_scale;
  if (!SIG) {
    if (has_sink) {  // a virtual key of score `sink` without a value
      const float m_fin = fmaxf(m, sink), f = expf(m - m_fin);
      l = l * f + expf(sink - m_fin);
      inv_l *= f;
    }
    inv_l /= l;
  }
  TA* o = out + (size_t)t * ldo + (size_t)h * DV;
#pragma unroll
  for (int n = 0; n < kMaxVChunks; ++n) {
    const int c = lane + 64 * n;
    if (c < DV) {
      float y = acc[n] * inv_l;
      if (gate) y *= 1.0f / (1.0f + expf(-(float)gate[(size_t)t * ldg + (size_t)h * DV + c]));
      o[c] = (TA)y;
    }
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void sigmoid_split_reduce_kernel(const float* __restrict__ part, int nsplit,
                                                                   TA* __restrict__ out, int ldo, int T, int HDV,
                                                                   float out_scale) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)T * HDV) return;
  const int t = (int)(e / HDV), c = (int)(e % HDV);
  float a = 0.f;
  for (int sp = 0; sp < nsplit; ++sp) a += part[(size_t)sp * T * HDV + e];
  out[(size_t)t * ldo + c] = (TA)(a * out_scale);
}

// out = sum_s acc_s exp(m_s - M) / sum_s l_s exp(m_s - M), M = max_s m_s (a split without keys has m = -inf, l = 0)
template <typename TA>
__global__ __launch_bounds__(256) void softmax_split_reduce_kernel(const float* __restrict__ part, int nsplit,
                                                                   TA* __restrict__ out, int ldo, int T, int H, int DV,
                                                                   const TA* __restrict__ gate, int ldg, float out_scale,
                                                                   int has_sink, float sink) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)T * H * DV) return;
  const int th = (int)(e / DV), c = (int)(e % DV), t = th / H, h = th - t * H;
  const size_t TH = (size_t)T * H, W = DV + 2;
  float M = has_sink ? sink : -INFINITY;
  for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, part[((size_t)sp * TH + th) * W + DV]);
  float num = 0.f, den = has_sink ? expf(sink - M) : 0.f;
  for (int sp = 0; sp < nsplit; ++sp) {
    const float* p = part + ((size_t)sp * TH + th) * W;
    const float f = expf(p[DV] - M);
    num = fmaf(p[c], f, num);
    den = fmaf(p[DV + 1], f, den);
  }
  float y = num / den * out_scale;
  if (gate) y *= 1.0f / (1.0f + expf(-(float)gate[(size_t)t * ldg + (size_t)h * DV + c]));
  out[(size_t)t * ldo + (size_t)h * DV + c] = (TA)y;
}

// ---- prompt portions in bf16: query tiles on the matrix cores ------------------------------------------------------
// One wave64 per (32 consecutive queries of a sequence, head); the 4 waves of a workgroup take 4 neighbouring heads of
// the same tile, so with GQA their K / V reads meet in L1. S^T = K.Q^T on v_mfma_f32_32x32x16_bf16 leaves one query per
// lane (both lane halves hold 16 of the block's 32 keys), so cap, distance penalty and the online softmax are
// in-register fp32. P.V runs on the same MFMA with the fp32 weights split into two bf16 terms (p = hi + lo, relative
// error 2^-17: below one rounding of the bf16 values they multiply), accumulated in fp32. K rows and V^T page rows are
// read straight from the paged cache into MFMA fragments (16-byte / 8-byte loads; the key order inside a 16-key step is
// the accumulator's row order, so no shuffle is needed between the two products).
typedef __bf16 bf16x4v __attribute__((ext_vector_type(4)));
constexpr int kTileQ = 32;
constexpr int kMfmaMinLen = 8;   // shorter portions (and decoded tokens) stay on the one-wave-per-row kernel
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMasked = -1e30f;

__device__ __forceinline__ float max_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// tanh through one v_exp_f32 and one reciprocal; a short odd polynomial where the quotient form would cancel
__device__ __forceinline__ float tanh_fast(float y) {
  const float e = __builtin_amdgcn_exp2f(2.0f * kLog2e * y);
  const float big = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
  const float y2 = y * y;
  const float small = y * (1.0f + y2 * (-0.33333334f + y2 * (0.13333334f - 0.053968254f * y2)));
  return fabsf(y) < 0.25f ? small : big;
}

template <int DK, int DV, bool SIG>
__global__ __launch_bounds__(256) void window_attention_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int* __restrict__ block_tables, int maxb, const int* __restrict__ cu_q, const int* __restrict__ ctx, int S,
    bf16* __restrict__ out, int ldo, int H, int G, float scale, float softcap, int window, const float* __restrict__ r1,
    const float* __restrict__ r2, const bf16* __restrict__ gate, int ldg, const float* __restrict__ sig_bias,
    float out_scale, int chunk, const float* __restrict__ hscale, int has_sink, float sink) {
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wid;
  if (h >= H) return;
  if (hscale) scale *= hscale[h];
  // tile -> (sequence, first row): sequences of at least kMfmaMinLen rows own ceil(len / 32) tiles each
  int s = 0, seen = 0, len = 0;
  for (; s < S; ++s) {
    len = cu_q[s + 1] - cu_q[s];
    const int nt = len >= kMfmaMinLen ? (len + kTileQ - 1) / kTileQ : 0;
    if ((int)blockIdx.x < seen + nt) break;
    seen += nt;
  }
  if (s == S) return;
  const int row0 = ((int)blockIdx.x - seen) * kTileQ, nrows = min(kTileQ, len - row0);
  const int qi = lane & 31, hb = lane >> 5, g = h / (H / G);
  const bool valid = qi < nrows;
  const int t = cu_q[s] + row0 + min(qi, nrows - 1);
  const int pos0 = ctx[s] - len + row0;             // position of the tile's first query
  const int pos = pos0 + min(qi, nrows - 1), last = pos0 + nrows - 1;
  int first = window > 0 ? max(0, pos0 - window + 1) : 0;
  if (chunk > 0) first = max(first, pos0 / chunk * chunk);
  const int qfirst = chunk > 0 ? pos / chunk * chunk : 0;  // the first key this lane's query sees in chunk mode
  const int* bt = block_tables + (size_t)s * maxb;
  bf16x8 qf[DK / 16];
  const bf16* qr = q + ((size_t)t * H + h) * DK + 8 * hb;
#pragma unroll
  for (int i = 0; i < DK / 16; ++i) qf[i] = load8(qr + 16 * i);
  f32x16 acc_o[DV / 32];
#pragma unroll
  for (int i = 0; i < DV / 32; ++i) acc_o[i] = f32x16{};
  float m_run = kMasked, l_run = 0.f;
  const float b1 = r1 ? r1[h] : 0.f, b2 = r1 ? r2[h] : 0.f;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const float pb = (SIG && sig_bias) ? sig_bias[h] : 0.f;
  for (int kb = first & ~31; kb <= last; kb += 32) {
    // ---- S^T block: rows = keys kb .. kb + 31, columns = the tile's queries
    const int kn = min(kb + qi, last);  // keys past the tile's last position: any valid row (masked below)
    const bf16* kr = k_cache + (((size_t)bt[kn >> 4] * G + g) * 16 + (kn & 15)) * DK + 8 * hb;
    f32x16 sc = f32x16{};
#pragma unroll
    for (int i = 0; i < DK / 16; ++i) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(load8(kr + 16 * i), qf[i], sc, 0, 0, 0);
    float mt = kMasked;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int dist = pos - (kb + (r & 3) + 8 * (r >> 2) + 4 * hb);
      float x = sc[r] * scale;
      if (softcap > 0.f) x = softcap * tanh_fast(x * inv_cap);
      if (r1) x -= b1 * (0.6931471805599453f * __builtin_amdgcn_logf(fmaf(b2, (float)max(dist, 0), 1.0f)));
      const bool ok = valid && dist >= 0 && (window <= 0 || dist < window) && pos - dist >= qfirst;
      x = ok ? x : kMasked;
      sc[r] = x;
      mt = fmaxf(mt, x);
    }
    if (SIG) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        sc[r] = sc[r] > 0.5f * kMasked
                    ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-(sc[r] + pb) * kLog2e)) : 0.f;
    } else {
      mt = max_halves(mt);
      const float m_new = fmaxf(m_run, mt);
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * kLog2e);
      m_run = m_new;
      float rs = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = sc[r] > 0.5f * kMasked ? __builtin_amdgcn_exp2f((sc[r] - m_new) * kLog2e) : 0.f;
        sc[r] = p;
        rs += p;
      }
      l_run = l_run * alpha + rs;
#pragma unroll
      for (int i = 0; i < DV / 32; ++i) acc_o[i] *= alpha;
    }
    // ---- O^T += V^T . P^T, one 16-key page per step
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int kp = kb + 16 * ks;
      if (kp > last) break;
      bf16x8 ph, pl;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = sc[8 * ks + e];
        ph[e] = (bf16)p;
        pl[e] = (bf16)(p - (float)ph[e]);
      }
      const bf16* vr = v_cache + (((size_t)bt[kp >> 4] * G + g) * DV + qi) * 16 + 4 * hb;
#pragma unroll
      for (int i = 0; i < DV / 32; ++i) {
        const bf16x4v a = *reinterpret_cast<const bf16x4v*>(vr + (size_t)32 * i * 16);
        const bf16x4v b = *reinterpret_cast<const bf16x4v*>(vr + (size_t)32 * i * 16 + 8);
        const bf16x8 vf = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, ph, acc_o[i], 0, 0, 0);
        acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pl, acc_o[i], 0, 0, 0);
      }
    }
  }
  float l = sum_halves(l_run);
  if (!valid) return;
  float inv_l = out_scale;
  if (!SIG) {
    if (has_sink) {  // a virtual key of score `sink` without a value
      const float m_fin = fmaxf(m_run, sink), f = expf(m_run - m_fin);
      l = l * f + expf(sink - m_fin);
      inv_l *= f;
    }
    inv_l /= l;
  }
  bf16* o = out + (size_t)t * ldo + (size_t)h * DV;
  const bf16* gr = gate ? gate + (size_t)t * ldg + (size_t)h * DV : nullptr;
#pragma unroll
  for (int i = 0; i < DV / 32; ++i) {
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int c = 32 * i + 8 * r4 + 4 * hb;
      bf16x4v y;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = acc_o[i][4 * r4 + e] * inv_l;
        if (gr) v *= 1.0f / (1.0f + __expf(-(float)gr[c + e]));
        y[e] = (bf16)v;
      }
      *reinterpret_cast<bf16x4v*>(o + c) = y;
    }
  }
}

template <int DK, int DV>
void launch_window_mfma(const void* q, const void* k_cache, const void* v_cache, const int* block_tables, int maxb,
                        const int* cu_q, const int* ctx, int S, void* out, int ldo, int T, int H, int G, float scale,
                        float softcap, int window, const float* r1, const float* r2, const void* gate, int ldg,
                        const float* sig_bias, int sig, float out_scale, hipStream_t st, int chunk, const float* hscale,
                        int has_sink, float sink) {
  const dim3 grid((T + kTileQ - 1) / kTileQ + S, (H + 3) / 4);
  if (sig)
    window_attention_mfma_kernel<DK, DV, true><<<grid, 256, 0, st>>>(
        (const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, block_tables, maxb, cu_q, ctx, S, (bf16*)out, ldo, H,
        G, scale, softcap, window, r1, r2, (const bf16*)gate, ldg, sig_bias, out_scale, chunk, hscale, has_sink, sink);
  else
    window_attention_mfma_kernel<DK, DV, false><<<grid, 256, 0, st>>>(
        (const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, block_tables, maxb, cu_q, ctx, S, (bf16*)out, ldo, H,
        G, scale, softcap, window, r1, r2, (const bf16*)gate, ldg, sig_bias, out_scale, chunk, hscale, has_sink, sink);
}

}  // namespace

void gai_qknorm_kv_write(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* wq,
                         const float* wk, const int* slots, void* q_out, void* k_cache, void* v_cache, int T, int H,
                         int G, int DK, int DV, float eps, int dt, hipStream_t st) {
  if (T == 0) return;
  if (dt)
    qknorm_kv_write_kernel<float><<<T, 256, 0, st>>>((const float*)q, ldq, (const float*)k, ldk, (const float*)v, ldv, wq,
                                                     wk, slots, (float*)q_out, (float*)k_cache, (float*)v_cache, H, G,
                                                     DK, DV, eps);
  else
    qknorm_kv_write_kernel<bf16><<<T, 256, 0, st>>>((const bf16*)q, ldq, (const bf16*)k, ldk, (const bf16*)v, ldv, wq, wk,
                                                    slots, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, H, G, DK, DV,
                                                    eps);
  GAI_LAUNCH_CHECK();
}

void gai_headnorm_kv_write(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* wq,
                           const float* wk, const int* slots, const int* positions, void* q_out, void* k_cache,
                           void* v_cache, int T, int H, int G, int DK, int DV, float eps, float temp_coef, int temp_every,
                           int dt, hipStream_t st) {
  if (T == 0) return;
  if (temp_every < 1) gai_launch_error(__FILE__, __LINE__, "headnorm_kv_write: temperature period must be >= 1");
  if (dt)
    headnorm_kv_write_kernel<float><<<T, 256, 0, st>>>((const float*)q, ldq, (const float*)k, ldk, (const float*)v, ldv,
                                                       wq, wk, slots, positions, (float*)q_out, (float*)k_cache,
                                                       (float*)v_cache, H, G, DK, DV, eps, temp_coef, temp_every);
  else
    headnorm_kv_write_kernel<bf16><<<T, 256, 0, st>>>((const bf16*)q, ldq, (const bf16*)k, ldk, (const bf16*)v, ldv, wq,
                                                      wk, slots, positions, (bf16*)q_out, (bf16*)k_cache,
                                                      (bf16*)v_cache, H, G, DK, DV, eps, temp_coef, temp_every);
  GAI_LAUNCH_CHECK();
}

void gai_latent_kv_write(const void* q, int ldq, const void* dkv, int ldk, const float* nw, const float* inv_freq,
                         float mag, const int* positions, const int* slots, void* q_cat, void* k_cache, void* v_cache,
                         int T, int H, int DN, int DR, int R, float eps, int dt, hipStream_t st, int ROT) {
  if (T == 0) return;
  if (ROT % 2 || ROT < 0 || ROT > DR || R < 1)
    gai_launch_error(__FILE__, __LINE__, "latent_kv_write: an even number of rotated channels within DR, latent size >= 1");
  const size_t lds = (size_t)(ROT > 0 ? ROT : 1) * sizeof(float);
  if (dt)
    latent_kv_write_kernel<float><<<T, 256, lds, st>>>((const float*)q, ldq, (const float*)dkv, ldk, nw, inv_freq, mag,
                                                       positions, slots, (float*)q_cat, (float*)k_cache,
                                                       (float*)v_cache, H, DN, DR, R, eps, ROT);
  else
    latent_kv_write_kernel<bf16><<<T, 256, lds, st>>>((const bf16*)q, ldq, (const bf16*)dkv, ldk, nw, inv_freq, mag,
                                                      positions, slots, (bf16*)q_cat, (bf16*)k_cache, (bf16*)v_cache, H,
                                                      DN, DR, R, eps, ROT);
  GAI_LAUNCH_CHECK();
}

// dt_in / dt: 0 = bf16, 1 = fp32 (inputs may be fp32 while the cache is bf16: the output of an fp32 convolution)
void gai_rotary_kv_write(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const int* positions,
                         const int* slots, void* q_out, void* k_cache, void* v_cache, int T, int H, int G, int DK, int DV,
                         int ROT, float base, int dt_in, int dt, hipStream_t st) {
  if (T == 0) return;
  if (ROT % 2 || ROT < 0 || ROT > DK) gai_launch_error(__FILE__, __LINE__, "rotary_kv_write: an even number of rotated channels within a head");
  if (!dt_in && dt) gai_launch_error(__FILE__, __LINE__, "rotary_kv_write: bf16 inputs go with a bf16 cache");
  const size_t lds = (size_t)(ROT > 0 ? ROT : 1) * sizeof(float);
#define GAI_ROT(TI, TA)                                                                                              \
  rotary_kv_write_kernel<TI, TA><<<T, 256, lds, st>>>((const TI*)q, ldq, (const TI*)k, ldk, (const TI*)v, ldv, positions, \
                                                      slots, (TA*)q_out, (TA*)k_cache, (TA*)v_cache, H, G, DK, DV, ROT, \
                                                      base)
  if (dt_in && dt) GAI_ROT(float, float); else if (dt_in) GAI_ROT(float, bf16); else GAI_ROT(bf16, bf16);
#undef GAI_ROT
  GAI_LAUNCH_CHECK();
}

// Key splits of a decode step (every row a single token): enough waves to give each SIMD a few
int gai_sigmoid_attention_splits(int T, int S, int H) {
  if (T != S || T * H >= 2048) return 1;
  int n = 4096 / (T * H);
  return n > 16 ? 16 : (n < 1 ? 1 : n);
}

void gai_window_attention(const void* q, const void* k_cache, const void* v_cache, const int* block_tables, int maxb,
                          const int* cu_q, const int* ctx, int S, void* out, int ldo, int T, int H, int G, int DK, int DV,
                          float scale, float softcap, int window, const float* r1, const float* r2, const void* gate,
                          int ldg, const float* sig_bias, int sig, float out_scale, int dt, hipStream_t st,
                          float* part, int chunk, const float* hscale, int has_sink, float sink) {
  if (T == 0 || S == 0) return;
  if (sig && (chunk > 0 || hscale || has_sink))
    gai_launch_error(__FILE__, __LINE__, "window_attention: chunks, head scales and sinks go with the softmax mode");
  if (DV > 64 * kMaxVChunks) gai_launch_error(__FILE__, __LINE__, "window_attention: value head size above 512");
  if (H % G) gai_launch_error(__FILE__, __LINE__, "window_attention: heads must be a multiple of kv heads");
  const int TH = T * H, grid = (TH + 3) / 4;
  const size_t lds = 4 * (size_t)(DK + 64) * sizeof(float);
  // bf16 steps with prompt portions (more rows than sequences): portions of >= kMfmaMinLen rows go to the query-tiled
  // matrix-core kernel for the head sizes it is instantiated for; the rest runs below
  int skip_len = 0x7fffffff;
  if (!dt && T > S && (!gate || ldg % 4 == 0) && ldo % 4 == 0) {
#define GAI_WIN(K_, V_)                                                                                              \
  if (DK == K_ && DV == V_) {                                                                                        \
    launch_window_mfma<K_, V_>(q, k_cache, v_cache, block_tables, maxb, cu_q, ctx, S, out, ldo, T, H, G, scale,      \
                               softcap, window, r1, r2, gate, ldg, sig_bias, sig, out_scale, st, chunk, hscale,       \
                               has_sink, sink);                                                                      \
    skip_len = kMfmaMinLen;                                                                                          \
  }
    GAI_WIN(64, 64) GAI_WIN(64, 128) GAI_WIN(128, 64) GAI_WIN(128, 128) GAI_WIN(256, 256)
    // latent rows: key row = latent + rotated part, value row = latent
    GAI_WIN(96, 64) GAI_WIN(192, 128) GAI_WIN(320, 256)
#undef GAI_WIN
    GAI_LAUNCH_CHECK();
  }
  const int nsplit = part ? gai_sigmoid_attention_splits(T, S, H) : 1;
#define GAI_ROW(TA, SIG_)                                                                                            \
  window_attention_kernel<TA, SIG_><<<dim3(grid, nsplit), 256, lds, st>>>(                                           \
      (const TA*)q, (const TA*)k_cache, (const TA*)v_cache, block_tables, maxb, cu_q, ctx, S, (TA*)out, ldo, TH, H, G, \
      DK, DV, scale, softcap, window, r1, r2, (const TA*)gate, ldg, skip_len, sig_bias, out_scale, nsplit, part,    \
      chunk, hscale, has_sink, sink)
  if (dt) {
    if (sig) GAI_ROW(float, true); else GAI_ROW(float, false);
  } else {
    if (sig) GAI_ROW(bf16, true); else GAI_ROW(bf16, false);
  }
#undef GAI_ROW
  if (nsplit > 1 && !sig) {
    const long n = (long)T * H * DV;
    if (dt)
      softmax_split_reduce_kernel<float><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(part, nsplit, (float*)out, ldo, T, H,
                                                                                       DV, (const float*)gate, ldg,
                                                                                       out_scale, has_sink, sink);
    else
      softmax_split_reduce_kernel<bf16><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(part, nsplit, (bf16*)out, ldo, T, H,
                                                                                      DV, (const bf16*)gate, ldg,
                                                                                      out_scale, has_sink, sink);
  } else if (nsplit > 1) {
    const long n = (long)T * H * DV;
    if (dt)
      sigmoid_split_reduce_kernel<float><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(part, nsplit, (float*)out, ldo, T,
                                                                                       H * DV, out_scale);
    else
      sigmoid_split_reduce_kernel<bf16><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(part, nsplit, (bf16*)out, ldo, T,
                                                                                      H * DV, out_scale);
  }
  GAI_LAUNCH_CHECK();
}
