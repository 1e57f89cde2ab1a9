// Normalisations around a 32-bit residual stream (hybrid decoders whose residual sum, norms and recurrent
// inputs stay in fp32 while the matrix products run in bf16).
//
//   add_rmsnorm_f32   res += mult * delta;  out = res * rsqrt(mean(res^2) + eps) * w      (w = nullptr: out = res)
//   poly_norm         y = a N(z) + b N(z^2) + c N(z^3) + e,  N(t) = t * rsqrt(mean(t^2) + eps) over the row
//   head_norm_gate    y = o * rsqrt(mean_head(o^2) + eps) * nw * act(gate)   (act: silu | sigmoid), one head per wave
//   embed_scale_f32   out = table[id] * scale as fp32 (+ pos_table[position]: learned absolute positions)
//   gated_norm_add    g = y * sigmoid(gate) (gate = nullptr: g = y);  res += g * rsqrt(mean(g^2) + eps) * wpost;  out = rmsnorm(res) * wnext
//                     (post-norm gated residual: the closing norm of a sublayer, the residual add and the opening norm
//                     of the next sublayer in one pass)
//   gate_group_norm   g = y * silu(z);  out = g * rsqrt(mean_group(g^2) + eps) * w, the row cut into equal groups
//   add_dyt_f32       res += delta (+ extra);  out = tanh(alpha * res) * w + b   (dynamic tanh: a norm without statistics,
//                     so the pass is purely element-wise: four elements per thread, no reduction)
//   act_mul           out = act(a) (* b), act: silu | squared ReLU | cap * tanh(a / cap) | tanh GELU, or the clamped gated
//                     activation min(a, cap) * sigmoid(1.702 min(a, cap)) * (clamp(b, +-cap) + 1); fp32 arithmetic, a / b column
//                     slices of wider rows, out bf16 or fp32
//
// Activations (delta, z, gate, out, y) are bf16 or fp32 (template TA); every statistic and product is fp32.
// One wave64 per row for the row norms (D of a few thousand: the row is re-read from L2 in the second pass).
#include "gai_common.h"
#include "gai_kernels.h"

using namespace gai;

namespace {

template <typename TD, typename TA>
__global__ __launch_bounds__(256) void add_rmsnorm_f32_kernel(float* __restrict__ res, const TD* __restrict__ delta,
                                                              int ldd, float mult, const float* __restrict__ w,
                                                              TA* __restrict__ out, int T, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  float* r = res + (size_t)row * D;
  float s = 0.f;
  if (delta) {
    const TD* d = delta + (size_t)row * ldd;
    for (int i = lane; i < D; i += 64) {
      const float v = r[i] + mult * (float)d[i];
      r[i] = v;
      s += v * v;
    }
  } else {
    for (int i = lane; i < D; i += 64) {
      const float v = r[i];
      s += v * v;
    }
  }
  if (!out) return;
  TA* o = out + (size_t)row * D;
  if (!w) {
    for (int i = lane; i < D; i += 64) o[i] = (TA)r[i];
    return;
  }
  s = wave_sum(s);
  const float inv = 1.0f / sqrtf(s / D + eps);
  for (int i = lane; i < D; i += 64) o[i] = (TA)(r[i] * inv * w[i]);
}

// Few rows (decode steps): one workgroup per row instead of one wave, the summed values kept in registers between the
// passes (rows up to 256 * kAddWideRegs wide; wider rows re-read them).
constexpr int kAddWideRegs = 16;

template <typename TD, typename TA>
__global__ __launch_bounds__(256) void add_rmsnorm_f32_wide_kernel(float* __restrict__ res, const TD* __restrict__ delta,
                                                                   int ldd, float mult, const float* __restrict__ w,
                                                                   TA* __restrict__ out, int D, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  float* r = res + (size_t)row * D;
  const TD* d = delta ? delta + (size_t)row * ldd : nullptr;
  float v[kAddWideRegs];
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kAddWideRegs; ++q) {
    const int i = tid + 256 * q;
    v[q] = 0.f;
    if (i < D) {
      v[q] = d ? r[i] + mult * (float)d[i] : r[i];
      if (d) r[i] = v[q];
      s += v[q] * v[q];
    }
  }
  for (int i = tid + 256 * kAddWideRegs; i < D; i += 256) {
    const float x = d ? r[i] + mult * (float)d[i] : r[i];
    if (d) r[i] = x;
    s += x * x;
  }
  if (!out) return;
  TA* o = out + (size_t)row * D;
  float inv = 1.0f;
  if (w) {
    s = block_sum(s, scratch);
    inv = 1.0f / sqrtf(s / D + eps);
  }
#pragma unroll
  for (int q = 0; q < kAddWideRegs; ++q) {
    const int i = tid + 256 * q;
    if (i < D) o[i] = (TA)(w ? v[q] * inv * w[i] : v[q]);
  }
  for (int i = tid + 256 * kAddWideRegs; i < D; i += 256) o[i] = (TA)(w ? r[i] * inv * w[i] : r[i]);
}

template <typename TA>
__global__ __launch_bounds__(256) void poly_norm_kernel(const TA* __restrict__ z, TA* __restrict__ y,
                                                        const float* __restrict__ coef, int F, float eps) {
  __shared__ float scratch[16];
  const TA* zr = z + (size_t)blockIdx.x * F;
  TA* yr = y + (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int i = threadIdx.x; i < F; i += 256) {
    const float v = (float)zr[i], v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  s1 = block_sum(s1, scratch);
  s2 = block_sum(s2, scratch);
  s3 = block_sum(s3, scratch);
  const float a = coef[0] / sqrtf(s1 / F + eps), b = coef[1] / sqrtf(s2 / F + eps), c = coef[2] / sqrtf(s3 / F + eps);
  const float e = coef[3];
  for (int i = threadIdx.x; i < F; i += 256) {
    const float v = (float)zr[i];
    yr[i] = (TA)(a * v + b * v * v + c * v * v * v + e);
  }
}

// few wide rows (a whole-row norm in a decode step): one workgroup per (token, head), values kept in registers
template <typename TA>
__global__ __launch_bounds__(256) void head_norm_gate_wide_kernel(const float* __restrict__ o, const TA* __restrict__ gate,
                                                                  int ldg, const float* __restrict__ nw, int nw_per_head,
                                                                  int act, TA* __restrict__ y, int ldy, int H, int DV,
                                                                  float eps) {
  constexpr int kMax = 32;  // DV <= 8192
  __shared__ float scratch[16];
  const int th = blockIdx.x, t = th / H, h = th % H, tid = threadIdx.x;
  const float* orow = o + (size_t)th * DV;
  float v[kMax];
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kMax; ++q) {
    const int i = tid + 256 * q;
    v[q] = i < DV ? orow[i] : 0.f;
    s += v[q] * v[q];
  }
  s = block_sum(s, scratch);
  const float inv = 1.0f / sqrtf(s / DV + eps);
  const TA* g = gate + (size_t)t * ldg + (size_t)h * DV;
  const float* wr = nw + (nw_per_head ? (size_t)h * DV : 0);
  TA* yr = y + (size_t)t * ldy + (size_t)h * DV;
#pragma unroll
  for (int q = 0; q < kMax; ++q) {
    const int i = tid + 256 * q;
    if (i < DV) {
      const float gv = (float)g[i];
      const float sg = 1.0f / (1.0f + expf(-gv));
      yr[i] = (TA)(v[q] * inv * wr[i] * (act == 0 ? gv * sg : sg));
    }
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const TA* __restrict__ gate,
                                                             int ldg, const float* __restrict__ nw, int nw_per_head,
                                                             int act, TA* __restrict__ y, int ldy, int TH, int H,
                                                             int DV, float eps) {
  const int lane = threadIdx.x & 63;
  const int th = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (th >= TH) return;
  const int t = th / H, h = th % H;
  const float* orow = o + (size_t)th * DV;
  float s = 0.f;
  for (int i = lane; i < DV; i += 64) s += orow[i] * orow[i];
  s = wave_sum(s);
  const float inv = 1.0f / sqrtf(s / DV + eps);
  const TA* g = gate + (size_t)t * ldg + (size_t)h * DV;
  const float* wr = nw + (nw_per_head ? (size_t)h * DV : 0);
  TA* yr = y + (size_t)t * ldy + (size_t)h * DV;
  for (int i = lane; i < DV; i += 64) {
    const float gv = (float)g[i];
    const float sg = 1.0f / (1.0f + expf(-gv));
    yr[i] = (TA)(orow[i] * inv * wr[i] * (act == 0 ? gv * sg : sg));
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void embed_scale_f32_kernel(const int* __restrict__ ids, const TA* __restrict__ table,
                                                              float scale, float* __restrict__ out, int T, int D,
                                                              int V, const int* __restrict__ positions,
                                                              const TA* __restrict__ pos_table, int P) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const TA* e = table + (size_t)id * D;
  float* o = out + (size_t)row * D;
  if (pos_table) {
    int p = positions[row];
    p = p < 0 ? 0 : (p >= P ? P - 1 : p);
    const TA* pe = pos_table + (size_t)p * D;
    for (int i = lane; i < D; i += 64) o[i] = (float)e[i] * scale + (float)pe[i];
  } else {
    for (int i = lane; i < D; i += 64) o[i] = (float)e[i] * scale;
  }
}

template <typename TY, typename TG, typename TA>
__global__ __launch_bounds__(256) void gated_norm_add_kernel(float* __restrict__ res, const TY* __restrict__ y, int ldy,
                                                             const TG* __restrict__ gate, int ldg,
                                                             const float* __restrict__ wpost,
                                                             const float* __restrict__ wnext, TA* __restrict__ out,
                                                             int T, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= T) return;
  float* r = res + (size_t)row * D;
  const TY* yr = y + (size_t)row * ldy;
  const TG* gr = gate + (size_t)row * ldg;
  float s = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float g = gate ? (float)yr[i] / (1.0f + expf(-(float)gr[i])) : (float)yr[i];
    s += g * g;
  }
  s = wave_sum(s);
  const float inv = 1.0f / sqrtf(s / D + eps);
  float s2 = 0.f;
  for (int i = lane; i < D; i += 64) {
    const float g = gate ? (float)yr[i] / (1.0f + expf(-(float)gr[i])) : (float)yr[i];
    const float v = r[i] + g * inv * wpost[i];
    r[i] = v;
    s2 += v * v;
  }
  if (!out) return;
  TA* o = out + (size_t)row * D;
  if (!wnext) {
    for (int i = lane; i < D; i += 64) o[i] = (TA)r[i];
    return;
  }
  s2 = wave_sum(s2);
  const float inv2 = 1.0f / sqrtf(s2 / D + eps);
  for (int i = lane; i < D; i += 64) o[i] = (TA)(r[i] * inv2 * wnext[i]);
}

// Few rows (decode steps): one workgroup per row instead of one wave, the gated values kept in registers between the
// passes (rows up to 256 * kWideRegs wide; wider rows recompute them).
constexpr int kWideRegs = 16;

template <typename TY, typename TG, typename TA>
__global__ __launch_bounds__(256) void gated_norm_add_wide_kernel(float* __restrict__ res, const TY* __restrict__ y,
                                                                  int ldy, const TG* __restrict__ gate, int ldg,
                                                                  const float* __restrict__ wpost,
                                                                  const float* __restrict__ wnext, TA* __restrict__ out,
                                                                  int D, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, tid = threadIdx.x;
  float* r = res + (size_t)row * D;
  const TY* yr = y + (size_t)row * ldy;
  const TG* gr = gate + (size_t)row * ldg;
  float g[kWideRegs];
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kWideRegs; ++q) {
    const int i = tid + 256 * q;
    g[q] = i < D ? (gate ? (float)yr[i] / (1.0f + expf(-(float)gr[i])) : (float)yr[i]) : 0.f;
    s += g[q] * g[q];
  }
  for (int i = tid + 256 * kWideRegs; i < D; i += 256) {
    const float v = gate ? (float)yr[i] / (1.0f + expf(-(float)gr[i])) : (float)yr[i];
    s += v * v;
  }
  s = block_sum(s, scratch);
  const float inv = 1.0f / sqrtf(s / D + eps);
  float s2 = 0.f;
#pragma unroll
  for (int q = 0; q < kWideRegs; ++q) {
    const int i = tid + 256 * q;
    if (i < D) {
      g[q] = r[i] + g[q] * inv * wpost[i];
      r[i] = g[q];
      s2 += g[q] * g[q];
    }
  }
  for (int i = tid + 256 * kWideRegs; i < D; i += 256) {
    const float v = r[i] + (gate ? (float)yr[i] / (1.0f + expf(-(float)gr[i])) : (float)yr[i]) * inv * wpost[i];
    r[i] = v;
    s2 += v * v;
  }
  if (!out) return;
  TA* o = out + (size_t)row * D;
  if (!wnext) {
    for (int i = tid; i < D; i += 256) o[i] = (TA)r[i];
    return;
  }
  s2 = block_sum(s2, scratch);
  const float inv2 = 1.0f / sqrtf(s2 / D + eps);
#pragma unroll
  for (int q = 0; q < kWideRegs; ++q) {
    const int i = tid + 256 * q;
    if (i < D) o[i] = (TA)(g[q] * inv2 * wnext[i]);
  }
  for (int i = tid + 256 * kWideRegs; i < D; i += 256) o[i] = (TA)(r[i] * inv2 * wnext[i]);
}

template <typename TA>
__global__ __launch_bounds__(256) void gate_group_norm_wide_kernel(const float* __restrict__ y, const TA* __restrict__ z,
                                                                   int ldz, const float* __restrict__ w,
                                                                   TA* __restrict__ out, int NG, int GS, float eps) {
  __shared__ float scratch[16];
  const int tg = blockIdx.x, tid = threadIdx.x;
  const int t = tg / NG, g = tg - t * NG;
  const float* yr = y + ((size_t)t * NG + g) * GS;
  const TA* zr = z + (size_t)t * ldz + (size_t)g * GS;
  float v[kWideRegs];
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < kWideRegs; ++q) {
    const int i = tid + 256 * q;
    float x = 0.f;
    if (i < GS) {
      const float zv = (float)zr[i];
      x = yr[i] * zv / (1.0f + expf(-zv));
    }
    v[q] = x;
    s += x * x;
  }
  for (int i = tid + 256 * kWideRegs; i < GS; i += 256) {
    const float zv = (float)zr[i];
    const float x = yr[i] * zv / (1.0f + expf(-zv));
    s += x * x;
  }
  s = block_sum(s, scratch);
  const float inv = 1.0f / sqrtf(s / GS + eps);
  const float* wr = w + (size_t)g * GS;
  TA* o = out + ((size_t)t * NG + g) * GS;
#pragma unroll
  for (int q = 0; q < kWideRegs; ++q) {
    const int i = tid + 256 * q;
    if (i < GS) o[i] = (TA)(v[q] * inv * wr[i]);
  }
  for (int i = tid + 256 * kWideRegs; i < GS; i += 256) {
    const float zv = (float)zr[i];
    o[i] = (TA)(yr[i] * zv / (1.0f + expf(-zv)) * inv * wr[i]);
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void gate_group_norm_kernel(const float* __restrict__ y, const TA* __restrict__ z,
                                                              int ldz, const float* __restrict__ w, TA* __restrict__ out,
                                                              int TG, int NG, int GS, float eps) {
  const int lane = threadIdx.x & 63;
  const int tg = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tg >= TG) return;
  const int t = tg / NG, g = tg - t * NG;
  const float* yr = y + ((size_t)t * NG + g) * GS;
  const TA* zr = z + (size_t)t * ldz + (size_t)g * GS;
  float s = 0.f;
  for (int i = lane; i < GS; i += 64) {
    const float zv = (float)zr[i];
    const float v = yr[i] * zv / (1.0f + expf(-zv));
    s += v * v;
  }
  s = wave_sum(s);
  const float inv = 1.0f / sqrtf(s / GS + eps);
  const float* wr = w + (size_t)g * GS;
  TA* o = out + ((size_t)t * NG + g) * GS;
  for (int i = lane; i < GS; i += 64) {
    const float zv = (float)zr[i];
    o[i] = (TA)(yr[i] * zv / (1.0f + expf(-zv)) * inv * wr[i]);
  }
}

// ---- dynamic tanh norm fused with the residual add --------------------------------------------------------------------
template <typename TD, typename TA, int VEC>
__global__ __launch_bounds__(256) void add_dyt_f32_kernel(float* __restrict__ res, const TD* __restrict__ delta, int ldd,
                                                          const float* __restrict__ extra, float alpha,
                                                          const float* __restrict__ w, const float* __restrict__ b,
                                                          TA* __restrict__ out, int T, int D) {
  const int per = D / VEC;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)T * per) return;
  const int row = (int)(e / per), c0 = (int)(e % per) * VEC;
  float* r = res + (size_t)row * D + c0;
  float v[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) v[i] = r[i];
  if (delta) {
    const TD* d = delta + (size_t)row * ldd + c0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] += (float)d[i];
  }
  if (extra) {
    const float* x = extra + (size_t)row * D + c0;
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] += x[i];
  }
  if (delta || extra) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) r[i] = v[i];
  }
  if (!out) return;
  TA* o = out + (size_t)row * D + c0;
#pragma unroll
  for (int i = 0; i < VEC; ++i) o[i] = (TA)fmaf(tanhf(alpha * v[i]), w[c0 + i], b[c0 + i]);
}

constexpr float kGluSlope = 1.702f;  // slope of the sigmoid in the clamped gated activation

template <typename TI, typename TO, int VEC>
__global__ __launch_bounds__(256) void act_mul_kernel(const TI* __restrict__ a, int lda, const TI* __restrict__ b, int ldb,
                                                      TO* __restrict__ out, int T, int C, int act, float cap) {
  const int per = C / VEC;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)T * per) return;
  const int row = (int)(e / per), c = (int)(e % per) * VEC;
  struct alignas(sizeof(TI) * VEC) VI { TI v[VEC]; };
  struct alignas(sizeof(TO) * VEC) VO { TO v[VEC]; };
  const VI xa = *reinterpret_cast<const VI*>(a + (size_t)row * lda + c);
  VI xb;
  if (b) xb = *reinterpret_cast<const VI*>(b + (size_t)row * ldb + c);
  VO yo;
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    const float x = (float)xa.v[i];
    float y;
    if (act == 0) y = x / (1.0f + expf(-x));
    else if (act == 1) y = fmaxf(x, 0.f) * fmaxf(x, 0.f);
    else if (act == 2) y = cap * tanhf(x / cap);
    else if (act == 3) y = 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    else {  // clamped gated activation of (a, b) with limit cap
      const float g = fminf(x, cap), u = fminf(fmaxf((float)xb.v[i], -cap), cap);
      y = g / (1.0f + expf(-kGluSlope * g)) * (u + 1.0f);
    }
    if (b && act != 4) y *= (float)xb.v[i];
    yo.v[i] = (TO)y;
  }
  *reinterpret_cast<VO*>(out + (size_t)row * C + c) = yo;
}

}  // namespace

void gai_add_rmsnorm_f32(float* res, const void* delta, int ldd, float mult, const float* w, void* out, int T, int D,
                         float eps, int dt_delta, int dt_out, hipStream_t st) {
  if (T == 0) return;
  const int grid = (T + 3) / 4;
  const bool wide = T <= 512 && D >= 512;  // few rows: a workgroup per row
#define GAI_ARN(TD, TA)                                                                                              \
  if (wide)                                                                                                          \
    add_rmsnorm_f32_wide_kernel<TD, TA><<<T, 256, 0, st>>>(res, (const TD*)delta, ldd, mult, w, (TA*)out, D, eps);   \
  else                                                                                                               \
    add_rmsnorm_f32_kernel<TD, TA><<<grid, 256, 0, st>>>(res, (const TD*)delta, ldd, mult, w, (TA*)out, T, D, eps)
  if (dt_delta && dt_out) { GAI_ARN(float, float); }
  else if (dt_delta) { GAI_ARN(float, bf16); }
  else if (dt_out) { GAI_ARN(bf16, float); }
  else { GAI_ARN(bf16, bf16); }
#undef GAI_ARN
  GAI_LAUNCH_CHECK();
}

void gai_poly_norm(const void* z, void* y, const float* coef, int T, int F, float eps, int dt, hipStream_t st) {
  if (T == 0) return;
  if (dt)
    poly_norm_kernel<float><<<T, 256, 0, st>>>((const float*)z, (float*)y, coef, F, eps);
  else
    poly_norm_kernel<bf16><<<T, 256, 0, st>>>((const bf16*)z, (bf16*)y, coef, F, eps);
  GAI_LAUNCH_CHECK();
}

void gai_head_norm_gate(const float* o, const void* gate, int ldg, const float* nw, int nw_per_head, int act, void* y,
                        int ldy, int T, int H, int DV, float eps, int dt, hipStream_t st) {
  if (T == 0) return;
  const int TH = T * H, grid = (TH + 3) / 4;
  if (TH <= 256 && DV >= 1024 && DV <= 8192) {  // few wide rows: a single wave per row would walk it alone
    if (dt)
      head_norm_gate_wide_kernel<float><<<TH, 256, 0, st>>>(o, (const float*)gate, ldg, nw, nw_per_head, act, (float*)y,
                                                            ldy, H, DV, eps);
    else
      head_norm_gate_wide_kernel<bf16><<<TH, 256, 0, st>>>(o, (const bf16*)gate, ldg, nw, nw_per_head, act, (bf16*)y, ldy,
                                                           H, DV, eps);
    GAI_LAUNCH_CHECK();
    return;
  }
  if (dt)
    head_norm_gate_kernel<float><<<grid, 256, 0, st>>>(o, (const float*)gate, ldg, nw, nw_per_head, act, (float*)y, ldy,
                                                        TH, H, DV, eps);
  else
    head_norm_gate_kernel<bf16><<<grid, 256, 0, st>>>(o, (const bf16*)gate, ldg, nw, nw_per_head, act, (bf16*)y, ldy, TH,
                                                       H, DV, eps);
  GAI_LAUNCH_CHECK();
}

void gai_embed_scale_f32(const int* ids, const void* table, float scale, float* out, int T, int D, int V, int dt,
                         hipStream_t st, const int* positions, const void* pos_table, int P) {
  if (T == 0) return;
  const int grid = (T + 3) / 4;
  if (dt)
    embed_scale_f32_kernel<float><<<grid, 256, 0, st>>>(ids, (const float*)table, scale, out, T, D, V, positions,
                                                        (const float*)pos_table, P);
  else
    embed_scale_f32_kernel<bf16><<<grid, 256, 0, st>>>(ids, (const bf16*)table, scale, out, T, D, V, positions,
                                                       (const bf16*)pos_table, P);
  GAI_LAUNCH_CHECK();
}

void gai_gated_norm_add_f32(float* res, const void* y, int ldy, int dt_y, const void* gate, int ldg, int dt_gate,
                            const float* wpost, const float* wnext, void* out, int dt_out, int T, int D, float eps,
                            hipStream_t st) {
  if (T == 0) return;
  const int grid = (T + 3) / 4;
  const bool wide = T <= 512 && D >= 512;  // few rows: a workgroup per row
#define GAI_GNA(TY, TG, TA)                                                                                          \
  if (wide)                                                                                                          \
    gated_norm_add_wide_kernel<TY, TG, TA><<<T, 256, 0, st>>>(res, (const TY*)y, ldy, (const TG*)gate, ldg, wpost,   \
                                                              wnext, (TA*)out, D, eps);                              \
  else                                                                                                               \
    gated_norm_add_kernel<TY, TG, TA><<<grid, 256, 0, st>>>(res, (const TY*)y, ldy, (const TG*)gate, ldg, wpost,     \
                                                            wnext, (TA*)out, T, D, eps)
  if (!gate) dt_gate = dt_y;  // no gate: the gate type is not read
  if (dt_y && dt_gate && (dt_out || !out)) { GAI_GNA(float, float, float); }
  else if (dt_y && dt_gate) { GAI_GNA(float, float, bf16); }
  else if (!dt_y && !dt_gate && (!dt_out || !out)) { GAI_GNA(bf16, bf16, bf16); }
  else if (!dt_y && dt_gate && (!dt_out || !out)) { GAI_GNA(bf16, float, bf16); }
  else gai_launch_error(__FILE__, __LINE__, "gated_norm_add_f32: unsupported dtype combination");
#undef GAI_GNA
  GAI_LAUNCH_CHECK();
}

void gai_gate_group_norm(const float* y, const void* z, int ldz, const float* w, void* out, int T, int NG, int GS,
                         float eps, int dt, hipStream_t st) {
  if (T == 0) return;
  const int TG = T * NG, grid = (TG + 3) / 4;
  if (TG <= 512 && GS >= 512) {  // few long groups: a workgroup per group
    if (dt)
      gate_group_norm_wide_kernel<float><<<TG, 256, 0, st>>>(y, (const float*)z, ldz, w, (float*)out, NG, GS, eps);
    else
      gate_group_norm_wide_kernel<bf16><<<TG, 256, 0, st>>>(y, (const bf16*)z, ldz, w, (bf16*)out, NG, GS, eps);
    GAI_LAUNCH_CHECK();
    return;
  }
  if (dt)
    gate_group_norm_kernel<float><<<grid, 256, 0, st>>>(y, (const float*)z, ldz, w, (float*)out, TG, NG, GS, eps);
  else
    gate_group_norm_kernel<bf16><<<grid, 256, 0, st>>>(y, (const bf16*)z, ldz, w, (bf16*)out, TG, NG, GS, eps);
  GAI_LAUNCH_CHECK();
}

void gai_add_dyt_f32(float* res, const void* delta, int ldd, const float* extra, float alpha, const float* w,
                     const float* b, void* out, int T, int D, int dt_delta, int dt_out, hipStream_t st) {
  if (T == 0) return;
  const bool v4 = D % 4 == 0 && (!delta || ldd % 4 == 0);
  const long n = (long)T * (v4 ? D / 4 : D);
  const unsigned grid = (unsigned)((n + 255) / 256);
#define GAI_DYT(TD, TA)                                                                                               \
  do {                                                                                                                \
    if (v4) add_dyt_f32_kernel<TD, TA, 4><<<grid, 256, 0, st>>>(res, (const TD*)delta, ldd, extra, alpha, w, b,       \
                                                                (TA*)out, T, D);                                      \
    else add_dyt_f32_kernel<TD, TA, 1><<<grid, 256, 0, st>>>(res, (const TD*)delta, ldd, extra, alpha, w, b,          \
                                                             (TA*)out, T, D);                                         \
  } while (0)
  if (dt_delta && dt_out) GAI_DYT(float, float);
  else if (dt_delta) GAI_DYT(float, bf16);
  else if (dt_out) GAI_DYT(bf16, float);
  else GAI_DYT(bf16, bf16);
#undef GAI_DYT
  GAI_LAUNCH_CHECK();
}

void gai_act_mul(const void* a, int lda, const void* b, int ldb, void* out, int T, int C, int act, float cap, int dt_in,
                 int dt_out, hipStream_t st) {
  if (T == 0 || C == 0) return;
  if (act < 0 || act > 4)
    gai_launch_error(__FILE__, __LINE__, "act_mul: act 0 (silu), 1 (squared ReLU), 2 (tanh cap), 3 (tanh GELU) or 4 (clamped gate)");
  if ((act == 2 || act == 4) && !(cap > 0.f)) gai_launch_error(__FILE__, __LINE__, "act_mul: the cap / limit must be positive");
  if (act == 4 && !b) gai_launch_error(__FILE__, __LINE__, "act_mul: the clamped gated activation takes two operands");
  // four elements per thread where rows, strides and base addresses allow aligned vector accesses
  const size_t esz = dt_in ? 4 : 2;
  const bool v4 = C % 4 == 0 && lda % 4 == 0 && (!b || ldb % 4 == 0) && (uintptr_t)a % (4 * esz) == 0 &&
                  (!b || (uintptr_t)b % (4 * esz) == 0) && (uintptr_t)out % 16 == 0;
  const long n = (long)T * (v4 ? C / 4 : C);
  const unsigned grid = (unsigned)((n + 255) / 256);
#define GAI_AM(TI, TO)                                                                                                \
  do {                                                                                                                \
    if (v4) act_mul_kernel<TI, TO, 4><<<grid, 256, 0, st>>>((const TI*)a, lda, (const TI*)b, ldb, (TO*)out, T, C, act, cap); \
    else act_mul_kernel<TI, TO, 1><<<grid, 256, 0, st>>>((const TI*)a, lda, (const TI*)b, ldb, (TO*)out, T, C, act, cap);    \
  } while (0)
  if (dt_in && dt_out) GAI_AM(float, float);
  else if (dt_in) GAI_AM(float, bf16);
  else if (dt_out) GAI_AM(bf16, float);
  else GAI_AM(bf16, bf16);
#undef GAI_AM
  GAI_LAUNCH_CHECK();
}
