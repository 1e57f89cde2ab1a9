// Recurrent sequence mixers over a per-sequence fp32 state pool (slot = one live sequence):
//
//   token_shift_mix   m_s[t] = h[t] + (h[t-1] - h[t]) * mu_s   for NM mixes; h[-1] of a portion comes from the pool
//   conv_silu         short causal depthwise convolution over time (last tap = current token) (+ bias) + SiLU (or no
//                     activation); the inputs before a portion's first token come from the pool (zeros for a fresh
//                     sequence)
//   state_tail_write  keep the last NR input rows of every sequence in the pool (token shift: NR = 1; conv: taps - 1)
//   wkv_scan          S [DK, DV] per head:  o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T,
//                     w_t = exp(-exp(wpre_t + w0))
//   delta_prep        token-parallel inputs of the delta rule: unit-norm q (x DK^-1/2) and k per head, per-channel
//                     decay exp(-exp(A_log_h) softplus(a + dt_bias)), write strength sigmoid(b)
//   delta_scan        S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//   rglru_gates       real-gated linear recurrent unit, token-parallel part: block-diagonal gates r, i = sigmoid(W u + b)
//                     in fp32, a = exp(-c r softplus(lam)), b = sqrt(1 - a^2) i u
//   rglru_scan        S <- a_t S + b_t per channel; o_t = scale * S_t * act(y_t)
//   ssd_scan          state-space scan with one decay per head: S [N, DV], dt_t = softplus(dt + dt_bias),
//                     S <- exp(-exp(A_log) dt_t) S + dt_t B_t x_t^T;  o_t = S^T C_t + D x_t  (the output reads the
//                     UPDATED state); with a fixed decay per head, step size one and no skip term it is linear
//                     attention with a constant decay: S <- decay_h S + k_t v_t^T, o_t = S^T q_t
//   selective_scan    state-space scan with a decay per channel AND state element, everything input-dependent:
//                     dt_c = softplus(dt + dt_bias); S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;
//                     y_c = sum_n S[c, n] C_n + D_c x_c; out = y * silu(z)
//
//   decay_gate        token-parallel fp32 gates of a recurrence from their logits: sigmoid(x), sigmoid(x)^(1 / p) (through
//                     its logarithm -softplus(-x) / p) or exp(-p sigmoid(x))
//   unit_key_removal  per head the unit key u = k / sqrt(sum k^2 + eps) and the removal vector sigmoid(a + bias) * u
//   dplr_scan         diagonal decay plus a rank-one removal: S <- diag(w_t) S - av_t (bv_t^T S) + k_t v_t^T (decay and removal
//                     both act on S_(t-1)), o_t = scale * S^T q_t; without av / bv it is gated linear attention
//
// A batch is S sequences of rows [cu[s], cu[s+1]) with pool slot slots[s] (device vectors: graph-capturable); a decoded
// token is a sequence of one row, a prompt portion a longer one. The scans keep the state in VGPRs for the whole
// portion and read / write the pool once. Two shapes per recurrence:
//   * decode steps (one row per sequence): one workgroup per (head, sequence), thread (rg, j) owns rows
//     [64 rg, 64 rg + 64) of state column j - the state streams through coalesced, the step is state-bandwidth bound;
//   * steps with prompt portions: the column-sliced kernels further down (one wave64 per block of state columns, no
//     workgroup barrier in the token loop).
#include "gai_common.h"
#include "gai_kernels.h"

using namespace gai;

namespace {

constexpr int kRows = 64;     // state rows per thread
constexpr int kMaxRG = 4;     // DK <= 256
constexpr int kMaxDK = kRows * kMaxRG;

template <typename TA>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(const TA* __restrict__ h, const float* __restrict__ mu,
                                                              int NM, const float* __restrict__ shift_state,
                                                              const int* __restrict__ cu, const int* __restrict__ slots,
                                                              int S, TA* __restrict__ out, int T, int D) {
  const int t = blockIdx.x;
  int lo = 0, hi = S;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  const bool head = cu[lo] == t;
  const float* prev_s = shift_state + (size_t)slots[lo] * D;
  const TA* cur = h + (size_t)t * D;
  for (int i = threadIdx.x; i < D; i += 256) {
    const float x = (float)cur[i];
    const float xp = head ? prev_s[i] : (float)cur[i - D];
    const float d = xp - x;
    for (int n = 0; n < NM; ++n) out[((size_t)n * T + t) * D + i] = (TA)(x + d * mu[(size_t)n * D + i]);
  }
}

// One thread per (sequence, channel): read every value the new tail needs, then write (the tail may overlap itself).
template <typename TA>
__global__ __launch_bounds__(256) void state_tail_write_kernel(const TA* __restrict__ x, int ldx, float* __restrict__ state,
                                                               const int* __restrict__ cu, const int* __restrict__ slots,
                                                               int C, int NR) {
  const int s = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int b = cu[s], L = cu[s + 1] - b;
  if (L <= 0) return;
  float* st = state + (size_t)slots[s] * NR * C + c;
  float keep[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    if (r < NR) {
      const int src = L - NR + r;  // row of the portion; negative: older, from the pool
      keep[r] = src >= 0 ? (float)x[(size_t)(b + src) * ldx + c] : st[(size_t)(NR + src) * C];
    }
  }
#pragma unroll
  for (int r = 0; r < 8; ++r)
    if (r < NR) st[(size_t)r * C] = keep[r];
}

template <typename TA>
__global__ __launch_bounds__(256) void conv_silu_kernel(const TA* __restrict__ x, int ldx, const float* __restrict__ w,
                                                        const float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots, int S, float* __restrict__ y,
                                                        int C, int K, const float* __restrict__ bias, int act) {
  const int t = blockIdx.x;
  int lo = 0, hi = S;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid;
  }
  const int rel = t - cu[lo];
  const float* st = state + (size_t)slots[lo] * (K - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {  // few rows: channel tiles across blockIdx.y
    float a = 0.f;
    for (int i = 0; i < K; ++i) {
      const int src = rel - (K - 1) + i;
      const float xv = src >= 0 ? (float)x[(size_t)(t - (K - 1) + i) * ldx + c] : st[(size_t)(K - 1 + src) * C + c];
      a = fmaf(xv, w[(size_t)c * K + i], a);
    }
    if (bias) a += bias[c];
    y[(size_t)t * C + c] = act ? a / (1.0f + expf(-a)) : a;
  }
}

template <typename TA>
__global__ __launch_bounds__(1024) void wkv_scan_kernel(const TA* __restrict__ r, const TA* __restrict__ k,
                                                        const TA* __restrict__ v, int ld, const float* __restrict__ wpre,
                                                        const float* __restrict__ w0, const float* __restrict__ u,
                                                        float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots, float* __restrict__ out, int H,
                                                        int D) {
  extern __shared__ float lds[];  // us[D] | buf[2][3][D] (r, k, w) | red[2][RG][D]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int RG = (D + kRows - 1) / kRows;
  const int j = tid % D, rg = tid / D;
  const int row0 = rg * kRows, nrow = min(kRows, D - row0);
  float* us = lds;
  float* buf = us + D;
  float* red = buf + 6 * D;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* Sg = state + (((size_t)slots[s] * H + h) * D + row0) * D + j;
  float col[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) col[i] = i < nrow ? Sg[(size_t)i * D] : 0.f;
  if (tid < D) us[tid] = u[(size_t)h * D + tid];
  for (int t = t0; t < t1; ++t) {
    const int b = (t - t0) & 1;
    float* rb = buf + b * 3 * D;
    if (tid < D) {
      const size_t o = (size_t)t * ld + (size_t)h * D + tid;
      rb[tid] = (float)r[o];
      rb[D + tid] = (float)k[o];
      rb[2 * D + tid] = expf(-expf(wpre[((size_t)t * H + h) * D + tid] + w0[(size_t)h * D + tid]));
    }
    const float vj = (float)v[(size_t)t * ld + (size_t)h * D + j];
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      if (i < nrow) {
        const float kv = rb[D + row0 + i] * vj;
        acc = fmaf(rb[row0 + i], fmaf(us[row0 + i], kv, col[i]), acc);
        col[i] = fmaf(rb[2 * D + row0 + i], col[i], kv);
      }
    }
    if (RG == 1) {
      out[((size_t)t * H + h) * D + j] = acc;
    } else {
      red[(b * RG + rg) * D + j] = acc;
      __syncthreads();
      if (rg == 0) {
        float o = 0.f;
        for (int g = 0; g < RG; ++g) o += red[(b * RG + g) * D + j];
        out[((size_t)t * H + h) * D + j] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRows; ++i)
    if (i < nrow) Sg[(size_t)i * D] = col[i];
}

template <typename TA>
__global__ __launch_bounds__(256) void delta_prep_kernel(const float* __restrict__ qkv, int ld, const TA* __restrict__ a,
                                                         int lda, const TA* __restrict__ bp, int ldb,
                                                         const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                         float* __restrict__ qn, float* __restrict__ kn,
                                                         float* __restrict__ decay, float* __restrict__ beta, int H, int G,
                                                         int DK) {
  const int t = blockIdx.x, wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* row = qkv + (size_t)t * ld;
  const float qscale = 1.0f / sqrtf((float)DK);
  for (int gh = wid; gh < 2 * G; gh += 4) {  // q heads then k heads
    const float* src = row + (size_t)gh * DK;
    float s = 0.f;
    for (int i = lane; i < DK; i += 64) s += src[i] * src[i];
    s = wave_sum(s);
    const float inv = (1.0f / sqrtf(s + 1e-6f)) * (gh < G ? qscale : 1.0f);
    float* dst = gh < G ? qn + ((size_t)t * G + gh) * DK : kn + ((size_t)t * G + (gh - G)) * DK;
    for (int i = lane; i < DK; i += 64) dst[i] = src[i] * inv;
  }
  const int HD = H * DK;
  for (int i = threadIdx.x; i < HD; i += 256) {
    const float x = (float)a[(size_t)t * lda + i] + dt_bias[i];
    const float sp = x > 20.f ? x : log1pf(expf(x));
    decay[(size_t)t * HD + i] = expf(-expf(A_log[i / DK]) * sp);
  }
  for (int i = threadIdx.x; i < H; i += 256) beta[(size_t)t * H + i] = 1.0f / (1.0f + expf(-(float)bp[(size_t)t * ldb + i]));
}

__global__ __launch_bounds__(1024) void delta_scan_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                          const float* __restrict__ v, int ldv,
                                                          const float* __restrict__ decay, const float* __restrict__ beta,
                                                          float* __restrict__ state, const int* __restrict__ cu,
                                                          const int* __restrict__ slots, float* __restrict__ out, int H,
                                                          int G, int DK, int DV) {
  extern __shared__ float lds[];  // buf[2][3][DK] (q, k, g) | red[2][2][RG][DV]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int RG = (DK + kRows - 1) / kRows;
  const int j = tid % DV, rg = tid / DV;
  const int row0 = rg * kRows, nrow = min(kRows, DK - row0);
  const int g = h / (H / G);
  float* buf = lds;
  float* red = buf + 6 * DK;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* Sg = state + (((size_t)slots[s] * H + h) * DK + row0) * DV + j;
  float col[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) col[i] = i < nrow ? Sg[(size_t)i * DV] : 0.f;
  for (int t = t0; t < t1; ++t) {
    const int b = (t - t0) & 1;
    float* qb = buf + b * 3 * DK;
    for (int i = tid; i < DK; i += blockDim.x) {
      qb[i] = q[((size_t)t * G + g) * DK + i];
      qb[DK + i] = k[((size_t)t * G + g) * DK + i];
      qb[2 * DK + i] = decay[((size_t)t * H + h) * DK + i];
    }
    const float vj = v[(size_t)t * ldv + (size_t)h * DV + j];
    const float bt = beta[(size_t)t * H + h];
    __syncthreads();
    float mm = 0.f;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      if (i < nrow) {
        col[i] *= qb[2 * DK + row0 + i];
        mm = fmaf(col[i], qb[DK + row0 + i], mm);
      }
    }
    if (RG > 1) {
      float* rm = red + ((b * 2 + 0) * RG) * DV;
      rm[rg * DV + j] = mm;
      __syncthreads();
      mm = 0.f;
      for (int x = 0; x < RG; ++x) mm += rm[x * DV + j];
    }
    const float uj = bt * (vj - mm);
    float oo = 0.f;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      if (i < nrow) {
        col[i] = fmaf(qb[DK + row0 + i], uj, col[i]);
        oo = fmaf(col[i], qb[row0 + i], oo);
      }
    }
    if (RG == 1) {
      out[((size_t)t * H + h) * DV + j] = oo;
    } else {
      float* ro = red + ((b * 2 + 1) * RG) * DV;
      ro[rg * DV + j] = oo;
      __syncthreads();
      if (rg == 0) {
        float o = 0.f;
        for (int x = 0; x < RG; ++x) o += ro[x * DV + j];
        out[((size_t)t * H + h) * DV + j] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRows; ++i)
    if (i < nrow) Sg[(size_t)i * DV] = col[i];
}

// ---- prompt portions: one wave64 per (head, sequence, block of state columns) -------------------------------------
// The columns of S evolve independently of each other, so a long portion is spread over many waves per head instead
// of one workgroup: lane (jj, rg) owns rows [rg R, rg R + R) of column jj (64 / RGS columns x RGS row groups), the token
// inputs of 8 tokens at a time are staged in LDS by the wave itself (prefetched into registers one round ahead), and
// the row-group reductions are DPP adds: no workgroup barrier and no LDS shuffle anywhere in the token loop. LDS
// rows past DK stay zero, so the token loop has no row guard (branch-free: its LDS reads are issued in batches).
constexpr int kTB = 8;

template <int R>
__device__ __forceinline__ int lds_row(int row) { return row + row / R; }  // row groups land in different banks

// Sum over the RGS row groups of a column, in every lane of the group. The row groups of one column sit in RGS
// neighbouring lanes (RGS <= 16: inside one DPP row), so the butterfly is 2 - 4 v_add_f32 with DPP operands (quad
// permutes, then half-row and row mirrors - the mirrored partner holds its group's total in every lane) and never
// goes through the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int RGS>
__device__ __forceinline__ float rowgroup_sum(float v) {
  static_assert(RGS == 4 || RGS == 8 || RGS == 16, "row groups of one column share a DPP row");
  v += dpp_f<0xB1>(v);                       // quad_perm [1, 0, 3, 2]
  v += dpp_f<0x4E>(v);                       // quad_perm [2, 3, 0, 1]
  if (RGS >= 8) v += dpp_f<0x141>(v);        // row_half_mirror
  if (RGS >= 16) v += dpp_f<0x140>(v);       // row_mirror
  return v;
}

// Sum over J = 2^k neighbouring lanes (aligned groups), in every lane: DPP inside a row of 16, the crossbar beyond it.
template <int J>
__device__ __forceinline__ float lanegroup_sum(float v) {
  if (J >= 2) v += dpp_f<0xB1>(v);
  if (J >= 4) v += dpp_f<0x4E>(v);
  if (J >= 8) v += dpp_f<0x141>(v);
  if (J >= 16) v += dpp_f<0x140>(v);
  if (J >= 32) v += __shfl_xor(v, 16, 64);
  if (J >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}

// decay of every (token, head, channel) ahead of the serial scan: exp(-exp(wpre + w0)), token-parallel
__global__ __launch_bounds__(256) void wkv_decay_kernel(const float* __restrict__ wpre, const float* __restrict__ w0,
                                                        float* __restrict__ wdecay, size_t n, int HD) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) wdecay[i] = expf(-expf(wpre[i] + w0[i % HD]));
}

template <typename TA, int R, int RGS>
__global__ __launch_bounds__(64) void wkv_scan_cols_kernel(const TA* __restrict__ r, const TA* __restrict__ k,
                                                           const TA* __restrict__ v, int ld,
                                                           const float* __restrict__ wdecay, const float* __restrict__ u,
                                                           float* __restrict__ state, const int* __restrict__ cu,
                                                           const int* __restrict__ slots, float* __restrict__ out, int H,
                                                           int D) {
  constexpr int COLS = 64 / RGS, NP = kTB * RGS * R / 64, LD = RGS * R + RGS;
  extern __shared__ float lds[];
  const int h = blockIdx.x, s = blockIdx.y, cb = blockIdx.z, lane = threadIdx.x;
  const int jj = lane / RGS, rg = lane % RGS, j = cb * COLS + jj;
  const bool on = j < D;
  const int row0 = rg * R, nrow = max(0, min(R, D - row0));
  float* rs = lds;
  float* ks = rs + kTB * LD;
  float* ws = ks + kTB * LD;
  float* vs = ws + kTB * LD;  // [kTB][COLS]
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  for (int x = lane; x < 3 * kTB * LD; x += 64) lds[x] = 0.f;
  float* Sg = state + (((size_t)slots[s] * H + h) * D + row0) * D + j;
  float col[R], ur[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    col[i] = (on && i < nrow) ? Sg[(size_t)i * D] : 0.f;
    ur[i] = i < nrow ? u[(size_t)h * D + row0 + i] : 0.f;
  }
  // staging map without divisions: lane = (token of the round, 1 of 8 parts); a part walks its token's row with stride 8
  constexpr int NPART = 64 / kTB;
  static_assert(NP * NPART >= RGS * R, "staging covers a full row");
  const int stt = lane / NPART, spart = lane % NPART;
  float pr[NP], pk[NP], pw[NP], pv[2];
  auto fetch = [&](int tb) {
    const int n = min(kTB, t1 - tb);
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < D) {
        const size_t o = (size_t)(tb + stt) * ld + (size_t)h * D + i;
        pr[x] = (float)r[o];
        pk[x] = (float)k[o];
        pw[x] = wdecay[((size_t)(tb + stt) * H + h) * D + i];
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int idx = x * 64 + lane, tt = idx / COLS, c = cb * COLS + idx % COLS;
      pv[x] = (tt < n && c < D) ? (float)v[(size_t)(tb + tt) * ld + (size_t)h * D + c] : 0.f;
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += kTB) {
    const int n = min(kTB, t1 - tb);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < D) {
        const int a = stt * LD + lds_row<R>(i);
        rs[a] = pr[x];
        ks[a] = pk[x];
        ws[a] = pw[x];
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
      if (x * 64 + lane < kTB * COLS) vs[x * 64 + lane] = pv[x];
    __builtin_amdgcn_wave_barrier();
    if (tb + kTB < t1) fetch(tb + kTB);
    for (int tt = 0; tt < n; ++tt) {
      const float vj = vs[tt * COLS + jj];
      const int a = tt * LD + row0 + rg;
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        const float kv0 = ks[a + i] * vj, kv1 = ks[a + i + 1] * vj;
        acc0 = fmaf(rs[a + i], fmaf(ur[i], kv0, col[i]), acc0);
        acc1 = fmaf(rs[a + i + 1], fmaf(ur[i + 1], kv1, col[i + 1]), acc1);
        col[i] = fmaf(ws[a + i], col[i], kv0);
        col[i + 1] = fmaf(ws[a + i + 1], col[i + 1], kv1);
      }
      const float acc = rowgroup_sum<RGS>(acc0 + acc1);
      if (rg == 0 && on) out[((size_t)(tb + tt) * H + h) * D + j] = acc;
    }
  }
  if (on) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < nrow) Sg[(size_t)i * D] = col[i];
  }
}

template <int R, int RGS>
__global__ __launch_bounds__(64) void delta_scan_cols_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                             const float* __restrict__ v, int ldv,
                                                             const float* __restrict__ decay, const float* __restrict__ beta,
                                                             float* __restrict__ state, const int* __restrict__ cu,
                                                             const int* __restrict__ slots, float* __restrict__ out, int H,
                                                             int G, int DK, int DV) {
  constexpr int COLS = 64 / RGS, NP = kTB * RGS * R / 64, LD = RGS * R + RGS;
  extern __shared__ float lds[];
  const int h = blockIdx.x, s = blockIdx.y, cb = blockIdx.z, lane = threadIdx.x;
  const int jj = lane / RGS, rg = lane % RGS, j = cb * COLS + jj;
  const bool on = j < DV;
  const int row0 = rg * R, nrow = max(0, min(R, DK - row0));
  const int g = h / (H / G);
  float* qs = lds;
  float* ks = qs + kTB * LD;
  float* gs = ks + kTB * LD;
  float* vs = gs + kTB * LD;     // [kTB][COLS]
  float* bs = vs + kTB * COLS;   // [kTB]
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  for (int x = lane; x < 3 * kTB * LD; x += 64) lds[x] = 0.f;
  float* Sg = state + (((size_t)slots[s] * H + h) * DK + row0) * DV + j;
  float col[R];
#pragma unroll
  for (int i = 0; i < R; ++i) col[i] = (on && i < nrow) ? Sg[(size_t)i * DV] : 0.f;
  constexpr int NPART = 64 / kTB;
  static_assert(NP * NPART >= RGS * R, "staging covers a full row");
  const int stt = lane / NPART, spart = lane % NPART;
  float pq[NP], pk[NP], pg[NP], pv[2], pb = 0.f;
  auto fetch = [&](int tb) {
    const int n = min(kTB, t1 - tb);
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < DK) {
        pq[x] = q[((size_t)(tb + stt) * G + g) * DK + i];
        pk[x] = k[((size_t)(tb + stt) * G + g) * DK + i];
        pg[x] = decay[((size_t)(tb + stt) * H + h) * DK + i];
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int idx = x * 64 + lane, tt = idx / COLS, c = cb * COLS + idx % COLS;
      pv[x] = (tt < n && c < DV) ? v[(size_t)(tb + tt) * ldv + (size_t)h * DV + c] : 0.f;
    }
    if (lane < n) pb = beta[(size_t)(tb + lane) * H + h];
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += kTB) {
    const int n = min(kTB, t1 - tb);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < DK) {
        const int a = stt * LD + lds_row<R>(i);
        qs[a] = pq[x];
        ks[a] = pk[x];
        gs[a] = pg[x];
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
      if (x * 64 + lane < kTB * COLS) vs[x * 64 + lane] = pv[x];
    if (lane < kTB) bs[lane] = pb;
    __builtin_amdgcn_wave_barrier();
    if (tb + kTB < t1) fetch(tb + kTB);
    for (int tt = 0; tt < n; ++tt) {
      const float vj = vs[tt * COLS + jj], bt = bs[tt];
      const int a = tt * LD + row0 + rg;
      float m0 = 0.f, m1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        col[i] *= gs[a + i];
        col[i + 1] *= gs[a + i + 1];
        m0 = fmaf(col[i], ks[a + i], m0);
        m1 = fmaf(col[i + 1], ks[a + i + 1], m1);
      }
      const float uj = bt * (vj - rowgroup_sum<RGS>(m0 + m1));
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        col[i] = fmaf(ks[a + i], uj, col[i]);
        col[i + 1] = fmaf(ks[a + i + 1], uj, col[i + 1]);
        o0 = fmaf(col[i], qs[a + i], o0);
        o1 = fmaf(col[i + 1], qs[a + i + 1], o1);
      }
      const float oo = rowgroup_sum<RGS>(o0 + o1);
      if (rg == 0 && on) out[((size_t)(tb + tt) * H + h) * DV + j] = oo;
    }
  }
  if (on) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < nrow) Sg[(size_t)i * DV] = col[i];
  }
}

// ---- diagonal decay plus rank-one removal (gated linear attention, generalised delta rule) --------------------------
// The two shapes of delta_scan: decode steps with one workgroup per (head, sequence) and coalesced state streaming,
// prompt portions with one wave64 per block of state columns. q / k / v come in the activation dtype (column slices of
// a projection output), decay and the removal vectors in fp32; all arithmetic fp32.
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename TA>
__global__ __launch_bounds__(256) void decay_gate_kernel(const TA* __restrict__ z, int ldz, const float* __restrict__ bias,
                                                         int kind, float param, float* __restrict__ out, int T, int C) {
  const long e = (long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long)T * C) return;
  const int t = (int)(e / C), c = (int)(e % C);
  const float x = (float)z[(size_t)t * ldz + c] + (bias ? bias[c] : 0.f);
  float y;
  if (kind == 0) y = sigmoid_f(x);
  else if (kind == 1) {  // sigmoid(x)^(1 / param) = exp(-softplus(-x) / param)
    const float sp = -x > 20.f ? -x : log1pf(expf(-x));
    y = expf(-sp / param);
  } else y = expf(-param * sigmoid_f(x));
  out[e] = y;
}

template <typename TA>
__global__ __launch_bounds__(256) void unit_key_removal_kernel(const TA* __restrict__ k, int ldk, const TA* __restrict__ a,
                                                               int lda, const float* __restrict__ a_bias,
                                                               float* __restrict__ av, float* __restrict__ bv, int TH,
                                                               int H, int DK, float eps) {
  const int lane = threadIdx.x & 63;
  const int th = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (th >= TH) return;
  const int t = th / H, h = th - t * H;
  const TA* kr = k + (size_t)t * ldk + (size_t)h * DK;
  const TA* ar = a + (size_t)t * lda + (size_t)h * DK;
  float ss = 0.f;
  for (int i = lane; i < DK; i += 64) {
    const float x = (float)kr[i];
    ss += x * x;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss + eps);
  for (int i = lane; i < DK; i += 64) {
    const float u = (float)kr[i] * inv;
    const float rate = sigmoid_f((float)ar[i] + (a_bias ? a_bias[(size_t)h * DK + i] : 0.f));
    bv[(size_t)th * DK + i] = u;
    av[(size_t)th * DK + i] = rate * u;
  }
}

template <typename TA, bool RANK1>
__global__ __launch_bounds__(1024) void dplr_scan_kernel(const TA* __restrict__ q, int ldq, const TA* __restrict__ k, int ldk,
                                                         const TA* __restrict__ v, int ldv, const float* __restrict__ decay,
                                                         const float* __restrict__ av, const float* __restrict__ bv,
                                                         float* __restrict__ state, const int* __restrict__ cu,
                                                         const int* __restrict__ slots, float* __restrict__ out, int H,
                                                         int DK, int DV, float q_scale) {
  extern __shared__ float lds[];  // buf[2][5][DK] (q, k, w, a, b) | red[2][2][RG][DV]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int RG = (DK + kRows - 1) / kRows;
  const int j = tid % DV, rg = tid / DV;
  const int row0 = rg * kRows, nrow = min(kRows, DK - row0);
  float* buf = lds;
  float* red = buf + 10 * DK;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* Sg = state + (((size_t)slots[s] * H + h) * DK + row0) * DV + j;
  float col[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) col[i] = i < nrow ? Sg[(size_t)i * DV] : 0.f;
  for (int t = t0; t < t1; ++t) {
    const int b = (t - t0) & 1;
    float* qb = buf + b * 5 * DK;
    for (int i = tid; i < DK; i += blockDim.x) {
      const size_t o = ((size_t)t * H + h) * DK + i;
      qb[i] = (float)q[(size_t)t * ldq + (size_t)h * DK + i];
      qb[DK + i] = (float)k[(size_t)t * ldk + (size_t)h * DK + i];
      qb[2 * DK + i] = decay[o];
      if (RANK1) {
        qb[3 * DK + i] = av[o];
        qb[4 * DK + i] = bv[o];
      }
    }
    const float vj = (float)v[(size_t)t * ldv + (size_t)h * DV + j];
    __syncthreads();
    float mm = 0.f;
    if (RANK1) {
#pragma unroll
      for (int i = 0; i < kRows; ++i)
        if (i < nrow) mm = fmaf(col[i], qb[4 * DK + row0 + i], mm);
      if (RG > 1) {
        float* rm = red + ((b * 2 + 0) * RG) * DV;
        rm[rg * DV + j] = mm;
        __syncthreads();
        mm = 0.f;
        for (int x = 0; x < RG; ++x) mm += rm[x * DV + j];
      }
    }
    float oo = 0.f;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      if (i < nrow) {
        float c = fmaf(qb[2 * DK + row0 + i], col[i], qb[DK + row0 + i] * vj);
        if (RANK1) c = fmaf(-qb[3 * DK + row0 + i], mm, c);
        col[i] = c;
        oo = fmaf(c, qb[row0 + i], oo);
      }
    }
    if (RG == 1) {
      out[((size_t)t * H + h) * DV + j] = oo * q_scale;
    } else {
      float* ro = red + ((b * 2 + 1) * RG) * DV;
      ro[rg * DV + j] = oo;
      __syncthreads();
      if (rg == 0) {
        float o = 0.f;
        for (int x = 0; x < RG; ++x) o += ro[x * DV + j];
        out[((size_t)t * H + h) * DV + j] = o * q_scale;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRows; ++i)
    if (i < nrow) Sg[(size_t)i * DV] = col[i];
}

// MODE 0: whole portions, state from / to the pool. A long portion of few sequences leaves most SIMDs without a wave, and
// the recurrence is linear in S (S_t = A_t S_(t-1) + k_t v_t^T with A_t = diag(w_t) - av_t bv_t^T), so such a step is cut
// into chunks of kDplrChunk tokens that run side by side:
//   MODE 1: a chunk from a zero state, no outputs: its final state Q and its transition - without removal the product
//           of its decays per key channel (P), with removal the DK x DK matrix M = A_n ... A_1, obtained by running the
//           homogeneous recurrence on the columns of the identity (DK more columns of the same kernel, v = 0);
//   carry:  per sequence S <- diag(P) S + Q or S <- M S + Q over its chunks, leaving every chunk's entry state in Q's
//           place (and the pool's final state);
//   MODE 2: the chunk again from its entry state, outputs written.
// Only the association of the fp32 products differs from the serial order.
constexpr int kDplrChunk = 256;

__device__ __forceinline__ bool dplr_chunk_of(const int* __restrict__ cu, int S, int idx, int& s, int& t0, int& t1) {
  int seen = 0;
  for (s = 0; s < S; ++s) {
    const int len = cu[s + 1] - cu[s], nc = (len + kDplrChunk - 1) / kDplrChunk;
    if (idx < seen + nc) {
      t0 = cu[s] + (idx - seen) * kDplrChunk;
      t1 = min(t0 + kDplrChunk, cu[s + 1]);
      return true;
    }
    seen += nc;
  }
  return false;
}

template <typename TA, int R, int RGS, bool RANK1, int MODE>
__global__ __launch_bounds__(64) void dplr_scan_cols_kernel(const TA* __restrict__ q, int ldq, const TA* __restrict__ k,
                                                            int ldk, const TA* __restrict__ v, int ldv,
                                                            const float* __restrict__ decay, const float* __restrict__ av,
                                                            const float* __restrict__ bv, float* __restrict__ state,
                                                            const int* __restrict__ cu, const int* __restrict__ slots,
                                                            float* __restrict__ out, int H, int DK, int DV,
                                                            float q_scale, int S, float* __restrict__ Qbuf,
                                                            float* __restrict__ Tbuf) {
  constexpr int COLS = 64 / RGS, NP = kTB * RGS * R / 64, LD = RGS * R + RGS, NA = RANK1 ? 5 : 3;
  extern __shared__ float lds[];
  const int h = blockIdx.x, cb = blockIdx.z, lane = threadIdx.x;
  int s = blockIdx.y, t0, t1;
  if (MODE == 0) {
    t0 = cu[s];
    t1 = cu[s + 1];
  } else if (!dplr_chunk_of(cu, S, blockIdx.y, s, t0, t1)) {
    return;
  }
  const int jj = lane / RGS, rg = lane % RGS, j = cb * COLS + jj;
  // MODE 1 with removal: columns DV .. DV + DK - 1 are the columns of the chunk's transition matrix
  const bool is_m = MODE == 1 && RANK1 && j >= DV;
  const int jm = j - DV;
  const bool on = j < DV || (is_m && jm < DK);
  const int row0 = rg * R, nrow = max(0, min(R, DK - row0));
  float* qs = lds;
  float* ks = qs + kTB * LD;
  float* ws = ks + kTB * LD;
  float* as = ws + kTB * LD;     // RANK1 only
  float* bs = as + kTB * LD;
  float* vs = lds + NA * kTB * LD;  // [kTB][COLS]
  if (t1 <= t0) return;
  for (int x = lane; x < NA * kTB * LD; x += 64) lds[x] = 0.f;
  // MODE 0: the pool's slot; MODE 1 / 2: the chunk's own [H, DK, DV] image in Qbuf (MODE 2 reads its entry state
  // there), the transition matrix columns in Tbuf [chunk, H, DK, DK]
  const int lds_s = is_m ? DK : DV;
  float* Sg = MODE == 0 ? state + (((size_t)slots[s] * H + h) * DK + row0) * DV + j
              : is_m    ? Tbuf + (((size_t)blockIdx.y * H + h) * DK + row0) * DK + jm
                        : Qbuf + (((size_t)blockIdx.y * H + h) * DK + row0) * DV + j;
  float col[R], pprod[(MODE == 1 && !RANK1) ? R : 1];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (MODE == 1) col[i] = (is_m && row0 + i == jm) ? 1.f : 0.f;
    else col[i] = (on && i < nrow) ? Sg[(size_t)i * lds_s] : 0.f;
    if (MODE == 1 && !RANK1) pprod[i] = 1.f;
  }
  constexpr int NPART = 64 / kTB;
  static_assert(NP * NPART >= RGS * R, "staging covers a full row");
  const int stt = lane / NPART, spart = lane % NPART;
  float pq[NP], pk[NP], pw[NP], pa[RANK1 ? NP : 1], pb[RANK1 ? NP : 1], pv[2];
  auto fetch = [&](int tb) {
    const int n = min(kTB, t1 - tb);
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < DK) {
        const size_t o = ((size_t)(tb + stt) * H + h) * DK + i;
        pq[x] = (float)q[(size_t)(tb + stt) * ldq + (size_t)h * DK + i];
        pk[x] = (float)k[(size_t)(tb + stt) * ldk + (size_t)h * DK + i];
        pw[x] = decay[o];
        if (RANK1) {
          pa[x] = av[o];
          pb[x] = bv[o];
        }
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const int idx = x * 64 + lane, tt = idx / COLS, c = cb * COLS + idx % COLS;
      pv[x] = (tt < n && c < DV) ? (float)v[(size_t)(tb + tt) * ldv + (size_t)h * DV + c] : 0.f;
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += kTB) {
    const int n = min(kTB, t1 - tb);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int x = 0; x < NP; ++x) {
      const int i = spart + NPART * x;
      if (stt < n && i < DK) {
        const int a = stt * LD + lds_row<R>(i);
        qs[a] = pq[x];
        ks[a] = pk[x];
        ws[a] = pw[x];
        if (RANK1) {
          as[a] = pa[x];
          bs[a] = pb[x];
        }
      }
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
      if (x * 64 + lane < kTB * COLS) vs[x * 64 + lane] = pv[x];
    __builtin_amdgcn_wave_barrier();
    if (tb + kTB < t1) fetch(tb + kTB);
    for (int tt = 0; tt < n; ++tt) {
      const float vj = vs[tt * COLS + jj];
      const int a = tt * LD + row0 + rg;
      float mm = 0.f;
      if (RANK1) {
        float m0 = 0.f, m1 = 0.f;
#pragma unroll
        for (int i = 0; i < R; i += 2) {
          m0 = fmaf(col[i], bs[a + i], m0);
          m1 = fmaf(col[i + 1], bs[a + i + 1], m1);
        }
        mm = rowgroup_sum<RGS>(m0 + m1);
      }
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        float c0 = fmaf(ws[a + i], col[i], ks[a + i] * vj);
        float c1 = fmaf(ws[a + i + 1], col[i + 1], ks[a + i + 1] * vj);
        if (RANK1) {
          c0 = fmaf(-as[a + i], mm, c0);
          c1 = fmaf(-as[a + i + 1], mm, c1);
        }
        col[i] = c0;
        col[i + 1] = c1;
        if (MODE == 1 && !RANK1) {
          pprod[i] *= ws[a + i];
          pprod[i + 1] *= ws[a + i + 1];
        }
        if (MODE != 1) {
          o0 = fmaf(c0, qs[a + i], o0);
          o1 = fmaf(c1, qs[a + i + 1], o1);
        }
      }
      if (MODE != 1) {
        const float oo = rowgroup_sum<RGS>(o0 + o1);
        if (rg == 0 && on) out[((size_t)(tb + tt) * H + h) * DV + j] = oo * q_scale;
      }
    }
  }
  if (on && MODE != 2) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < nrow) Sg[(size_t)i * lds_s] = col[i];
  }
  if (MODE == 1 && !RANK1 && cb == 0 && jj == 0) {  // the chunk's decay product per key channel
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < nrow) Tbuf[((size_t)blockIdx.y * H + h) * DK + row0 + i] = pprod[i];
  }
}

// S <- diag(P) S + Q over the chunks of a sequence; Q[chunk] is replaced by the chunk's entry state
__global__ __launch_bounds__(256) void dplr_chunk_carry_diag_kernel(const float* __restrict__ Pbuf, float* __restrict__ Qbuf,
                                                                    float* __restrict__ state, const int* __restrict__ cu,
                                                                    const int* __restrict__ slots, int H, int DK, int DV) {
  const int e = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y, s = blockIdx.z, ND = DK * DV;
  if (e >= ND) return;
  const int len = cu[s + 1] - cu[s];
  if (len <= 0) return;
  int first = 0;
  for (int x = 0; x < s; ++x) first += (cu[x + 1] - cu[x] + kDplrChunk - 1) / kDplrChunk;
  const int nc = (len + kDplrChunk - 1) / kDplrChunk, row = e / DV;
  float* sp = state + ((size_t)slots[s] * H + h) * ND + e;
  float Sv = *sp;
  for (int n = 0; n < nc; ++n) {
    float* qp = Qbuf + ((size_t)(first + n) * H + h) * ND + e;
    const float qv = *qp;
    *qp = Sv;
    Sv = fmaf(Pbuf[((size_t)(first + n) * H + h) * DK + row], Sv, qv);
  }
  *sp = Sv;
}

// S <- M S + Q over the chunks of a sequence (M: the chunk's DK x DK transition); one workgroup per (block of kCarryCols
// state columns, head, sequence), thread r owns row r of the block, the block's current S sits in LDS
constexpr int kCarryCols = 16;

__global__ __launch_bounds__(256) void dplr_chunk_carry_full_kernel(const float* __restrict__ Mbuf, float* __restrict__ Qbuf,
                                                                    float* __restrict__ state, const int* __restrict__ cu,
                                                                    const int* __restrict__ slots, int H, int DK, int DV) {
  extern __shared__ float Sc[];  // [DK][kCarryCols]
  const int c0 = blockIdx.x * kCarryCols, h = blockIdx.y, s = blockIdx.z, r = threadIdx.x;
  const int len = cu[s + 1] - cu[s];
  if (len <= 0) return;
  int first = 0;
  for (int x = 0; x < s; ++x) first += (cu[x + 1] - cu[x] + kDplrChunk - 1) / kDplrChunk;
  const int nc = (len + kDplrChunk - 1) / kDplrChunk, ncol = min(kCarryCols, DV - c0);
  float* sp = state + (((size_t)slots[s] * H + h) * DK + r) * DV + c0;
  if (r < DK)
    for (int c = 0; c < kCarryCols; ++c) Sc[r * kCarryCols + c] = c < ncol ? sp[c] : 0.f;
  __syncthreads();
  for (int n = 0; n < nc; ++n) {
    float acc[kCarryCols];
    if (r < DK) {
      float* qp = Qbuf + (((size_t)(first + n) * H + h) * DK + r) * DV + c0;
#pragma unroll
      for (int c = 0; c < kCarryCols; ++c) {
        acc[c] = c < ncol ? qp[c] : 0.f;
        if (c < ncol) qp[c] = Sc[r * kCarryCols + c];
      }
      const float* mr = Mbuf + (((size_t)(first + n) * H + h) * DK + r) * DK;
      for (int kk = 0; kk < DK; ++kk) {
        const float m = mr[kk];
#pragma unroll
        for (int c = 0; c < kCarryCols; ++c) acc[c] = fmaf(m, Sc[kk * kCarryCols + c], acc[c]);
      }
    }
    __syncthreads();
    if (r < DK) {
#pragma unroll
      for (int c = 0; c < kCarryCols; ++c) Sc[r * kCarryCols + c] = acc[c];
    }
    __syncthreads();
  }
  if (r < DK)
    for (int c = 0; c < ncol; ++c) sp[c] = Sc[r * kCarryCols + c];
}

// ---- real-gated linear recurrent unit -----------------------------------------------------------------------------
// Gates: one workgroup per (tile of kGT tokens, block of the block-diagonal matrices). The tile's u rows sit in LDS;
// thread c owns output channel c of the block for all kGT tokens and walks the block's input channels: the two weight
// reads are coalesced over the threads ([block, in, out] layout), the u reads are LDS broadcasts. All fp32 FMA: these
// gates steer a recurrence, so they are not rounded to the matrix cores' input format.

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <int kGT>  // tokens per workgroup: 16, or fewer for wide blocks (the tile's u rows must fit in LDS)
__global__ __launch_bounds__(256) void rglru_gates_kernel(const float* __restrict__ u, const float* __restrict__ wa_t,
                                                          const float* __restrict__ ba, const float* __restrict__ wi_t,
                                                          const float* __restrict__ bi, const float* __restrict__ lam,
                                                          float cdecay, float* __restrict__ a_out,
                                                          float* __restrict__ b_out, int T, int W, int BS) {
  extern __shared__ __attribute__((aligned(16))) float us[];  // [kGT][BS]
  const int t0 = blockIdx.x * kGT, blk = blockIdx.y, nt = min(kGT, T - t0);
  for (int x = threadIdx.x; x < kGT * BS; x += 256) {
    const int tt = x / BS, k = x - tt * BS;
    us[x] = tt < nt ? u[(size_t)(t0 + tt) * W + (size_t)blk * BS + k] : 0.f;
  }
  __syncthreads();
  const float* wa = wa_t + (size_t)blk * BS * BS;
  const float* wi = wi_t + (size_t)blk * BS * BS;
  for (int c = threadIdx.x; c < BS; c += 256) {
    float ar[kGT], ai[kGT];
#pragma unroll
    for (int tt = 0; tt < kGT; ++tt) ar[tt] = ai[tt] = 0.f;
    int k = 0;
    if ((BS & 3) == 0) {  // four input channels per iteration: one 16-byte LDS broadcast per token instead of four reads
      for (; k < BS; k += 4) {
        float xa[4], xi[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          xa[q] = wa[(size_t)(k + q) * BS + c];
          xi[q] = wi[(size_t)(k + q) * BS + c];
        }
#pragma unroll
        for (int tt = 0; tt < kGT; ++tt) {
          const float4 uv = *reinterpret_cast<const float4*>(us + tt * BS + k);
          ar[tt] = fmaf(xa[0], uv.x, ar[tt]);
          ai[tt] = fmaf(xi[0], uv.x, ai[tt]);
          ar[tt] = fmaf(xa[1], uv.y, ar[tt]);
          ai[tt] = fmaf(xi[1], uv.y, ai[tt]);
          ar[tt] = fmaf(xa[2], uv.z, ar[tt]);
          ai[tt] = fmaf(xi[2], uv.z, ai[tt]);
          ar[tt] = fmaf(xa[3], uv.w, ar[tt]);
          ai[tt] = fmaf(xi[3], uv.w, ai[tt]);
        }
      }
    }
    for (; k < BS; ++k) {
      const float xa = wa[(size_t)k * BS + c], xi = wi[(size_t)k * BS + c];
#pragma unroll
      for (int tt = 0; tt < kGT; ++tt) {
        const float uv = us[tt * BS + k];
        ar[tt] = fmaf(xa, uv, ar[tt]);
        ai[tt] = fmaf(xi, uv, ai[tt]);
      }
    }
    const int ch = blk * BS + c;
    const float sp = softplus_f(lam[ch]), rb = ba[ch], ib = bi[ch];
#pragma unroll
    for (int tt = 0; tt < kGT; ++tt) {
      if (tt < nt) {
        const float r = 1.0f / (1.0f + expf(-(ar[tt] + rb)));
        const float ig = 1.0f / (1.0f + expf(-(ai[tt] + ib)));
        const float la = -cdecay * r * sp;
        const size_t o = (size_t)(t0 + tt) * W + ch;
        a_out[o] = expf(la);
        b_out[o] = sqrtf(-expm1f(2.0f * la)) * ig * us[tt * BS + c];
      }
    }
  }
}

// Few tokens (decode steps): the same gates with the work of one block spread over many workgroups - one per
// (4 tokens, block, 64 output channels), the block's input channels cut into 4 interleaved slices (one per wave) whose
// partial sums meet in LDS - so that the gate matrices stream through all CUs instead of one workgroup per block.
constexpr int kGS = 4;  // tokens per workgroup

__global__ __launch_bounds__(256) void rglru_gates_split_kernel(const float* __restrict__ u, const float* __restrict__ wa_t,
                                                                const float* __restrict__ ba,
                                                                const float* __restrict__ wi_t,
                                                                const float* __restrict__ bi, const float* __restrict__ lam,
                                                                float cdecay, float* __restrict__ a_out,
                                                                float* __restrict__ b_out, int T, int W, int BS) {
  extern __shared__ __attribute__((aligned(16))) float us[];  // [kGS][BS] | red[4][2 kGS][64]
  float* red = us + kGS * BS;
  const int t0 = blockIdx.x * kGS, blk = blockIdx.y, c0 = blockIdx.z * 64, nt = min(kGS, T - t0);
  const int cl = threadIdx.x & 63, ks = threadIdx.x >> 6, c = c0 + cl;
  for (int x = threadIdx.x; x < kGS * BS; x += 256) {
    const int tt = x / BS, k = x - tt * BS;
    us[x] = tt < nt ? u[(size_t)(t0 + tt) * W + (size_t)blk * BS + k] : 0.f;
  }
  __syncthreads();
  float ar[kGS], ai[kGS];
#pragma unroll
  for (int tt = 0; tt < kGS; ++tt) ar[tt] = ai[tt] = 0.f;
  if (c < BS) {
    const float* wa = wa_t + (size_t)blk * BS * BS + c;
    const float* wi = wi_t + (size_t)blk * BS * BS + c;
#pragma unroll 4
    for (int k = ks; k < BS; k += 4) {
      const float xa = wa[(size_t)k * BS], xi = wi[(size_t)k * BS];
#pragma unroll
      for (int tt = 0; tt < kGS; ++tt) {
        const float uv = us[tt * BS + k];
        ar[tt] = fmaf(xa, uv, ar[tt]);
        ai[tt] = fmaf(xi, uv, ai[tt]);
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < kGS; ++tt) {
    red[(ks * 2 * kGS + tt) * 64 + cl] = ar[tt];
    red[(ks * 2 * kGS + kGS + tt) * 64 + cl] = ai[tt];
  }
  __syncthreads();
  if (ks != 0 || c >= BS) return;
  const int ch = blk * BS + c;
  const float sp = softplus_f(lam[ch]), rb = ba[ch], ib = bi[ch];
#pragma unroll
  for (int tt = 0; tt < kGS; ++tt) {
    if (tt < nt) {
      float sr = 0.f, si = 0.f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sr += red[(q * 2 * kGS + tt) * 64 + cl];
        si += red[(q * 2 * kGS + kGS + tt) * 64 + cl];
      }
      const float r = 1.0f / (1.0f + expf(-(sr + rb)));
      const float ig = 1.0f / (1.0f + expf(-(si + ib)));
      const float la = -cdecay * r * sp;
      const size_t o = (size_t)(t0 + tt) * W + ch;
      a_out[o] = expf(la);
      b_out[o] = sqrtf(-expm1f(2.0f * la)) * ig * us[tt * BS + c];
    }
  }
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// One thread per (sequence, channel); the loads of a step do not depend on the recurrence, so four steps are in flight.
template <typename TA>
__global__ __launch_bounds__(256) void rglru_scan_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         const TA* __restrict__ y, int ldy, float* __restrict__ state,
                                                         const int* __restrict__ cu, const int* __restrict__ slots,
                                                         TA* __restrict__ out, int ldo, int W, int gelu, float scale) {
  const int s = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= W) return;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* sp = state + (size_t)slots[s] * W + c;
  float S = *sp;
  int t = t0;
  for (; t + 4 <= t1; t += 4) {
    float av[4], bv[4], yv[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      av[x] = a[(size_t)(t + x) * W + c];
      bv[x] = b[(size_t)(t + x) * W + c];
      yv[x] = (float)y[(size_t)(t + x) * ldy + c];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      S = fmaf(av[x], S, bv[x]);
      out[(size_t)(t + x) * ldo + c] = (TA)(scale * S * (gelu ? gelu_tanh_f(yv[x]) : yv[x]));
    }
  }
  for (; t < t1; ++t) {
    S = fmaf(a[(size_t)t * W + c], S, b[(size_t)t * W + c]);
    const float yv = (float)y[(size_t)t * ldy + c];
    out[(size_t)t * ldo + c] = (TA)(scale * S * (gelu ? gelu_tanh_f(yv) : yv));
  }
  *sp = S;
}

// Prompt portions: the recurrence is linear, so a portion is cut into chunks of kChunk tokens that run side by side.
//   pass 1 (chunk-parallel): P = product of a over the chunk, Q = the chunk's final state from a zero start;
//   pass 2 (one thread per sequence and channel): walks the chunks, S <- P S + Q, and leaves every chunk's entry state;
//   pass 3 (chunk-parallel): the recurrence inside the chunk from its entry state, outputs written.
// Chunk (s, n) covers rows [cu[s] + n kChunk, ...) of sequence s; blockIdx.y walks them in sequence order.
constexpr int kChunk = 64;

template <int L = kChunk>
__device__ __forceinline__ bool chunk_of(const int* __restrict__ cu, int S, int idx, int& s, int& t0, int& t1) {
  int seen = 0;
  for (s = 0; s < S; ++s) {
    const int len = cu[s + 1] - cu[s], nc = (len + L - 1) / L;
    if (idx < seen + nc) {
      t0 = cu[s] + (idx - seen) * L;
      t1 = min(t0 + L, cu[s + 1]);
      return true;
    }
    seen += nc;
  }
  return false;
}

__global__ __launch_bounds__(256) void rglru_chunk_reduce_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                 const int* __restrict__ cu, int S, float* __restrict__ P,
                                                                 float* __restrict__ Q, int W) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  int s, t0, t1;
  if (c >= W || !chunk_of(cu, S, blockIdx.y, s, t0, t1)) return;
  float p = 1.f, q = 0.f;
  int t = t0;
  for (; t + 4 <= t1; t += 4) {
    float av[4], bv[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      av[x] = a[(size_t)(t + x) * W + c];
      bv[x] = b[(size_t)(t + x) * W + c];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      q = fmaf(av[x], q, bv[x]);
      p *= av[x];
    }
  }
  for (; t < t1; ++t) {
    const float av = a[(size_t)t * W + c];
    q = fmaf(av, q, b[(size_t)t * W + c]);
    p *= av;
  }
  P[(size_t)blockIdx.y * W + c] = p;
  Q[(size_t)blockIdx.y * W + c] = q;
}

__global__ __launch_bounds__(256) void rglru_chunk_carry_kernel(const float* __restrict__ P, const float* __restrict__ Q,
                                                                float* __restrict__ Sin, float* __restrict__ state,
                                                                const int* __restrict__ cu, const int* __restrict__ slots,
                                                                int W) {
  const int s = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= W) return;
  const int len = cu[s + 1] - cu[s];
  if (len <= 0) return;
  int first = 0;
  for (int x = 0; x < s; ++x) first += (cu[x + 1] - cu[x] + kChunk - 1) / kChunk;
  const int nc = (len + kChunk - 1) / kChunk;
  float* sp = state + (size_t)slots[s] * W + c;
  float Sv = *sp;
  for (int n = 0; n < nc; ++n) {
    const size_t o = (size_t)(first + n) * W + c;
    Sin[o] = Sv;
    Sv = fmaf(P[o], Sv, Q[o]);
  }
  *sp = Sv;
}

template <typename TA>
__global__ __launch_bounds__(256) void rglru_chunk_apply_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                                const TA* __restrict__ y, int ldy,
                                                                const float* __restrict__ Sin, const int* __restrict__ cu,
                                                                int S, TA* __restrict__ out, int ldo, int W, int gelu,
                                                                float scale) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  int s, t0, t1;
  if (c >= W || !chunk_of(cu, S, blockIdx.y, s, t0, t1)) return;
  float Sv = Sin[(size_t)blockIdx.y * W + c];
  int t = t0;
  for (; t + 4 <= t1; t += 4) {
    float av[4], bv[4], yv[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      av[x] = a[(size_t)(t + x) * W + c];
      bv[x] = b[(size_t)(t + x) * W + c];
      yv[x] = (float)y[(size_t)(t + x) * ldy + c];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      Sv = fmaf(av[x], Sv, bv[x]);
      out[(size_t)(t + x) * ldo + c] = (TA)(scale * Sv * (gelu ? gelu_tanh_f(yv[x]) : yv[x]));
    }
  }
  for (; t < t1; ++t) {
    Sv = fmaf(a[(size_t)t * W + c], Sv, b[(size_t)t * W + c]);
    const float yv = (float)y[(size_t)t * ldy + c];
    out[(size_t)t * ldo + c] = (TA)(scale * Sv * (gelu ? gelu_tanh_f(yv) : yv));
  }
}

// ---- state-space scan with a scalar decay per head ----------------------------------------------------------------
// The two shapes of wkv_scan / delta_scan: decode steps with one workgroup per (head, sequence), prompt portions with
// one wave64 per block of state columns.
template <typename TA>
__global__ __launch_bounds__(1024) void ssd_scan_kernel(const float* __restrict__ x, const float* __restrict__ Bm,
                                                        const float* __restrict__ Cm, int ld, const TA* __restrict__ dt,
                                                        int lddt, const float* __restrict__ dt_bias,
                                                        const float* __restrict__ A_log, const float* __restrict__ Dskip,
                                                        float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots, float* __restrict__ out, int H,
                                                        int G, int N, int DV, const float* __restrict__ fixed) {
  extern __shared__ float lds[];  // buf[2][2][N] (B, C) | red[2][RG][DV]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int RG = (N + kRows - 1) / kRows;
  const int j = tid % DV, rg = tid / DV;
  const int row0 = rg * kRows, nrow = min(kRows, N - row0);
  const int g = h / (H / G);
  float* buf = lds;
  float* red = buf + 4 * N;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* Sg = state + (((size_t)slots[s] * H + h) * N + row0) * DV + j;
  float col[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) col[i] = i < nrow ? Sg[(size_t)i * DV] : 0.f;
  // fixed: one constant decay per head, step size one, no skip term (constant-decay linear attention)
  const float negA = fixed ? 0.f : -expf(A_log[h]), dskip = Dskip ? Dskip[h] : 0.f, dtb = fixed ? 0.f : dt_bias[h];
  const float fdec = fixed ? fixed[h] : 0.f;
  for (int t = t0; t < t1; ++t) {
    const int b = (t - t0) & 1;
    float* bb = buf + b * 2 * N;
    for (int i = tid; i < N; i += blockDim.x) {
      bb[i] = Bm[(size_t)t * ld + (size_t)g * N + i];
      bb[N + i] = Cm[(size_t)t * ld + (size_t)g * N + i];
    }
    const float xj = x[(size_t)t * ld + (size_t)h * DV + j];
    const float dtv = fixed ? 1.0f : softplus_f((float)dt[(size_t)t * lddt + h] + dtb);
    const float dec = fixed ? fdec : expf(negA * dtv), dx = dtv * xj;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      if (i < nrow) {
        col[i] = fmaf(dec, col[i], bb[row0 + i] * dx);
        acc = fmaf(col[i], bb[N + row0 + i], acc);
      }
    }
    if (RG == 1) {
      out[((size_t)t * H + h) * DV + j] = fmaf(dskip, xj, acc);
    } else {
      red[(b * RG + rg) * DV + j] = acc;
      __syncthreads();
      if (rg == 0) {
        float o = 0.f;
        for (int q = 0; q < RG; ++q) o += red[(b * RG + q) * DV + j];
        out[((size_t)t * H + h) * DV + j] = fmaf(dskip, xj, o);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kRows; ++i)
    if (i < nrow) Sg[(size_t)i * DV] = col[i];
}

// MODE 0: whole portions, state from / to the pool. A long portion of few sequences leaves most SIMDs with one wave
// and nothing to hide its latencies behind; the recurrence is linear in S (one scalar decay per head and token), so such
// a step is cut into chunks of kSsdChunk tokens that run side by side:
//   MODE 1: a chunk from a zero state, no outputs: its final state Q and the product P of its decays;
//   carry:  per sequence S <- P S + Q over its chunks, leaving every chunk's entry state (and the pool's final state);
//   MODE 2: the chunk again from its entry state, outputs written.
constexpr int kSsdChunk = 256;

template <typename TA, int R, int RGS, int MODE>
__global__ __launch_bounds__(64) void ssd_scan_cols_kernel(const float* __restrict__ x, const float* __restrict__ Bm,
                                                           const float* __restrict__ Cm, int ld,
                                                           const TA* __restrict__ dt, int lddt,
                                                           const float* __restrict__ dt_bias,
                                                           const float* __restrict__ A_log,
                                                           const float* __restrict__ Dskip, float* __restrict__ state,
                                                           const int* __restrict__ cu, const int* __restrict__ slots,
                                                           float* __restrict__ out, int H, int G, int N, int DV, int S,
                                                           float* __restrict__ Pbuf, float* __restrict__ Qbuf,
                                                           const float* __restrict__ fixed) {
  constexpr int COLS = 64 / RGS, NP = kTB * RGS * R / 64, LD = RGS * R + RGS;
  extern __shared__ float lds[];
  const int h = blockIdx.x, cb = blockIdx.z, lane = threadIdx.x;
  int s = blockIdx.y, t0, t1;
  if (MODE == 0) {
    t0 = cu[s];
    t1 = cu[s + 1];
  } else if (!chunk_of<kSsdChunk>(cu, S, blockIdx.y, s, t0, t1)) {
    return;
  }
  const int jj = lane / RGS, rg = lane % RGS, j = cb * COLS + jj;
  const bool on = j < DV;
  const int row0 = rg * R, nrow = max(0, min(R, N - row0));
  const int g = h / (H / G);
  float* Bs = lds;
  float* Cs = Bs + kTB * LD;
  float* xs = Cs + kTB * LD;     // [kTB][COLS]
  float* ds = xs + kTB * COLS;   // [2][kTB]: step size, decay
  if (t1 <= t0) return;
  for (int q = lane; q < 2 * kTB * LD; q += 64) lds[q] = 0.f;
  // MODE 0: the pool's slot; MODE 1 / 2: the chunk's own [H, N, DV] image in Qbuf (MODE 2 reads its entry state there)
  float* Sg = (MODE == 0 ? state + (((size_t)slots[s] * H + h) * N + row0) * DV
                         : Qbuf + (((size_t)blockIdx.y * H + h) * N + row0) * DV) + j;
  float col[R];
  float pprod = 1.f;
#pragma unroll
  for (int i = 0; i < R; ++i) col[i] = (MODE != 1 && on && i < nrow) ? Sg[(size_t)i * DV] : 0.f;
  const float negA = fixed ? 0.f : -expf(A_log[h]), dskip = Dskip ? Dskip[h] : 0.f, dtb = fixed ? 0.f : dt_bias[h];
  const float fdec = fixed ? fixed[h] : 0.f;
  constexpr int NPART = 64 / kTB;
  static_assert(NP * NPART >= RGS * R, "staging covers a full row");
  const int stt = lane / NPART, spart = lane % NPART;
  float pB[NP], pC[NP], pv[2], pdt = 0.f, pdec = 0.f;
  auto fetch = [&](int tb) {
    const int n = min(kTB, t1 - tb);
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int i = spart + NPART * q;
      if (stt < n && i < N) {
        const size_t o = (size_t)(tb + stt) * ld + (size_t)g * N + i;
        pB[q] = Bm[o];
        pC[q] = Cm[o];
      }
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int idx = q * 64 + lane, tt = idx / COLS, c = cb * COLS + idx % COLS;
      pv[q] = (tt < n && c < DV) ? x[(size_t)(tb + tt) * ld + (size_t)h * DV + c] : 0.f;
    }
    if (lane < n) {
      pdt = fixed ? 1.0f : softplus_f((float)dt[(size_t)(tb + lane) * lddt + h] + dtb);
      pdec = fixed ? fdec : expf(negA * pdt);
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += kTB) {
    const int n = min(kTB, t1 - tb);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int i = spart + NPART * q;
      if (stt < n && i < N) {
        const int a = stt * LD + lds_row<R>(i);
        Bs[a] = pB[q];
        Cs[a] = pC[q];
      }
    }
#pragma unroll
    for (int q = 0; q < 2; ++q)
      if (q * 64 + lane < kTB * COLS) xs[q * 64 + lane] = pv[q];
    if (lane < kTB) {
      ds[lane] = pdt;
      ds[kTB + lane] = pdec;
    }
    __builtin_amdgcn_wave_barrier();
    if (tb + kTB < t1) fetch(tb + kTB);
    for (int tt = 0; tt < n; ++tt) {
      const float xj = xs[tt * COLS + jj], dec = ds[kTB + tt], dx = ds[tt] * xj;
      const int a = tt * LD + row0 + rg;
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int i = 0; i < R; i += 2) {
        col[i] = fmaf(dec, col[i], Bs[a + i] * dx);
        col[i + 1] = fmaf(dec, col[i + 1], Bs[a + i + 1] * dx);
        acc0 = fmaf(col[i], Cs[a + i], acc0);
        acc1 = fmaf(col[i + 1], Cs[a + i + 1], acc1);
      }
      if (MODE == 1) {
        pprod *= dec;
      } else {
        const float acc = rowgroup_sum<RGS>(acc0 + acc1);
        if (rg == 0 && on) out[((size_t)(tb + tt) * H + h) * DV + j] = fmaf(dskip, xj, acc);
      }
    }
  }
  if (MODE != 2 && on) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < nrow) Sg[(size_t)i * DV] = col[i];
  }
  if (MODE == 1 && cb == 0 && lane == 0) Pbuf[(size_t)blockIdx.y * H + h] = pprod;
}

// S <- P S + Q over the chunks of a sequence; Q[chunk] is replaced by the chunk's entry state
__global__ __launch_bounds__(256) void ssd_chunk_carry_kernel(const float* __restrict__ Pbuf, float* __restrict__ Qbuf,
                                                              float* __restrict__ state, const int* __restrict__ cu,
                                                              const int* __restrict__ slots, int H, int ND) {
  const int e = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y, s = blockIdx.z;
  if (e >= ND) return;
  const int len = cu[s + 1] - cu[s];
  if (len <= 0) return;
  int first = 0;
  for (int q = 0; q < s; ++q) first += (cu[q + 1] - cu[q] + kSsdChunk - 1) / kSsdChunk;
  const int nc = (len + kSsdChunk - 1) / kSsdChunk;
  float* sp = state + ((size_t)slots[s] * H + h) * ND + e;
  float Sv = *sp;
  for (int n = 0; n < nc; ++n) {
    float* qp = Qbuf + ((size_t)(first + n) * H + h) * ND + e;
    const float q = *qp;
    *qp = Sv;
    Sv = fmaf(Pbuf[(size_t)(first + n) * H + h], Sv, q);
  }
  *sp = Sv;
}

// ---- selective state-space scan: a decay per channel and state element ----------------------------------------------
// Every (channel, state element) pair is its own scalar recurrence, so there is nothing to contract but the N states of
// a channel at the output: J = 2^k lanes share a channel, each keeping PER states in registers (PER J >= N), and the
// output sum is a J-lane butterfly. One wave64 per (64 / J channels, sequence). PER = 4 streams the state with the fewest
// lanes (decode steps, many sequences); PER = 1 gives a long portion of few sequences four times the waves, each with a
// quarter of the serial work per token. Tokens go through in tiles of kST:
//   A  the tile's step sizes, inputs and gates - fetched into registers one tile ahead, so their latency hides behind
//      the serial part - become softplus(dt + bias), dt * x in LDS (token-parallel: no lane repeats another's softplus),
//      B_t and C_t (shared by all channels) go to LDS too;
//   B  the serial part, a few tokens at a time: decays exp2(dt A) (A pre-multiplied by log2 e), dt x B and C of those
//      tokens first (independent, pipelined), then one FMA per state and token on the dependency chain, then the
//      butterflies of all those tokens; the channel's sums land in LDS;
//   C  token-parallel epilogue: (sum + D x) * silu(z), stored with the lanes along the channels.
// The same kernel serves prompt portions and single decoded tokens (a sequence of one row).
constexpr int kST = 16;
constexpr int kSelBC = 8;    // B / C tile elements a lane prefetches (state sizes up to 32); larger states load in place

template <typename TA, int J, int PER>
__global__ __launch_bounds__(64) void selective_scan_kernel(
    const float* __restrict__ x, int ldx, const float* __restrict__ dt, int lddt, const float* __restrict__ dt_bias,
    const float* __restrict__ A, const TA* __restrict__ Bm, int ldb, const TA* __restrict__ Cm, int ldc,
    const float* __restrict__ Dskip, const TA* __restrict__ z, int ldz, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ slots, TA* __restrict__ out, int ldo, int I, int N) {
  constexpr int CH = 64 / J, NE = kST * CH, NQ = (NE + 63) / 64, NP = PER * J;
  extern __shared__ float lds[];  // B[kST][NP] | C[kST][NP] | dt[NE] | dt x[NE] | y[NE]; NP >= N, the padding stays 0
  const int s = blockIdx.y, lane = threadIdx.x;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  float* Bs = lds;
  float* Cs = Bs + kST * NP;
  float* dtS = Cs + kST * NP;
  for (int e = lane; e < 2 * kST * NP; e += 64) lds[e] = 0.f;
  __syncthreads();
  float* dxS = dtS + NE;
  float* yS = dxS + NE;
  const int c0 = blockIdx.x * CH, cl = lane / J, j = lane % J, c = c0 + cl;
  const bool on = c < I;
  // lane j of a channel owns the states j, j + J, j + 2 J, j + 3 J; those past N are padding: decay exponent 0, B = C = 0
  // in LDS, so they stay 0 and the serial part needs no bounds
  float a2[PER], st[PER];
  float* Sg = state + ((size_t)slots[s] * I + (on ? c : 0)) * N;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const bool ok = on && j + J * i < N;
    a2[i] = ok ? A[(size_t)c * N + j + J * i] * 1.4426950408889634f : 0.f;
    st[i] = ok ? Sg[j + J * i] : 0.f;
  }
  // the tile elements (token, channel) this lane stages and finishes: e = lane + 64 q -> (e / CH, e % CH)
  float bq[NQ], dq[NQ], rdt[NQ], rx[NQ], cx[NQ], cz[NQ];
  TA rz[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int ch = c0 + (lane + 64 * q) % CH;
    bq[q] = ch < I ? dt_bias[ch] : 0.f;
    dq[q] = ch < I ? Dskip[ch] : 0.f;
  }
  const bool bc_regs = kST * N <= 64 * kSelBC;
  TA rb[kSelBC], rc[kSelBC];
  int bt[kSelBC], bi[kSelBC];
#pragma unroll
  for (int q = 0; q < kSelBC; ++q) {
    bt[q] = (lane + 64 * q) / N;
    bi[q] = (lane + 64 * q) - bt[q] * N;
  }
  // Loads only, from clamped (always valid) addresses: nothing here waits for the data, so the next tile's inputs are
  // in flight while the serial part of this tile runs. Rows past the portion's end repeat its last row; they are
  // staged but never used.
  auto fetch = [&](int tb) {
    const int last = min(kST, t1 - tb) - 1;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = lane + 64 * q;
      const size_t t = (size_t)(tb + min(e / CH, last));
      const int ch = min(c0 + e % CH, I - 1);
      rdt[q] = dt[t * lddt + ch];
      rx[q] = x[t * ldx + ch];
      rz[q] = z[t * ldz + ch];
    }
    if (bc_regs) {
#pragma unroll
      for (int q = 0; q < kSelBC; ++q) {
        const size_t t = (size_t)(tb + min(bt[q], last));
        rb[q] = Bm[t * ldb + bi[q]];
        rc[q] = Cm[t * ldc + bi[q]];
      }
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += kST) {
    const int n = min(kST, t1 - tb);
    // ---- A: registers -> LDS
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = lane + 64 * q;
      if (e < NE) {
        const float dtv = softplus_f(rdt[q] + bq[q]);
        dtS[e] = dtv;
        dxS[e] = dtv * rx[q];
      }
      cx[q] = rx[q];
      cz[q] = (float)rz[q];
    }
    if (bc_regs) {
#pragma unroll
      for (int q = 0; q < kSelBC; ++q) {
        const int e = lane + 64 * q;
        if (e < kST * N) {
          Bs[bt[q] * NP + bi[q]] = (float)rb[q];
          Cs[bt[q] * NP + bi[q]] = (float)rc[q];
        }
      }
    } else {
      for (int e = lane; e < n * N; e += 64) {
        const int tt = e / N, i = e - tt * N;
        Bs[tt * NP + i] = (float)Bm[(size_t)(tb + tt) * ldb + i];
        Cs[tt * NP + i] = (float)Cm[(size_t)(tb + tt) * ldc + i];
      }
    }
    __syncthreads();
    if (tb + kST < t1) fetch(tb + kST);  // in flight during the serial part
    // ---- B: the recurrence, SUB tokens at a time: everything off the dependency chain (decays, dt x B, C) is computed
    // for the SUB tokens first, so the chain itself is one FMA per state and token; rows past the portion's end are
    // staged (repeats of its last row) and made neutral here
    constexpr int SUB = kST / PER;
    for (int ts = 0; ts < n; ts += SUB) {
      float dec[PER][SUB], dxb[PER][SUB], ccv[PER][SUB], accv[SUB];
#pragma unroll
      for (int u = 0; u < SUB; ++u) {
        const int tt = ts + u;
        const bool live = tt < n;
        const float dtv = dtS[tt * CH + cl], dx = dxS[tt * CH + cl];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          dec[i][u] = live ? __builtin_amdgcn_exp2f(dtv * a2[i]) : 1.0f;
          dxb[i][u] = live ? dx * Bs[tt * NP + j + J * i] : 0.f;
          ccv[i][u] = Cs[tt * NP + j + J * i];
        }
      }
#pragma unroll
      for (int u = 0; u < SUB; ++u) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          st[i] = fmaf(dec[i][u], st[i], dxb[i][u]);
          acc = fmaf(st[i], ccv[i][u], acc);
        }
        accv[u] = acc;
      }
#pragma unroll
      for (int u = 0; u < SUB; ++u) accv[u] = lanegroup_sum<J>(accv[u]);
      if (j == 0) {
#pragma unroll
        for (int u = 0; u < SUB; ++u) yS[(ts + u) * CH + cl] = accv[u];
      }
    }
    __syncthreads();
    // ---- C: skip term, gate, store
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int e = lane + 64 * q, tt = e / CH, ch = c0 + e % CH;
      if (e < NE && tt < n && ch < I) {
        const float zv = cz[q];
        out[(size_t)(tb + tt) * ldo + ch] = (TA)(fmaf(dq[q], cx[q], yS[e]) * (zv / (1.0f + expf(-zv))));
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < PER; ++i)
    if (on && j + J * i < N) Sg[j + J * i] = st[i];
}

// Single-token steps (every sequence brings one row): no tiles to stage - a thread owns four neighbouring states of a
// channel (one 16-byte state load and store where N % 4 == 0), J lanes a channel; the step is state-bandwidth bound.
// Longer sequences would be walked token by token (correct, not fast): the launcher sends them to the tiled kernel.
template <typename TA, int J>
__global__ __launch_bounds__(256) void selective_step_kernel(
    const float* __restrict__ x, int ldx, const float* __restrict__ dt, int lddt, const float* __restrict__ dt_bias,
    const float* __restrict__ A, const TA* __restrict__ Bm, int ldb, const TA* __restrict__ Cm, int ldc,
    const float* __restrict__ Dskip, const TA* __restrict__ z, int ldz, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ slots, TA* __restrict__ out, int ldo, int I, int N) {
  const int s = blockIdx.y;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  const int g = blockIdx.x * 256 + threadIdx.x, c = g / J, j = g % J, n0 = 4 * j;
  const bool on = c < I;
  float* Sg = state + ((size_t)slots[s] * I + (on ? c : 0)) * N + n0;
  const bool vec = on && (N & 3) == 0 && n0 < N;
  float a2[4], st[4];
  if (vec) {
    const float4 a = *reinterpret_cast<const float4*>(A + (size_t)c * N + n0);
    const float4 v = *reinterpret_cast<const float4*>(Sg);
    a2[0] = a.x, a2[1] = a.y, a2[2] = a.z, a2[3] = a.w;
    st[0] = v.x, st[1] = v.y, st[2] = v.z, st[3] = v.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = on && n0 + i < N;
      a2[i] = ok ? A[(size_t)c * N + n0 + i] : 0.f;
      st[i] = ok ? Sg[i] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) a2[i] *= 1.4426950408889634f;
  const float dtb = on ? dt_bias[c] : 0.f, dsk = on ? Dskip[c] : 0.f;
  for (int t = t0; t < t1; ++t) {
    const float xv = on ? x[(size_t)t * ldx + c] : 0.f;
    const float dtv = softplus_f((on ? dt[(size_t)t * lddt + c] : 0.f) + dtb);
    const float dx = dtv * xv;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (on && n0 + i < N) {
        const float bv = (float)Bm[(size_t)t * ldb + n0 + i], cv = (float)Cm[(size_t)t * ldc + n0 + i];
        st[i] = fmaf(__builtin_amdgcn_exp2f(dtv * a2[i]), st[i], dx * bv);
        acc = fmaf(st[i], cv, acc);
      }
    }
    acc = lanegroup_sum<J>(acc);
    if (on && j == 0) {
      const float zv = (float)z[(size_t)t * ldz + c];
      out[(size_t)t * ldo + c] = (TA)(fmaf(dsk, xv, acc) * (zv / (1.0f + expf(-zv))));
    }
  }
  if (vec) {
    *reinterpret_cast<float4*>(Sg) = make_float4(st[0], st[1], st[2], st[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (on && n0 + i < N) Sg[i] = st[i];
  }
}

}  // namespace

void gai_token_shift_mix(const void* h, const float* mu, int NM, const float* shift_state, const int* cu,
                         const int* slots, int S, void* out, int T, int D, int dt, hipStream_t st) {
  if (T == 0) return;
  if (dt)
    token_shift_mix_kernel<float><<<T, 256, 0, st>>>((const float*)h, mu, NM, shift_state, cu, slots, S, (float*)out, T, D);
  else
    token_shift_mix_kernel<bf16><<<T, 256, 0, st>>>((const bf16*)h, mu, NM, shift_state, cu, slots, S, (bf16*)out, T, D);
  GAI_LAUNCH_CHECK();
}

void gai_state_tail_write(const void* x, int ldx, float* state, const int* cu, const int* slots, int S, int C, int NR,
                          int dt, hipStream_t st) {
  if (S == 0 || NR == 0) return;
  if (NR > 8) gai_launch_error(__FILE__, __LINE__, "state_tail_write: more than 8 rows kept");
  const dim3 grid((C + 255) / 256, S);
  if (dt)
    state_tail_write_kernel<float><<<grid, 256, 0, st>>>((const float*)x, ldx, state, cu, slots, C, NR);
  else
    state_tail_write_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)x, ldx, state, cu, slots, C, NR);
  GAI_LAUNCH_CHECK();
}

void gai_conv_silu(const void* x, int ldx, const float* w, const float* state, const int* cu, const int* slots, int S,
                   float* y, int T, int C, int K, int dt, hipStream_t st, const float* bias, int act) {
  if (T == 0) return;
  const dim3 grid(T, T <= 256 ? (unsigned)((C + 255) / 256 < 16 ? (C + 255) / 256 : 16) : 1u);
  if (dt)
    conv_silu_kernel<float><<<grid, 256, 0, st>>>((const float*)x, ldx, w, state, cu, slots, S, y, C, K, bias, act);
  else
    conv_silu_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)x, ldx, w, state, cu, slots, S, y, C, K, bias, act);
  GAI_LAUNCH_CHECK();
}

void gai_wkv_scan(const void* r, const void* k, const void* v, int ld, const float* wpre, const float* w0,
                  const float* u, float* state, const int* cu, const int* slots, int S, int T, float* out, int H, int D,
                  int dt, float* ws, hipStream_t st) {
  if (S == 0) return;
  if (D > kMaxDK) gai_launch_error(__FILE__, __LINE__, "wkv_scan: head size above 256");
  if (T > S && ws) {  // some sequence brings more than one row: the column-sliced scan (ws: [T, H * D] decays)
    const size_t nw = (size_t)T * H * D;
    wkv_decay_kernel<<<(unsigned)((nw + 255) / 256), 256, 0, st>>>(wpre, w0, ws, nw, H * D);
#define GAI_WKV(TA, R, RGS)                                                                                          \
  do {                                                                                                               \
    const dim3 grid(H, S, (D + 64 / RGS - 1) / (64 / RGS));                                                          \
    const size_t lds = (size_t)(3 * kTB * (RGS * R + RGS) + kTB * (64 / RGS)) * sizeof(float);                       \
    wkv_scan_cols_kernel<TA, R, RGS><<<grid, 64, lds, st>>>((const TA*)r, (const TA*)k, (const TA*)v, ld, ws, u,    \
                                                            state, cu, slots, out, H, D);                           \
  } while (0)
    if (dt) {
      if (D <= 64) GAI_WKV(float, 8, 8); else if (D <= 128) GAI_WKV(float, 8, 16); else GAI_WKV(float, 16, 16);
    } else {
      if (D <= 64) GAI_WKV(bf16, 8, 8); else if (D <= 128) GAI_WKV(bf16, 8, 16); else GAI_WKV(bf16, 16, 16);
    }
#undef GAI_WKV
    GAI_LAUNCH_CHECK();
    return;
  }
  const int RG = (D + kRows - 1) / kRows;
  if (D > kMaxDK || D * RG > 1024) gai_launch_error(__FILE__, __LINE__, "wkv_scan: head size above 256");
  const dim3 grid(H, S);
  const size_t lds = (size_t)(7 * D + 2 * RG * D) * sizeof(float);
  if (dt)
    wkv_scan_kernel<float><<<grid, D * RG, lds, st>>>((const float*)r, (const float*)k, (const float*)v, ld, wpre, w0, u,
                                                      state, cu, slots, out, H, D);
  else
    wkv_scan_kernel<bf16><<<grid, D * RG, lds, st>>>((const bf16*)r, (const bf16*)k, (const bf16*)v, ld, wpre, w0, u,
                                                     state, cu, slots, out, H, D);
  GAI_LAUNCH_CHECK();
}

void gai_delta_prep(const float* qkv, int ld, const void* a, int lda, const void* b, int ldb, const float* A_log,
                    const float* dt_bias, float* qn, float* kn, float* decay, float* beta, int T, int H, int G, int DK,
                    int dt, hipStream_t st) {
  if (T == 0) return;
  if (dt)
    delta_prep_kernel<float><<<T, 256, 0, st>>>(qkv, ld, (const float*)a, lda, (const float*)b, ldb, A_log, dt_bias, qn,
                                                kn, decay, beta, H, G, DK);
  else
    delta_prep_kernel<bf16><<<T, 256, 0, st>>>(qkv, ld, (const bf16*)a, lda, (const bf16*)b, ldb, A_log, dt_bias, qn, kn,
                                               decay, beta, H, G, DK);
  GAI_LAUNCH_CHECK();
}

void gai_delta_scan(const float* q, const float* k, const float* v, int ldv, const float* decay, const float* beta,
                    float* state, const int* cu, const int* slots, int S, int T, float* out, int H, int G, int DK,
                    int DV, hipStream_t st) {
  if (S == 0) return;
  if (H % G) gai_launch_error(__FILE__, __LINE__, "delta_scan: heads must be a multiple of key heads");
  if (DK > kMaxDK) gai_launch_error(__FILE__, __LINE__, "delta_scan: key head size above 256");
  if (T > S) {  // some sequence brings more than one row: the column-sliced scan
#define GAI_DELTA(R, RGS)                                                                                            \
  do {                                                                                                               \
    const dim3 grid(H, S, (DV + 64 / RGS - 1) / (64 / RGS));                                                         \
    const size_t lds = (size_t)(3 * kTB * (RGS * R + RGS) + kTB * (64 / RGS) + kTB) * sizeof(float);                 \
    delta_scan_cols_kernel<R, RGS><<<grid, 64, lds, st>>>(q, k, v, ldv, decay, beta, state, cu, slots, out, H, G,   \
                                                          DK, DV);                                                   \
  } while (0)
    if (DK <= 64) GAI_DELTA(8, 8); else if (DK <= 128) GAI_DELTA(8, 16); else GAI_DELTA(16, 16);
#undef GAI_DELTA
    GAI_LAUNCH_CHECK();
    return;
  }
  const int RG = (DK + kRows - 1) / kRows;
  if (DK > kMaxDK || DV * RG > 1024) gai_launch_error(__FILE__, __LINE__, "delta_scan: head sizes above 256");
  if (H % G) gai_launch_error(__FILE__, __LINE__, "delta_scan: heads must be a multiple of key heads");
  const dim3 grid(H, S);
  const size_t lds = (size_t)(6 * DK + 4 * RG * DV) * sizeof(float);
  delta_scan_kernel<<<grid, DV * RG, lds, st>>>(q, k, v, ldv, decay, beta, state, cu, slots, out, H, G, DK, DV);
  GAI_LAUNCH_CHECK();
}

void gai_decay_gate(const void* z, int ldz, const float* bias, int kind, float param, float* out, int T, int C, int dt,
                    hipStream_t st) {
  if (T == 0 || C == 0) return;
  if (kind < 0 || kind > 2) gai_launch_error(__FILE__, __LINE__, "decay_gate: kind 0 (sigmoid), 1 (sigmoid root) or 2 (exp of sigmoid)");
  if (kind == 1 && !(param > 0.f)) gai_launch_error(__FILE__, __LINE__, "decay_gate: the root must be positive");
  const unsigned grid = (unsigned)(((long)T * C + 255) / 256);
  if (dt)
    decay_gate_kernel<float><<<grid, 256, 0, st>>>((const float*)z, ldz, bias, kind, param, out, T, C);
  else
    decay_gate_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)z, ldz, bias, kind, param, out, T, C);
  GAI_LAUNCH_CHECK();
}

void gai_unit_key_removal(const void* k, int ldk, const void* a, int lda, const float* a_bias, float* av, float* bv, int T,
                          int H, int DK, float eps, int dt, hipStream_t st) {
  if (T == 0) return;
  const int TH = T * H, grid = (TH + 3) / 4;
  if (dt)
    unit_key_removal_kernel<float><<<grid, 256, 0, st>>>((const float*)k, ldk, (const float*)a, lda, a_bias, av, bv, TH, H,
                                                          DK, eps);
  else
    unit_key_removal_kernel<bf16><<<grid, 256, 0, st>>>((const bf16*)k, ldk, (const bf16*)a, lda, a_bias, av, bv, TH, H, DK,
                                                         eps);
  GAI_LAUNCH_CHECK();
}

// fp32 elements of the scratch that the chunked scan of such a step needs (0: the step runs unchunked)
size_t gai_dplr_scan_ws_floats(int T, int S, int H, int DK, int DV, int rank1) {
  const int RGS = DK <= 64 ? 8 : 16;
  const long waves = (long)H * S * ((DV + 64 / RGS - 1) / (64 / RGS));
  if (T <= S || T < 2 * kDplrChunk || waves >= 4096) return 0;  // single tokens, short portions, or SIMDs already full
  const size_t NC = (size_t)T / kDplrChunk + S;
  return NC * H * ((size_t)DK * DV + (rank1 ? (size_t)DK * DK : (size_t)DK));
}

void gai_dplr_scan(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const float* decay,
                   const float* av, const float* bv, float* state, const int* cu, const int* slots, int S, int T,
                   float* out, int H, int DK, int DV, float q_scale, int dt, hipStream_t st, float* ws) {
  if (S == 0 || T == 0) return;
  if (DK > kMaxDK) gai_launch_error(__FILE__, __LINE__, "dplr_scan: key head size above 256");
  if ((av == nullptr) != (bv == nullptr)) gai_launch_error(__FILE__, __LINE__, "dplr_scan: the two removal vectors come together");
  const bool r1 = av != nullptr;
  if (T > S) {  // some sequence brings more than one row: the column-sliced scan
    const bool chunked = ws && gai_dplr_scan_ws_floats(T, S, H, DK, DV, r1) > 0;
    const int NC = T / kDplrChunk + S;
    float* Qbuf = ws;
    float* Tbuf = ws ? ws + (size_t)NC * H * DK * DV : nullptr;
#define GAI_DPLR_L(TA, R, RGS, R1, MODE, NY, NCOL)                                                                   \
  do {                                                                                                               \
    const dim3 grid(H, NY, ((NCOL) + 64 / RGS - 1) / (64 / RGS));                                                    \
    const size_t lds = (size_t)((R1 ? 5 : 3) * kTB * (RGS * R + RGS) + kTB * (64 / RGS)) * sizeof(float);            \
    dplr_scan_cols_kernel<TA, R, RGS, R1, MODE><<<grid, 64, lds, st>>>(                                              \
        (const TA*)q, ldq, (const TA*)k, ldk, (const TA*)v, ldv, decay, av, bv, state, cu, slots, out, H, DK, DV,    \
        q_scale, S, Qbuf, Tbuf);                                                                                     \
  } while (0)
#define GAI_DPLR_C(TA, R, RGS, R1)                                                                                   \
  do {                                                                                                               \
    if (chunked) {                                                                                                   \
      GAI_DPLR_L(TA, R, RGS, R1, 1, NC, R1 ? DV + DK : DV);                                                          \
      if (R1)                                                                                                        \
        dplr_chunk_carry_full_kernel<<<dim3((DV + kCarryCols - 1) / kCarryCols, H, S), 256,                          \
                                       (size_t)DK * kCarryCols * sizeof(float), st>>>(Tbuf, Qbuf, state, cu, slots,  \
                                                                                      H, DK, DV);                    \
      else                                                                                                           \
        dplr_chunk_carry_diag_kernel<<<dim3((DK * DV + 255) / 256, H, S), 256, 0, st>>>(Tbuf, Qbuf, state, cu,       \
                                                                                       slots, H, DK, DV);            \
      GAI_DPLR_L(TA, R, RGS, R1, 2, NC, DV);                                                                         \
    } else {                                                                                                         \
      GAI_DPLR_L(TA, R, RGS, R1, 0, S, DV);                                                                          \
    }                                                                                                                \
  } while (0)
#define GAI_DPLR_S(TA, R1)                                                                                           \
  do {                                                                                                               \
    if (DK <= 64) GAI_DPLR_C(TA, 8, 8, R1); else if (DK <= 128) GAI_DPLR_C(TA, 8, 16, R1);                           \
    else GAI_DPLR_C(TA, 16, 16, R1);                                                                                 \
  } while (0)
    if (dt) { if (r1) GAI_DPLR_S(float, true); else GAI_DPLR_S(float, false); }
    else { if (r1) GAI_DPLR_S(bf16, true); else GAI_DPLR_S(bf16, false); }
#undef GAI_DPLR_S
#undef GAI_DPLR_C
#undef GAI_DPLR_L
    GAI_LAUNCH_CHECK();
    return;
  }
  const int RG = (DK + kRows - 1) / kRows;
  if (DV * RG > 1024) gai_launch_error(__FILE__, __LINE__, "dplr_scan: head sizes above 256");
  const dim3 grid(H, S);
  const size_t lds = (size_t)(10 * DK + 4 * RG * DV) * sizeof(float);
#define GAI_DPLR(TA, R1)                                                                                             \
  dplr_scan_kernel<TA, R1><<<grid, DV * RG, lds, st>>>((const TA*)q, ldq, (const TA*)k, ldk, (const TA*)v, ldv, decay, \
                                                       av, bv, state, cu, slots, out, H, DK, DV, q_scale)
  if (dt) { if (r1) GAI_DPLR(float, true); else GAI_DPLR(float, false); }
  else { if (r1) GAI_DPLR(bf16, true); else GAI_DPLR(bf16, false); }
#undef GAI_DPLR
  GAI_LAUNCH_CHECK();
}

void gai_rglru_gates(const float* u, const float* wa_t, const float* ba, const float* wi_t, const float* bi,
                     const float* lam, float cdecay, float* a_out, float* b_out, int T, int W, int NB, hipStream_t st) {
  if (T == 0) return;
  if (NB < 1 || W % NB) gai_launch_error(__FILE__, __LINE__, "rglru_gates: width must be a multiple of the blocks");
  const int BS = W / NB;
  if (BS > 3584) gai_launch_error(__FILE__, __LINE__, "rglru_gates: block size above 3584");
  if (T <= 64 && BS <= 3072) {  // decode-sized steps
    const dim3 grid((T + kGS - 1) / kGS, NB, (BS + 63) / 64);
    const size_t lds2 = (size_t)(kGS * BS + 4 * 2 * kGS * 64) * sizeof(float);
    rglru_gates_split_kernel<<<grid, 256, lds2, st>>>(u, wa_t, ba, wi_t, bi, lam, cdecay, a_out, b_out, T, W, BS);
    GAI_LAUNCH_CHECK();
    return;
  }
#define GAI_GATES(GT)                                                                                                \
  rglru_gates_kernel<GT><<<dim3((T + GT - 1) / GT, NB), 256, (size_t)GT * BS * sizeof(float), st>>>(                 \
      u, wa_t, ba, wi_t, bi, lam, cdecay, a_out, b_out, T, W, BS)
  if (BS <= 1024) GAI_GATES(16); else if (BS <= 2048) GAI_GATES(8); else GAI_GATES(4);
#undef GAI_GATES
  GAI_LAUNCH_CHECK();
}

int gai_rglru_scan_chunks(int T, int S) { return T / kChunk + S; }

void gai_rglru_scan(const float* a, const float* b, const void* y, int ldy, float* state, const int* cu,
                    const int* slots, int S, int T, void* out, int ldo, int W, int gelu, float scale, int dt, float* ws,
                    hipStream_t st) {
  if (S == 0 || T == 0) return;
  if (T > S && ws) {  // some sequence brings more than one row: chunk-parallel scan (ws: [3][T / kChunk + S][W])
    const int NC = gai_rglru_scan_chunks(T, S);
    float* P = ws;
    float* Q = ws + (size_t)NC * W;
    float* Sin = ws + 2 * (size_t)NC * W;
    const dim3 gc((W + 255) / 256, NC), gs((W + 255) / 256, S);
    rglru_chunk_reduce_kernel<<<gc, 256, 0, st>>>(a, b, cu, S, P, Q, W);
    rglru_chunk_carry_kernel<<<gs, 256, 0, st>>>(P, Q, Sin, state, cu, slots, W);
    if (dt)
      rglru_chunk_apply_kernel<float><<<gc, 256, 0, st>>>(a, b, (const float*)y, ldy, Sin, cu, S, (float*)out, ldo, W,
                                                          gelu, scale);
    else
      rglru_chunk_apply_kernel<bf16><<<gc, 256, 0, st>>>(a, b, (const bf16*)y, ldy, Sin, cu, S, (bf16*)out, ldo, W, gelu,
                                                         scale);
    GAI_LAUNCH_CHECK();
    return;
  }
  const dim3 grid((W + 255) / 256, S);
  if (dt)
    rglru_scan_kernel<float><<<grid, 256, 0, st>>>(a, b, (const float*)y, ldy, state, cu, slots, (float*)out, ldo, W,
                                                   gelu, scale);
  else
    rglru_scan_kernel<bf16><<<grid, 256, 0, st>>>(a, b, (const bf16*)y, ldy, state, cu, slots, (bf16*)out, ldo, W, gelu,
                                                  scale);
  GAI_LAUNCH_CHECK();
}

// fp32 elements of the scratch that the chunked scan of such a step needs (0: the step runs unchunked)
size_t gai_ssd_scan_ws_floats(int T, int S, int H, int N, int DV) {
  const int RGS = N <= 64 ? 8 : 16;
  const long waves = (long)H * S * ((DV + 64 / RGS - 1) / (64 / RGS));
  if (T <= S || T < 2 * kSsdChunk || waves >= 4096) return 0;  // single tokens, short portions, or SIMDs already full
  const size_t NC = (size_t)T / kSsdChunk + S;
  return NC * H * ((size_t)N * DV + 1);
}

void gai_ssd_scan(const float* x, const float* B, const float* C, int ld, const void* dt, int lddt,
                  const float* dt_bias, const float* A_log, const float* D, float* state, const int* cu,
                  const int* slots, int S, int T, float* out, int H, int G, int N, int DV, int dtt, float* ws,
                  hipStream_t st, const float* fixed) {
  if (S == 0) return;
  if (!fixed && (!dt || !dt_bias || !A_log || !D))
    gai_launch_error(__FILE__, __LINE__, "ssd_scan: step sizes, their bias, A_log and D, or a fixed decay per head");
  if (H % G) gai_launch_error(__FILE__, __LINE__, "ssd_scan: heads must be a multiple of groups");
  if (N > kMaxDK) gai_launch_error(__FILE__, __LINE__, "ssd_scan: state size above 256");
  if (T > S) {  // some sequence brings more than one row: the column-sliced scan
    const bool chunked = ws && gai_ssd_scan_ws_floats(T, S, H, N, DV) > 0;
    const int NC = T / kSsdChunk + S;
    float* Qbuf = ws;
    float* Pbuf = ws ? ws + (size_t)NC * H * N * DV : nullptr;
#define GAI_SSD_L(TA, R, RGS, MODE, NY)                                                                              \
  do {                                                                                                               \
    const dim3 grid(H, NY, (DV + 64 / RGS - 1) / (64 / RGS));                                                        \
    const size_t lds = (size_t)(2 * kTB * (RGS * R + RGS) + kTB * (64 / RGS) + 2 * kTB) * sizeof(float);             \
    ssd_scan_cols_kernel<TA, R, RGS, MODE><<<grid, 64, lds, st>>>(x, B, C, ld, (const TA*)dt, lddt, dt_bias, A_log,  \
                                                                  D, state, cu, slots, out, H, G, N, DV, S, Pbuf,   \
                                                                  Qbuf, fixed);                                      \
  } while (0)
#define GAI_SSD(TA, R, RGS)                                                                                          \
  do {                                                                                                               \
    if (chunked) {                                                                                                   \
      GAI_SSD_L(TA, R, RGS, 1, NC);                                                                                  \
      ssd_chunk_carry_kernel<<<dim3((N * DV + 255) / 256, H, S), 256, 0, st>>>(Pbuf, Qbuf, state, cu, slots, H,      \
                                                                                N * DV);                             \
      GAI_SSD_L(TA, R, RGS, 2, NC);                                                                                  \
    } else {                                                                                                         \
      GAI_SSD_L(TA, R, RGS, 0, S);                                                                                   \
    }                                                                                                                \
  } while (0)
    if (dtt) {
      if (N <= 64) GAI_SSD(float, 8, 8); else if (N <= 128) GAI_SSD(float, 8, 16); else GAI_SSD(float, 16, 16);
    } else {
      if (N <= 64) GAI_SSD(bf16, 8, 8); else if (N <= 128) GAI_SSD(bf16, 8, 16); else GAI_SSD(bf16, 16, 16);
    }
#undef GAI_SSD
#undef GAI_SSD_L
    GAI_LAUNCH_CHECK();
    return;
  }
  const int RG = (N + kRows - 1) / kRows;
  if (DV * RG > 1024) gai_launch_error(__FILE__, __LINE__, "ssd_scan: value head size times state row groups above 1024");
  const dim3 grid(H, S);
  const size_t lds = (size_t)(4 * N + 2 * RG * DV) * sizeof(float);
  if (dtt)
    ssd_scan_kernel<float><<<grid, DV * RG, lds, st>>>(x, B, C, ld, (const float*)dt, lddt, dt_bias, A_log, D, state, cu,
                                                       slots, out, H, G, N, DV, fixed);
  else
    ssd_scan_kernel<bf16><<<grid, DV * RG, lds, st>>>(x, B, C, ld, (const bf16*)dt, lddt, dt_bias, A_log, D, state, cu,
                                                      slots, out, H, G, N, DV, fixed);
  GAI_LAUNCH_CHECK();
}

void gai_selective_scan(const float* x, int ldx, const float* dt, int lddt, const float* dt_bias, const float* A,
                        const void* B, int ldb, const void* C, int ldc, const float* D, const void* z, int ldz,
                        float* state, const int* cu, const int* slots, int S, int T, void* out, int ldo, int I, int N,
                        int dtt, hipStream_t st) {
  if (S == 0) return;
  if (N < 1 || N > 256) gai_launch_error(__FILE__, __LINE__, "selective_scan: 1 <= state size <= 256");
  int J4 = 1, J1 = 1;
  while (J4 * 4 < N) J4 <<= 1;  // 4 states per lane
  while (J1 < N) J1 <<= 1;      // 1 state per lane
  if (T == S) {  // single-token steps
    const dim3 sgrid((unsigned)(((size_t)I * J4 + 255) / 256), S);
#define GAI_STEP(TA, J_)                                                                                              \
  selective_step_kernel<TA, J_><<<sgrid, 256, 0, st>>>(x, ldx, dt, lddt, dt_bias, A, (const TA*)B, ldb, (const TA*)C, \
                                                       ldc, D, (const TA*)z, ldz, state, cu, slots, (TA*)out, ldo, I, N)
#define GAI_STEP_J(TA)                                                                                                \
  switch (J4) {                                                                                                       \
    case 1: GAI_STEP(TA, 1); break;                                                                                   \
    case 2: GAI_STEP(TA, 2); break;                                                                                   \
    case 4: GAI_STEP(TA, 4); break;                                                                                   \
    case 8: GAI_STEP(TA, 8); break;                                                                                   \
    case 16: GAI_STEP(TA, 16); break;                                                                                 \
    case 32: GAI_STEP(TA, 32); break;                                                                                 \
    default: GAI_STEP(TA, 64); break;                                                                                 \
  }
    if (dtt) { GAI_STEP_J(float) } else { GAI_STEP_J(bf16) }
#undef GAI_STEP_J
#undef GAI_STEP
    GAI_LAUNCH_CHECK();
    return;
  }
  // portions (more rows than sequences) that would leave SIMDs idle with 4 states per lane spread over 4 x the waves
  const bool spread = T > S && N <= 64 && (long)S * ((I * J4 + 63) / 64) < 2048;
  const int J = spread ? J1 : J4, PER = spread ? 1 : 4, CH = 64 / J;
  const dim3 grid((unsigned)((I + CH - 1) / CH), S);
  const size_t lds = (size_t)(2 * kST * PER * J + 3 * kST * CH) * sizeof(float);
#define GAI_SEL(TA, J_, P_)                                                                                           \
  selective_scan_kernel<TA, J_, P_><<<grid, 64, lds, st>>>(x, ldx, dt, lddt, dt_bias, A, (const TA*)B, ldb,           \
                                                           (const TA*)C, ldc, D, (const TA*)z, ldz, state, cu, slots, \
                                                           (TA*)out, ldo, I, N)
#define GAI_SEL_J(TA, P_)                                                                                             \
  switch (J) {                                                                                                        \
    case 1: GAI_SEL(TA, 1, P_); break;                                                                                \
    case 2: GAI_SEL(TA, 2, P_); break;                                                                                \
    case 4: GAI_SEL(TA, 4, P_); break;                                                                                \
    case 8: GAI_SEL(TA, 8, P_); break;                                                                                \
    case 16: GAI_SEL(TA, 16, P_); break;                                                                              \
    case 32: GAI_SEL(TA, 32, P_); break;                                                                              \
    default: GAI_SEL(TA, 64, P_); break;                                                                              \
  }
  if (dtt) {
    if (PER == 1) { GAI_SEL_J(float, 1) } else { GAI_SEL_J(float, 4) }
  } else {
    if (PER == 1) { GAI_SEL_J(bf16, 1) } else { GAI_SEL_J(bf16, 4) }
  }
#undef GAI_SEL_J
#undef GAI_SEL
  GAI_LAUNCH_CHECK();
}
