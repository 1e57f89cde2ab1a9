// PyTorch bindings of the sequence-mixer kernels with a 32-bit residual / state (norm_f32.hip, attention_window.hip,
// recurrent.hip). Shape / dtype checks on the host, a launch on the current stream, no allocation: graph-capturable.
// Activation tensors are bf16 or fp32 (all of one call alike); per-channel tables and states are fp32.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include "gai_kernels.h"

namespace {

using at::Tensor;
using c10::optional;

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

int act_dt(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name, " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat ? 1 : 0;
}
void same_dt(const Tensor& t, int dt, const char* name) { TORCH_CHECK(act_dt(t, name) == dt, name, ": dtype differs"); }
const float* f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be a contiguous fp32 GPU tensor");
  return t.data_ptr<float>();
}
float* f32w(Tensor& t, const char* name) { return const_cast<float*>(f32(t, name)); }
const int* i32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, " must be a contiguous int32 GPU tensor");
  return t.data_ptr<int>();
}
// [rows, cols] view with unit column stride (a column slice of a wider projection output)
int row_stride(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be 2-D with contiguous rows");
  return (int)t.stride(0);
}

void add_rmsnorm_f32(Tensor& res, const optional<Tensor>& delta, double mult, const optional<Tensor>& w,
                     const optional<Tensor>& out, double eps) {
  float* r = f32w(res, "res");
  TORCH_CHECK(res.dim() == 2, "add_rmsnorm_f32: res [T, D]");
  const int T = res.size(0), D = res.size(1);
  int dd = 0, od = 0, ldd = 0;
  if (delta) {
    dd = act_dt(*delta, "delta");
    ldd = row_stride(*delta, "delta");
    TORCH_CHECK(delta->size(0) == T && delta->size(1) == D, "add_rmsnorm_f32: delta shape");
  }
  if (out) {
    od = act_dt(*out, "out");
    TORCH_CHECK(out->is_contiguous() && out->numel() == (int64_t)T * D, "add_rmsnorm_f32: out shape");
  }
  TORCH_CHECK(delta || out, "add_rmsnorm_f32: nothing to do");
  if (w) TORCH_CHECK(w->numel() == D, "add_rmsnorm_f32: weight size");
  gai_add_rmsnorm_f32(r, delta ? delta->data_ptr() : nullptr, ldd, (float)mult, w ? f32(*w, "w") : nullptr,
                      out ? out->data_ptr() : nullptr, T, D, (float)eps, dd, od, cur_stream());
}

void poly_norm(const Tensor& z, const Tensor& coef, double eps, Tensor& y) {
  const int dt = act_dt(z, "z");
  same_dt(y, dt, "y");
  TORCH_CHECK(z.dim() == 2 && z.is_contiguous() && y.is_contiguous() && y.numel() == z.numel(), "poly_norm: shapes");
  TORCH_CHECK(coef.numel() == 4, "poly_norm: four coefficients");
  gai_poly_norm(z.data_ptr(), y.data_ptr(), f32(coef, "coef"), z.size(0), z.size(1), (float)eps, dt, cur_stream());
}

void head_norm_gate(const Tensor& o, const Tensor& gate, const Tensor& nw, int64_t act, double eps, Tensor& y) {
  TORCH_CHECK(o.dim() == 3, "head_norm_gate: o [T, H, DV]");
  const int T = o.size(0), H = o.size(1), DV = o.size(2);
  const int dt = act_dt(gate, "gate");
  same_dt(y, dt, "y");
  const int ldg = row_stride(gate, "gate");
  const int ldy = row_stride(y, "y");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == H * DV && y.size(0) == T && y.size(1) == H * DV,
              "head_norm_gate: gate / y shapes");
  TORCH_CHECK(nw.numel() == DV || nw.numel() == H * DV, "head_norm_gate: norm weight size");
  TORCH_CHECK(act == 0 || act == 1, "head_norm_gate: act 0 (silu) or 1 (sigmoid)");
  gai_head_norm_gate(f32(o, "o"), gate.data_ptr(), ldg, f32(nw, "nw"), nw.numel() == H * DV && H > 1 ? 1 : 0, (int)act,
                     y.data_ptr(), ldy, T, H, DV, (float)eps, dt, cur_stream());
}

void embed_scale_f32(const Tensor& ids, const Tensor& table, double scale, Tensor& out,
                     const optional<Tensor>& positions, const optional<Tensor>& pos_table) {
  const int dt = act_dt(table, "table");
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous(), "embed_scale_f32: table [V, D]");
  const int T = ids.numel(), D = table.size(1);
  TORCH_CHECK(out.numel() == (int64_t)T * D, "embed_scale_f32: out shape");
  TORCH_CHECK(positions.has_value() == pos_table.has_value(), "embed_scale_f32: positions and their table come together");
  int P = 0;
  if (pos_table) {
    same_dt(*pos_table, dt, "pos_table");
    TORCH_CHECK(pos_table->dim() == 2 && pos_table->is_contiguous() && pos_table->size(1) == D && pos_table->size(0) >= 1 &&
                    positions->numel() >= T, "embed_scale_f32: position table [P, D], one position per token");
    P = pos_table->size(0);
  }
  gai_embed_scale_f32(i32(ids, "ids"), table.data_ptr(), (float)scale, f32w(out, "out"), T, D, table.size(0), dt,
                      cur_stream(), positions ? i32(*positions, "positions") : nullptr,
                      pos_table ? pos_table->data_ptr() : nullptr, P);
}

void gated_norm_add_f32(Tensor& res, const Tensor& y, const optional<Tensor>& gate, const Tensor& wpost, double eps,
                        const optional<Tensor>& wnext, optional<Tensor> out) {
  TORCH_CHECK(res.dim() == 2, "gated_norm_add_f32: res [T, D]");
  float* r = f32w(res, "res");
  const int T = res.size(0), D = res.size(1);
  const int dty = act_dt(y, "y"), dtg = gate ? act_dt(*gate, "gate") : dty;
  TORCH_CHECK(y.size(0) == T && y.size(1) == D && (!gate || (gate->size(0) == T && gate->size(1) == D)) &&
                  wpost.numel() == D, "gated_norm_add_f32: y / gate / weight shapes");
  int dto = 0;
  if (out) {
    dto = act_dt(*out, "out");
    TORCH_CHECK(out->is_contiguous() && out->numel() == (int64_t)T * D, "gated_norm_add_f32: out shape");
  }
  if (wnext) TORCH_CHECK(wnext->numel() == D, "gated_norm_add_f32: next norm weight size");
  gai_gated_norm_add_f32(r, y.data_ptr(), row_stride(y, "y"), dty, gate ? gate->data_ptr() : nullptr,
                         gate ? row_stride(*gate, "gate") : 0, dtg,
                         f32(wpost, "wpost"), wnext ? f32(*wnext, "wnext") : nullptr, out ? out->data_ptr() : nullptr,
                         dto, T, D, (float)eps, cur_stream());
}

void gate_group_norm(const Tensor& y, const Tensor& z, const Tensor& w, int64_t groups, double eps, Tensor& out) {
  TORCH_CHECK(y.dim() == 2, "gate_group_norm: y [T, C]");
  const int T = y.size(0), C = y.size(1);
  const int dt = act_dt(z, "z");
  same_dt(out, dt, "out");
  TORCH_CHECK(groups >= 1 && C % groups == 0 && z.size(0) == T && z.size(1) == C && w.numel() == C &&
                  out.is_contiguous() && out.numel() == (int64_t)T * C, "gate_group_norm: shapes");
  gai_gate_group_norm(f32(y, "y"), z.data_ptr(), row_stride(z, "z"), f32(w, "w"), out.data_ptr(), T, (int)groups,
                      C / (int)groups, (float)eps, dt, cur_stream());
}

void check_cache(const Tensor& kc, const Tensor& vc, int dt, int G, int DK, int DV) {
  same_dt(kc, dt, "k_cache");
  same_dt(vc, dt, "v_cache");
  TORCH_CHECK(kc.dim() == 4 && vc.dim() == 4 && kc.is_contiguous() && vc.is_contiguous(), "kv cache: 4-D contiguous");
  TORCH_CHECK(kc.size(1) == G && kc.size(2) == 16 && kc.size(3) == DK, "k_cache must be [pages, G, 16, DK]");
  TORCH_CHECK(vc.size(0) == kc.size(0) && vc.size(1) == G && vc.size(2) == DV && vc.size(3) == 16,
              "v_cache must be [pages, G, DV, 16]");
}

void qknorm_kv_write(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& wq, const Tensor& wk,
                     const Tensor& slots, Tensor& q_out, Tensor& k_cache, Tensor& v_cache, int64_t H, int64_t G,
                     int64_t DK, int64_t DV, double eps) {
  const int dt = act_dt(q, "q");
  same_dt(k, dt, "k");
  same_dt(v, dt, "v");
  same_dt(q_out, dt, "q_out");
  check_cache(k_cache, v_cache, dt, G, DK, DV);
  const int T = q.size(0);
  TORCH_CHECK(q.size(1) == H * DK && k.size(0) == T && k.size(1) == G * DK && v.size(0) == T && v.size(1) == G * DV,
              "qknorm_kv_write: projection shapes");
  TORCH_CHECK(wq.numel() == H * DK && wk.numel() == G * DK && slots.numel() >= T && q_out.is_contiguous() &&
                  q_out.numel() == (int64_t)T * H * DK, "qknorm_kv_write: weight / slot / output shapes");
  gai_qknorm_kv_write(q.data_ptr(), row_stride(q, "q"), k.data_ptr(), row_stride(k, "k"), v.data_ptr(),
                      row_stride(v, "v"), f32(wq, "wq"), f32(wk, "wk"), i32(slots, "slots"), q_out.data_ptr(),
                      k_cache.data_ptr(), v_cache.data_ptr(), T, H, G, DK, DV, (float)eps, dt, cur_stream());
}

void headnorm_kv_write(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& wq, const Tensor& wk,
                       const Tensor& slots, const optional<Tensor>& positions, Tensor& q_out, Tensor& k_cache,
                       Tensor& v_cache, int64_t H, int64_t G, int64_t DK, int64_t DV, double eps, double temp_coef,
                       int64_t temp_every) {
  const int dt = act_dt(q, "q");
  same_dt(k, dt, "k");
  same_dt(v, dt, "v");
  same_dt(q_out, dt, "q_out");
  check_cache(k_cache, v_cache, dt, G, DK, DV);
  const int T = q.size(0);
  TORCH_CHECK(q.size(1) == H * DK && k.size(0) == T && k.size(1) == G * DK && v.size(0) == T && v.size(1) == G * DV,
              "headnorm_kv_write: projection shapes");
  TORCH_CHECK(wq.numel() == DK && wk.numel() == DK && slots.numel() >= T && q_out.is_contiguous() &&
                  q_out.numel() == (int64_t)T * H * DK, "headnorm_kv_write: weight / slot / output shapes");
  if (positions) TORCH_CHECK(positions->numel() >= T && temp_every >= 1, "headnorm_kv_write: one position per token");
  gai_headnorm_kv_write(q.data_ptr(), row_stride(q, "q"), k.data_ptr(), row_stride(k, "k"), v.data_ptr(),
                        row_stride(v, "v"), f32(wq, "wq"), f32(wk, "wk"), i32(slots, "slots"),
                        positions ? i32(*positions, "positions") : nullptr, q_out.data_ptr(), k_cache.data_ptr(),
                        v_cache.data_ptr(), T, H, G, DK, DV, (float)eps, (float)temp_coef, (int)temp_every, dt,
                        cur_stream());
}

void window_attention(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& block_tables,
                      const Tensor& cu_q, const Tensor& ctx, Tensor& out, int64_t H, int64_t G, int64_t DK, int64_t DV,
                      double scale, double softcap, int64_t window, const optional<Tensor>& r1,
                      const optional<Tensor>& r2, const optional<Tensor>& gate, const optional<Tensor>& sig_bias,
                      bool sigmoid, double out_scale, const optional<Tensor>& part, int64_t chunk,
                      const optional<Tensor>& head_scale, const optional<double>& sink) {
  const int dt = act_dt(q, "q");
  same_dt(out, dt, "out");
  check_cache(k_cache, v_cache, dt, G, DK, DV);
  TORCH_CHECK(q.is_contiguous() && q.numel() % (H * DK) == 0, "window_attention: q shape");
  const int T = q.numel() / (H * DK);
  const int S = ctx.numel();
  const int ldo = row_stride(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * DV && cu_q.numel() == S + 1 && block_tables.dim() == 2 &&
                  block_tables.size(0) >= S, "window_attention: out / cu_q / block table shapes");
  if (sig_bias) TORCH_CHECK(sigmoid && sig_bias->numel() == H, "window_attention: one sigmoid bias per head");
  if (head_scale) TORCH_CHECK(!sigmoid && head_scale->numel() == H, "window_attention: one score scale per head, softmax mode");
  TORCH_CHECK(chunk >= 0 && (!sigmoid || (chunk == 0 && !sink)), "window_attention: chunks and sinks go with the softmax mode");
  if (sigmoid) TORCH_CHECK(!gate && !r1 && softcap == 0.0, "window_attention: sigmoid mode takes no cap, distance term or gate");
  TORCH_CHECK(r1.has_value() == r2.has_value(), "window_attention: r1 and r2 come together");
  if (r1) TORCH_CHECK(r1->numel() == H && r2->numel() == H, "window_attention: one distance pair per head");
  int ldg = 0;
  if (gate) {  // output multiplied by sigmoid(gate), [T, H * DV] rows of a wider projection
    same_dt(*gate, dt, "gate");
    ldg = row_stride(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == H * DV, "window_attention: gate shape");
  }
  float* partp = nullptr;
  if (part) {  // scratch of the key-split decode form (softmax mode keeps a maximum and a denominator per row too)
    TORCH_CHECK(part->is_cuda() && part->scalar_type() == at::kFloat && part->is_contiguous() &&
                    part->numel() >= (int64_t)gai_sigmoid_attention_splits(T, S, H) * T * H * (sigmoid ? DV : DV + 2),
                "window_attention: split scratch too small");
    partp = part->data_ptr<float>();
  }
  gai_window_attention(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), i32(block_tables, "block_tables"),
                       block_tables.size(1), i32(cu_q, "cu_q"), i32(ctx, "ctx"), S, out.data_ptr(), ldo, T, H, G, DK, DV,
                       (float)scale, (float)softcap, (int)window, r1 ? f32(*r1, "r1") : nullptr,
                       r2 ? f32(*r2, "r2") : nullptr, gate ? gate->data_ptr() : nullptr, ldg,
                       sig_bias ? f32(*sig_bias, "sig_bias") : nullptr, sigmoid ? 1 : 0, (float)out_scale, dt,
                       cur_stream(), partp, (int)chunk, head_scale ? f32(*head_scale, "head_scale") : nullptr, sink ? 1 : 0,
                       sink ? (float)*sink : 0.f);
}

void rotary_kv_write(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& positions, const Tensor& slots,
                     Tensor& q_out, Tensor& k_cache, Tensor& v_cache, int64_t H, int64_t G, int64_t DK, int64_t DV,
                     int64_t rot, double base) {
  const int di = act_dt(q, "q"), dt = act_dt(k_cache, "k_cache");
  same_dt(k, di, "k");
  same_dt(v, di, "v");
  same_dt(q_out, dt, "q_out");
  check_cache(k_cache, v_cache, dt, G, DK, DV);
  const int T = q.size(0);
  TORCH_CHECK(q.size(1) == H * DK && k.size(0) == T && k.size(1) == G * DK && v.size(0) == T && v.size(1) == G * DV,
              "rotary_kv_write: projection shapes");
  TORCH_CHECK(slots.numel() >= T && positions.numel() >= T && q_out.is_contiguous() && q_out.numel() == (int64_t)T * H * DK,
              "rotary_kv_write: slot / position / output shapes");
  TORCH_CHECK(di == 1 || dt == 0, "rotary_kv_write: bf16 inputs go with a bf16 cache");
  gai_rotary_kv_write(q.data_ptr(), row_stride(q, "q"), k.data_ptr(), row_stride(k, "k"), v.data_ptr(), row_stride(v, "v"),
                      i32(positions, "positions"), i32(slots, "slots"), q_out.data_ptr(), k_cache.data_ptr(),
                      v_cache.data_ptr(), T, H, G, DK, DV, (int)rot, (float)base, di, dt, cur_stream());
}

void decay_gate(const Tensor& z, const optional<Tensor>& bias, int64_t kind, double param, Tensor& out) {
  const int dt = act_dt(z, "z");
  const int T = z.size(0), C = z.size(1);
  TORCH_CHECK(kind >= 0 && kind <= 2 && out.numel() == (int64_t)T * C, "decay_gate: kind 0 .. 2, out [T, C]");
  if (bias) TORCH_CHECK(bias->numel() == C, "decay_gate: one bias per channel");
  gai_decay_gate(z.data_ptr(), row_stride(z, "z"), bias ? f32(*bias, "bias") : nullptr, (int)kind, (float)param,
                 f32w(out, "out"), T, C, dt, cur_stream());
}

void unit_key_removal(const Tensor& k, const Tensor& a, const optional<Tensor>& a_bias, int64_t H, int64_t DK, double eps,
                      Tensor& av, Tensor& bv) {
  const int dt = act_dt(k, "k");
  same_dt(a, dt, "a");
  const int T = k.size(0);
  TORCH_CHECK(k.size(1) == H * DK && a.size(0) == T && a.size(1) == H * DK && av.numel() == (int64_t)T * H * DK &&
                  bv.numel() == av.numel(), "unit_key_removal: k / a [T, H * DK]");
  if (a_bias) TORCH_CHECK(a_bias->numel() == H * DK, "unit_key_removal: one bias per channel");
  gai_unit_key_removal(k.data_ptr(), row_stride(k, "k"), a.data_ptr(), row_stride(a, "a"),
                       a_bias ? f32(*a_bias, "a_bias") : nullptr, f32w(av, "av"), f32w(bv, "bv"), T, H, DK, (float)eps, dt,
                       cur_stream());
}

void dplr_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& decay, const optional<Tensor>& av,
               const optional<Tensor>& bv, Tensor& state, const Tensor& cu, const Tensor& slots, Tensor& out,
               double q_scale, const optional<Tensor>& ws) {
  const int dt = act_dt(q, "q");
  same_dt(k, dt, "k");
  same_dt(v, dt, "v");
  TORCH_CHECK(state.dim() == 4, "dplr_scan: state [slots, H, DK, DV]");
  const int T = q.size(0), H = state.size(1), DK = state.size(2), DV = state.size(3), S = slots.numel();
  TORCH_CHECK(q.size(1) == H * DK && k.size(0) == T && k.size(1) == H * DK && v.size(0) == T && v.size(1) == H * DV &&
                  decay.numel() == (int64_t)T * H * DK && out.numel() == (int64_t)T * H * DV && cu.numel() == S + 1,
              "dplr_scan: q / k / decay [T, H * DK], v [T, H * DV], out [T, H, DV]");
  TORCH_CHECK(av.has_value() == bv.has_value(), "dplr_scan: the two removal vectors come together");
  if (av) TORCH_CHECK(av->numel() == decay.numel() && bv->numel() == decay.numel(), "dplr_scan: av / bv [T, H * DK]");
  float* wsp = nullptr;
  if (ws) {  // scratch of the chunk-parallel form
    TORCH_CHECK(ws->is_cuda() && ws->scalar_type() == at::kFloat && ws->is_contiguous() &&
                    (size_t)ws->numel() >= gai_dplr_scan_ws_floats(T, S, H, DK, DV, av ? 1 : 0),
                "dplr_scan: chunk scratch too small");
    wsp = ws->data_ptr<float>();
  }
  gai_dplr_scan(q.data_ptr(), row_stride(q, "q"), k.data_ptr(), row_stride(k, "k"), v.data_ptr(), row_stride(v, "v"),
                f32(decay, "decay"), av ? f32(*av, "av") : nullptr, bv ? f32(*bv, "bv") : nullptr, f32w(state, "state"),
                i32(cu, "cu"), i32(slots, "slots"), S, T, f32w(out, "out"), H, DK, DV, (float)q_scale, dt, cur_stream(),
                wsp);
}

int64_t dplr_scan_ws_floats(int64_t T, int64_t S, int64_t H, int64_t DK, int64_t DV, bool rank1) {
  return (int64_t)gai_dplr_scan_ws_floats((int)T, (int)S, (int)H, (int)DK, (int)DV, rank1 ? 1 : 0);
}

void token_shift_mix(const Tensor& h, const Tensor& mu, const Tensor& shift_state, const Tensor& cu, const Tensor& slots,
                     Tensor& out) {
  const int dt = act_dt(h, "h");
  same_dt(out, dt, "out");
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && mu.dim() == 2 && mu.size(1) == h.size(1), "token_shift_mix: shapes");
  const int T = h.size(0), D = h.size(1), NM = mu.size(0), S = slots.numel();
  TORCH_CHECK(out.is_contiguous() && out.numel() == (int64_t)NM * T * D && cu.numel() == S + 1 &&
                  shift_state.dim() == 2 && shift_state.size(1) == D, "token_shift_mix: out / cu / state shapes");
  gai_token_shift_mix(h.data_ptr(), f32(mu, "mu"), NM, f32(shift_state, "shift_state"), i32(cu, "cu"),
                      i32(slots, "slots"), S, out.data_ptr(), T, D, dt, cur_stream());
}

void state_tail_write(const Tensor& x, Tensor& state, const Tensor& cu, const Tensor& slots) {
  const int dt = act_dt(x, "x");
  const int ldx = row_stride(x, "x");
  const int C = x.size(1), S = slots.numel();
  TORCH_CHECK(state.dim() == 3 && state.size(2) == C && cu.numel() == S + 1, "state_tail_write: state [slots, rows, C]");
  gai_state_tail_write(x.data_ptr(), ldx, f32w(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S, C,
                       (int)state.size(1), dt, cur_stream());
}

void conv_silu(const Tensor& x, const Tensor& w, const Tensor& state, const Tensor& cu, const Tensor& slots, Tensor& y,
               const optional<Tensor>& bias, bool act) {
  const int dt = act_dt(x, "x");
  const int ldx = row_stride(x, "x");
  const int T = x.size(0), C = x.size(1), K = w.size(1), S = slots.numel();
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && K >= 1, "conv_silu: weight [C, taps]");
  TORCH_CHECK(state.dim() == 3 && state.size(1) == K - 1 && state.size(2) == C && cu.numel() == S + 1 &&
                  y.numel() == (int64_t)T * C, "conv_silu: state / cu / y shapes");
  if (bias) TORCH_CHECK(bias->numel() == C, "conv_silu: one bias per channel");
  gai_conv_silu(x.data_ptr(), ldx, f32(w, "w"), f32(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S,
                f32w(y, "y"), T, C, K, dt, cur_stream(), bias ? f32(*bias, "bias") : nullptr, act ? 1 : 0);
}

void rglru_gates(const Tensor& u, const Tensor& wa_t, const Tensor& ba, const Tensor& wi_t, const Tensor& bi,
                 const Tensor& lam, double cdecay, Tensor& a, Tensor& b) {
  TORCH_CHECK(u.dim() == 2 && wa_t.dim() == 3 && wa_t.size(1) == wa_t.size(2), "rglru_gates: u [T, W], gates [blocks, in, out]");
  const int T = u.size(0), W = u.size(1), NB = wa_t.size(0);
  TORCH_CHECK(NB * wa_t.size(1) == W && wi_t.sizes() == wa_t.sizes() && ba.numel() == W && bi.numel() == W &&
                  lam.numel() == W && a.numel() == (int64_t)T * W && b.numel() == a.numel(), "rglru_gates: shapes");
  gai_rglru_gates(f32(u, "u"), f32(wa_t, "wa_t"), f32(ba, "ba"), f32(wi_t, "wi_t"), f32(bi, "bi"), f32(lam, "lam"),
                  (float)cdecay, f32w(a, "a"), f32w(b, "b"), T, W, NB, cur_stream());
}

int64_t rglru_scan_ws_floats(int64_t T, int64_t S, int64_t W) { return 3 * (int64_t)gai_rglru_scan_chunks(T, S) * W; }

void rglru_scan(const Tensor& a, const Tensor& b, const Tensor& y, Tensor& state, const Tensor& cu, const Tensor& slots,
                Tensor& out, bool gelu, double out_scale, const optional<Tensor>& ws) {
  TORCH_CHECK(a.dim() == 2 && state.dim() == 2, "rglru_scan: a [T, W], state [slots, W]");
  const int T = a.size(0), W = a.size(1), S = slots.numel();
  const int dt = act_dt(y, "y");
  same_dt(out, dt, "out");
  TORCH_CHECK(b.numel() == a.numel() && y.size(0) == T && y.size(1) == W && out.size(0) == T && out.size(1) == W &&
                  state.size(1) == W && cu.numel() == S + 1, "rglru_scan: shapes");
  float* wsp = nullptr;
  if (ws) {
    TORCH_CHECK(ws->is_cuda() && ws->scalar_type() == at::kFloat && ws->is_contiguous() &&
                    ws->numel() >= rglru_scan_ws_floats(T, S, W), "rglru_scan: workspace too small");
    wsp = ws->data_ptr<float>();
  }
  gai_rglru_scan(f32(a, "a"), f32(b, "b"), y.data_ptr(), row_stride(y, "y"), f32w(state, "state"), i32(cu, "cu"),
                 i32(slots, "slots"), S, T, out.data_ptr(), row_stride(out, "out"), W, gelu ? 1 : 0, (float)out_scale,
                 dt, wsp, cur_stream());
}

int64_t ssd_scan_ws_floats(int64_t T, int64_t S, int64_t H, int64_t N, int64_t DV) {
  return (int64_t)gai_ssd_scan_ws_floats(T, S, H, N, DV);
}

void ssd_scan(const Tensor& x, const Tensor& B, const Tensor& C, const Tensor& dt, const Tensor& dt_bias,
              const Tensor& A_log, const Tensor& D, Tensor& state, const Tensor& cu, const Tensor& slots, Tensor& out,
              int64_t G, const optional<Tensor>& ws) {
  TORCH_CHECK(state.dim() == 4, "ssd_scan: state [slots, H, N, DV]");
  const int H = state.size(1), N = state.size(2), DV = state.size(3), S = slots.numel();
  auto f32row = [](const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.scalar_type() == at::kFloat && t.stride(1) == 1, name, " must be fp32 rows");
    return (int)t.stride(0);
  };
  const int ld = f32row(x, "x");
  TORCH_CHECK(f32row(B, "B") == ld && f32row(C, "C") == ld, "ssd_scan: x / B / C must be views of one fp32 buffer");
  const int T = x.size(0);
  const int dtt = act_dt(dt, "dt");
  TORCH_CHECK(x.size(1) == H * DV && B.size(0) == T && B.size(1) == G * N && C.size(0) == T && C.size(1) == G * N &&
                  dt.size(0) == T && dt.size(1) == H && dt_bias.numel() == H && A_log.numel() == H && D.numel() == H &&
                  cu.numel() == S + 1 && out.numel() == (int64_t)T * H * DV && G >= 1 && H % G == 0,
              "ssd_scan: shapes");
  float* wsp = nullptr;
  if (ws) {
    TORCH_CHECK(ws->is_cuda() && ws->scalar_type() == at::kFloat && ws->is_contiguous() &&
                    ws->numel() >= ssd_scan_ws_floats(T, S, H, N, DV), "ssd_scan: workspace too small");
    wsp = ws->data_ptr<float>();
  }
  gai_ssd_scan(x.data_ptr<float>(), B.data_ptr<float>(), C.data_ptr<float>(), ld, dt.data_ptr(), row_stride(dt, "dt"),
               f32(dt_bias, "dt_bias"), f32(A_log, "A_log"), f32(D, "D"), f32w(state, "state"), i32(cu, "cu"),
               i32(slots, "slots"), S, T, f32w(out, "out"), H, (int)G, N, DV, dtt, wsp, cur_stream());
}

void wkv_scan(const Tensor& r, const Tensor& k, const Tensor& v, const Tensor& wpre, const Tensor& w0, const Tensor& u,
              Tensor& state, const Tensor& cu, const Tensor& slots, Tensor& out, const optional<Tensor>& ws) {
  const int dt = act_dt(r, "r");
  same_dt(k, dt, "k");
  same_dt(v, dt, "v");
  TORCH_CHECK(state.dim() == 4 && state.size(2) == state.size(3), "wkv_scan: state [slots, H, D, D]");
  const int H = state.size(1), D = state.size(2), S = slots.numel();
  const int ld = row_stride(r, "r");
  TORCH_CHECK(row_stride(k, "k") == ld && row_stride(v, "v") == ld && r.size(1) == H * D && k.size(1) == H * D &&
                  v.size(1) == H * D, "wkv_scan: r / k / v must be equal-stride [T, H * D] views");
  const int T = r.size(0);
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && wpre.numel() == (int64_t)T * H * D && w0.numel() == H * D &&
                  u.numel() == H * D && cu.numel() == S + 1 && out.numel() == (int64_t)T * H * D,
              "wkv_scan: decay / bonus / cu / out shapes");
  float* wsp = nullptr;  // scratch for the decays of a step with prompt portions (absent: the per-sequence kernel runs)
  if (ws) {
    TORCH_CHECK(ws->is_cuda() && ws->scalar_type() == at::kFloat && ws->is_contiguous() && ws->numel() >= wpre.numel(),
                "wkv_scan: workspace must be fp32 [T, H * D]");
    wsp = ws->data_ptr<float>();
  }
  gai_wkv_scan(r.data_ptr(), k.data_ptr(), v.data_ptr(), ld, f32(wpre, "wpre"), f32(w0, "w0"), f32(u, "u"),
               f32w(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S, T, f32w(out, "out"), H, D, dt, wsp, cur_stream());
}

void delta_prep(const Tensor& qkv, const Tensor& a, const Tensor& b, const Tensor& A_log, const Tensor& dt_bias,
                Tensor& qn, Tensor& kn, Tensor& decay, Tensor& beta, int64_t H, int64_t G, int64_t DK) {
  const int dt = act_dt(a, "a");
  same_dt(b, dt, "b");
  TORCH_CHECK(qkv.dim() == 2 && qkv.scalar_type() == at::kFloat && qkv.stride(1) == 1 && qkv.size(1) >= 2 * G * DK,
              "delta_prep: qkv fp32 [T, >= 2 G DK]");
  const int T = qkv.size(0);
  TORCH_CHECK(a.size(0) == T && a.size(1) == H * DK && b.size(0) == T && b.size(1) == H && A_log.numel() == H &&
                  dt_bias.numel() == H * DK, "delta_prep: a / b / A_log / dt_bias shapes");
  TORCH_CHECK(qn.numel() == (int64_t)T * G * DK && kn.numel() == qn.numel() && decay.numel() == (int64_t)T * H * DK &&
                  beta.numel() == (int64_t)T * H, "delta_prep: output shapes");
  gai_delta_prep(qkv.data_ptr<float>(), (int)qkv.stride(0), a.data_ptr(), row_stride(a, "a"), b.data_ptr(),
                 row_stride(b, "b"), f32(A_log, "A_log"), f32(dt_bias, "dt_bias"), f32w(qn, "qn"), f32w(kn, "kn"),
                 f32w(decay, "decay"), f32w(beta, "beta"), T, H, G, DK, dt, cur_stream());
}

void delta_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& decay, const Tensor& beta, Tensor& state,
                const Tensor& cu, const Tensor& slots, Tensor& out, int64_t G) {
  TORCH_CHECK(state.dim() == 4, "delta_scan: state [slots, H, DK, DV]");
  const int H = state.size(1), DK = state.size(2), DV = state.size(3), S = slots.numel();
  TORCH_CHECK(v.dim() == 2 && v.scalar_type() == at::kFloat && v.stride(1) == 1 && v.size(1) == H * DV,
              "delta_scan: v fp32 [T, H * DV]");
  const int T = v.size(0);
  TORCH_CHECK(q.numel() == (int64_t)T * G * DK && k.numel() == q.numel() && decay.numel() == (int64_t)T * H * DK &&
                  beta.numel() == (int64_t)T * H && cu.numel() == S + 1 && out.numel() == (int64_t)T * H * DV,
              "delta_scan: q / k / decay / beta / cu / out shapes");
  gai_delta_scan(f32(q, "q"), f32(k, "k"), v.data_ptr<float>(), (int)v.stride(0), f32(decay, "decay"), f32(beta, "beta"),
                 f32w(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S, T, f32w(out, "out"), H, G, DK, DV,
                 cur_stream());
}

void add_dyt_f32(Tensor& res, const optional<Tensor>& delta, const optional<Tensor>& extra, double alpha,
                 const optional<Tensor>& w, const optional<Tensor>& b, const optional<Tensor>& out) {
  float* r = f32w(res, "res");
  TORCH_CHECK(res.dim() == 2, "add_dyt_f32: res [T, D]");
  const int T = res.size(0), D = res.size(1);
  int dd = 0, od = 0, ldd = 0;
  if (delta) {
    dd = act_dt(*delta, "delta");
    ldd = row_stride(*delta, "delta");
    TORCH_CHECK(delta->size(0) == T && delta->size(1) == D, "add_dyt_f32: delta shape");
  }
  if (extra) TORCH_CHECK(extra->numel() == (int64_t)T * D, "add_dyt_f32: extra shape");
  if (out) {
    od = act_dt(*out, "out");
    TORCH_CHECK(out->is_contiguous() && out->numel() == (int64_t)T * D && w && b && w->numel() == D && b->numel() == D,
                "add_dyt_f32: out [T, D] needs weight and bias [D]");
  }
  TORCH_CHECK(delta || extra || out, "add_dyt_f32: nothing to do");
  gai_add_dyt_f32(r, delta ? delta->data_ptr() : nullptr, ldd, extra ? f32(*extra, "extra") : nullptr, (float)alpha,
                  out ? f32(*w, "w") : nullptr, out ? f32(*b, "b") : nullptr, out ? out->data_ptr() : nullptr, T, D, dd,
                  od, cur_stream());
}

void act_mul(const Tensor& a, const optional<Tensor>& b, int64_t act, double cap, Tensor& out) {
  const int di = act_dt(a, "a"), dout = act_dt(out, "out");
  const int lda = row_stride(a, "a");
  const int T = a.size(0), C = a.size(1);
  int ldb = 0;
  if (b) {
    same_dt(*b, di, "b");
    ldb = row_stride(*b, "b");
    TORCH_CHECK(b->size(0) == T && b->size(1) == C, "act_mul: b shape");
  }
  TORCH_CHECK(out.is_contiguous() && out.numel() == (int64_t)T * C, "act_mul: out shape");
  gai_act_mul(a.data_ptr(), lda, b ? b->data_ptr() : nullptr, ldb, out.data_ptr(), T, C, (int)act, (float)cap, di, dout,
              cur_stream());
}

void latent_kv_write(const Tensor& q, const Tensor& dkv, const Tensor& nw, const Tensor& inv_freq, double mag,
                     const Tensor& positions, const Tensor& slots, Tensor& q_cat, Tensor& k_cache, Tensor& v_cache,
                     int64_t H, int64_t DN, int64_t DR, int64_t R, double eps) {
  const int dt = act_dt(q, "q");
  same_dt(dkv, dt, "dkv");
  same_dt(q_cat, dt, "q_cat");
  same_dt(k_cache, dt, "k_cache");
  same_dt(v_cache, dt, "v_cache");
  const int ldq = row_stride(q, "q"), ldk = row_stride(dkv, "dkv");
  const int T = q.size(0);
  TORCH_CHECK(q.size(1) == H * (DN + DR) && dkv.size(0) == T && dkv.size(1) == R + DR && nw.numel() == R &&
                  2 * inv_freq.numel() <= DR && positions.numel() >= T && slots.numel() >= T &&
                  q_cat.is_contiguous() && q_cat.numel() == (int64_t)T * H * (R + DR),
              "latent_kv_write: shapes");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() && k_cache.size(1) == 1 && k_cache.size(2) == 16 &&
                  k_cache.size(3) == R + DR && v_cache.dim() == 4 && v_cache.is_contiguous() && v_cache.size(1) == 1 &&
                  v_cache.size(2) == R && v_cache.size(3) == 16 && v_cache.size(0) == k_cache.size(0),
              "latent_kv_write: cache pages K [pages, 1, 16, R + DR], V^T [pages, 1, R, 16]");
  gai_latent_kv_write(q.data_ptr(), ldq, dkv.data_ptr(), ldk, f32(nw, "norm weight"),
                      inv_freq.numel() ? f32(inv_freq, "inv_freq") : nullptr, (float)mag, i32(positions, "positions"),
                      i32(slots, "slots"), q_cat.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), T, (int)H, (int)DN,
                      (int)DR, (int)R, (float)eps, dt, cur_stream(), 2 * (int)inv_freq.numel());
}

void linear_attention_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& decay, Tensor& state,
                           const Tensor& cu, const Tensor& slots, Tensor& out, const optional<Tensor>& ws) {
  TORCH_CHECK(state.dim() == 4, "linear_attention_scan: state [slots, H, DK, DV]");
  const int H = state.size(1), N = state.size(2), DV = state.size(3), S = slots.numel();
  auto f32row = [](const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.scalar_type() == at::kFloat && t.stride(1) == 1, name, " must be fp32 rows");
    return (int)t.stride(0);
  };
  const int ld = f32row(v, "v");
  TORCH_CHECK(f32row(k, "k") == ld && f32row(q, "q") == ld, "linear_attention_scan: q / k / v must be views of one fp32 buffer");
  const int T = v.size(0);
  TORCH_CHECK(v.size(1) == H * DV && k.size(0) == T && k.size(1) == H * N && q.size(0) == T && q.size(1) == H * N &&
                  decay.numel() == H && cu.numel() == S + 1 && out.numel() == (int64_t)T * H * DV,
              "linear_attention_scan: shapes");
  float* wsp = nullptr;
  if (ws) {
    TORCH_CHECK(ws->is_cuda() && ws->scalar_type() == at::kFloat && ws->is_contiguous() &&
                    ws->numel() >= ssd_scan_ws_floats(T, S, H, N, DV), "linear_attention_scan: workspace too small");
    wsp = ws->data_ptr<float>();
  }
  gai_ssd_scan(v.data_ptr<float>(), k.data_ptr<float>(), q.data_ptr<float>(), ld, nullptr, 0, nullptr, nullptr, nullptr,
               f32w(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S, T, f32w(out, "out"), H, H, N, DV, 1, wsp,
               cur_stream(), f32(decay, "decay"));
}

void selective_scan(const Tensor& x, const Tensor& dt, const Tensor& dt_bias, const Tensor& A, const Tensor& B,
                    const Tensor& C, const Tensor& D, const Tensor& z, Tensor& state, const Tensor& cu,
                    const Tensor& slots, Tensor& out) {
  TORCH_CHECK(state.dim() == 3, "selective_scan: state [slots, I, N]");
  const int I = state.size(1), N = state.size(2), S = slots.numel(), T = x.size(0);
  auto f32row = [](const Tensor& t, const char* name) {
    TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.scalar_type() == at::kFloat && t.stride(1) == 1, name, " must be fp32 rows");
    return (int)t.stride(0);
  };
  const int ldx = f32row(x, "x"), lddt = f32row(dt, "dt");
  const int dtt = act_dt(B, "B");
  same_dt(C, dtt, "C");
  same_dt(z, dtt, "z");
  same_dt(out, dtt, "out");
  TORCH_CHECK(x.size(1) == I && dt.size(0) == T && dt.size(1) == I && dt_bias.numel() == I && A.numel() == (int64_t)I * N &&
                  B.size(0) == T && B.size(1) == N && C.size(0) == T && C.size(1) == N && D.numel() == I &&
                  z.size(0) == T && z.size(1) == I && cu.numel() == S + 1 && out.is_contiguous() &&
                  out.numel() == (int64_t)T * I,
              "selective_scan: shapes");
  gai_selective_scan(x.data_ptr<float>(), ldx, dt.data_ptr<float>(), lddt, f32(dt_bias, "dt_bias"), f32(A, "A"),
                     B.data_ptr(), row_stride(B, "B"), C.data_ptr(), row_stride(C, "C"), f32(D, "D"), z.data_ptr(),
                     row_stride(z, "z"), f32w(state, "state"), i32(cu, "cu"), i32(slots, "slots"), S, T, out.data_ptr(), I,
                     I, N, dtt, cur_stream());
}

}  // namespace

void gai_bind_seq_ops(pybind11::module_& m) {
  m.def("add_dyt_f32", &add_dyt_f32);
  m.def("act_mul", &act_mul);
  m.def("latent_kv_write", &latent_kv_write);
  m.def("linear_attention_scan", &linear_attention_scan);
  m.def("selective_scan", &selective_scan);
  m.def("add_rmsnorm_f32", &add_rmsnorm_f32);
  m.def("poly_norm", &poly_norm);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("embed_scale_f32", &embed_scale_f32);
  m.def("qknorm_kv_write", &qknorm_kv_write);
  m.def("window_attention", &window_attention);
  m.def("rotary_kv_write", &rotary_kv_write);
  m.def("decay_gate", &decay_gate);
  m.def("unit_key_removal", &unit_key_removal);
  m.def("dplr_scan", &dplr_scan);
  m.def("dplr_scan_ws_floats", &dplr_scan_ws_floats);
  m.def("sigmoid_attention_splits", [](int64_t T, int64_t S, int64_t H) { return (int64_t)gai_sigmoid_attention_splits(T, S, H); });
  m.def("token_shift_mix", &token_shift_mix);
  m.def("state_tail_write", &state_tail_write);
  m.def("conv_silu", &conv_silu);
  m.def("wkv_scan", &wkv_scan);
  m.def("delta_prep", &delta_prep);
  m.def("delta_scan", &delta_scan);
  m.def("gated_norm_add_f32", &gated_norm_add_f32);
  m.def("gate_group_norm", &gate_group_norm);
  m.def("headnorm_kv_write", &headnorm_kv_write);
  m.def("rglru_gates", &rglru_gates);
  m.def("rglru_scan", &rglru_scan);
  m.def("rglru_scan_ws_floats", &rglru_scan_ws_floats);
  m.def("ssd_scan", &ssd_scan);
  m.def("ssd_scan_ws_floats", &ssd_scan_ws_floats);
}
