// torch.ops.bfly.* registrations of csrc/kernels/parlayer.hip (csrc/include/bfly_parlayer.h).
// Shapes, strides and index tensors are validated on the host before any launch.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "bfly_parlayer.h"

namespace {

using at::Tensor;
using c10::optional;

inline hipStream_t cur_stream() { return at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

inline bool is_f32(const Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, "expected a bf16 or f32 tensor");
  return t.scalar_type() == at::kFloat;
}
#define CHK_GPU(t) TORCH_CHECK((t).is_cuda(), #t " must be a GPU tensor")
#define CHK_SAME(a, b) TORCH_CHECK((a).scalar_type() == (b).scalar_type(), #a " and " #b " must have one element type")
#define CHK_F32(t) TORCH_CHECK((t).scalar_type() == at::kFloat && (t).is_contiguous(), #t " must be contiguous f32")
#define CHK_I32(t) TORCH_CHECK((t).scalar_type() == at::kInt && (t).is_contiguous(), #t " must be contiguous int32")
// [T, heads, size] view into rows: unit stride inside a head, heads packed
#define CHK_HEADS(t)                                                                                      \
  TORCH_CHECK((t).dim() == 3 && (t).stride(2) == 1 && ((t).size(1) == 1 || (t).stride(1) == (t).size(2)), \
              #t " must be a [T, heads, size] view with packed heads")

const void* opt_rows(const optional<Tensor>& y, const Tensor& like, int64_t T, int64_t W, const char* what) {
  if (!y.has_value()) return nullptr;
  TORCH_CHECK(y->is_cuda() && y->scalar_type() == like.scalar_type() && y->dim() == 2 && y->is_contiguous() &&
                  y->size(0) == T && y->size(1) == W, what, ": a sublayer output must be contiguous [T, W] of the output type");
  return y->data_ptr();
}

void par_norm_shift(const Tensor& x, const optional<Tensor>& ya, const optional<Tensor>& yb,
                    const optional<Tensor>& x_out, const Tensor& norm_a, const optional<Tensor>& norm_b, double eps,
                    double offset, const optional<Tensor>& shift, const optional<Tensor>& state,
                    const optional<Tensor>& state_slots, const Tensor& row_seq, const Tensor& row_cu,
                    const Tensor& positions, Tensor& ha, const optional<Tensor>& hb) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(norm_a); CHK_I32(row_seq); CHK_I32(row_cu); CHK_I32(positions);
  TORCH_CHECK(x.dim() == 2, "par_norm_shift: x [T, W]");
  const int64_t T = x.size(0), W = x.size(1), nseq = row_cu.numel() - 1;
  TORCH_CHECK(ha.is_cuda() && ha.dim() == 2 && ha.is_contiguous() && ha.size(0) == T && ha.size(1) == W, "par_norm_shift: ha");
  const bool f32 = is_f32(ha);
  const void* yap = opt_rows(ya, ha, T, W, "par_norm_shift");
  const void* ybp = opt_rows(yb, ha, T, W, "par_norm_shift");
  float* xo = nullptr;
  if (yap || ybp) {
    TORCH_CHECK(x_out.has_value(), "par_norm_shift: the updated residual needs a buffer");
    CHK_F32(*x_out);
    TORCH_CHECK(x_out->sizes() == x.sizes() && x_out->data_ptr() != x.data_ptr(),
                "par_norm_shift: x_out must be another [T, W] buffer than x (rows read their neighbours' old values)");
    xo = x_out->data_ptr<float>();
  }
  TORCH_CHECK(norm_a.numel() == W && nseq >= 0 && row_seq.numel() == T && positions.numel() == T, "par_norm_shift: shapes");
  const float *nb = nullptr, *sh = nullptr;
  void* hbp = nullptr;
  if (norm_b.has_value()) {
    CHK_F32(*norm_b);
    TORCH_CHECK(norm_b->numel() == W && hb.has_value(), "par_norm_shift: norm_b [W] with hb");
    CHK_SAME(*hb, ha);
    TORCH_CHECK(hb->is_contiguous() && hb->sizes() == ha.sizes(), "par_norm_shift: hb");
    nb = norm_b->data_ptr<float>();
    hbp = hb->data_ptr();
  }
  float* st = nullptr;
  const int* sl = nullptr;
  if (shift.has_value()) {
    CHK_F32(*shift);
    TORCH_CHECK(shift->numel() == W, "par_norm_shift: shift [W]");
    sh = shift->data_ptr<float>();
    TORCH_CHECK(state.has_value() && state_slots.has_value(), "par_norm_shift: a shift needs the state pool and slots");
    CHK_F32(*state); CHK_I32(*state_slots);
    TORCH_CHECK(state->dim() == 2 && state->size(1) == W && state_slots->numel() == nseq,
                "par_norm_shift: state [slots, W], one slot per sequence");
    st = state->data_ptr<float>();
    sl = state_slots->data_ptr<int>();
  }
  bfly::launch_par_norm_shift(x.data_ptr<float>(), yap, ybp, xo, norm_a.data_ptr<float>(), nb, (float)eps, (float)offset,
                              sh, st, sl, row_seq.data_ptr<int>(), row_cu.data_ptr<int>(), positions.data_ptr<int>(),
                              ha.data_ptr(), hbp, (int)T, (int)W, f32, cur_stream());
}

void par_final(const Tensor& x, const optional<Tensor>& ya, const optional<Tensor>& yb, const Tensor& norm_w, double eps,
               double offset, const optional<Tensor>& idx, Tensor& out) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(norm_w);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous() && out.is_cuda(), "par_final: layouts");
  const int64_t T = x.size(0), W = x.size(1);
  const void* yap = opt_rows(ya, out, T, W, "par_final");
  const void* ybp = opt_rows(yb, out, T, W, "par_final");
  const long* ip = nullptr;
  int64_t R = T;
  if (idx.has_value()) {
    TORCH_CHECK(idx->scalar_type() == at::kLong && idx->is_contiguous() && idx->is_cuda(), "par_final: idx must be int64");
    ip = reinterpret_cast<const long*>(idx->data_ptr<int64_t>());
    R = idx->numel();
  }
  TORCH_CHECK(out.size(0) == R && out.size(1) == W && norm_w.numel() == W, "par_final: shapes");
  bfly::launch_par_final(x.data_ptr<float>(), yap, ybp, norm_w.data_ptr<float>(), (float)eps, (float)offset, ip,
                         out.data_ptr(), (int)R, (int)W, is_f32(out), cur_stream());
}

void rope_table(const Tensor& positions, const Tensor& inv_freq, Tensor& cs) {
  CHK_GPU(positions); CHK_I32(positions); CHK_F32(inv_freq); CHK_F32(cs);
  const int64_t T = positions.numel(), n = inv_freq.numel();
  TORCH_CHECK(cs.dim() == 3 && cs.size(0) == T && cs.size(1) == 2 && cs.size(2) == n, "rope_table: cs [T, 2, n]");
  bfly::launch_rope_table(positions.data_ptr<int>(), inv_freq.data_ptr<float>(), (int)n, cs.data_ptr<float>(), (int)T,
                          cur_stream());
}

void qk_norm_rope_kv(const Tensor& q, const Tensor& k, const Tensor& v, const optional<Tensor>& qn_w,
                     const optional<Tensor>& kn_w, double eps, const optional<Tensor>& cs,
                     const Tensor& slots, Tensor& k_cache, Tensor& v_cache, const optional<Tensor>& q_out) {
  CHK_GPU(q); CHK_HEADS(q); CHK_HEADS(k); CHK_HEADS(v); CHK_SAME(k, q); CHK_SAME(v, q); CHK_SAME(k_cache, q);
  CHK_SAME(v_cache, q); CHK_I32(slots);
  const int64_t T = q.size(0), Hq = q.size(1), D = q.size(2), Gk = k.size(1), Gv = v.size(1), Dv = v.size(2);
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D && slots.numel() == T,
              "qk_norm_rope_kv: row counts / head sizes");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous(),
              "qk_norm_rope_kv: cache layouts");
  const int64_t bs = k_cache.size(2), Dp = k_cache.size(3), Dvp = v_cache.size(2);
  TORCH_CHECK(k_cache.size(1) == Gk && v_cache.size(1) == Gv && v_cache.size(3) == bs && Dp >= D && Dvp >= Dv &&
                  v_cache.size(0) == k_cache.size(0), "qk_norm_rope_kv: cache shapes K [blocks, Gk, BS, >= D], V [blocks, Gv, >= Dv, BS]");
  int64_t nrot = 0;
  const float* csp = nullptr;
  if (cs.has_value()) {
    CHK_F32(*cs);
    TORCH_CHECK(cs->dim() == 3 && cs->size(0) == T && cs->size(1) == 2, "qk_norm_rope_kv: cs [T, 2, n]");
    nrot = cs->size(2);
    csp = cs->data_ptr<float>();
  }
  void* qo = nullptr;
  if (q_out.has_value()) {
    CHK_SAME(*q_out, q);
    TORCH_CHECK(q_out->dim() == 3 && q_out->is_contiguous() && q_out->size(0) == T && q_out->size(1) == Hq &&
                    q_out->size(2) == Dp, "qk_norm_rope_kv: q_out [T, Hq, padded D]");
    qo = q_out->data_ptr();
  } else {
    TORCH_CHECK(!qn_w.has_value() && nrot == 0 && Dp == D, "qk_norm_rope_kv: queries that are normed, rotated or padded need q_out");
  }
  TORCH_CHECK(D >= 1 && Dp <= 512 && 2 * nrot <= D, "qk_norm_rope_kv: head size <= 512, rotated dims <= D");
  const float *qn = nullptr, *kn = nullptr;
  if (qn_w.has_value()) { CHK_F32(*qn_w); TORCH_CHECK(qn_w->numel() == D, "qk_norm_rope_kv: qn_w [D]"); qn = qn_w->data_ptr<float>(); }
  if (kn_w.has_value()) { CHK_F32(*kn_w); TORCH_CHECK(kn_w->numel() == D, "qk_norm_rope_kv: kn_w [D]"); kn = kn_w->data_ptr<float>(); }
  bfly::launch_qk_norm_rope_kv(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), qn, kn,
                               (float)eps, csp, (int)nrot, slots.data_ptr<int>(), qo, k_cache.data_ptr(), v_cache.data_ptr(), (int)T,
                               (int)Hq, (int)Gk, (int)Gv, (int)D, (int)Dp, (int)Dv, (int)Dvp, (int)bs, is_f32(q),
                               cur_stream());
}

void diff_combine(const Tensor& a, double lam, double eps, double out_mul, const optional<Tensor>& gate, int64_t Dv,
                  Tensor& out) {
  CHK_GPU(a); CHK_F32(a);
  TORCH_CHECK(a.dim() == 3 && a.size(1) % 2 == 0 && out.dim() == 2 && out.is_contiguous() && out.is_cuda(), "diff_combine: layouts");
  const int64_t T = a.size(0), H = a.size(1) / 2, Dvp = a.size(2);
  TORCH_CHECK(Dv >= 1 && Dv <= Dvp && Dv <= 512 && out.size(0) == T && out.size(1) == H * Dv, "diff_combine: shapes");
  const void* gp = nullptr;
  int64_t gld = 0;
  if (gate.has_value()) {
    CHK_SAME(*gate, out);
    TORCH_CHECK(gate->dim() == 2 && gate->stride(1) == 1 && gate->size(0) == T && gate->size(1) == H * Dv, "diff_combine: gate [T, H * Dv]");
    gp = gate->data_ptr();
    gld = gate->stride(0);
  }
  bfly::launch_diff_combine(a.data_ptr<float>(), (float)lam, (float)eps, (float)out_mul, gp, gld, out.data_ptr(), (int)T,
                            (int)H, (int)Dv, (int)Dvp, is_f32(out), cur_stream());
}

void glu_clamp(const Tensor& gu, double limit, double alpha, double up_offset, int64_t group, Tensor& out) {
  CHK_GPU(gu); CHK_SAME(gu, out);
  TORCH_CHECK(gu.dim() == 2 && gu.stride(1) == 1 && gu.size(1) % 2 == 0 && out.dim() == 2 && out.is_contiguous(), "glu_clamp: layouts");
  const int64_t T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(out.size(0) == T && out.size(1) == F, "glu_clamp: out [T, F]");
  TORCH_CHECK(group >= 0 && (group == 0 || F % group == 0), "glu_clamp: the interleave group must divide F");
  bfly::launch_glu_clamp(gu.data_ptr(), gu.stride(0), (float)limit, (float)alpha, (float)up_offset, out.data_ptr(), (int)T,
                         (int)F, (int)group, is_f32(gu), cur_stream());
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(bfly, m) {
  m.def("par_norm_shift(Tensor x, Tensor? ya, Tensor? yb, Tensor(a!)? x_out, Tensor norm_a, Tensor? norm_b, float eps, "
        "float offset, Tensor? shift, Tensor(b!)? state, Tensor? state_slots, Tensor row_seq, Tensor row_cu, "
        "Tensor positions, Tensor(c!) ha, Tensor(d!)? hb) -> ()");
  m.def("par_final(Tensor x, Tensor? ya, Tensor? yb, Tensor norm_w, float eps, float offset, Tensor? idx, "
        "Tensor(a!) out) -> ()");
  m.def("rope_table(Tensor positions, Tensor inv_freq, Tensor(a!) cs) -> ()");
  m.def("qk_norm_rope_kv(Tensor q, Tensor k, Tensor v, Tensor? qn_w, Tensor? kn_w, float eps, Tensor? cs, Tensor slots, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor(c!)? q_out) -> ()");
  m.def("diff_combine(Tensor a, float lam, float eps, float out_mul, Tensor? gate, int Dv, Tensor(a!) out) -> ()");
  m.def("glu_clamp(Tensor gu, float limit, float alpha, float up_offset, int group, Tensor(a!) out) -> ()");
}

TORCH_LIBRARY_IMPL(bfly, CUDA, m) {
  m.impl("par_norm_shift", &par_norm_shift);
  m.impl("par_final", &par_final);
  m.impl("rope_table", &rope_table);
  m.impl("qk_norm_rope_kv", &qk_norm_rope_kv);
  m.impl("diff_combine", &diff_combine);
  m.impl("glu_clamp", &glu_clamp);
}
