// torch.ops.bfly.* registrations of csrc/kernels/delta.hip (csrc/include/bfly_delta.h).
// Shapes, strides and index tensors are validated on the host before any launch.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "bfly_delta.h"

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
constexpr int64_t kMaxRowLds = 15 * 1024;      // floats of a row staged in LDS

const float* opt_f32(const optional<Tensor>& t, int64_t n, const char* what) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->numel() == n, what);
  return t->data_ptr<float>();
}

void post_norm_add_norm(Tensor& x, const Tensor& y, const Tensor& nw, const Tensor& nb, double eps, double mult,
                        const optional<Tensor>& extra, const optional<Tensor>& nw2, const optional<Tensor>& nb2,
                        const optional<Tensor>& h) {
  CHK_GPU(x); CHK_GPU(y); CHK_F32(x); CHK_F32(nw); CHK_F32(nb);
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.is_contiguous() && y.sizes() == x.sizes(), "post_norm_add_norm: layouts");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(W >= 1 && W <= kMaxRowLds && nw.numel() == W && nb.numel() == W, "post_norm_add_norm: width / norm weights");
  const float* ep = opt_f32(extra, T * W, "post_norm_add_norm: extra f32 [T, W]");
  TORCH_CHECK(nw2.has_value() == h.has_value() && nw2.has_value() == nb2.has_value(),
              "post_norm_add_norm: the second norm needs weight, bias and an output");
  const float* w2 = opt_f32(nw2, W, "post_norm_add_norm: second norm weight [W]");
  const float* b2 = opt_f32(nb2, W, "post_norm_add_norm: second norm bias [W]");
  void* hp = nullptr;
  if (h.has_value()) {
    CHK_SAME(*h, y);
    TORCH_CHECK(h->is_cuda() && h->is_contiguous() && h->sizes() == x.sizes(), "post_norm_add_norm: h [T, W]");
    hp = h->data_ptr();
  }
  bfly::launch_post_norm_add_norm(x.data_ptr<float>(), y.data_ptr(), nw.data_ptr<float>(), nb.data_ptr<float>(),
                                  (float)eps, (float)mult, ep, w2, b2, hp, (int)T, (int)W, is_f32(y), cur_stream());
}

// shared checks of a packed step's description
void check_step(const Tensor& state_slots, const Tensor& row_cu, const Tensor& positions, int64_t T, int64_t slots,
                const char* what) {
  CHK_I32(state_slots); CHK_I32(row_cu); CHK_I32(positions);
  TORCH_CHECK(state_slots.is_cuda() && row_cu.is_cuda() && positions.is_cuda(), what, ": step tensors on the GPU");
  TORCH_CHECK(row_cu.numel() == state_slots.numel() + 1 && positions.numel() == T, what, ": row_cu / positions");
  (void)slots;      // slot numbers come from the block manager that sized the pool
}

void short_conv_act(const Tensor& z, const Tensor& w, const optional<Tensor>& state,
                    const optional<Tensor>& state_slots, const Tensor& row_cu, const Tensor& positions, int64_t act,
                    Tensor& out) {
  CHK_GPU(z); CHK_GPU(w); CHK_F32(w); CHK_I32(row_cu); CHK_I32(positions);
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && out.dim() == 2 && out.is_contiguous() && out.is_cuda() &&
                  out.sizes() == z.sizes(), "short_conv_act: z [T, C] rows, out [T, C]");
  const int64_t T = z.size(0), C = z.size(1), nseq = row_cu.numel() - 1;
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && w.size(1) >= 1, "short_conv_act: w [C, taps]");
  const int64_t taps = w.size(1);
  TORCH_CHECK(nseq >= 0 && positions.numel() == T && (act == 0 || act == 1), "short_conv_act: row_cu / positions / act");
  const float* sp = nullptr;
  const int* slp = nullptr;
  if (taps > 1 && state.has_value() && state_slots.has_value()) {
    CHK_F32(*state); CHK_I32(*state_slots);
    TORCH_CHECK(state->is_cuda() && state->dim() == 3 && state->size(1) == taps - 1 && state->size(2) == C &&
                    state_slots->numel() == nseq, "short_conv_act: state [slots, taps - 1, C] / slots [nseq]");
    sp = state->data_ptr<float>();
    slp = state_slots->data_ptr<int>();
  }
  const bool f32 = is_f32(z), of32 = is_f32(out);
  TORCH_CHECK(of32 || !f32, "short_conv_act: f32 rows give f32 output");
  bfly::launch_short_conv_act(z.data_ptr(), z.stride(0), w.data_ptr<float>(), sp, slp, row_cu.data_ptr<int>(), (int)nseq,
                              positions.data_ptr<int>(), out.data_ptr(), (int)T, (int)C, (int)taps, (int)act, f32, of32,
                              cur_stream());
}

void short_conv_state_update(const Tensor& z, Tensor& state, const Tensor& state_slots, const Tensor& row_cu,
                             const Tensor& positions) {
  CHK_GPU(z); CHK_GPU(state); CHK_F32(state);
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && state.dim() == 3 && state.size(2) == z.size(1),
              "short_conv_state_update: z [T, C], state [slots, n, C]");
  check_step(state_slots, row_cu, positions, z.size(0), state.size(0), "short_conv_state_update");
  bfly::launch_short_conv_state_update(z.data_ptr(), z.stride(0), state.data_ptr<float>(), state_slots.data_ptr<int>(),
                                       row_cu.data_ptr<int>(), (int)state_slots.numel(), positions.data_ptr<int>(),
                                       (int)z.size(1), (int)state.size(1), is_f32(z), cur_stream());
}

#define CHK_HEADS_F32(t)                                                                                     \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kFloat && (t).dim() == 3 && (t).stride(2) == 1 &&    \
                  (t).stride(1) == (t).size(2), #t " must be f32 [T, heads, size] with contiguous heads")

void delta_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& b, const Tensor& a, const Tensor& a_log,
                const Tensor& dt_bias, Tensor& state, const Tensor& state_slots, const Tensor& row_cu,
                const Tensor& positions, double q_scale, double unit_eps, Tensor& o) {
  CHK_HEADS_F32(q); CHK_HEADS_F32(k); CHK_HEADS_F32(v);
  CHK_GPU(b); CHK_GPU(a); CHK_SAME(a, b); CHK_GPU(a_log); CHK_GPU(dt_bias); CHK_GPU(state); CHK_GPU(o);
  CHK_F32(a_log); CHK_F32(dt_bias); CHK_F32(state); CHK_F32(o);
  const int64_t T = q.size(0), G = q.size(1), D = q.size(2), H = v.size(1), Dv = v.size(2);
  TORCH_CHECK(k.size(0) == T && k.size(1) == G && k.size(2) == D && v.size(0) == T && G >= 1 && H % G == 0,
              "delta_scan: q / k [T, G, D], v [T, H, Dv] with H a multiple of G");
  TORCH_CHECK(b.dim() == 2 && a.dim() == 2 && b.stride(1) == 1 && a.stride(1) == 1 && b.size(0) == T && a.size(0) == T &&
                  b.size(1) == H && a.size(1) == H && a_log.numel() == H && dt_bias.numel() == H,
              "delta_scan: b / a [T, H], a_log / dt_bias [H]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == Dv && state.size(3) == D,
              "delta_scan: state [slots, H, Dv, D]");
  check_step(state_slots, row_cu, positions, T, state.size(0), "delta_scan");
  TORCH_CHECK(o.dim() == 3 && o.size(0) == T && o.size(1) == H && o.size(2) == Dv, "delta_scan: o");
  const int rc = bfly::launch_delta_scan(q.data_ptr<float>(), q.stride(0), k.data_ptr<float>(), k.stride(0),
                                         v.data_ptr<float>(), v.stride(0), b.data_ptr(), b.stride(0), a.data_ptr(),
                                         a.stride(0), a_log.data_ptr<float>(), dt_bias.data_ptr<float>(),
                                         state.data_ptr<float>(), state_slots.data_ptr<int>(), row_cu.data_ptr<int>(),
                                         (int)state_slots.numel(), positions.data_ptr<int>(), (float)q_scale,
                                         (float)unit_eps, o.data_ptr<float>(), (int)T, (int)H, (int)G, (int)D, (int)Dv,
                                         is_f32(b), cur_stream());
  TORCH_CHECK(rc == 0, "delta_scan: key size ", D, " not supported (<= 256)");
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(bfly, m) {
  m.def("post_norm_add_norm(Tensor(a!) x, Tensor y, Tensor nw, Tensor nb, float eps, float mult, Tensor? extra, "
        "Tensor? nw2, Tensor? nb2, Tensor(b!)? h) -> ()");
  m.def("short_conv_act(Tensor z, Tensor w, Tensor? state, Tensor? state_slots, Tensor row_cu, Tensor positions, "
        "int act, Tensor(a!) out) -> ()");
  m.def("short_conv_state_update(Tensor z, Tensor(a!) state, Tensor state_slots, Tensor row_cu, Tensor positions) -> ()");
  m.def("delta_scan(Tensor q, Tensor k, Tensor v, Tensor b, Tensor a, Tensor a_log, Tensor dt_bias, Tensor(a!) state, "
        "Tensor state_slots, Tensor row_cu, Tensor positions, float q_scale, float unit_eps, Tensor(b!) o) -> ()");
}

TORCH_LIBRARY_IMPL(bfly, CUDA, m) {
  m.impl("post_norm_add_norm", &post_norm_add_norm);
  m.impl("short_conv_act", &short_conv_act);
  m.impl("short_conv_state_update", &short_conv_state_update);
  m.impl("delta_scan", &delta_scan);
}
