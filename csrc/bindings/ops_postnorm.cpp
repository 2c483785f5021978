// torch.ops.bfly.* registrations of csrc/kernels/postnorm.hip (csrc/include/bfly_postnorm.h).
// Shapes, strides and index tensors are validated on the host before any launch.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "bfly_postnorm.h"

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

void embed_scaled(const Tensor& ids, const Tensor& table, double scale, Tensor& out) {
  CHK_GPU(ids); CHK_GPU(table); CHK_I32(ids); CHK_F32(out);
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && out.dim() == 2, "embed_scaled: layouts");
  const int64_t T = ids.numel(), W = table.size(1);
  TORCH_CHECK(out.size(0) == T && out.size(1) == W && table.size(0) >= 1, "embed_scaled: shapes");
  bfly::launch_embed_scaled(ids.data_ptr<int>(), table.data_ptr(), (float)scale, out.data_ptr<float>(), (int)T, (int)W,
                            (int)table.size(0), is_f32(table), cur_stream());
}

void conv_mix(const Tensor& x, const optional<Tensor>& w, const optional<Tensor>& state,
              const optional<Tensor>& state_slots, const Tensor& row_cu, const Tensor& positions, Tensor& out) {
  CHK_GPU(x); CHK_F32(x); CHK_I32(row_cu); CHK_I32(positions);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous() && out.sizes() == x.sizes(), "conv_mix: layouts");
  const int64_t T = x.size(0), W = x.size(1), nseq = row_cu.numel() - 1;
  TORCH_CHECK(nseq >= 0 && positions.numel() == T, "conv_mix: row_cu / positions");
  const float *wp = nullptr, *sp = nullptr;
  const int* slp = nullptr;
  int64_t taps = 0;
  if (w.has_value()) {
    CHK_F32(*w);
    TORCH_CHECK(w->dim() == 2 && w->size(0) == W, "conv_mix: w [W, taps]");
    taps = w->size(1);
    wp = w->data_ptr<float>();
    if (taps > 1) {
      TORCH_CHECK(state.has_value() && state_slots.has_value(), "conv_mix: taps > 1 needs the history pool and slots");
      CHK_F32(*state); CHK_I32(*state_slots);
      TORCH_CHECK(state->dim() == 3 && state->size(1) == taps - 1 && state->size(2) == W && state_slots->numel() == nseq,
                  "conv_mix: state [slots, taps - 1, W], one slot per sequence");
      sp = state->data_ptr<float>();
      slp = state_slots->data_ptr<int>();
    }
  }
  bfly::launch_conv_mix(x.data_ptr<float>(), wp, sp, slp, row_cu.data_ptr<int>(), (int)nseq, positions.data_ptr<int>(),
                        out.data_ptr(), (int)T, (int)W, (int)taps, is_f32(out), cur_stream());
}

void conv_state_update(const Tensor& x, Tensor& state, const Tensor& state_slots, const Tensor& row_cu,
                       const Tensor& positions) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(state); CHK_I32(state_slots); CHK_I32(row_cu); CHK_I32(positions);
  const int64_t T = x.size(0), W = x.size(1), nseq = row_cu.numel() - 1;
  TORCH_CHECK(x.dim() == 2 && state.dim() == 3 && state.size(2) == W && state_slots.numel() == nseq &&
                  positions.numel() == T, "conv_state_update: shapes");
  bfly::launch_conv_state_update(x.data_ptr<float>(), state.data_ptr<float>(), state_slots.data_ptr<int>(),
                                 row_cu.data_ptr<int>(), (int)nseq, positions.data_ptr<int>(), (int)W,
                                 (int)state.size(1), cur_stream());
}

void post_norm_add(const Tensor& x, const Tensor& y, const Tensor& nw, const Tensor& nb, double eps,
                   const Tensor& scale, Tensor& out, const optional<Tensor>& cast) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(nw); CHK_F32(nb); CHK_F32(scale); CHK_F32(out);
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.is_contiguous() && y.sizes() == x.sizes() && out.sizes() == x.sizes(),
              "post_norm_add: layouts");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(nw.numel() == W && nb.numel() == W && scale.numel() == W && W <= kMaxRowLds, "post_norm_add: shapes");
  void* cp = nullptr;
  if (cast.has_value()) {
    CHK_SAME(*cast, y);
    TORCH_CHECK(cast->is_contiguous() && cast->sizes() == x.sizes(), "post_norm_add: cast");
    cp = cast->data_ptr();
  }
  bfly::launch_post_norm_add(x.data_ptr<float>(), y.data_ptr(), nw.data_ptr<float>(), nb.data_ptr<float>(), (float)eps,
                             scale.data_ptr<float>(), out.data_ptr<float>(), cp, (int)T, (int)W, is_f32(y), cur_stream());
}

void post_norm_add_avg(Tensor& x, const optional<Tensor>& y, const optional<Tensor>& nw, const optional<Tensor>& nb,
                       double eps, const optional<Tensor>& scale, Tensor& stack, int64_t index, const Tensor& avg) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(stack); CHK_F32(avg);
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(x.dim() == 2 && stack.dim() == 3 && stack.size(1) == T && stack.size(2) == W && index >= 0 &&
                  index < stack.size(0) && avg.numel() == index + 1 && W <= kMaxRowLds, "post_norm_add_avg: shapes");
  const void* yp = nullptr;
  const float *wp = nullptr, *bp = nullptr, *sp = nullptr;
  bool f32 = true;
  if (y.has_value()) {
    TORCH_CHECK(nw.has_value() && nb.has_value() && scale.has_value(), "post_norm_add_avg: y needs norm weights and scale");
    CHK_F32(*nw); CHK_F32(*nb); CHK_F32(*scale);
    TORCH_CHECK(y->dim() == 2 && y->is_contiguous() && y->sizes() == x.sizes() && nw->numel() == W && nb->numel() == W &&
                    scale->numel() == W, "post_norm_add_avg: y / norm shapes");
    f32 = is_f32(*y);
    yp = y->data_ptr(); wp = nw->data_ptr<float>(); bp = nb->data_ptr<float>(); sp = scale->data_ptr<float>();
  }
  bfly::launch_post_norm_add_avg(x.data_ptr<float>(), yp, wp, bp, (float)eps, sp, stack.data_ptr<float>(), T * W,
                                 (int)index, avg.data_ptr<float>(), (int)T, (int)W, f32, cur_stream());
}

void latent_prep(const Tensor& z, int64_t Q, int64_t R, int64_t rd, int64_t H, const optional<Tensor>& qn_w,
                 const Tensor& kvn_w, double eps, const Tensor& positions, const Tensor& inv_freq, const Tensor& slots,
                 Tensor& k_cache, Tensor& v_cache, const optional<Tensor>& cq, const optional<Tensor>& gate) {
  CHK_GPU(z); CHK_F32(kvn_w); CHK_I32(positions); CHK_F32(inv_freq); CHK_I32(slots);
  CHK_SAME(k_cache, z); CHK_SAME(v_cache, z);
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && Q >= 0 && R >= 1 && rd >= 0 && H >= 0 && z.size(1) >= Q + R + rd + H,
              "latent_prep: z [T, >= Q + R + rd + H]");
  const int64_t T = z.size(0);
  // Q == 0: no query latent (no weight, no output); H == 0: no gates
  TORCH_CHECK((Q > 0) == qn_w.has_value() && (Q > 0) == cq.has_value() && (H > 0) == gate.has_value(),
              "latent_prep: the query latent needs its norm weight and output, the gates their output");
  if (Q > 0) { CHK_F32(*qn_w); CHK_SAME(*cq, z); TORCH_CHECK(qn_w->numel() == Q, "latent_prep: query norm weight [Q]"); }
  if (H > 0) CHK_F32(*gate);
  TORCH_CHECK(kvn_w.numel() == R && positions.numel() == T && slots.numel() == T &&
                  2 * inv_freq.numel() <= rd, "latent_prep: norm weights / positions / slots / frequencies");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous() &&
                  k_cache.size(1) == 1 && v_cache.size(1) == 1 && k_cache.size(3) >= R + rd && v_cache.size(2) >= R &&
                  v_cache.size(3) == k_cache.size(2) && v_cache.size(0) == k_cache.size(0),
              "latent_prep: caches K [blocks, 1, BS, >= R + rd], V [blocks, 1, >= R, BS]");
  TORCH_CHECK((Q == 0 || (cq->is_contiguous() && cq->dim() == 2 && cq->size(0) == T && cq->size(1) == Q)) &&
                  (H == 0 || gate->numel() == T * H), "latent_prep: outputs");
  // slots are produced by the block manager for this cache: blocks * BS bounds them
  bfly::launch_latent_prep(z.data_ptr(), z.stride(0), (int)Q, (int)R, (int)rd, (int)H,
                           Q > 0 ? qn_w->data_ptr<float>() : nullptr,
                           kvn_w.data_ptr<float>(), (float)eps, positions.data_ptr<int>(), inv_freq.data_ptr<float>(),
                           (int)inv_freq.numel(), slots.data_ptr<int>(), k_cache.data_ptr(), v_cache.data_ptr(),
                           (int)k_cache.size(2), (int)k_cache.size(3), (int)v_cache.size(2),
                           Q > 0 ? cq->data_ptr() : nullptr, H > 0 ? gate->data_ptr<float>() : nullptr, (int)T,
                           is_f32(z), cur_stream());
}

void rope_heads_copy(const Tensor& src, Tensor& dst, const Tensor& positions, const Tensor& inv_freq) {
  CHK_GPU(src); CHK_SAME(src, dst); CHK_I32(positions); CHK_F32(inv_freq);
  TORCH_CHECK(src.dim() == 3 && dst.dim() == 3 && src.size(0) == dst.size(0) && src.size(1) == dst.size(1) &&
                  dst.size(2) >= src.size(2) && src.stride(2) == 1 && dst.stride(2) == 1,
              "rope_heads_copy: src [T, H, n], dst [T, H, >= n] views with unit inner stride");
  const int64_t T = src.size(0), H = src.size(1), n = src.size(2);
  TORCH_CHECK(positions.numel() == T && 2 * inv_freq.numel() <= n, "rope_heads_copy: positions / rotated dims");
  bfly::launch_rope_heads_copy(src.data_ptr(), src.stride(0), src.stride(1), dst.data_ptr(), dst.stride(0), dst.stride(1),
                               positions.data_ptr<int>(), inv_freq.data_ptr<float>(), (int)inv_freq.numel(), (int)T,
                               (int)H, (int)n, (int)dst.size(2), is_f32(src), cur_stream());
}

void layer_norm_rows(const Tensor& x, const Tensor& nw, const Tensor& nb, double eps, const optional<Tensor>& idx,
                     Tensor& out) {
  CHK_GPU(x); CHK_F32(x); CHK_F32(nw); CHK_F32(nb);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.is_contiguous(), "layer_norm_rows: layouts");
  const int64_t W = x.size(1);
  const long* ip = nullptr;
  int64_t R = x.size(0);
  if (idx.has_value()) {
    TORCH_CHECK(idx->scalar_type() == at::kLong && idx->is_contiguous(), "layer_norm_rows: idx int64");
    ip = idx->data_ptr<long>();
    R = idx->numel();
  }
  TORCH_CHECK(out.size(0) == R && out.size(1) == W && nw.numel() == W && nb.numel() == W && W <= kMaxRowLds,
              "layer_norm_rows: shapes");
  bfly::launch_layer_norm_rows(x.data_ptr<float>(), nw.data_ptr<float>(), nb.data_ptr<float>(), (float)eps, ip,
                               out.data_ptr(), (int)R, (int)W, is_f32(out), cur_stream());
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(bfly, m) {
  m.def("embed_scaled(Tensor ids, Tensor table, float scale, Tensor(a!) out) -> ()");
  m.def("conv_mix(Tensor x, Tensor? w, Tensor? state, Tensor? state_slots, Tensor row_cu, Tensor positions, "
        "Tensor(a!) out) -> ()");
  m.def("conv_state_update(Tensor x, Tensor(a!) state, Tensor state_slots, Tensor row_cu, Tensor positions) -> ()");
  m.def("post_norm_add(Tensor x, Tensor y, Tensor nw, Tensor nb, float eps, Tensor scale, Tensor(a!) out, "
        "Tensor(b!)? cast) -> ()");
  m.def("post_norm_add_avg(Tensor(a!) x, Tensor? y, Tensor? nw, Tensor? nb, float eps, Tensor? scale, Tensor(b!) stack, "
        "int index, Tensor avg) -> ()");
  m.def("latent_prep(Tensor z, int q_rank, int kv_rank, int rot_dim, int heads, Tensor? qn_w, Tensor kvn_w, float eps, "
        "Tensor positions, Tensor inv_freq, Tensor slots, Tensor(a!) k_cache, Tensor(b!) v_cache, Tensor(c!)? cq, "
        "Tensor(d!)? gate) -> ()");
  m.def("rope_heads_copy(Tensor src, Tensor(a!) dst, Tensor positions, Tensor inv_freq) -> ()");
  m.def("layer_norm_rows(Tensor x, Tensor nw, Tensor nb, float eps, Tensor? idx, Tensor(a!) out) -> ()");
}

TORCH_LIBRARY_IMPL(bfly, CUDA, m) {
  m.impl("embed_scaled", &embed_scaled);
  m.impl("conv_mix", &conv_mix);
  m.impl("conv_state_update", &conv_state_update);
  m.impl("post_norm_add", &post_norm_add);
  m.impl("post_norm_add_avg", &post_norm_add_avg);
  m.impl("latent_prep", &latent_prep);
  m.impl("rope_heads_copy", &rope_heads_copy);
  m.impl("layer_norm_rows", &layer_norm_rows);
}
