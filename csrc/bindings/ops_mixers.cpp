// torch.ops.bfly.* registrations of the shape-generic kernels (csrc/include/bfly_mixers.h):
// generic GEMM, residual streams, partial rotary + paged append, windowed paged attention,
// gated linear attention, score-routed MoE. Activations and weights are bf16 or f32 (one type per
// call); shapes, strides and index tensors are validated on the host before any launch.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include "bfly_kernels.h"
#include "bfly_mixers.h"

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
// [T, heads, dim] view of a (possibly wider) row: heads packed, rows strided
#define CHK_HEADS(t) \
  TORCH_CHECK((t).dim() == 3 && (t).stride(2) == 1 && (t).stride(1) == (t).size(2), #t " must be [T, heads, dim] rows")

void gemm_any(const Tensor& x, const Tensor& w, const optional<Tensor>& bias, int64_t act, double a0, double a1,
              Tensor& out) {
  CHK_GPU(x); CHK_GPU(w); CHK_GPU(out); CHK_SAME(x, w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && out.dim() == 2, "gemm_any: 2-D operands");
  TORCH_CHECK(x.stride(1) == 1 && w.stride(1) == 1 && out.stride(1) == 1, "gemm_any: unit inner strides");
  const int64_t M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(w.size(1) == K && out.size(0) == M && out.size(1) == N, "gemm_any: shapes");
  TORCH_CHECK(act >= 0 && act <= 2, "gemm_any: act");
  const bool f32 = is_f32(x);
  const bool of32 = out.scalar_type() == at::kFloat;
  TORCH_CHECK(of32 || out.scalar_type() == x.scalar_type(), "gemm_any: out type");
  const void* b = nullptr;
  if (bias.has_value()) {
    CHK_SAME(*bias, x);
    TORCH_CHECK(bias->numel() == N && bias->is_contiguous(), "gemm_any: bias");
    b = bias->data_ptr();
  }
  bfly::launch_gemm_any(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), b, out.data_ptr(), out.stride(0), (int)M,
                        (int)N, (int)K, (int)act, (float)a0, (float)a1, f32, of32 && !f32, cur_stream());
}

// out[t, h] = w[h] x[t, h]: x [T, H, K], out [T, H, N] (views into wider rows), w [H, N, K]
void linear_heads(const Tensor& x, const Tensor& w, Tensor& out) {
  CHK_GPU(x); CHK_GPU(w); CHK_GPU(out); CHK_SAME(x, w); CHK_SAME(x, out);
  TORCH_CHECK(x.dim() == 3 && w.dim() == 3 && out.dim() == 3 && w.is_contiguous() && x.stride(2) == 1 &&
                  out.stride(2) == 1, "linear_heads: x [T, H, K], w [H, N, K], out [T, H, N]");
  const int64_t T = x.size(0), H = x.size(1), K = x.size(2), N = w.size(1);
  TORCH_CHECK(w.size(0) == H && w.size(2) == K && out.size(0) == T && out.size(1) == H && out.size(2) == N &&
                  H <= 65535, "linear_heads: shapes");
  bfly::launch_gemm_any(x.data_ptr(), x.stride(0), w.data_ptr(), K, nullptr, out.data_ptr(), out.stride(0), (int)T,
                        (int)N, (int)K, 0, 0.f, 0.f, is_f32(x), false, cur_stream(), (int)H, x.stride(1), N * K,
                        out.stride(1));
}

void act_(Tensor& x, int64_t act, double a0, double a1) {
  CHK_GPU(x);
  TORCH_CHECK(x.is_contiguous() && act >= 0 && act <= 2, "act_: contiguous, act 0..2");
  bfly::launch_act(x.data_ptr(), x.numel(), (int)act, (float)a0, (float)a1, is_f32(x), cur_stream());
}

void embed_norm_streams(const Tensor& ids, const Tensor& table, const Tensor& norm_w, double eps, double offset,
                        Tensor& xs) {
  CHK_GPU(ids); CHK_GPU(table); CHK_I32(ids); CHK_F32(norm_w); CHK_F32(xs);
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && xs.dim() == 3, "embed_norm_streams: layouts");
  const int64_t T = ids.numel(), S = xs.size(1), W = table.size(1);
  TORCH_CHECK(xs.size(0) == T && xs.size(2) == W && norm_w.numel() == W, "embed_norm_streams: shapes");
  bfly::launch_embed_norm_streams(ids.data_ptr<int>(), table.data_ptr(), norm_w.data_ptr<float>(), (float)eps,
                                  (float)offset, xs.data_ptr<float>(), (int)T, (int)S, (int)W, (int)table.size(0),
                                  is_f32(table), cur_stream());
}

void hc_pre(const Tensor& xs, const Tensor& w_in, const Tensor& norm_w, double eps, double offset, Tensor& out) {
  CHK_GPU(xs); CHK_F32(xs); CHK_F32(w_in); CHK_F32(norm_w);
  TORCH_CHECK(xs.dim() == 3 && out.dim() == 2 && out.is_contiguous(), "hc_pre: layouts");
  const int64_t T = xs.size(0), S = xs.size(1), W = xs.size(2);
  TORCH_CHECK(w_in.numel() == S && norm_w.numel() == W && out.size(0) == T && out.size(1) == W, "hc_pre: shapes");
  bfly::launch_hc_pre(xs.data_ptr<float>(), w_in.data_ptr<float>(), norm_w.data_ptr<float>(), (float)eps, (float)offset,
                      out.data_ptr(), (int)T, (int)S, (int)W, is_f32(out), cur_stream());
}

void hc_post(Tensor& xs, const Tensor& y, const Tensor& mix, const Tensor& w_out) {
  CHK_GPU(xs); CHK_F32(xs); CHK_F32(mix); CHK_F32(w_out);
  TORCH_CHECK(xs.dim() == 3 && y.dim() == 2 && y.is_contiguous(), "hc_post: layouts");
  const int64_t T = xs.size(0), S = xs.size(1), W = xs.size(2);
  TORCH_CHECK(S <= 16, "hc_post: at most 16 residual streams");
  TORCH_CHECK(mix.numel() == S * S && w_out.numel() == S && y.size(0) == T && y.size(1) == W, "hc_post: shapes");
  bfly::launch_hc_post(xs.data_ptr<float>(), y.data_ptr(), mix.data_ptr<float>(), w_out.data_ptr<float>(), (int)T,
                       (int)S, (int)W, is_f32(y), cur_stream());
}

void hc_post_pre(Tensor& xs, const Tensor& y, const Tensor& mix, const Tensor& w_out, const Tensor& w_in2,
                 const Tensor& norm_w2, double eps, double offset, Tensor& out) {
  CHK_GPU(xs); CHK_F32(xs); CHK_F32(mix); CHK_F32(w_out); CHK_F32(w_in2); CHK_F32(norm_w2); CHK_SAME(y, out);
  TORCH_CHECK(xs.dim() == 3 && y.dim() == 2 && y.is_contiguous() && out.dim() == 2 && out.is_contiguous(),
              "hc_post_pre: layouts");
  const int64_t T = xs.size(0), S = xs.size(1), W = xs.size(2);
  TORCH_CHECK(S <= 16, "hc_post_pre: at most 16 residual streams");
  TORCH_CHECK(mix.numel() == S * S && w_out.numel() == S && w_in2.numel() == S && norm_w2.numel() == W &&
                  y.size(0) == T && y.size(1) == W && out.size(0) == T && out.size(1) == W, "hc_post_pre: shapes");
  bfly::launch_hc_post_pre(xs.data_ptr<float>(), y.data_ptr(), mix.data_ptr<float>(), w_out.data_ptr<float>(),
                           w_in2.data_ptr<float>(), norm_w2.data_ptr<float>(), (float)eps, (float)offset, out.data_ptr(),
                           (int)T, (int)S, (int)W, is_f32(y), cur_stream());
}

void hc_final(const Tensor& xs, const Tensor& norm_w, double eps, double offset, const optional<Tensor>& idx,
              Tensor& out) {
  CHK_GPU(xs); CHK_F32(xs); CHK_F32(norm_w);
  TORCH_CHECK(xs.dim() == 3 && out.dim() == 2 && out.is_contiguous(), "hc_final: layouts");
  const int64_t S = xs.size(1), W = xs.size(2);
  const long* ip = nullptr;
  int64_t R = xs.size(0);
  if (idx.has_value()) {
    TORCH_CHECK(idx->scalar_type() == at::kLong && idx->is_contiguous(), "hc_final: idx int64");
    ip = idx->data_ptr<long>();
    R = idx->numel();
  }
  TORCH_CHECK(out.size(0) == R && out.size(1) == W && norm_w.numel() == W, "hc_final: shapes");
  bfly::launch_hc_final(xs.data_ptr<float>(), norm_w.data_ptr<float>(), (float)eps, (float)offset, ip, out.data_ptr(),
                        (int)R, (int)S, (int)W, is_f32(out), cur_stream());
}

void rope_partial_kv(Tensor& q, const optional<Tensor>& k, const optional<Tensor>& v, const Tensor& positions,
                     const Tensor& inv_freq, const optional<Tensor>& slots, const optional<Tensor>& k_cache,
                     const optional<Tensor>& v_cache) {
  CHK_GPU(q); CHK_HEADS(q); CHK_I32(positions); CHK_F32(inv_freq);
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  const int64_t nrot = inv_freq.numel();
  TORCH_CHECK(positions.numel() == T && 2 * nrot <= D, "rope_partial_kv: positions / rotated dims");
  void *kp = nullptr, *kc = nullptr, *vc = nullptr;
  const void* vp = nullptr;
  const int* sp = nullptr;
  int64_t G = 1, Dv = 1, bs = 1, kld = 0, vld = 0;
  if (k.has_value()) {
    TORCH_CHECK(v.has_value() && slots.has_value() && k_cache.has_value() && v_cache.has_value(),
                "rope_partial_kv: k needs v, slots and both caches");
    const Tensor &K = *k, &V = *v, &KC = *k_cache, &VC = *v_cache;
    CHK_HEADS(K); CHK_HEADS(V); CHK_SAME(K, q); CHK_SAME(V, q); CHK_SAME(KC, q); CHK_SAME(VC, q); CHK_I32(*slots);
    G = K.size(1); Dv = V.size(2);
    TORCH_CHECK(K.size(0) == T && V.size(0) == T && K.size(2) == D && V.size(1) == G && slots->numel() == T,
                "rope_partial_kv: k / v shapes");
    TORCH_CHECK(KC.dim() == 4 && VC.dim() == 4 && KC.is_contiguous() && VC.is_contiguous() && KC.size(1) == G &&
                    KC.size(3) == D && VC.size(0) == KC.size(0) && VC.size(1) == G && VC.size(3) == KC.size(2) &&
                    VC.size(2) == Dv,
                "rope_partial_kv: caches must be K [blocks, G, BS, D], V [blocks, G, Dv, BS]");
    bs = KC.size(2);
    // slots are produced by the block manager for this cache: blocks * BS bounds them
    kp = K.data_ptr(); vp = V.data_ptr(); kc = KC.data_ptr(); vc = VC.data_ptr(); sp = slots->data_ptr<int>();
    kld = K.stride(0); vld = V.stride(0);
  }
  bfly::launch_rope_partial_kv(q.data_ptr(), q.stride(0), kp, kld, vp, vld, positions.data_ptr<int>(),
                               inv_freq.data_ptr<float>(), (int)nrot, sp, kc, vc, (int)T, (int)H, (int)G, (int)D,
                               (int)Dv, (int)bs, is_f32(q), cur_stream());
}

void row_seq(const Tensor& row_cu, Tensor& out) {
  CHK_GPU(row_cu); CHK_I32(row_cu); CHK_I32(out);
  TORCH_CHECK(row_cu.numel() >= 1, "row_seq: row_cu");
  bfly::launch_row_seq(row_cu.data_ptr<int>(), (int)row_cu.numel() - 1, out.data_ptr<int>(), (int)out.numel(),
                       cur_stream());
}

void attn_window_paged(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& tables,
                       const Tensor& row_seq_t, const Tensor& row_cu, const Tensor& positions, double scale,
                       int64_t window, int64_t keep_first, const optional<Tensor>& sink,
                       const optional<Tensor>& out_scale, bool fold_heads, const optional<Tensor>& part, Tensor& out,
                       int64_t chunk, double softcap, const optional<Tensor>& dist_a, const optional<Tensor>& dist_b,
                       double qt_coef, int64_t qt_every, int64_t maps) {
  CHK_GPU(q); CHK_HEADS(q); CHK_SAME(k_cache, q); CHK_SAME(v_cache, q);
  bfly::AttnMod md;
  md.out_f32 = out.scalar_type() == at::kFloat && !is_f32(q);
  TORCH_CHECK(md.out_f32 || out.scalar_type() == q.scalar_type(), "attn_window_paged: out must be f32 or of q's type");
  TORCH_CHECK(chunk >= 0 && softcap >= 0 && qt_every >= 1 && maps >= 1, "attn_window_paged: modifiers");
  md.chunk = (int)chunk;
  md.softcap = (float)softcap;
  md.qt_coef = (float)qt_coef;
  md.qt_every = (int)qt_every;
  md.maps = (int)maps;
  CHK_I32(tables); CHK_I32(row_seq_t); CHK_I32(positions);
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous(),
              "attn_window_paged: caches");
  const int64_t G = v_cache.size(1), bs = k_cache.size(2), Dv = v_cache.size(2);
  TORCH_CHECK(k_cache.size(3) == D && k_cache.size(1) == G * maps && v_cache.size(3) == bs &&
                  v_cache.size(0) == k_cache.size(0),
              "attn_window_paged: cache shapes K [blocks, G * maps, BS, D], V [blocks, G, Dv, BS]");
  CHK_I32(row_cu);
  TORCH_CHECK(row_cu.numel() == tables.size(0) + 1, "attn_window_paged: row_cu");
  TORCH_CHECK(G > 0 && H % (G * maps) == 0 && Dv <= 512 && D <= 4096, "attn_window_paged: head counts / sizes");
  TORCH_CHECK(dist_a.has_value() || !dist_b.has_value(), "attn_window_paged: dist_b needs dist_a");
  if (dist_a.has_value()) {      // (a, b): logarithmic, a alone: linear
    CHK_F32(*dist_a);
    TORCH_CHECK(dist_a->is_cuda() && dist_a->numel() == H, "attn_window_paged: distance bias [H]");
    md.dist_a = dist_a->data_ptr<float>();
    if (dist_b.has_value()) {
      CHK_F32(*dist_b);
      TORCH_CHECK(dist_b->is_cuda() && dist_b->numel() == H, "attn_window_paged: distance bias [H]");
      md.dist_b = dist_b->data_ptr<float>();
    }
  }
  TORCH_CHECK(tables.dim() == 2 && row_seq_t.numel() == T && positions.numel() == T, "attn_window_paged: index shapes");
  const float *sinkp = nullptr, *gatep = nullptr;
  if (sink.has_value()) {
    CHK_F32(*sink);
    TORCH_CHECK(sink->numel() == H, "attn_window_paged: sink [H]");
    sinkp = sink->data_ptr<float>();
  }
  if (out_scale.has_value()) {
    CHK_F32(*out_scale);
    TORCH_CHECK(out_scale->numel() == T * H, "attn_window_paged: out_scale [T, H]");
    gatep = out_scale->data_ptr<float>();
  }
  TORCH_CHECK(!fold_heads || G == 1, "attn_window_paged: fold_heads needs one shared key / value head");
  float* partp = nullptr;
  int64_t part_n = 0;
  if (part.has_value()) {
    CHK_F32(*part);
    partp = part->data_ptr<float>();
    part_n = part->numel();
  }
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3 && out.size(0) == T && out.size(1) == H && out.size(2) == Dv,
              "attn_window_paged: out");
  TORCH_CHECK(window >= 1 && keep_first >= 0, "attn_window_paged: window >= 1, keep_first >= 0");
  if (!is_f32(q) && bfly::launch_attn_window_mfma(q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                                  tables.data_ptr<int>(), (int)tables.size(1), row_cu.data_ptr<int>(),
                                                  (int)tables.size(0), positions.data_ptr<int>(), (float)scale,
                                                  (int)window, (int)keep_first, sinkp, gatep, out.data_ptr(),
                                                  (int)T, (int)H, (int)G, (int)D, (int)Dv, (int)bs, fold_heads, partp,
                                                  (long)part_n, cur_stream(), md))
    return;
  bfly::launch_attn_window_paged(q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                 tables.data_ptr<int>(), (int)tables.size(1), row_seq_t.data_ptr<int>(),
                                 (int)tables.size(0), positions.data_ptr<int>(), (float)scale, (int)window,
                                 (int)keep_first, sinkp, gatep, out.data_ptr(), (int)T, (int)H, (int)G, (int)D,
                                 (int)Dv, (int)bs, is_f32(q), cur_stream(), md);
}

void gla_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& z, Tensor& state,
              const Tensor& state_slots, const Tensor& row_cu, const Tensor& positions, double tau, double q_scale,
              Tensor& o) {
  CHK_GPU(q); CHK_HEADS(q); CHK_HEADS(k); CHK_HEADS(v); CHK_SAME(k, q); CHK_SAME(v, q); CHK_SAME(z, q);
  CHK_F32(state); CHK_F32(o); CHK_I32(state_slots); CHK_I32(row_cu); CHK_I32(positions);
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2), Dv = v.size(2);
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D && v.size(0) == T && v.size(1) == H, "gla_scan: q/k/v");
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && z.size(0) == T && z.size(1) == H * D, "gla_scan: z [T, H * D]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == Dv, "gla_scan: state");
  const int64_t nseq = state_slots.numel();
  TORCH_CHECK(row_cu.numel() == nseq + 1 && positions.numel() == T, "gla_scan: row_cu / positions");
  TORCH_CHECK(o.dim() == 3 && o.size(0) == T && o.size(1) == H && o.size(2) == Dv, "gla_scan: o");
  TORCH_CHECK(tau > 0, "gla_scan: tau");
  const int rc = bfly::launch_gla_scan(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                                       z.data_ptr(), z.stride(0), state.data_ptr<float>(), state_slots.data_ptr<int>(),
                                       row_cu.data_ptr<int>(), (int)nseq, positions.data_ptr<int>(), (float)tau,
                                       (float)q_scale, o.data_ptr<float>(), (int)T, (int)H, (int)D, (int)Dv, is_f32(q),
                                       cur_stream());
  TORCH_CHECK(rc == 0, "gla_scan: key size ", D, " not supported (<= 256)");
}

void gla_out(const Tensor& o, const Tensor& g, const Tensor& norm_w, double eps, Tensor& out) {
  CHK_GPU(o); CHK_F32(o); CHK_F32(norm_w); CHK_SAME(g, out);
  TORCH_CHECK(o.dim() == 3 && g.dim() == 2 && g.stride(1) == 1 && out.is_contiguous(), "gla_out: layouts");
  const int64_t T = o.size(0), H = o.size(1), Dv = o.size(2);
  TORCH_CHECK(g.size(0) == T && g.size(1) == H * Dv && out.numel() == T * H * Dv && norm_w.numel() == Dv, "gla_out: shapes");
  bfly::launch_gla_out(o.data_ptr<float>(), g.data_ptr(), g.stride(0), norm_w.data_ptr<float>(), (float)eps,
                       out.data_ptr(), (int)T, (int)H, (int)Dv, is_f32(out), cur_stream());
}

void router_logits(const Tensor& x, const Tensor& wr, Tensor& logits) {
  CHK_GPU(x); CHK_SAME(x, wr); CHK_F32(logits);
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && wr.dim() == 2 && wr.is_contiguous(), "router_logits: layouts");
  const int64_t T = x.size(0), Hd = x.size(1), E = wr.size(0);
  TORCH_CHECK(wr.size(1) == Hd && logits.dim() == 2 && logits.size(0) == T && logits.size(1) == E, "router_logits: shapes");
  bfly::launch_router_logits(x.data_ptr(), x.stride(0), wr.data_ptr(), logits.data_ptr<float>(), (int)T, (int)E, (int)Hd,
                             is_f32(x), cur_stream());
}

void moe_topk_scores(const Tensor& logits, const optional<Tensor>& bias, int64_t top_k, int64_t scoring, bool renorm,
                     Tensor& ids, Tensor& w, const optional<Tensor>& select_bias) {
  CHK_GPU(logits); CHK_F32(logits); CHK_I32(ids); CHK_F32(w);
  const float* bp = nullptr;
  if (bias.has_value()) {
    CHK_F32(*bias);
    TORCH_CHECK(bias->numel() == logits.size(1), "moe_topk_scores: bias [E]");
    bp = bias->data_ptr<float>();
  }
  const float* sbp = nullptr;
  if (select_bias.has_value()) {
    CHK_F32(*select_bias);
    TORCH_CHECK(select_bias->is_cuda() && select_bias->numel() == logits.size(1), "moe_topk_scores: select_bias [E]");
    sbp = select_bias->data_ptr<float>();
  }
  TORCH_CHECK(logits.dim() == 2, "moe_topk_scores: logits [T, E]");
  const int64_t T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(E >= 1 && E <= 1024 && top_k >= 1 && top_k <= E, "moe_topk_scores: experts / top_k");
  TORCH_CHECK(ids.numel() == T * top_k && w.numel() == T * top_k, "moe_topk_scores: outputs");
  bfly::launch_moe_topk_scores(logits.data_ptr<float>(), bp, (int)top_k, (int)scoring, renorm, ids.data_ptr<int>(),
                               w.data_ptr<float>(), (int)T, (int)E, cur_stream(), sbp);
}

int64_t moe_sort_max_tiles(int64_t TK, int64_t E) { return bfly::moe_sort_max_tiles((int)TK, (int)E); }

// work: int32 [TK + (E + 1) + 2 * max_tiles + 1] = perm | offsets | tiles | ntiles
void moe_glu_ffn(const Tensor& x, const Tensor& topk_ids, const Tensor& topk_w, const Tensor& gate_up_w,
                 const Tensor& down_w, double limit, double alpha, double up_offset, bool scale_input, Tensor& work,
                 Tensor& hmid, Tensor& y, Tensor& out, int64_t plain_act) {
  CHK_GPU(x); CHK_SAME(x, gate_up_w); CHK_SAME(x, down_w); CHK_SAME(x, hmid); CHK_SAME(x, out);
  CHK_I32(topk_ids); CHK_F32(topk_w); CHK_I32(work); CHK_F32(y);
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && gate_up_w.dim() == 3 && down_w.dim() == 3 &&
                  gate_up_w.is_contiguous() && down_w.is_contiguous(), "moe_glu_ffn: layouts");
  const int64_t T = x.size(0), Hd = x.size(1), E = gate_up_w.size(0), F = down_w.size(2);
  TORCH_CHECK(topk_ids.dim() == 2 && topk_ids.size(0) == T && topk_w.numel() == topk_ids.numel(), "moe_glu_ffn: routing");
  const int64_t K = topk_ids.size(1), TK = T * K;
  TORCH_CHECK(plain_act == bfly::ACT_NONE || plain_act == bfly::ACT_RELU2, "moe_glu_ffn: plain experts take relu2");
  TORCH_CHECK(E <= 1024 && gate_up_w.size(1) == (plain_act ? F : 2 * F) && gate_up_w.size(2) == Hd &&
                  down_w.size(0) == E && down_w.size(1) == Hd,
              "moe_glu_ffn: weights [E, 2F, H] (plain experts: [E, F, H]) / [E, H, F]");
  const int64_t mt = bfly::moe_sort_max_tiles((int)TK, (int)E);
  TORCH_CHECK(work.numel() >= TK + E + 1 + 2 * mt + 1, "moe_glu_ffn: work buffer");
  TORCH_CHECK(hmid.is_contiguous() && hmid.numel() >= TK * F && y.numel() >= TK * Hd && out.is_contiguous() &&
                  out.size(0) == T && out.size(1) == Hd, "moe_glu_ffn: buffers");
  if (TK == 0) return;
  int* perm = work.data_ptr<int>();
  int* offsets = perm + TK;
  int* tiles = offsets + E + 1;
  int* ntiles = tiles + 2 * mt;
  hipStream_t s = cur_stream();
  const bool f32 = is_f32(x);
  const int tr = bfly::moe_tile_rows((int)TK, (int)E, f32);
  bfly::launch_moe_sort(topk_ids.data_ptr<int>(), (int)TK, (int)E, perm, offsets, tiles, ntiles, tr, s);
  // scores on the expert's input (the row is scaled and the outputs are summed) or on its output
  bfly::launch_moe_glu_up(x.data_ptr(), x.stride(0), scale_input ? topk_w.data_ptr<float>() : nullptr, (int)K, perm,
                          offsets, tiles, ntiles, (int)mt, gate_up_w.data_ptr(), (float)limit, (float)alpha,
                          (float)up_offset, hmid.data_ptr(), (int)Hd, (int)F, f32, tr, s, (int)plain_act);
  bfly::launch_moe_down(hmid.data_ptr(), perm, offsets, tiles, ntiles, (int)mt, down_w.data_ptr(), y.data_ptr<float>(),
                        (int)Hd, (int)F, f32, tr, s);
  bfly::launch_moe_sum(y.data_ptr<float>(), scale_input ? nullptr : topk_w.data_ptr<float>(), (int)K, out.data_ptr(),
                       (int)T, (int)Hd, f32, s);
}

void sample_greedy_f32(const Tensor& logits, int64_t vstart, Tensor& out_ids, Tensor& out_scores, bool check_finite) {
  CHK_GPU(logits); CHK_I32(out_ids); CHK_F32(out_scores);
  TORCH_CHECK(logits.scalar_type() == at::kFloat && logits.dim() == 2 && logits.stride(1) == 1, "sample_greedy_f32: logits");
  const int64_t rows = logits.size(0);
  TORCH_CHECK(out_ids.numel() == rows && out_scores.numel() == rows && logits.size(1) >= 1, "sample_greedy_f32: outputs");
  bfly::launch_sample_greedy_f32(logits.data_ptr<float>(), logits.stride(0), (int)rows, (int)logits.size(1), (int)vstart,
                                 out_ids.data_ptr<int>(), out_scores.data_ptr<float>(), cur_stream(), check_finite ? 1 : 0);
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(bfly, m) {
  m.def("sample_greedy_f32(Tensor logits, int vstart, Tensor(a!) out_ids, Tensor(b!) out_scores, bool check_finite) -> ()");
  m.def("gemm_any(Tensor x, Tensor w, Tensor? bias, int act, float a0, float a1, Tensor(a!) out) -> ()");
  m.def("linear_heads(Tensor x, Tensor w, Tensor(a!) out) -> ()");
  m.def("act_(Tensor(a!) x, int act, float a0, float a1) -> ()");
  m.def("embed_norm_streams(Tensor ids, Tensor table, Tensor norm_w, float eps, float offset, Tensor(a!) xs) -> ()");
  m.def("hc_pre(Tensor xs, Tensor w_in, Tensor norm_w, float eps, float offset, Tensor(a!) out) -> ()");
  m.def("hc_post(Tensor(a!) xs, Tensor y, Tensor mix, Tensor w_out) -> ()");
  m.def("hc_post_pre(Tensor(a!) xs, Tensor y, Tensor mix, Tensor w_out, Tensor w_in2, Tensor norm_w2, float eps, "
        "float offset, Tensor(b!) out) -> ()");
  m.def("hc_final(Tensor xs, Tensor norm_w, float eps, float offset, Tensor? idx, Tensor(a!) out) -> ()");
  m.def("rope_partial_kv(Tensor(a!) q, Tensor(b!)? k, Tensor? v, Tensor positions, Tensor inv_freq, Tensor? slots, "
        "Tensor(c!)? k_cache, Tensor(d!)? v_cache) -> ()");
  m.def("row_seq(Tensor row_cu, Tensor(a!) out) -> ()");
  m.def("attn_window_paged(Tensor q, Tensor k_cache, Tensor v_cache, Tensor tables, Tensor row_seq, Tensor row_cu, "
        "Tensor positions, float scale, int window, int keep_first, Tensor? sink, Tensor? out_scale, bool fold_heads, "
        "Tensor(b!)? part, Tensor(a!) out, int chunk=0, float softcap=0., Tensor? dist_a=None, Tensor? dist_b=None, "
        "float qt_coef=0., int qt_every=1, int maps=1) -> ()");
  m.def("gla_scan(Tensor q, Tensor k, Tensor v, Tensor z, Tensor(a!) state, Tensor state_slots, Tensor row_cu, "
        "Tensor positions, float tau, float q_scale, Tensor(b!) o) -> ()");
  m.def("gla_out(Tensor o, Tensor g, Tensor norm_w, float eps, Tensor(a!) out) -> ()");
  m.def("router_logits(Tensor x, Tensor wr, Tensor(a!) logits) -> ()");
  m.def("moe_topk_scores(Tensor logits, Tensor? bias, int top_k, int scoring, bool renorm, Tensor(a!) ids, "
        "Tensor(b!) w, Tensor? select_bias=None) -> ()");
  m.def("moe_sort_max_tiles(int tk, int experts) -> int", &moe_sort_max_tiles);
  m.def("moe_glu_ffn(Tensor x, Tensor topk_ids, Tensor topk_w, Tensor gate_up_w, Tensor down_w, float limit, "
        "float alpha, float up_offset, bool scale_input, Tensor(a!) work, Tensor(b!) hmid, Tensor(c!) y, "
        "Tensor(d!) out, int plain_act=0) -> ()");
}

TORCH_LIBRARY_IMPL(bfly, CUDA, m) {
  m.impl("sample_greedy_f32", &sample_greedy_f32);
  m.impl("gemm_any", &gemm_any);
  m.impl("linear_heads", &linear_heads);
  m.impl("act_", &act_);
  m.impl("embed_norm_streams", &embed_norm_streams);
  m.impl("hc_pre", &hc_pre);
  m.impl("hc_post", &hc_post);
  m.impl("hc_post_pre", &hc_post_pre);
  m.impl("hc_final", &hc_final);
  m.impl("rope_partial_kv", &rope_partial_kv);
  m.impl("row_seq", &row_seq);
  m.impl("attn_window_paged", &attn_window_paged);
  m.impl("gla_scan", &gla_scan);
  m.impl("gla_out", &gla_out);
  m.impl("router_logits", &router_logits);
  m.impl("moe_topk_scores", &moe_topk_scores);
  m.impl("moe_glu_ffn", &moe_glu_ffn);
}
