// Host-side launch API of the shape-generic kernels: GEMM for any (M, N, K) in bf16 or f32,
// parallel residual streams (hyper-connections) with offset-weight RMS norms, partial
// interleaved rotary + paged append, windowed paged attention with kept first tokens and a sink
// logit, gated linear attention with pooled per-sequence state, score-routed MoE with clamped
// GLU experts. Every launcher is stream-ordered, allocation-free and synchronisation-free.
// `f32`: the activation / weight element type is float (else bf16); accumulation, norms,
// softmax, rotary angles, recurrent state and router scores are f32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bfly {

enum AnyAct { ACT_NONE = 0, ACT_RELU2 = 1, ACT_XIELU = 2 };

// out[M, N] = act(x[M, K] w[N, K]^T + bias[N]); `out_f32`: out is float whatever the inputs. act:
// squared ReLU, or xIELU with coefficients (a0, a1): v > 0: a0 v^2 + v / 2, else a1 (exp(v) - 1 - v) + v / 2.
// batch > 1: `batch` independent problems (one per head, say) whose x / w / out start bx / bw / bo
// elements apart, in one launch.
void launch_gemm_any(const void* x, long ldx, const void* w, long ldw, const void* bias, void* out, long ldo,
                     int M, int N, int K, int act, float a0, float a1, bool f32, bool out_f32, hipStream_t s,
                     int batch = 1, long bx = 0, long bw = 0, long bo = 0);
// x <- act(x) elementwise (n elements)
void launch_act(void* x, long n, int act, float a0, float a1, bool f32, hipStream_t s);

// xs[t, s, :] = rms(table[ids[t]]) * (w + offset) for every stream s; xs f32 [T, S, W]
void launch_embed_norm_streams(const int* ids, const void* table, const float* norm_w, float eps, float offset,
                               float* xs, int T, int S, int W, int vocab, bool f32, hipStream_t s);
// out[t] = rms(sum_s w_in[s] xs[t, s]) * (w + offset)
void launch_hc_pre(const float* xs, const float* w_in, const float* norm_w, float eps, float offset, void* out,
                   int T, int S, int W, bool f32, hipStream_t s);
// xs[t, r] <- sum_s mix[s, r] xs[t, s] + w_out[r] y[t]   (all streams at once from the old ones)
void launch_hc_post(float* xs, const void* y, const float* mix, const float* w_out, int T, int S, int W, bool f32,
                    hipStream_t s);
// launch_hc_post, then launch_hc_pre of the next sublayer (w_in2, norm_w2) on the updated streams
void launch_hc_post_pre(float* xs, const void* y, const float* mix, const float* w_out, const float* w_in2,
                        const float* norm_w2, float eps, float offset, void* out, int T, int S, int W, bool f32,
                        hipStream_t s);
// out[i] = rms(sum_s xs[idx[i], s]) * (w + offset); idx == nullptr: every row
void launch_hc_final(const float* xs, const float* norm_w, float eps, float offset, const long* idx, void* out,
                     int R, int S, int W, bool f32, hipStream_t s);

// Rotate pairs (2i, 2i+1), i < nrot, of every q and k head by positions[t] * inv_freq[i]; append
// k / v rows to cache slot slots[t] (>= 0): K [blocks, G, BS, D], V [blocks, G, Dv, BS]. k == nullptr: q only.
void launch_rope_partial_kv(void* q, long q_ld, void* k, long k_ld, const void* v, long v_ld, const int* positions,
                            const float* inv_freq, int nrot, const int* slots, void* k_cache, void* v_cache,
                            int T, int H, int G, int D, int Dv, int block_size, bool f32, hipStream_t s);
// row_seq[t] = the sequence whose row range [row_cu[s], row_cu[s+1]) holds row t, else -1
void launch_row_seq(const int* row_cu, int nseq, int* row_seq, int T, hipStream_t s);
// Score modifiers of the paged attention kernels, all off by default. Order: scale (with the
// temperature), cap, distance bias, mask.
struct AttnMod {
  int chunk = 0;                  // > 0: instead of the window, a row sees its own chunk of `chunk` positions
                                  // (j >= p - p % chunk)
  float softcap = 0.f;            // > 0: s <- cap tanh(s / cap)
  const float* dist_a = nullptr;  // [H] (with dist_b): s <- s - a[h] ln(1 + b[h] (p - j))
  const float* dist_b = nullptr;  // nullptr with dist_a set: the linear form s <- s - a[h] (p - j)
  float qt_coef = 0.f;            // the score scale of a row at p is multiplied by
  int qt_every = 1;               // 1 + coef ln(floor((p + 1) / every) + 1)
  int maps = 1;                   // key heads per value head: K [blocks, G * maps, BS, D]; query heads are ordered
                                  // (head, map) and head (h, m) reads key head (g(h), m) and value head g(h)
  bool out_f32 = false;           // out is float whatever the inputs
};

// Row t of sequence row_seq[t] (-1: padding row, output zero) at position p sees cached keys
// j <= p with p - j < window or j < keep_first; the softmax denominator includes exp(sink[h])
// (sink == nullptr: an ordinary softmax); out_scale (nullable) [T, H] multiplies each head's output.
// out [T, H, Dv] contiguous. Dv <= 512.
void launch_attn_window_paged(const void* q, long q_ld, const void* k_cache, const void* v_cache, const int* tables,
                              int max_blocks, const int* row_seq, int nseq, const int* positions, float scale,
                              int window, int keep_first, const float* sink, const float* out_scale, void* out, int T,
                              int H, int G, int D, int Dv, int block_size, bool f32, hipStream_t s,
                              const AttnMod& md = AttnMod());

// The MFMA form of launch_attn_window_paged over row_cu (bf16, 32-token pages, D and Dv in {32, 64,
// 96, 128, 192, 256}, 16-byte aligned q rows): false if the shape has no such form. `fold` (G == 1):
// tiles run over (token, head) pairs, so a token's heads share the pages they read. `part` (nullable,
// part_floats f32): scratch for steps of few tiles, whose pages are then split over several
// workgroups per tile (T * H * (Dv + 2) floats per split).
bool launch_attn_window_mfma(const void* q, long q_ld, const void* k_cache, const void* v_cache, const int* tables,
                             int max_blocks, const int* row_cu, int nseq, const int* positions, float scale, int window,
                             int keep_first, const float* sink, const float* out_scale, void* out, int T, int H, int G,
                             int D, int Dv, int block_size, bool fold, float* part, long part_floats, hipStream_t s,
                             const AttnMod& md = AttnMod());

// Gated linear attention scan over packed rows (see ops.gla_scan). Returns < 0 if D > 256.
int launch_gla_scan(const void* q, long q_ld, const void* k, long k_ld, const void* v, long v_ld, const void* z,
                    long z_ld, float* state, const int* state_slots, const int* row_cu, int nseq,
                    const int* positions, float tau, float q_scale, float* o, int T, int H, int D, int Dv, bool f32,
                    hipStream_t s);
// out[t, h * Dv + j] = rms(o[t, h])[j] * w[j] * silu(g[t, h * Dv + j])
void launch_gla_out(const float* o, const void* g, long g_ld, const float* norm_w, float eps, void* out, int T, int H,
                    int Dv, bool f32, hipStream_t s);

// logits[t, e] = x[t] . wr[e] in f32, one wave per pair (for steps of a few rows)
void launch_router_logits(const void* x, long ldx, const void* wr, float* logits, int T, int E, int Hd, bool f32,
                          hipStream_t s);
// Router choice from f32 logits [T, E] (+ bias [E], nullable): scoring 0 softmax / 1 sigmoid, top-k
// (ties: lowest id), optional renorm. select_bias [E] (nullable) is added to the scores for the choice
// only; the weights are the chosen experts' plain scores. E <= 1024.
void launch_moe_topk_scores(const float* logits, const float* bias, int top_k, int scoring, bool renorm, int* ids,
                            float* w, int T, int E, hipStream_t s, const float* select_bias = nullptr);
// Group the T*K (token, choice) pairs by expert: perm [TK] pair indices grouped by expert,
// offsets [E + 1], tiles [max_tiles][2] = (expert, first row) of every tile_rows-row tile, ntiles [1].
void launch_moe_sort(const int* ids, int TK, int E, int* perm, int* offsets, int* tiles, int* ntiles, int tile_rows,
                     hipStream_t s);
int moe_sort_max_tiles(int TK, int E);
// rows per tile of the grouped expert GEMMs for this problem (64, or 128 for large bf16 groups)
int moe_tile_rows(int TK, int E, bool f32);
// hmid[r, f] = g' sigmoid(alpha g') (u' + up_offset), (g', u') the clamped gate / up products of
// expert e(r) on (w x) for grouped row r (topk_w == nullptr: on x itself). plain_act != ACT_NONE: experts
// without a gate, gate_up_w [E, F, Hd] and hmid = act(up product) (ACT_RELU2)
void launch_moe_glu_up(const void* x, long ldx, const float* topk_w, int K, const int* perm, const int* offsets,
                       const int* tiles, const int* ntiles, int max_tiles, const void* gate_up_w, float limit,
                       float alpha, float up_offset, void* hmid, int Hd, int F, bool f32, int tile_rows, hipStream_t s,
                       int plain_act = ACT_NONE);
// y[perm[r], :] = down_e(r) hmid[r]     (y f32, pair order)
void launch_moe_down(const void* hmid, const int* perm, const int* offsets, const int* tiles, const int* ntiles,
                     int max_tiles, const void* down_w, float* y, int Hd, int F, bool f32, int tile_rows, hipStream_t s);
// out[t] = sum_j wts[t * K + j] y[t * K + j]   (wts == nullptr: the plain sum)
void launch_moe_sum(const float* y, const float* wts, int K, void* out, int T, int Hd, bool f32, hipStream_t s);

}  // namespace bfly
