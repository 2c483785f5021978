// Post-norm residual stacks with latent attention, generic in every size and in the activation
// type (bf16 or f32; the residual, norms, angles and gates are f32 in both):
//   embed_scaled_kernel        x = table[token] * scale (f32)
//   conv_mix_kernel            h_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j) per channel over the
//                              rows of a sequence; rows before the step come from the per-sequence
//                              history pool, zeros before position 0
//   conv_state_update_kernel   the pool takes the last taps - 1 inputs of every sequence
//   post_norm_add_kernel       out = x + scale * layer_norm(y), optionally also rounded for the
//                              next GEMM
//   post_norm_add_avg_kernel   the same update (or none), the result stored as a layer's output,
//                              and the residual replaced by a weighted sum of all outputs so far
//   latent_prep_kernel         RMS norms of the query and key/value latents, rotary on the shared
//                              key part, sigmoid gates, append to the paged caches
//   rope_heads_copy_kernel     rotated copy of a slice of every head
//   layer_norm_rows_kernel     layer norm of chosen rows
// Rows of a step are packed: sequence s owns rows row_cu[s] .. row_cu[s+1].
#include <algorithm>

#include "bfly_common.h"
#include "bfly_postnorm.h"

namespace bfly {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                           float scale, float* __restrict__ out, int W, int vocab) {
  const long t = blockIdx.x;
  const int id = min(max(ids[t], 0), vocab - 1);
  const T* row = table + (long)id * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) out[t * W + c] = (float)row[c] * scale;
}

// the sequence whose row range holds row t (row_cu is non-decreasing; -1: none)
__device__ __forceinline__ int seq_of_row(const int* __restrict__ row_cu, int nseq, int t) {
  int lo = 0, hi = nseq;            // the last s with row_cu[s] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (row_cu[mid] <= t) lo = mid; else hi = mid;
  }
  return (nseq > 0 && row_cu[lo] <= t && t < row_cu[lo + 1]) ? lo : -1;
}

// one thread per (row, V consecutive channels): the taps' loads are independent of one another
// (V = 4 when the width allows 16-byte accesses)
template <typename TO, int V>
__global__ __launch_bounds__(256) void conv_mix_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       const float* __restrict__ state,
                                                       const int* __restrict__ state_slots,
                                                       const int* __restrict__ row_cu, int nseq,
                                                       const int* __restrict__ positions, TO* __restrict__ out,
                                                       int W, int taps) {
  typedef float fv __attribute__((ext_vector_type(V)));
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= W) return;
  const fv xc = *reinterpret_cast<const fv*>(x + (long)t * W + c);
  const int s = (w && taps > 0) ? seq_of_row(row_cu, nseq, t) : -1;
  fv h = xc;
  if (s >= 0) {                      // (else: no convolution, or a row outside every sequence)
    const int a = row_cu[s], p = positions[t];
    const int slot = state_slots ? state_slots[s] : -1;
    const int n = taps - 1;
    for (int j = 0; j < taps; ++j) {
      const int d = n - j;           // the input d steps back
      fv v;
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = 0.f;
      if (d == 0) v = xc;
      else if (t - d >= a) v = *reinterpret_cast<const fv*>(x + (long)(t - d) * W + c);
      else if (p - d >= 0 && slot >= 0)
        v = *reinterpret_cast<const fv*>(state + ((long)slot * n + (n - (d - (t - a)))) * W + c);
#pragma unroll
      for (int e = 0; e < V; ++e) h[e] = fmaf(w[(long)(c + e) * taps + j], v[e], h[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) out[(long)t * W + c + e] = (TO)h[e];
}

// The same for up to 8 taps with RB consecutive rows per workgroup: a thread keeps the last
// taps - 1 inputs of its channels in registers and slides over the rows, so a row costs one load
// of x; the history is fetched anew (earlier rows, the pool, or zeros) at the block's first row
// and wherever a new sequence begins. Taps are summed in the same order as above.
template <typename TO, int V>
__global__ __launch_bounds__(256) void conv_mix_rows_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const float* __restrict__ state,
                                                            const int* __restrict__ state_slots,
                                                            const int* __restrict__ row_cu, int nseq,
                                                            const int* __restrict__ positions, TO* __restrict__ out,
                                                            int W, int taps, int T, int RB) {
  typedef float fv __attribute__((ext_vector_type(V)));
  constexpr int MAXN = 7;
  const int t0 = blockIdx.x * RB, t1 = min(T, t0 + RB);
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= W) return;
  const int n = taps - 1;
  fv wv[MAXN + 1], hist[MAXN];
#pragma unroll
  for (int j = 0; j <= MAXN; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) wv[j][e] = j < taps ? w[(long)(c + e) * taps + j] : 0.f;
  int s = -1, send = t0;
  bool fetch = true;
  for (int t = t0; t < t1; ++t) {
    if (t >= send) {
      s = seq_of_row(row_cu, nseq, t);
      send = s >= 0 ? row_cu[s + 1] : t + 1;
      fetch = true;
    }
    const fv xc = *reinterpret_cast<const fv*>(x + (long)t * W + c);
    fv h = xc;
    if (s >= 0) {
      if (fetch) {
        const int a = row_cu[s], p = positions[t];
        const int slot = state_slots ? state_slots[s] : -1;
#pragma unroll
        for (int k = 0; k < MAXN; ++k) {
          if (k >= n) break;
          const int d = n - k;
          fv v;
#pragma unroll
          for (int e = 0; e < V; ++e) v[e] = 0.f;
          if (t - d >= a) v = *reinterpret_cast<const fv*>(x + (long)(t - d) * W + c);
          else if (p - d >= 0 && slot >= 0)
            v = *reinterpret_cast<const fv*>(state + ((long)slot * n + (n - (d - (t - a)))) * W + c);
          hist[k] = v;
        }
        fetch = false;
      }
#pragma unroll
      for (int k = 0; k < MAXN; ++k) {
        if (k >= n) break;
#pragma unroll
        for (int e = 0; e < V; ++e) h[e] = fmaf(wv[k][e], hist[k][e], h[e]);
      }
#pragma unroll
      for (int k = 0; k <= MAXN; ++k)
        if (k == n) {
#pragma unroll
          for (int e = 0; e < V; ++e) h[e] = fmaf(wv[k][e], xc[e], h[e]);
        }
#pragma unroll
      for (int k = 0; k < MAXN; ++k) {
        if (k + 1 < n) hist[k] = hist[k + 1];
        else if (k + 1 == n) hist[k] = xc;
      }
    }
    if constexpr (V == 4 && sizeof(TO) == 2) {
      bf16x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (bf16)h[e];
      *reinterpret_cast<bf16x4*>(out + (long)t * W + c) = o;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[(long)t * W + c + e] = (TO)h[e];
    }
  }
}

// one thread per (sequence, channel): entry i of the new history is old entry i + len while that
// exists (read before any entry at or above it is written), then the step's own rows
__global__ __launch_bounds__(256) void conv_state_update_kernel(const float* __restrict__ x, float* __restrict__ state,
                                                                const int* __restrict__ state_slots,
                                                                const int* __restrict__ row_cu,
                                                                const int* __restrict__ positions, int W, int n) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int a = row_cu[s], b = row_cu[s + 1], slot = state_slots[s];
  if (c >= W || b <= a || slot < 0) return;
  const int len = b - a, p0 = positions[a];
  float* S = state + (long)slot * n * W + c;
  for (int i = 0; i < n; ++i) {
    const int r = b - (n - i);       // the row that becomes entry i
    float v;
    if (r >= a) v = x[(long)r * W + c];
    else v = (p0 - (a - r) >= 0) ? S[(long)(i + len) * W] : 0.f;
    S[(long)i * W] = v;
  }
}

// mean and 1 / sqrt(var + eps) of the row staged in LDS (f32, two passes)
__device__ __forceinline__ void row_stats(const float* __restrict__ sy, int W, float eps, float* red, float& mean,
                                          float& rstd) {
  float a = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) a += sy[c];
  mean = block_sum(a, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = sy[c] - mean;
    q = fmaf(d, d, q);
  }
  rstd = 1.f / sqrtf(block_sum(q, red) / (float)W + eps);
}

template <typename T>
__global__ __launch_bounds__(1024) void post_norm_add_kernel(const float* __restrict__ x, const T* __restrict__ y,
                                                            const float* __restrict__ nw, const float* __restrict__ nb,
                                                            float eps, const float* __restrict__ scale,
                                                            float* __restrict__ out, T* __restrict__ cast, int W) {
  extern __shared__ float sy[];
  __shared__ float red[16];
  const long t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) sy[c] = (float)y[t * W + c];
  __syncthreads();
  float mean, rstd;
  row_stats(sy, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = x[t * W + c] + scale[c] * ((sy[c] - mean) * rstd * nw[c] + nb[c]);
    out[t * W + c] = v;
    if (cast) cast[t * W + c] = (T)v;
  }
}

template <typename T>
__global__ __launch_bounds__(1024) void post_norm_add_avg_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                const float* __restrict__ nw,
                                                                const float* __restrict__ nb, float eps,
                                                                const float* __restrict__ scale,
                                                                float* __restrict__ stack, long plane, int index,
                                                                const float* __restrict__ avg, int W) {
  extern __shared__ float sy[];
  __shared__ float red[16];
  const long t = blockIdx.x;
  float mean = 0.f, rstd = 0.f;
  if (y) {
    for (int c = threadIdx.x; c < W; c += blockDim.x) sy[c] = (float)y[t * W + c];
    __syncthreads();
    row_stats(sy, W, eps, red, mean, rstd);
  }
  const float wl = avg[index];
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = x[t * W + c];
    if (y) v += scale[c] * ((sy[c] - mean) * rstd * nw[c] + nb[c]);
    stack[(long)index * plane + t * W + c] = v;
    float acc = 0.f;
    for (int j = 0; j < index; ++j) acc = fmaf(avg[j], stack[(long)j * plane + t * W + c], acc);
    x[t * W + c] = fmaf(wl, v, acc);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ z, long z_ld, int Q, int R, int rd,
                                                          int H, const float* __restrict__ qn_w,
                                                          const float* __restrict__ kvn_w, float eps,
                                                          const int* __restrict__ positions,
                                                          const float* __restrict__ inv_freq, int nrot,
                                                          const int* __restrict__ slots, T* __restrict__ k_cache,
                                                          T* __restrict__ v_cache, int bs, int Dk, int Dvc,
                                                          T* __restrict__ cq, float* __restrict__ gate) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const T* zr = z + t * z_ld;
  float a = 0.f, b = 0.f;
  for (int i = threadIdx.x; i < Q; i += blockDim.x) { const float v = (float)zr[i]; a = fmaf(v, v, a); }
  for (int i = threadIdx.x; i < R; i += blockDim.x) { const float v = (float)zr[Q + i]; b = fmaf(v, v, b); }
  const float rq = Q > 0 ? 1.f / sqrtf(block_sum(a, red) / (float)Q + eps) : 0.f;     // (Q, H = 0: no query latent, no gates)
  const float rk = 1.f / sqrtf(block_sum(b, red) / (float)R + eps);
  for (int i = threadIdx.x; i < Q; i += blockDim.x) cq[t * Q + i] = (T)((float)zr[i] * rq * qn_w[i]);
  for (int i = threadIdx.x; i < H; i += blockDim.x) gate[t * H + i] = 1.f / (1.f + expf(-(float)zr[Q + R + rd + i]));
  const int slot = slots[t];
  if (slot < 0) return;
  const long blk = slot / bs, off = slot % bs;
  T* krow = k_cache + (blk * bs + off) * Dk;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const T c = (T)((float)zr[Q + i] * rk * kvn_w[i]);
    krow[i] = c;
    v_cache[(blk * Dvc + i) * bs + off] = c;
  }
  const float p = (float)positions[t];
  const T* kr = zr + Q + R;
  for (int i = threadIdx.x; i < rd / 2; i += blockDim.x) {
    const float u = (float)kr[2 * i], w = (float)kr[2 * i + 1];
    if (i < nrot) {
      double sd, cd;
      sincos((double)(p * inv_freq[i]), &sd, &cd);
      const float c = (float)cd, s = (float)sd;
      krow[R + 2 * i] = (T)(u * c - w * s);
      krow[R + 2 * i + 1] = (T)(w * c + u * s);
    } else {
      krow[R + 2 * i] = (T)u;
      krow[R + 2 * i + 1] = (T)w;
    }
  }
  if ((rd & 1) && threadIdx.x == 0) krow[R + rd - 1] = kr[rd - 1];
}

// dst heads may be wider than src heads (nd >= n): the tail is zero filled
template <typename T>
__global__ __launch_bounds__(256) void rope_heads_copy_kernel(const T* __restrict__ src, long s_ld, long s_hd,
                                                              T* __restrict__ dst, long d_ld, long d_hd,
                                                              const int* __restrict__ positions,
                                                              const float* __restrict__ inv_freq, int nrot, int H,
                                                              int n, int nd) {
  const long t = blockIdx.x;
  const float p = (float)positions[t];
  const int half = (nd + 1) / 2;
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int h = i / half, r = i % half;
    const T* sp = src + t * s_ld + h * s_hd + 2 * r;
    T* dp = dst + t * d_ld + h * d_hd + 2 * r;
    const bool two = 2 * r + 1 < nd;
    float u = 2 * r < n ? (float)sp[0] : 0.f, w = 2 * r + 1 < n ? (float)sp[1] : 0.f;
    if (r < nrot) {                                  // (2 nrot <= n: both elements exist)
      double sd, cd;
      sincos((double)(p * inv_freq[r]), &sd, &cd);
      const float c = (float)cd, s = (float)sd;
      const float u2 = u * c - w * s, w2 = w * c + u * s;
      u = u2;
      w = w2;
    }
    dp[0] = (T)u;
    if (two) dp[1] = (T)w;
  }
}

template <typename TO>
__global__ __launch_bounds__(1024) void layer_norm_rows_kernel(const float* __restrict__ x, const float* __restrict__ nw,
                                                              const float* __restrict__ nb, float eps,
                                                              const long* __restrict__ idx, TO* __restrict__ out,
                                                              int W) {
  extern __shared__ float sy[];
  __shared__ float red[16];
  const long i = blockIdx.x, t = idx ? idx[i] : i;
  for (int c = threadIdx.x; c < W; c += blockDim.x) sy[c] = x[t * W + c];
  __syncthreads();
  float mean, rstd;
  row_stats(sy, W, eps, red, mean, rstd);
  for (int c = threadIdx.x; c < W; c += blockDim.x) out[i * W + c] = (TO)((sy[c] - mean) * rstd * nw[c] + nb[c]);
}

}  // namespace

// threads of a one-row workgroup: about four elements per thread, whole waves, at most 1024
static int row_threads(int W) { return std::min(1024, std::max(64, (W / 4 + 63) / 64 * 64)); }

void launch_embed_scaled(const int* ids, const void* table, float scale, float* out, int T, int W, int vocab, bool f32,
                         hipStream_t s) {
  if (T <= 0) return;
  if (f32) embed_scaled_kernel<float><<<T, 256, 0, s>>>(ids, (const float*)table, scale, out, W, vocab);
  else embed_scaled_kernel<bf16><<<T, 256, 0, s>>>(ids, (const bf16*)table, scale, out, W, vocab);
}

void launch_conv_mix(const float* x, const float* w, const float* state, const int* state_slots, const int* row_cu,
                     int nseq, const int* positions, void* out, int T, int W, int taps, bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (w && taps >= 1 && taps <= 8) {
    // rows per workgroup: one for steps of few rows (every row its own sequence, as in decoding)
    const int RB = std::min(16, std::max(1, T / 512));
#define BFLY_CONV(TO, V)                                                                                     \
  conv_mix_rows_kernel<TO, V><<<dim3((T + RB - 1) / RB, (W / V + 255) / 256), 256, 0, s>>>(                  \
      x, w, state, state_slots, row_cu, nseq, positions, (TO*)out, W, taps, T, RB)
    if (W % 4 == 0) { if (f32) BFLY_CONV(float, 4); else BFLY_CONV(bf16, 4); }
    else { if (f32) BFLY_CONV(float, 1); else BFLY_CONV(bf16, 1); }
#undef BFLY_CONV
    return;
  }
  dim3 grid(T, (W + 255) / 256);
  if (f32)
    conv_mix_kernel<float, 1><<<grid, 256, 0, s>>>(x, w, state, state_slots, row_cu, nseq, positions, (float*)out, W, taps);
  else
    conv_mix_kernel<bf16, 1><<<grid, 256, 0, s>>>(x, w, state, state_slots, row_cu, nseq, positions, (bf16*)out, W, taps);
}

void launch_conv_state_update(const float* x, float* state, const int* state_slots, const int* row_cu, int nseq,
                              const int* positions, int W, int n, hipStream_t s) {
  if (nseq <= 0 || n <= 0) return;
  dim3 grid(nseq, (W + 255) / 256);
  conv_state_update_kernel<<<grid, 256, 0, s>>>(x, state, state_slots, row_cu, positions, W, n);
}

void launch_post_norm_add(const float* x, const void* y, const float* nw, const float* nb, float eps,
                          const float* scale, float* out, void* cast, int T, int W, bool f32, hipStream_t s) {
  if (T <= 0) return;
  const size_t sm = (size_t)W * sizeof(float);
  if (f32)
    post_norm_add_kernel<float><<<T, row_threads(W), sm, s>>>(x, (const float*)y, nw, nb, eps, scale, out, (float*)cast, W);
  else
    post_norm_add_kernel<bf16><<<T, row_threads(W), sm, s>>>(x, (const bf16*)y, nw, nb, eps, scale, out, (bf16*)cast, W);
}

void launch_post_norm_add_avg(float* x, const void* y, const float* nw, const float* nb, float eps, const float* scale,
                              float* stack, long plane, int index, const float* avg, int T, int W, bool f32,
                              hipStream_t s) {
  if (T <= 0) return;
  const size_t sm = (size_t)W * sizeof(float);
  if (f32)
    post_norm_add_avg_kernel<float><<<T, row_threads(W), sm, s>>>(x, (const float*)y, nw, nb, eps, scale, stack, plane, index, avg, W);
  else
    post_norm_add_avg_kernel<bf16><<<T, row_threads(W), sm, s>>>(x, (const bf16*)y, nw, nb, eps, scale, stack, plane, index, avg, W);
}

void launch_latent_prep(const void* z, long z_ld, int Q, int R, int rd, int H, const float* qn_w, const float* kvn_w,
                        float eps, const int* positions, const float* inv_freq, int nrot, const int* slots,
                        void* k_cache, void* v_cache, int block_size, int Dk, int Dvc, void* cq, float* gate, int T,
                        bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    latent_prep_kernel<float><<<T, 256, 0, s>>>((const float*)z, z_ld, Q, R, rd, H, qn_w, kvn_w, eps, positions, inv_freq,
                                                nrot, slots, (float*)k_cache, (float*)v_cache, block_size, Dk, Dvc,
                                                (float*)cq, gate);
  else
    latent_prep_kernel<bf16><<<T, 256, 0, s>>>((const bf16*)z, z_ld, Q, R, rd, H, qn_w, kvn_w, eps, positions, inv_freq,
                                               nrot, slots, (bf16*)k_cache, (bf16*)v_cache, block_size, Dk, Dvc,
                                               (bf16*)cq, gate);
}

void launch_rope_heads_copy(const void* src, long s_ld, long s_hd, void* dst, long d_ld, long d_hd,
                            const int* positions, const float* inv_freq, int nrot, int T, int H, int n, int nd, bool f32,
                            hipStream_t s) {
  if (T <= 0 || nd <= 0) return;
  if (f32)
    rope_heads_copy_kernel<float><<<T, 256, 0, s>>>((const float*)src, s_ld, s_hd, (float*)dst, d_ld, d_hd, positions,
                                                    inv_freq, nrot, H, n, nd);
  else
    rope_heads_copy_kernel<bf16><<<T, 256, 0, s>>>((const bf16*)src, s_ld, s_hd, (bf16*)dst, d_ld, d_hd, positions,
                                                   inv_freq, nrot, H, n, nd);
}

void launch_layer_norm_rows(const float* x, const float* nw, const float* nb, float eps, const long* idx, void* out,
                            int R, int W, bool f32, hipStream_t s) {
  if (R <= 0) return;
  const size_t sm = (size_t)W * sizeof(float);
  if (f32) layer_norm_rows_kernel<float><<<R, row_threads(W), sm, s>>>(x, nw, nb, eps, idx, (float*)out, W);
  else layer_norm_rows_kernel<bf16><<<R, row_threads(W), sm, s>>>(x, nw, nb, eps, idx, (bf16*)out, W);
}

}  // namespace bfly
