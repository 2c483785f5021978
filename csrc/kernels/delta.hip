// Sandwich-norm residual stacks with a gated delta rule, generic in every size and in the activation
// type (bf16 or f32; the residual, norms, decays, unit norms and the recurrent state are f32 in both):
//   post_norm_add_norm_kernel        x <- x + mult * layer_norm(y) (+ extra), then the next sublayer's
//                                    input layer_norm(x) with its own weight and bias
//   short_conv_act_kernel            y_t = act(sum_j w[:, j] z_(t - taps + 1 + j)) per channel over the
//                                    rows of a sequence; rows before the step come from the per-sequence
//                                    history pool, zeros before position 0
//   short_conv_state_update_kernel   the pool takes the last taps - 1 rows of every sequence
//   delta_scan_kernel                S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q per
//                                    (sequence, head), the state pooled per sequence
// Rows of a step are packed: sequence s owns rows row_cu[s] .. row_cu[s+1].
#include <algorithm>

#include "bfly_common.h"
#include "bfly_delta.h"

namespace bfly {

namespace {

// the sequence whose row range holds row t (row_cu is non-decreasing; -1: none)
__device__ __forceinline__ int seq_of_row(const int* __restrict__ row_cu, int nseq, int t) {
  int lo = 0, hi = nseq;            // the last s with row_cu[s] <= t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (row_cu[mid] <= t) lo = mid; else hi = mid;
  }
  return (nseq > 0 && row_cu[lo] <= t && t < row_cu[lo + 1]) ? lo : -1;
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

// One workgroup per row; the row of y, then the updated row of x, staged in LDS. V = 4 (W % 4 == 0):
// 16-byte accesses (8-byte for bf16); the statistics are the same two-pass sums either way.
template <typename T, int V>
__global__ __launch_bounds__(1024) void post_norm_add_norm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                 const float* __restrict__ nw,
                                                                 const float* __restrict__ nb, float eps, float mult,
                                                                 const float* __restrict__ extra,
                                                                 const float* __restrict__ nw2,
                                                                 const float* __restrict__ nb2, T* __restrict__ h,
                                                                 int W) {
  typedef float fv __attribute__((ext_vector_type(V)));
  typedef T tv __attribute__((ext_vector_type(V)));
  extern __shared__ __attribute__((aligned(16))) float sy[];
  __shared__ float red[16];
  const long t = blockIdx.x;
  for (int c = V * threadIdx.x; c < W; c += V * blockDim.x) {
    const tv yv = *reinterpret_cast<const tv*>(y + t * W + c);
    fv f;
#pragma unroll
    for (int e = 0; e < V; ++e) f[e] = (float)yv[e];
    *reinterpret_cast<fv*>(sy + c) = f;
  }
  __syncthreads();
  float mean, rstd;
  row_stats(sy, W, eps, red, mean, rstd);
  for (int c = V * threadIdx.x; c < W; c += V * blockDim.x) {
    const fv yv = *reinterpret_cast<const fv*>(sy + c), wv = *reinterpret_cast<const fv*>(nw + c),
             bv = *reinterpret_cast<const fv*>(nb + c);
    fv v = *reinterpret_cast<const fv*>(x + t * W + c);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = v[e] + mult * ((yv[e] - mean) * rstd * wv[e] + bv[e]);
    if (extra) {
      const fv ev = *reinterpret_cast<const fv*>(extra + t * W + c);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] += ev[e];
    }
    *reinterpret_cast<fv*>(x + t * W + c) = v;
    *reinterpret_cast<fv*>(sy + c) = v;      // (a thread rewrites only what it alone read after the barrier)
  }
  if (!h) return;
  __syncthreads();
  row_stats(sy, W, eps, red, mean, rstd);
  for (int c = V * threadIdx.x; c < W; c += V * blockDim.x) {
    const fv xv = *reinterpret_cast<const fv*>(sy + c), wv = *reinterpret_cast<const fv*>(nw2 + c),
             bv = *reinterpret_cast<const fv*>(nb2 + c);
    tv o;
#pragma unroll
    for (int e = 0; e < V; ++e) o[e] = (T)((xv[e] - mean) * rstd * wv[e] + bv[e]);
    *reinterpret_cast<tv*>(h + t * W + c) = o;
  }
}

// one thread per (row, channel); the taps are summed oldest first
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_act_kernel(const TI* __restrict__ z, long z_ld,
                                                             const float* __restrict__ w,
                                                             const float* __restrict__ state,
                                                             const int* __restrict__ state_slots,
                                                             const int* __restrict__ row_cu, int nseq,
                                                             const int* __restrict__ positions, TO* __restrict__ out,
                                                             int C, int taps, int act) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int s = seq_of_row(row_cu, nseq, t);
  float acc = 0.f;
  if (s >= 0) {
    const int a = row_cu[s], p = positions[t];
    const int slot = state_slots ? state_slots[s] : -1;
    const int n = taps - 1;
    for (int j = 0; j < taps; ++j) {
      const int d = n - j;           // the input d steps back
      float v = 0.f;
      if (t - d >= a) v = (float)z[(long)(t - d) * z_ld + c];
      else if (p - d >= 0 && slot >= 0) v = state[((long)slot * n + (n - (d - (t - a)))) * C + c];
      acc = fmaf(w[(long)c * taps + j], v, acc);
    }
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  out[(long)t * C + c] = (TO)acc;
}

// The same for up to 8 taps and C % 4 == 0 with RB consecutive rows per workgroup: a thread owns 4
// channels, keeps their last taps - 1 inputs in registers and slides over the rows, so a row costs one
// load of z; the history is fetched anew (earlier rows, the pool, or zeros) at the block's first row and
// wherever a new sequence begins. Taps are summed in the same order as above.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_act_rows_kernel(const TI* __restrict__ z, long z_ld,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ state,
                                                                  const int* __restrict__ state_slots,
                                                                  const int* __restrict__ row_cu, int nseq,
                                                                  const int* __restrict__ positions,
                                                                  TO* __restrict__ out, int C, int taps, int act, int T,
                                                                  int RB) {
  constexpr int MAXN = 7;
  typedef TI tiv __attribute__((ext_vector_type(4)));
  typedef TO tov __attribute__((ext_vector_type(4)));
  const int t0 = blockIdx.x * RB, t1 = min(T, t0 + RB);
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (c >= C) return;
  const int n = taps - 1;
  f32x4 wv[MAXN + 1], hist[MAXN];
#pragma unroll
  for (int j = 0; j <= MAXN; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) wv[j][e] = j < taps ? w[(long)(c + e) * taps + j] : 0.f;
  auto ld = [&](long row) {
    const tiv v = *reinterpret_cast<const tiv*>(z + row * z_ld + c);
    return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  };
  int s = -1, send = t0;
  bool fetch = true;
  for (int t = t0; t < t1; ++t) {
    if (t >= send) {
      s = seq_of_row(row_cu, nseq, t);
      send = s >= 0 ? row_cu[s + 1] : t + 1;
      fetch = true;
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (s >= 0) {
      const f32x4 zc = ld(t);
      if (fetch) {
        const int a = row_cu[s], p = positions[t];
        const int slot = state_slots ? state_slots[s] : -1;
#pragma unroll
        for (int k = 0; k < MAXN; ++k) {
          if (k >= n) break;
          const int d = n - k;
          f32x4 v = {0.f, 0.f, 0.f, 0.f};
          if (t - d >= a) v = ld(t - d);
          else if (p - d >= 0 && slot >= 0)
            v = *reinterpret_cast<const f32x4*>(state + ((long)slot * n + (n - (d - (t - a)))) * C + c);
          hist[k] = v;
        }
        fetch = false;
      }
#pragma unroll
      for (int k = 0; k < MAXN; ++k) {
        if (k >= n) break;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(wv[k][e], hist[k][e], acc[e]);
      }
#pragma unroll
      for (int k = 0; k <= MAXN; ++k)
        if (k == n) {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] = fmaf(wv[k][e], zc[e], acc[e]);
        }
#pragma unroll
      for (int k = 0; k < MAXN; ++k) {
        if (k + 1 < n) hist[k] = hist[k + 1];
        else if (k + 1 == n) hist[k] = zc;
      }
    }
    tov o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (TO)(act == 1 ? acc[e] / (1.f + expf(-acc[e])) : acc[e]);
    *reinterpret_cast<tov*>(out + (long)t * C + c) = o;
  }
}

// one thread per (sequence, channel): entry i of the new history is old entry i + len while that
// exists (read before any entry at or above it is written), then the step's own rows
template <typename TI>
__global__ __launch_bounds__(256) void short_conv_state_update_kernel(const TI* __restrict__ z, long z_ld,
                                                                      float* __restrict__ state,
                                                                      const int* __restrict__ state_slots,
                                                                      const int* __restrict__ row_cu,
                                                                      const int* __restrict__ positions, int C, int n) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int a = row_cu[s], b = row_cu[s + 1], slot = state_slots[s];
  if (c >= C || b <= a || slot < 0) return;
  const int len = b - a, p0 = positions[a];
  float* S = state + (long)slot * n * C + c;
  for (int i = 0; i < n; ++i) {
    const int r = b - (n - i);       // the row that becomes entry i
    float v;
    if (r >= a) v = (float)z[(long)r * z_ld + c];
    else v = (p0 - (a - r) >= 0) ? S[(long)(i + len) * C] : 0.f;
    S[(long)i * C] = v;
  }
}

// sum over the 8 lanes that share lane >> 3, in every lane, by three cross-lane moves inside a row of 16
// (neighbour, next pair, mirrored half row): no LDS traffic, so the token loop's LDS reads stay in flight
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float sum8(float v) {
  v += dpp_move<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);     // row_half_mirror: lane i of 8 <- lane 7 - i (the other quad's sum)
  return v;
}

// Workgroup = (sequence, head, 64-column slice of Dv), 8 waves; wave w owns 8 columns. A lane is
// (row group gg = lane & 7, column c = lane >> 3) and keeps the NR rows d = gg * NR .. + NR - 1 of its
// column's state in registers. The pool holds a head's state column by column ([Dv, D]: the rows a lane
// owns are contiguous, the eight lanes of a column cover it with 16-byte accesses). Tokens are staged
// 16 at a time: raw keys and queries go to LDS (rows past D are zero, so the row loop needs no bound),
// and per token the scalars of the update: decay g, write strength beta, 1 / |k|, q_scale / |q| (the
// unit norms are folded into scalars: S^T k = kn S^T k_raw and so on, so no element is normalised on
// its own). The next block's inputs travel to registers while the current block is computed. A token
// then costs a dot product of the lane's rows with k (four partial sums), three cross-lane moves to sum
// the eight row groups, one fused pass that updates the rows and accumulates the read-out, and three
// more moves: no barrier inside the token loop. The outputs of the 16 tokens leave through LDS.
template <typename T, int NR>
__global__ __launch_bounds__(512) void delta_scan_kernel(const float* __restrict__ q, long q_ld,
                                                         const float* __restrict__ k, long k_ld,
                                                         const float* __restrict__ v, long v_ld,
                                                         const T* __restrict__ bl, long b_ld, const T* __restrict__ al,
                                                         long a_ld, const float* __restrict__ a_log,
                                                         const float* __restrict__ dt_bias, float* __restrict__ state,
                                                         const int* __restrict__ state_slots,
                                                         const int* __restrict__ row_cu,
                                                         const int* __restrict__ positions, float q_scale,
                                                         float unit_eps, float* __restrict__ o, int H, int G, int D,
                                                         int Dv) {
  constexpr int TB = 16, DP = 8 * NR, NT = 512, KQ = TB * DP / NT, VN = TB * 64 / NT;
  __shared__ __attribute__((aligned(16))) float sk[TB * DP], sq[TB * DP];
  __shared__ float sv[TB][64], so[TB][64];
  __shared__ float sg[TB], sb[TB], skn[TB], sqn[TB];
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * 64;
  const int hk = h / (H / G);
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int cl = 8 * w + (lane >> 3), gg = lane & 7;
  const int col = c0 + cl;
  const bool live = col < Dv;
  const int r0 = row_cu[s], r1 = row_cu[s + 1];
  const int slot = state_slots[s];
  if (r1 <= r0) return;
  if (slot < 0) {      // padding sequence of a fixed-shape step: defined output, no state
    for (int i = threadIdx.x; i < (r1 - r0) * 64; i += NT)
      if (c0 + (i & 63) < Dv) o[((long)(r0 + (i >> 6)) * H + h) * Dv + c0 + (i & 63)] = 0.f;
    return;
  }
  float* S = state + (((long)slot * H + h) * Dv + col) * D;      // this lane's column
  const bool vec = (D & 3) == 0;
  float st[NR];
  const bool fresh = positions[r0] == 0;
#pragma unroll
  for (int i4 = 0; i4 < NR / 4; ++i4) {
    const int d = gg * NR + 4 * i4;
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (!fresh && live) {
      if (vec && d + 3 < D) x = *reinterpret_cast<const f32x4*>(S + d);
      else
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = d + j < D ? S[d + j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) st[4 * i4 + j] = x[j];
  }
  const float rate = expf(a_log[h]), dtb = dt_bias[h];
  // the inputs of a block of TB tokens, one slice per thread
  float rk[KQ], rq[KQ], rv[VN], ra = 0.f, rb = 0.f;
  auto fetch = [&](int t0) {
    const int nb = min(TB, r1 - t0);
#pragma unroll
    for (int j = 0; j < KQ; ++j) {
      const int i = threadIdx.x + j * NT, tt = i / DP, d = i - tt * DP;
      const bool ok = tt < nb && d < D;
      const long t = t0 + tt;
      rk[j] = ok ? k[t * k_ld + (long)hk * D + d] : 0.f;
      rq[j] = ok ? q[t * q_ld + (long)hk * D + d] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) {
      const int i = threadIdx.x + j * NT, tt = i >> 6, c = i & 63;
      rv[j] = (tt < nb && c0 + c < Dv) ? v[(long)(t0 + tt) * v_ld + (long)h * Dv + c0 + c] : 0.f;
    }
    if (threadIdx.x < nb) {
      ra = (float)al[(long)(t0 + threadIdx.x) * a_ld + h];
      rb = (float)bl[(long)(t0 + threadIdx.x) * b_ld + h];
    }
  };
  fetch(r0);
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nb = min(TB, r1 - t0);
#pragma unroll
    for (int j = 0; j < KQ; ++j) {
      sk[threadIdx.x + j * NT] = rk[j];
      sq[threadIdx.x + j * NT] = rq[j];
    }
#pragma unroll
    for (int j = 0; j < VN; ++j) sv[(threadIdx.x + j * NT) >> 6][threadIdx.x & 63] = rv[j];
    if (threadIdx.x < nb) {
      const float av = ra + dtb;
      const float sp = av > 20.f ? av : log1pf(expf(av));            // softplus
      sg[threadIdx.x] = expf(-rate * sp);
      sb[threadIdx.x] = 1.f / (1.f + expf(-rb));
    }
    __syncthreads();
    // unit norms: wave w sums the squares of tokens w and w + 8
    for (int tt = w; tt < nb; tt += 8) {
      float a = 0.f, b = 0.f;
      for (int d = lane; d < DP; d += 64) {
        a = fmaf(sk[tt * DP + d], sk[tt * DP + d], a);
        b = fmaf(sq[tt * DP + d], sq[tt * DP + d], b);
      }
      a = wave_sum(a);
      b = wave_sum(b);
      if (lane == 0) {
        skn[tt] = 1.f / sqrtf(a + unit_eps);
        sqn[tt] = q_scale / sqrtf(b + unit_eps);
      }
    }
    __syncthreads();
    if (t0 + TB < r1) fetch(t0 + TB);        // in flight during the token loop
    for (int tt = 0; tt < nb; ++tt) {
      const float vv = sv[tt][cl], g = sg[tt], bt = sb[tt], kn = skn[tt], qn = sqn[tt];
      const f32x4* pk = reinterpret_cast<const f32x4*>(sk + tt * DP + gg * NR);
      const f32x4* pq = reinterpret_cast<const f32x4*>(sq + tt * DP + gg * NR);
      f32x4 kr[NR / 4];
      f32x4 dp = {0.f, 0.f, 0.f, 0.f};      // four partial sums: short dependent chains
#pragma unroll
      for (int i4 = 0; i4 < NR / 4; ++i4) {
        kr[i4] = pk[i4];
#pragma unroll
        for (int j = 0; j < 4; ++j) dp[j] = fmaf(st[4 * i4 + j], kr[i4][j], dp[j]);
      }
      const float dot = sum8((dp[0] + dp[1]) + (dp[2] + dp[3]));
      // the decayed state's read at k is g kn dot; the write is k_unit u^T = k_raw (kn u)
      const float u = bt * (vv - g * (kn * dot));
      const float uk = kn * u;
      f32x4 pp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i4 = 0; i4 < NR / 4; ++i4) {
        const f32x4 q4 = pq[i4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          st[4 * i4 + j] = fmaf(g, st[4 * i4 + j], kr[i4][j] * uk);
          pp[j] = fmaf(q4[j], st[4 * i4 + j], pp[j]);
        }
      }
      const float po = sum8((pp[0] + pp[1]) + (pp[2] + pp[3]));
      if (gg == 0) so[tt][cl] = po * qn;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nb * 64; i += NT) {
      const int tt = i >> 6, c = i & 63;
      if (c0 + c < Dv) o[((long)(t0 + tt) * H + h) * Dv + c0 + c] = so[tt][c];
    }
    // (the next block's staging overwrites sk / sq / sv and the scalars, which every wave finished
    // reading at the barrier above; so is rewritten only after the next block's barriers)
  }
  if (live) {
#pragma unroll
    for (int i4 = 0; i4 < NR / 4; ++i4) {
      const int d = gg * NR + 4 * i4;
      if (vec && d + 3 < D) {
        *reinterpret_cast<f32x4*>(S + d) = f32x4{st[4 * i4], st[4 * i4 + 1], st[4 * i4 + 2], st[4 * i4 + 3]};
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (d + j < D) S[d + j] = st[4 * i4 + j];
      }
    }
  }
}

// threads of a one-row workgroup: about four elements per thread, whole waves, at most 1024
int row_threads(int W) { return std::min(1024, std::max(64, (W / 4 + 63) / 64 * 64)); }

}  // namespace

void launch_post_norm_add_norm(float* x, const void* y, const float* nw, const float* nb, float eps, float mult,
                               const float* extra, const float* nw2, const float* nb2, void* h, int T, int W, bool f32,
                               hipStream_t s) {
  if (T <= 0) return;
  const size_t sm = (size_t)W * sizeof(float);
#define BFLY_PNAN(TT, V)                                                                                          \
  post_norm_add_norm_kernel<TT, V><<<T, row_threads(W), sm, s>>>(x, (const TT*)y, nw, nb, eps, mult, extra, nw2, nb2, \
                                                                 (TT*)h, W)
  if (W % 4 == 0) { if (f32) BFLY_PNAN(float, 4); else BFLY_PNAN(bf16, 4); }
  else { if (f32) BFLY_PNAN(float, 1); else BFLY_PNAN(bf16, 1); }
#undef BFLY_PNAN
}

void launch_short_conv_act(const void* z, long z_ld, const float* w, const float* state, const int* state_slots,
                           const int* row_cu, int nseq, const int* positions, void* out, int T, int C, int taps, int act,
                           bool f32, bool out_f32, hipStream_t s) {
  if (T <= 0 || C <= 0) return;
  const size_t esz = f32 ? 4 : 2;
  if (taps <= 8 && C % 4 == 0 && z_ld % 4 == 0 && reinterpret_cast<uintptr_t>(z) % (4 * esz) == 0 && T >= 64) {
    // rows per workgroup: enough workgroups to fill the chip first
    const int RB = std::min(16, std::max(1, T / 512));
    dim3 g2((T + RB - 1) / RB, (C / 4 + 255) / 256);
#define BFLY_SCR(TI, TO)                                                                                             \
  short_conv_act_rows_kernel<TI, TO><<<g2, 256, 0, s>>>((const TI*)z, z_ld, w, state, state_slots, row_cu, nseq,     \
                                                        positions, (TO*)out, C, taps, act, T, RB)
    if (f32) BFLY_SCR(float, float);
    else if (out_f32) BFLY_SCR(bf16, float);
    else BFLY_SCR(bf16, bf16);
#undef BFLY_SCR
    return;
  }
  dim3 grid(T, (C + 255) / 256);
#define BFLY_SC(TI, TO)                                                                                              \
  short_conv_act_kernel<TI, TO><<<grid, 256, 0, s>>>((const TI*)z, z_ld, w, state, state_slots, row_cu, nseq, positions, \
                                                     (TO*)out, C, taps, act)
  if (f32) BFLY_SC(float, float);
  else if (out_f32) BFLY_SC(bf16, float);
  else BFLY_SC(bf16, bf16);
#undef BFLY_SC
}

void launch_short_conv_state_update(const void* z, long z_ld, float* state, const int* state_slots, const int* row_cu,
                                    int nseq, const int* positions, int C, int n, bool f32, hipStream_t s) {
  if (nseq <= 0 || n <= 0 || C <= 0) return;
  dim3 grid(nseq, (C + 255) / 256);
  if (f32)
    short_conv_state_update_kernel<float><<<grid, 256, 0, s>>>((const float*)z, z_ld, state, state_slots, row_cu,
                                                               positions, C, n);
  else
    short_conv_state_update_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)z, z_ld, state, state_slots, row_cu,
                                                              positions, C, n);
}

template <typename T>
static int delta_scan_t(const float* q, long q_ld, const float* k, long k_ld, const float* v, long v_ld, const T* b,
                        long b_ld, const T* a, long a_ld, const float* a_log, const float* dt_bias, float* state,
                        const int* state_slots, const int* row_cu, int nseq, const int* positions, float q_scale,
                        float unit_eps, float* o, int H, int G, int D, int Dv, hipStream_t s) {
  dim3 grid(nseq, H, (Dv + 63) / 64);
#define BFLY_DELTA(NR)                                                                                             \
  delta_scan_kernel<T, NR><<<grid, 512, 0, s>>>(q, q_ld, k, k_ld, v, v_ld, b, b_ld, a, a_ld, a_log, dt_bias, state, \
                                                state_slots, row_cu, positions, q_scale, unit_eps, o, H, G, D, Dv)
  if (D <= 32) BFLY_DELTA(4);
  else if (D <= 64) BFLY_DELTA(8);
  else if (D <= 128) BFLY_DELTA(16);
  else if (D <= 256) BFLY_DELTA(32);
  else return -1;
#undef BFLY_DELTA
  return 0;
}

int launch_delta_scan(const float* q, long q_ld, const float* k, long k_ld, const float* v, long v_ld, const void* b,
                      long b_ld, const void* a, long a_ld, const float* a_log, const float* dt_bias, float* state,
                      const int* state_slots, const int* row_cu, int nseq, const int* positions, float q_scale,
                      float unit_eps, float* o, int T, int H, int G, int D, int Dv, bool f32, hipStream_t s) {
  if (T <= 0 || nseq <= 0) return 0;
  if (f32)
    return delta_scan_t<float>(q, q_ld, k, k_ld, v, v_ld, (const float*)b, b_ld, (const float*)a, a_ld, a_log, dt_bias,
                               state, state_slots, row_cu, nseq, positions, q_scale, unit_eps, o, H, G, D, Dv, s);
  return delta_scan_t<bf16>(q, q_ld, k, k_ld, v, v_ld, (const bf16*)b, b_ld, (const bf16*)a, a_ld, a_log, dt_bias, state,
                            state_slots, row_cu, nseq, positions, q_scale, unit_eps, o, H, G, D, Dv, s);
}

}  // namespace bfly
