// Parallel layers with a token shift, per-head normed and half-rotated queries / keys with the
// paged append, the combination of differential attention maps, and the dense clamped GLU.
//   par_norm_shift_kernel   x' = x + (ya + yb); both sublayer inputs from one RMS statistic of x'
//                           (two weights stored around zero); the mixer's input is mixed with the
//                           previous token's (h + (h_prev - h) shift), whose last value per sequence
//                           lives in a pooled f32 state
//   par_final_kernel        the last layer's sum and the output norm of the rows that are asked for
//   qk_norm_rope_kv_kernel  RMS norm per head, rotation of dimension i with i + n, padded query
//                           copy, K rows and transposed V rows into the paged caches
//   diff_combine_kernel     a1 - lambda a2, unit RMS per head, constant factor, sigmoid gate
//   glu_clamp_kernel        min(g, L) sigmoid(alpha min(g, L)) (clamp(u, +-L) + offset)
// One workgroup per token row (one wave per head where heads are independent). The residual, the
// statistics, the state, angles and the combination are f32 whatever the activation type.
#include <algorithm>

#include "bfly_common.h"
#include "bfly_parlayer.h"

namespace bfly {

namespace {

// sum of squares of row r of x + (ya + yb), over the workgroup
template <typename T>
__device__ __forceinline__ float row_sumsq(const float* __restrict__ x, const T* __restrict__ ya,
                                           const T* __restrict__ yb, long r, int W, float* red) {
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = x[r * W + c];
    if (ya || yb) v += (ya ? (float)ya[r * W + c] : 0.f) + (yb ? (float)yb[r * W + c] : 0.f);
    ss = fmaf(v, v, ss);
  }
  return block_sum(ss, red);
}

template <typename T>
__device__ __forceinline__ float row_val(const float* __restrict__ x, const T* __restrict__ ya,
                                         const T* __restrict__ yb, long r, int W, int c) {
  float v = x[r * W + c];
  if (ya || yb) v += (ya ? (float)ya[r * W + c] : 0.f) + (yb ? (float)yb[r * W + c] : 0.f);
  return v;
}

// A row's workgroup recomputes the statistic of row t - 1 (and, for a sequence's first row of the
// step, of its last row, whose normed value it stores as the new state after it has read the old
// one): every value is derived from x, ya, yb alone, by the same operations in the same order, so
// the copies agree bit for bit and no workgroup reads what another one writes.
template <typename T>
__global__ __launch_bounds__(256) void par_norm_shift_kernel(const float* __restrict__ x, const T* __restrict__ ya,
                                                             const T* __restrict__ yb, float* __restrict__ x_out,
                                                             const float* __restrict__ norm_a,
                                                             const float* __restrict__ norm_b, float eps, float offset,
                                                             const float* __restrict__ shift, float* __restrict__ state,
                                                             const int* __restrict__ state_slots,
                                                             const int* __restrict__ row_seq,
                                                             const int* __restrict__ row_cu,
                                                             const int* __restrict__ positions, T* __restrict__ ha,
                                                             T* __restrict__ hb, int W) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int s = row_seq[t];
  if (s < 0) {          // padding row of a fixed-shape step
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      ha[t * W + c] = (T)0.f;
      if (hb) hb[t * W + c] = (T)0.f;
      if (x_out) x_out[t * W + c] = 0.f;
    }
    return;
  }
  const float invW = 1.f / (float)W;
  const float r = 1.f / sqrtf(row_sumsq(x, ya, yb, t, W, red) * invW + eps);
  const long a = row_cu[s], e = (long)row_cu[s + 1] - 1;
  const int slot = (shift && state_slots) ? state_slots[s] : -1;
  // where the previous token's value comes from: 1 the row before, 2 the state, 0 nothing
  const int src = !shift ? 0 : (t > a ? 1 : ((positions[t] > 0 && slot >= 0) ? 2 : 0));
  float rp = 0.f;
  if (src == 1) rp = 1.f / sqrtf(row_sumsq(x, ya, yb, t - 1, W, red) * invW + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = row_val(x, ya, yb, t, W, c);
    if (x_out) x_out[t * W + c] = v;
    const float n = v * r;
    float h = n * (norm_a[c] + offset);
    if (hb) hb[t * W + c] = (T)(n * (norm_b[c] + offset));
    if (shift) {
      float prev = 0.f;
      if (src == 1) prev = row_val(x, ya, yb, t - 1, W, c) * rp * (norm_a[c] + offset);
      else if (src == 2) prev = state[(long)slot * W + c];
      if (t == a && t == e && slot >= 0) state[(long)slot * W + c] = h;
      h = h + (prev - h) * shift[c];
    }
    ha[t * W + c] = (T)h;
  }
  if (shift && t == a && e > a && slot >= 0) {
    // (this thread read state[slot][c] above, for the same columns c it writes here)
    const float re = 1.f / sqrtf(row_sumsq(x, ya, yb, e, W, red) * invW + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x)
      state[(long)slot * W + c] = row_val(x, ya, yb, e, W, c) * re * (norm_a[c] + offset);
  }
}

// Four consecutive elements of a row as floats.
__device__ __forceinline__ f32x4 ld4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 ld4(const bf16* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void st4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void st4(bf16* p, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

// Row r of x + (ya + yb) into registers, VPT groups of four columns per thread (group k of thread
// i: columns 4 (i + 256 k) ...); returns the row's sum of squares over the workgroup. Every user
// sums in this one order, so the copies of a row's statistic agree bit for bit.
template <typename T, int VPT>
__device__ __forceinline__ float row_load4(const float* __restrict__ x, const T* __restrict__ ya,
                                           const T* __restrict__ yb, long r, int W, f32x4 (&v)[VPT], float* red) {
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int c = 4 * (threadIdx.x + 256 * k);
    v[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < W) {
      v[k] = ld4(x + r * W + c);
      if (ya || yb) {
        const f32x4 a = ya ? ld4(ya + r * W + c) : f32x4{0.f, 0.f, 0.f, 0.f};
        const f32x4 b = yb ? ld4(yb + r * W + c) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) v[k][i] += a[i] + b[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) ss = fmaf(v[k][i], v[k][i], ss);
  }
  return block_sum(ss, red);
}

// par_norm_shift_kernel for rows of W % 4 == 0, W <= 1024 VPT columns: each row is read once into
// registers with 16-byte (f32) / 8-byte (bf16) accesses.
template <typename T, int VPT>
__global__ __launch_bounds__(256) void par_norm_shift_vec_kernel(
    const float* __restrict__ x, const T* __restrict__ ya, const T* __restrict__ yb, float* __restrict__ x_out,
    const float* __restrict__ norm_a, const float* __restrict__ norm_b, float eps, float offset,
    const float* __restrict__ shift, float* __restrict__ state, const int* __restrict__ state_slots,
    const int* __restrict__ row_seq, const int* __restrict__ row_cu, const int* __restrict__ positions,
    T* __restrict__ ha, T* __restrict__ hb, int W) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const int s = row_seq[t];
  const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
  if (s < 0) {          // padding row of a fixed-shape step
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int c = 4 * (threadIdx.x + 256 * k);
      if (c >= W) continue;
      st4(ha + t * W + c, zero);
      if (hb) st4(hb + t * W + c, zero);
      if (x_out) st4(x_out + t * W + c, zero);
    }
    return;
  }
  const float invW = 1.f / (float)W;
  f32x4 v[VPT], pv[VPT];
  const float r = 1.f / sqrtf(row_load4<T, VPT>(x, ya, yb, t, W, v, red) * invW + eps);
  const long a = row_cu[s], e = (long)row_cu[s + 1] - 1;
  const int slot = (shift && state_slots) ? state_slots[s] : -1;
  const int src = !shift ? 0 : (t > a ? 1 : ((positions[t] > 0 && slot >= 0) ? 2 : 0));
  float rp = 0.f;
  if (src == 1) rp = 1.f / sqrtf(row_load4<T, VPT>(x, ya, yb, t - 1, W, pv, red) * invW + eps);
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int c = 4 * (threadIdx.x + 256 * k);
    if (c >= W) continue;
    if (x_out) st4(x_out + t * W + c, v[k]);
    const f32x4 wa = ld4(norm_a + c);
    f32x4 h, o;
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = v[k][i] * r * (wa[i] + offset);
    if (hb) {
      const f32x4 wb = ld4(norm_b + c);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = v[k][i] * r * (wb[i] + offset);
      st4(hb + t * W + c, o);
    }
    if (shift) {
      f32x4 prev = zero;
      if (src == 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) prev[i] = pv[k][i] * rp * (wa[i] + offset);
      } else if (src == 2) {
        prev = ld4(state + (long)slot * W + c);
      }
      if (t == a && t == e && slot >= 0) st4(state + (long)slot * W + c, h);
      const f32x4 sh = ld4(shift + c);
#pragma unroll
      for (int i = 0; i < 4; ++i) h[i] = h[i] + (prev[i] - h[i]) * sh[i];
    }
    st4(ha + t * W + c, h);
  }
  if (shift && t == a && e > a && slot >= 0) {
    // (this thread read state[slot] above, for the same columns it writes here)
    const float re = 1.f / sqrtf(row_load4<T, VPT>(x, ya, yb, e, W, pv, red) * invW + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      const int c = 4 * (threadIdx.x + 256 * k);
      if (c >= W) continue;
      const f32x4 wa = ld4(norm_a + c);
      f32x4 h;
#pragma unroll
      for (int i = 0; i < 4; ++i) h[i] = pv[k][i] * re * (wa[i] + offset);
      st4(state + (long)slot * W + c, h);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void par_final_kernel(const float* __restrict__ x, const T* __restrict__ ya,
                                                        const T* __restrict__ yb, const float* __restrict__ norm_w,
                                                        float eps, float offset, const long* __restrict__ idx,
                                                        T* __restrict__ out, int W) {
  __shared__ float red[16];
  const long i = blockIdx.x;
  const long t = idx ? idx[i] : i;
  const float r = 1.f / sqrtf(row_sumsq(x, ya, yb, t, W, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    out[i * W + c] = (T)(row_val(x, ya, yb, t, W, c) * r * (norm_w[c] + offset));
}

constexpr int kMaxHeadLane = 8;      // head sizes up to 512

// cs[t][0][f] = cos(positions[t] * inv_freq[f]), cs[t][1][f] = sin(...): the f32 frequencies, the
// product and the evaluation in f64. Once per step and rotation (every layer that shares the
// frequencies reads the same table).
__global__ void rope_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq, int nrot,
                                  float* __restrict__ cs, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / nrot;
  const int f = (int)(i % nrot);
  double sd, cd;
  sincos((double)positions[t] * (double)inv_freq[f], &sd, &cd);
  cs[(t * 2) * nrot + f] = (float)cd;
  cs[(t * 2 + 1) * nrot + f] = (float)sd;
}

// One workgroup per (token, group of 4 HPW heads), HPW heads per wave: the query heads, then the key
// heads; the workgroups of a token share the copy of its value rows. A head is normed in registers
// (lane l owns dims l, l + 64, ...: NL per lane), staged in LDS so that a rotated dimension finds its
// partner, and leaves rotated. A wave's HPW heads go through each phase together (all loads, all
// reductions, all hand-overs, all stores), so their latencies overlap: large steps take HPW = 4,
// steps of few rows HPW = 1 (more workgroups).
template <typename T, int HPW, int NL>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_kernel(const T* __restrict__ q, long q_ld, const T* __restrict__ k,
                                                              long k_ld, const T* __restrict__ v, long v_ld,
                                                              const float* __restrict__ qn_w,
                                                              const float* __restrict__ kn_w, float eps,
                                                              const float* __restrict__ cs, int nrot,
                                                              const int* __restrict__ slots, T* __restrict__ q_out,
                                                              T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq,
                                                              int Gk, int Gv, int D, int Dp, int Dv, int Dvp, int bs) {
  extern __shared__ float smem[];        // head staging [4][HPW][D]
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* scos = cs + t * 2 * nrot;       // the token's row of the step's rotation table
  const float* ssin = scos + nrot;
  const int slot = slots ? slots[t] : -1;
  const long blk = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  // q_out == nullptr: the queries need nothing (no norm, no rotation, no padding); key heads only
  const int h0 = 4 * HPW * blockIdx.y + wave + (q_out ? 0 : Hq);
  float val[HPW][NL];
  bool on[HPW];
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const int hh = h0 + 4 * u;
    on[u] = hh < Hq + Gk && (hh < Hq || slot >= 0);
    const T* src = hh < Hq ? q + t * q_ld + (long)hh * D : k + t * k_ld + (long)(hh - Hq) * D;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int d = lane + 64 * i;
      val[u][i] = (on[u] && d < D) ? (float)src[d] : 0.f;
    }
  }
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    const float* nw = h0 + 4 * u < Hq ? qn_w : kn_w;
    if (!nw || !on[u]) continue;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NL; ++i) ss = fmaf(val[u][i], val[u][i], ss);
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int d = lane + 64 * i;
      if (d < D) val[u][i] = val[u][i] * r * nw[d];
    }
  }
  if (nrot > 0) {
#pragma unroll
    for (int u = 0; u < HPW; ++u) {
      float* sh = smem + (long)(wave * HPW + u) * D;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int d = lane + 64 * i;
        if (d < D) sh[d] = val[u][i];
      }
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int d = lane + 64 * i;
      if (d < 2 * nrot) {
        const int f = d < nrot ? d : d - nrot;
        const float c = scos[f], sn = ssin[f];
#pragma unroll
        for (int u = 0; u < HPW; ++u) {
          const float* sh = smem + (long)(wave * HPW + u) * D;
          // pair (a, b) = dims (f, f + nrot): a' = a c - b s, b' = b c + a s
          val[u][i] = d < nrot ? val[u][i] * c - sh[d + nrot] * sn : val[u][i] * c + sh[d - nrot] * sn;
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < HPW; ++u) {
    if (!on[u]) continue;
    const int hh = h0 + 4 * u;
    if (hh < Hq) {
      T* dst = q_out + (t * Hq + hh) * Dp;
      for (int d = lane; d < Dp; d += 64) {       // (the padding past 64 NL stays in this loop's zero branch)
        float x = 0.f;
#pragma unroll
        for (int i = 0; i < NL; ++i)
          if (d == lane + 64 * i) x = val[u][i];
        dst[d] = (T)(d < D ? x : 0.f);
      }
    } else {
      T* dst = k_cache + ((blk * Gk + (hh - Hq)) * bs + off) * Dp;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int d = lane + 64 * i;
        if (d < D) dst[d] = (T)val[u][i];
      }
    }
  }
  if (slot < 0) return;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < Gv * Dv; i += gridDim.y * blockDim.x) {
    const int g = i / Dv, d = i % Dv;
    v_cache[((blk * Gv + g) * Dvp + d) * bs + off] = v[t * v_ld + i];
  }
}

// One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const float* __restrict__ a, float lam, float eps,
                                                          float out_mul, const T* __restrict__ gate, long gate_ld,
                                                          T* __restrict__ out, int H, int Dv, int Dvp) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* a1 = a + (t * 2 * H + 2 * h) * Dvp;
  const float* a2 = a1 + Dvp;
  float o[kMaxHeadLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxHeadLane; ++i) {
    const int d = lane + 64 * i;
    o[i] = d < Dv ? a1[d] - lam * a2[d] : 0.f;
    ss = fmaf(o[i], o[i], ss);
  }
  const float r = out_mul / sqrtf(wave_sum(ss) / (float)Dv + eps);
#pragma unroll
  for (int i = 0; i < kMaxHeadLane; ++i) {
    const int d = lane + 64 * i;
    if (d < Dv) {
      float y = o[i] * r;
      if (gate) y *= 1.f / (1.f + expf(-(float)gate[t * gate_ld + (long)h * Dv + d]));
      out[(t * H + h) * Dv + d] = (T)y;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void glu_clamp_kernel(const T* __restrict__ gu, long gu_ld, float limit, float alpha,
                                                        float up_offset, T* __restrict__ out, long n, int F,
                                                        int group) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long t = i / F;
    const int f = (int)(i % F);
    const int cg = group > 0 ? (f / group) * 2 * group + f % group : f;       // the gate's column
    const int cu = group > 0 ? cg + group : F + f;
    const float g = fminf((float)gu[t * gu_ld + cg], limit);
    const float u = fminf(fmaxf((float)gu[t * gu_ld + cu], -limit), limit);
    out[i] = (T)(g / (1.f + expf(-alpha * g)) * (u + up_offset));
  }
}

}  // namespace

void launch_par_norm_shift(const float* x, const void* ya, const void* yb, float* x_out, const float* norm_a,
                           const float* norm_b, float eps, float offset, const float* shift, float* state,
                           const int* state_slots, const int* row_seq, const int* row_cu, const int* positions,
                           void* ha, void* hb, int T, int W, bool f32, hipStream_t s) {
  if (T <= 0) return;
  const auto al = [](const void* p, size_t n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0; };
  const size_t ea = f32 ? 16 : 8;
  if (W % 4 == 0 && W <= 8192 && al(x, 16) && al(x_out, 16) && al(norm_a, 16) && al(norm_b, 16) && al(shift, 16) &&
      al(state, 16) && al(ya, ea) && al(yb, ea) && al(ha, ea) && al(hb, ea)) {
#define BFLY_PNS(TT, V)                                                                                          \
  par_norm_shift_vec_kernel<TT, V><<<T, 256, 0, s>>>(x, (const TT*)ya, (const TT*)yb, x_out, norm_a, norm_b, eps,   \
                                                    offset, shift, state, state_slots, row_seq, row_cu, positions, \
                                                    (TT*)ha, (TT*)hb, W)
#define BFLY_PNSV(TT)                \
  if (W <= 1024) BFLY_PNS(TT, 1);    \
  else if (W <= 2048) BFLY_PNS(TT, 2); \
  else if (W <= 4096) BFLY_PNS(TT, 4); \
  else BFLY_PNS(TT, 8)
    if (f32) { BFLY_PNSV(float); } else { BFLY_PNSV(bf16); }
#undef BFLY_PNSV
#undef BFLY_PNS
    return;
  }
  if (f32)
    par_norm_shift_kernel<float><<<T, 256, 0, s>>>(x, (const float*)ya, (const float*)yb, x_out, norm_a, norm_b, eps,
                                                   offset, shift, state, state_slots, row_seq, row_cu, positions,
                                                   (float*)ha, (float*)hb, W);
  else
    par_norm_shift_kernel<bf16><<<T, 256, 0, s>>>(x, (const bf16*)ya, (const bf16*)yb, x_out, norm_a, norm_b, eps,
                                                  offset, shift, state, state_slots, row_seq, row_cu, positions,
                                                  (bf16*)ha, (bf16*)hb, W);
}

void launch_par_final(const float* x, const void* ya, const void* yb, const float* norm_w, float eps, float offset,
                      const long* idx, void* out, int R, int W, bool f32, hipStream_t s) {
  if (R <= 0) return;
  if (f32)
    par_final_kernel<float><<<R, 256, 0, s>>>(x, (const float*)ya, (const float*)yb, norm_w, eps, offset, idx,
                                              (float*)out, W);
  else
    par_final_kernel<bf16><<<R, 256, 0, s>>>(x, (const bf16*)ya, (const bf16*)yb, norm_w, eps, offset, idx, (bf16*)out,
                                             W);
}

template <typename T>
static void qk_launch(const T* q, long q_ld, const T* k, long k_ld, const T* v, long v_ld, const float* qn_w,
                      const float* kn_w, float eps, const float* cs, int nrot, const int* slots, T* q_out, T* k_cache,
                      T* v_cache, int Tn, int Hq, int Gk, int Gv, int D, int Dp, int Dv, int Dvp, int bs, hipStream_t s) {
  const int heads = (q_out ? Hq : 0) + Gk;
  const bool big = (long)Tn * heads >= 4096;       // enough waves either way: several heads per wave
  const int hpw = big ? 4 : 1;
  const dim3 grid(Tn, (heads + 4 * hpw - 1) / (4 * hpw));
  const size_t sm = (size_t)(4 * hpw * D) * sizeof(float);
#define BFLY_QK(HPW, NL)                                                                                          \
  qk_norm_rope_kv_kernel<T, HPW, NL><<<grid, 256, sm, s>>>(q, q_ld, k, k_ld, v, v_ld, qn_w, kn_w, eps, cs, nrot, slots, \
                                                          q_out, k_cache, v_cache, Hq, Gk, Gv, D, Dp, Dv, Dvp, bs)
#define BFLY_QKN(HPW)              \
  if (D <= 64) BFLY_QK(HPW, 1);    \
  else if (D <= 128) BFLY_QK(HPW, 2); \
  else if (D <= 256) BFLY_QK(HPW, 4); \
  else BFLY_QK(HPW, 8)
  if (big) { BFLY_QKN(4); } else { BFLY_QKN(1); }
#undef BFLY_QKN
#undef BFLY_QK
}

void launch_qk_norm_rope_kv(const void* q, long q_ld, const void* k, long k_ld, const void* v, long v_ld,
                            const float* qn_w, const float* kn_w, float eps, const float* cs, int nrot,
                            const int* slots, void* q_out, void* k_cache,
                            void* v_cache, int T, int Hq, int Gk, int Gv, int D, int Dp, int Dv, int Dvp, int block_size,
                            bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    qk_launch<float>((const float*)q, q_ld, (const float*)k, k_ld, (const float*)v, v_ld, qn_w, kn_w, eps, cs, nrot, slots,
                     (float*)q_out, (float*)k_cache, (float*)v_cache, T, Hq, Gk, Gv, D, Dp, Dv, Dvp, block_size, s);
  else
    qk_launch<bf16>((const bf16*)q, q_ld, (const bf16*)k, k_ld, (const bf16*)v, v_ld, qn_w, kn_w, eps, cs, nrot, slots,
                    (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, T, Hq, Gk, Gv, D, Dp, Dv, Dvp, block_size, s);
}

void launch_rope_table(const int* positions, const float* inv_freq, int nrot, float* cs, int T, hipStream_t s) {
  const long n = (long)T * nrot;
  if (n <= 0) return;
  rope_table_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(positions, inv_freq, nrot, cs, n);
}

void launch_diff_combine(const float* a, float lam, float eps, float out_mul, const void* gate, long gate_ld,
                         void* out, int T, int H, int Dv, int Dvp, bool f32, hipStream_t s) {
  if (T <= 0) return;
  dim3 grid(T, H);
  if (f32)
    diff_combine_kernel<float><<<grid, 64, 0, s>>>(a, lam, eps, out_mul, (const float*)gate, gate_ld, (float*)out, H, Dv,
                                                   Dvp);
  else
    diff_combine_kernel<bf16><<<grid, 64, 0, s>>>(a, lam, eps, out_mul, (const bf16*)gate, gate_ld, (bf16*)out, H, Dv,
                                                  Dvp);
}

void launch_glu_clamp(const void* gu, long gu_ld, float limit, float alpha, float up_offset, void* out, int T, int F,
                      int group, bool f32, hipStream_t s) {
  const long n = (long)T * F;
  if (n <= 0) return;
  const unsigned grid = (unsigned)std::min<long>((n + 255) / 256, 65536);
  if (f32)
    glu_clamp_kernel<float><<<grid, 256, 0, s>>>((const float*)gu, gu_ld, limit, alpha, up_offset, (float*)out, n, F,
                                                 group);
  else
    glu_clamp_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)gu, gu_ld, limit, alpha, up_offset, (bf16*)out, n, F, group);
}

}  // namespace bfly
