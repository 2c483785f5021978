// Shape-generic GEMM family: any (M, N, K), bf16 or f32 operands, f32 accumulation in K order
// (the sum of an output element never depends on M or on the other rows of the batch).
// 64 x 64 output tile and 256 threads in both forms, operands staged through LDS with bounds
// checks, so no shape or alignment restriction. f32 operands: 16-deep K step, a 4 x 4 register
// block per thread on the VALU. bf16 operands: 64-deep K step staged as bf16, a 32 x 32 quadrant
// per wave as 2 x 2 MFMA 16x16x32 tiles (tile_mac_mfma below).
// The same tile core serves the plain projection (bias / squared-ReLU epilogues) and the two
// grouped expert GEMMs of a score-routed MoE with clamped GLU experts: rows are grouped by
// expert (moe_sort_kernel), the up kernel gathers token rows scaled by their routing score and
// applies the GLU to a (gate, up) accumulator pair, the down kernel scatters f32 rows back to
// (token, choice) order for a fixed-order sum.
#include <algorithm>

#include "bfly_common.h"
#include "bfly_mixers.h"

namespace bfly {

namespace {

constexpr int TM = 64, TN = 64, TK = 16, LDP = TM + 4;

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ T cvt(float v) { return (T)v; }

// epilogue activations: squared ReLU; xIELU with coefficients (a0, a1): v > 0: a0 v^2 + v / 2,
// else a1 (exp(v) - 1 - v) + v / 2
__device__ __forceinline__ float apply_act(float v, int act, float a0, float a1) {
  if (act == ACT_RELU2) { v = fmaxf(v, 0.f); return v * v; }
  if (act == ACT_XIELU) return v > 0.f ? fmaf(a0 * v, v, 0.5f * v) : fmaf(a1, expm1f(v) - v, 0.5f * v);
  return v;
}

// acc[i][j] += sum_k A(row0 + ty*4 + i, k) * B(col0 + tx*4 + j, k); la(r, k) / lb(c, k) return
// the operand element as float (0 outside the problem).
template <typename LA, typename LB>
__device__ __forceinline__ void tile_mac(float (&acc)[4][4], LA la, LB lb, int K, float (*As)[LDP], float (*Bs)[LDP]) {
  const int tid = threadIdx.x;
  const int lr = tid >> 2, lk = (tid & 3) * 4;      // staging: row lr, k lk..lk+3
  const int ty = tid >> 4, tx = tid & 15;
  for (int k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lr] = la(lr, k0 + lk + i);
      Bs[lk + i][lr] = lb(lr, k0 + lk + i);
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
}

template <typename T, typename TO>
__global__ __launch_bounds__(256) void gemm_any_kernel(const T* __restrict__ x, long ldx, const T* __restrict__ w,
                                                       long ldw, const T* __restrict__ bias, TO* __restrict__ out,
                                                       long ldo, int M, int N, int K, int act, float a0, float a1,
                                                       long bx, long bw, long bo) {
  __shared__ float As[TK][LDP], Bs[TK][LDP];
  const int row0 = blockIdx.y * TM, col0 = blockIdx.x * TN;
  x += blockIdx.z * bx;            // batched form: one problem per blockIdx.z (e.g. per head)
  w += blockIdx.z * bw;
  out += blockIdx.z * bo;
  float acc[4][4] = {};
  tile_mac(
      acc,
      [&](int r, int k) { return (row0 + r < M && k < K) ? ldf(x + (long)(row0 + r) * ldx + k) : 0.f; },
      [&](int c, int k) { return (col0 + c < N && k < K) ? ldf(w + (long)(col0 + c) * ldw + k) : 0.f; }, K, As, Bs);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c >= N) continue;
      float v = acc[i][j];
      if (bias) v += ldf(bias + c);
      out[(long)r * ldo + c] = cvt<TO>(apply_act(v, act, a0, a1));
    }
  }
}

template <typename T>
__global__ void act_kernel(T* x, long n, int act, float a0, float a1) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    x[i] = (T)apply_act((float)x[i], act, a0, a1);
}

// One workgroup. counts -> offsets -> placement (order inside an expert's group is arbitrary:
// every grouped row is computed on its own and lands at its pair index) -> list of tile_rows-row
// tiles.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int TKp, int E,
                                                        int* __restrict__ perm, int* __restrict__ offsets,
                                                        int* __restrict__ tiles, int* __restrict__ ntiles,
                                                        int tile_rows) {
  __shared__ int cnt[1025], cur[1024];
  for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < TKp; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cnt[e];
      offsets[e] = run;
      cur[e] = run;
      for (int r = 0; r < c; r += tile_rows) {
        tiles[2 * nt] = e;
        tiles[2 * nt + 1] = run + r;
        ++nt;
      }
      run += c;
    }
    offsets[E] = run;
    ntiles[0] = nt;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < TKp; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) perm[atomicAdd(&cur[e], 1)] = i;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_glu_up_kernel(const T* __restrict__ x, long ldx,
                                                         const float* __restrict__ topk_w, int Kc,
                                                         const int* __restrict__ perm, const int* __restrict__ offsets_e,
                                                         const int* __restrict__ tiles, const int* __restrict__ ntiles,
                                                         const T* __restrict__ gu_w, float limit, float alpha,
                                                         float up_offset, T* __restrict__ hmid, int Hd, int F,
                                                         int plain) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  __shared__ float As[TK][LDP], Bs[TK][LDP];
  __shared__ int tok[TM];
  __shared__ float wt[TM];
  const int e = tiles[2 * blockIdx.y], r0 = tiles[2 * blockIdx.y + 1];
  const int rend = offsets_e[e + 1];
  const int col0 = blockIdx.x * TN;
  if (threadIdx.x < TM) {
    const int r = r0 + threadIdx.x;
    int p = r < rend ? perm[r] : -1;
    tok[threadIdx.x] = p < 0 ? -1 : p / Kc;
    wt[threadIdx.x] = p < 0 ? 0.f : (topk_w ? topk_w[p] : 1.f);      // no scores: the row as it is
  }
  __syncthreads();
  // plain experts (no gate): F rows per expert, hmid = act(W x)
  const T* wg = gu_w + (long)e * (plain ? 1 : 2) * F * Hd;
  const T* wu = wg + (long)F * Hd;
  // the expert's input is the token row times its routing score, rounded to the activation type
  auto la = [&](int r, int k) {
    const int t = tok[r];
    return (t >= 0 && k < Hd) ? (float)cvt<T>(ldf(x + (long)t * ldx + k) * wt[r]) : 0.f;
  };
  float g[4][4] = {}, u[4][4] = {};
  tile_mac(g, la, [&](int c, int k) { return (col0 + c < F && k < Hd) ? ldf(wg + (long)(col0 + c) * Hd + k) : 0.f; },
           Hd, As, Bs);
  if (!plain)
    tile_mac(u, la, [&](int c, int k) { return (col0 + c < F && k < Hd) ? ldf(wu + (long)(col0 + c) * Hd + k) : 0.f; },
             Hd, As, Bs);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty * 4 + i;
    if (r >= rend) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c >= F) continue;
      if (plain) {
        hmid[(long)r * F + c] = cvt<T>(apply_act(g[i][j], plain, 0.f, 0.f));
        continue;
      }
      const float gg = fminf(g[i][j], limit);
      const float uu = fminf(fmaxf(u[i][j], -limit), limit);
      const float y = gg / (1.f + expf(-alpha * gg)) * (uu + up_offset);
      hmid[(long)r * F + c] = cvt<T>(y);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ hmid, const int* __restrict__ perm,
                                                       const int* __restrict__ offsets_e,
                                                       const int* __restrict__ tiles, const int* __restrict__ ntiles,
                                                       const T* __restrict__ down_w, float* __restrict__ y, int Hd,
                                                       int F) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  __shared__ float As[TK][LDP], Bs[TK][LDP];
  const int e = tiles[2 * blockIdx.y], r0 = tiles[2 * blockIdx.y + 1];
  const int rend = offsets_e[e + 1];
  const int col0 = blockIdx.x * TN;
  const T* wd = down_w + (long)e * Hd * F;
  float acc[4][4] = {};
  tile_mac(
      acc, [&](int r, int k) { return (r0 + r < rend && k < F) ? ldf(hmid + (long)(r0 + r) * F + k) : 0.f; },
      [&](int c, int k) { return (col0 + c < Hd && k < F) ? ldf(wd + (long)(col0 + c) * F + k) : 0.f; }, F, As, Bs);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty * 4 + i;
    if (r >= rend) continue;
    const long p = perm[r];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < Hd) y[p * Hd + c] = acc[i][j];
    }
  }
}

template <typename T>
__global__ void moe_sum_kernel(const float* __restrict__ y, const float* __restrict__ wts, int Kc, T* __restrict__ out,
                               long T_, int Hd) {
  const long n = T_ * Hd;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long t = i / Hd;
    const int c = (int)(i % Hd);
    float s = 0.f;
    if (wts) {
      for (int j = 0; j < Kc; ++j) s = fmaf(wts[t * Kc + j], y[(t * Kc + j) * Hd + c], s);
    } else {
      for (int j = 0; j < Kc; ++j) s += y[(t * Kc + j) * Hd + c];
    }
    out[i] = (T)s;
  }
}

// Router logits of a small step (a few rows): one wave per (token, expert), lanes split the
// hidden dim, f32 accumulation. Large steps use the f32-output GEMM instead.
template <typename T>
__global__ __launch_bounds__(256) void router_logits_kernel(const T* __restrict__ x, long ldx,
                                                            const T* __restrict__ wr, float* __restrict__ logits,
                                                            int E, int Hd) {
  const int t = blockIdx.x, e = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (e >= E) return;
  const T* xr = x + (long)t * ldx;
  const T* w = wr + (long)e * Hd;
  float a = 0.f;
  for (int k = lane; k < Hd; k += 64) a = fmaf(ldf(xr + k), ldf(w + k), a);
  a = wave_sum(a);
  if (lane == 0) logits[(long)t * E + e] = a;
}

// Router choice of one token per wave from its f32 logits [E]: softmax or sigmoid scores, K rounds
// of arg-max over the experts (ties to the lowest id).
__global__ __launch_bounds__(64) void moe_topk_scores_kernel(const float* __restrict__ logits,
                                                             const float* __restrict__ bias, int top_k, int scoring,
                                                             int renorm, int* __restrict__ ids, float* __restrict__ w,
                                                             int E, const float* __restrict__ sel) {
  __shared__ float sc[1024], raw[1024];
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) sc[e] = logits[(long)t * E + e] + (bias ? bias[e] : 0.f);
  __syncthreads();
  if (scoring == 0) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, sc[e]);
    mx = wave_max(mx);
    float den = 0.f;
    for (int e = lane; e < E; e += 64) den += expf(sc[e] - mx);
    den = wave_sum(den);
    __syncthreads();
    for (int e = lane; e < E; e += 64) sc[e] = expf(sc[e] - mx) / den;
  } else {
    for (int e = lane; e < E; e += 64) sc[e] = 1.f / (1.f + expf(-sc[e]));
  }
  __syncthreads();
  if (sel) {      // the choice is made among score + sel; the weight is the plain score
    for (int e = lane; e < E; e += 64) {
      raw[e] = sc[e];
      sc[e] += sel[e];
    }
    __syncthreads();
  }
  float sum = 0.f;
  for (int k = 0; k < top_k; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > bv) { bv = v; bi = e; }      // ascending e: the first maximum wins inside a lane
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (sel && bi < E) bv = raw[bi];
    sum += bv;
    if (lane == 0) {      // (a row of NaN scores selects nothing: id -1)
      const bool ok = bi < E;
      ids[(long)t * top_k + k] = ok ? bi : -1;
      w[(long)t * top_k + k] = ok ? bv : 0.f;
      if (ok) sc[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (renorm && lane == 0)
    for (int k = 0; k < top_k; ++k) w[(long)t * top_k + k] /= sum;
}

// ---------------------------------------------------------------------------------------
// bf16 tile core on the matrix pipe: the same 64 x 64 output tile and the same callers, but the
// operands are staged as bf16 (64-deep K step, 16-byte row segments, zero filled outside the
// problem) and each of the 4 waves owns a 32 x 32 quadrant as 2 x 2 MFMA 16x16x32 tiles. The K
// steps are accumulated in order, so a row's result does not depend on the rest of the batch.
// ---------------------------------------------------------------------------------------
constexpr int MK = 64, MLD = MK + 8;      // LDS row pitch 144 B: 16-byte aligned, off the bank stride

struct RowRef {
  const bf16* p;   // nullptr: a row of zeros
  float s;         // the row is multiplied by s and rounded to bf16 (1: as stored)
};

__device__ __forceinline__ bf16x8 load_row8(const RowRef r, int k, int K) {
  bf16x8 v;
  if (r.p == nullptr || k >= K) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16)0.f;
    return v;
  }
  if (k + 8 <= K && (reinterpret_cast<uintptr_t>(r.p + k) & 15) == 0) {
    v = *reinterpret_cast<const bf16x8*>(r.p + k);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (k + j < K) ? r.p[k + j] : (bf16)0.f;
  }
  if (r.s != 1.f) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16)((float)v[j] * r.s);
  }
  return v;
}

// acc[tn][tm][i] += sum_k X(m, k) W(n, k) over a (32 WT) x (32 WT) workgroup tile (WT = 2: 64 x 64,
// WT = 4: 128 x 128 for large row counts). Wave quadrant: m = 16 WT * (wave >> 1) + 16 tm +
// (lane & 15), n = 16 WT * (wave & 1) + 16 tn + 4 * (lane >> 4) + i; rowX(r) / rowW(c) give the
// r-th X row / c-th W row of the tile.
// Workgroup barrier that orders LDS traffic only. __syncthreads() also drains every global load
// in flight, which here are the next K step's prefetched segments: with it each K step would wait
// out a full memory latency.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
}

template <int WT, typename FX, typename FW>
__device__ __forceinline__ void tile_mac_mfma(f32x4 (&acc)[WT][WT], FX rowX, FW rowW, int K, bf16 (*Xs)[MLD],
                                              bf16 (*Ws)[MLD]) {
  constexpr int NS = WT / 2;                           // staged rows per thread and operand
  const int tid = threadIdx.x;
  const int lr = tid >> 2, lk = (tid & 3) * 16;        // staging: rows lr + 64 j, k lk .. lk + 15
  RowRef rx[NS], rw[NS];
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    rx[j] = rowX(lr + 64 * j);
    rw[j] = rowW(lr + 64 * j);
  }
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = (wave >> 1) * 16 * WT, wn = (wave & 1) * 16 * WT, r = lane & 15, g = lane >> 4;
  bf16x8 xv[NS][2], wv[NS][2];
#pragma unroll
  for (int j = 0; j < NS; ++j)
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      xv[j][e] = load_row8(rx[j], lk + 8 * e, K);
      wv[j][e] = load_row8(rw[j], lk + 8 * e, K);
    }
  for (int k0 = 0; k0 < K; k0 += MK) {
#pragma unroll
    for (int j = 0; j < NS; ++j)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        *reinterpret_cast<bf16x8*>(&Xs[lr + 64 * j][lk + 8 * e]) = xv[j][e];
        *reinterpret_cast<bf16x8*>(&Ws[lr + 64 * j][lk + 8 * e]) = wv[j][e];
      }
    lds_barrier();
    if (k0 + MK < K) {          // the next K step's segments travel while this one multiplies
#pragma unroll
      for (int j = 0; j < NS; ++j)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          xv[j][e] = load_row8(rx[j], k0 + MK + lk + 8 * e, K);
          wv[j][e] = load_row8(rw[j], k0 + MK + lk + 8 * e, K);
        }
    }
#pragma unroll
    for (int ks = 0; ks < MK; ks += 32) {
      bf16x8 xf[WT], wf[WT];
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        xf[t] = *reinterpret_cast<const bf16x8*>(&Xs[wm + 16 * t + r][ks + 8 * g]);
        wf[t] = *reinterpret_cast<const bf16x8*>(&Ws[wn + 16 * t + r][ks + 8 * g]);
      }
#pragma unroll
      for (int tn = 0; tn < WT; ++tn)
#pragma unroll
        for (int tm = 0; tm < WT; ++tm) acc[tn][tm] = mfma16(wf[tn], xf[tm], acc[tn][tm]);
    }
    lds_barrier();
  }
}

// tile_mac_mfma for two weight panels that share the X tile (an expert's gate and up rows): one K
// loop, X staged once, both panels' segments in flight together.
template <int WT, typename FX, typename FW, typename FV>
__device__ __forceinline__ void tile_mac_mfma2(f32x4 (&acc)[WT][WT], f32x4 (&acc2)[WT][WT], FX rowX, FW rowW, FV rowV,
                                               int K, bf16 (*Xs)[MLD], bf16 (*Ws)[MLD], bf16 (*Vs)[MLD]) {
  constexpr int NS = WT / 2;
  const int tid = threadIdx.x;
  const int lr = tid >> 2, lk = (tid & 3) * 16;
  RowRef rx[NS], rw[NS], rv[NS];
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    rx[j] = rowX(lr + 64 * j);
    rw[j] = rowW(lr + 64 * j);
    rv[j] = rowV(lr + 64 * j);
  }
  const int wave = tid >> 6, lane = tid & 63;
  const int wm = (wave >> 1) * 16 * WT, wn = (wave & 1) * 16 * WT, r = lane & 15, g = lane >> 4;
  bf16x8 xv[NS][2], wv[NS][2], vv[NS][2];
#pragma unroll
  for (int j = 0; j < NS; ++j)
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      xv[j][e] = load_row8(rx[j], lk + 8 * e, K);
      wv[j][e] = load_row8(rw[j], lk + 8 * e, K);
      vv[j][e] = load_row8(rv[j], lk + 8 * e, K);
    }
  for (int k0 = 0; k0 < K; k0 += MK) {
#pragma unroll
    for (int j = 0; j < NS; ++j)
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        *reinterpret_cast<bf16x8*>(&Xs[lr + 64 * j][lk + 8 * e]) = xv[j][e];
        *reinterpret_cast<bf16x8*>(&Ws[lr + 64 * j][lk + 8 * e]) = wv[j][e];
        *reinterpret_cast<bf16x8*>(&Vs[lr + 64 * j][lk + 8 * e]) = vv[j][e];
      }
    lds_barrier();
    if (k0 + MK < K) {
#pragma unroll
      for (int j = 0; j < NS; ++j)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          xv[j][e] = load_row8(rx[j], k0 + MK + lk + 8 * e, K);
          wv[j][e] = load_row8(rw[j], k0 + MK + lk + 8 * e, K);
          vv[j][e] = load_row8(rv[j], k0 + MK + lk + 8 * e, K);
        }
    }
#pragma unroll
    for (int ks = 0; ks < MK; ks += 32) {
      bf16x8 xf[WT], wf[WT];
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        xf[t] = *reinterpret_cast<const bf16x8*>(&Xs[wm + 16 * t + r][ks + 8 * g]);
        wf[t] = *reinterpret_cast<const bf16x8*>(&Ws[wn + 16 * t + r][ks + 8 * g]);
      }
#pragma unroll
      for (int tn = 0; tn < WT; ++tn)
#pragma unroll
        for (int tm = 0; tm < WT; ++tm) acc[tn][tm] = mfma16(wf[tn], xf[tm], acc[tn][tm]);
#pragma unroll
      for (int t = 0; t < WT; ++t) wf[t] = *reinterpret_cast<const bf16x8*>(&Vs[wn + 16 * t + r][ks + 8 * g]);
#pragma unroll
      for (int tn = 0; tn < WT; ++tn)
#pragma unroll
        for (int tm = 0; tm < WT; ++tm) acc2[tn][tm] = mfma16(wf[tn], xf[tm], acc2[tn][tm]);
    }
    lds_barrier();
  }
}

// f(m, n, value) over this lane's results of the tile
template <int WT, typename F>
__device__ __forceinline__ void tile_each(const f32x4 (&acc)[WT][WT], F f) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 16 * WT, wn = (wave & 1) * 16 * WT;
#pragma unroll
  for (int tn = 0; tn < WT; ++tn)
#pragma unroll
    for (int tm = 0; tm < WT; ++tm)
#pragma unroll
      for (int i = 0; i < 4; ++i) f(wm + 16 * tm + (lane & 15), wn + 16 * tn + 4 * (lane >> 4) + i, acc[tn][tm][i]);
}

#define BFLY_ZERO_ACC(a)                                    \
  f32x4 a[WT][WT];                                          \
  _Pragma("unroll") for (int _i = 0; _i < WT; ++_i)         \
      _Pragma("unroll") for (int _j = 0; _j < WT; ++_j) a[_i][_j] = f32x4{0.f, 0.f, 0.f, 0.f}

template <typename TO, int WT>
__global__ __launch_bounds__(256) void gemm_any_mfma_kernel(const bf16* __restrict__ x, long ldx,
                                                            const bf16* __restrict__ w, long ldw,
                                                            const bf16* __restrict__ bias, TO* __restrict__ out,
                                                            long ldo, int M, int N, int K, int act, float a0, float a1,
                                                            long bx, long bw, long bo) {
  constexpr int BT = 32 * WT;
  __shared__ __attribute__((aligned(16))) bf16 Xs[BT][MLD], Ws[BT][MLD];
  const int row0 = blockIdx.y * BT, col0 = blockIdx.x * BT;
  x += blockIdx.z * bx;
  w += blockIdx.z * bw;
  out += blockIdx.z * bo;
  BFLY_ZERO_ACC(acc);
  tile_mac_mfma<WT>(
      acc, [&](int r) { return RowRef{row0 + r < M ? x + (long)(row0 + r) * ldx : nullptr, 1.f}; },
      [&](int c) { return RowRef{col0 + c < N ? w + (long)(col0 + c) * ldw : nullptr, 1.f}; }, K, Xs, Ws);
  tile_each<WT>(acc, [&](int m, int n, float v) {
    const int r = row0 + m, c = col0 + n;
    if (r >= M || c >= N) return;
    if (bias) v += (float)bias[c];
    out[(long)r * ldo + c] = (TO)apply_act(v, act, a0, a1);
  });
}

// `tiles` lists (expert, first row) of every (32 WT)-row tile of the grouped rows
template <int WT>
__global__ __launch_bounds__(256) void moe_glu_up_mfma_kernel(const bf16* __restrict__ x, long ldx,
                                                              const float* __restrict__ topk_w, int Kc,
                                                              const int* __restrict__ perm,
                                                              const int* __restrict__ offsets_e,
                                                              const int* __restrict__ tiles,
                                                              const int* __restrict__ ntiles,
                                                              const bf16* __restrict__ gu_w, float limit, float alpha,
                                                              float up_offset, bf16* __restrict__ hmid, int Hd, int F,
                                                              int plain) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  constexpr int BT = 32 * WT;
  // small groups (decode): gate and up share one K loop, so both panels' weight segments are in
  // flight together; large groups (128-row tiles): two passes, which keep registers and LDS for
  // a second resident workgroup
  __shared__ __attribute__((aligned(16))) bf16 Xs[BT][MLD], Ws[BT][MLD], Vs[WT == 2 ? BT : 1][MLD];
  const int e = tiles[2 * blockIdx.y], r0 = tiles[2 * blockIdx.y + 1];
  const int rend = offsets_e[e + 1];
  const int col0 = blockIdx.x * BT;
  // plain experts (no gate): F rows per expert, hmid = act(W x)
  const bf16* wg = gu_w + (long)e * (plain ? 1 : 2) * F * Hd;
  const bf16* wu = wg + (long)F * Hd;
  // the expert's input row: the token row times its routing score, rounded to bf16
  auto rowX = [&](int r) {
    const int p = r0 + r < rend ? perm[r0 + r] : -1;
    return p < 0 ? RowRef{nullptr, 1.f} : RowRef{x + (long)(p / Kc) * ldx, topk_w ? topk_w[p] : 1.f};
  };
  BFLY_ZERO_ACC(g);
  BFLY_ZERO_ACC(u);
  auto rowG = [&](int c) { return RowRef{col0 + c < F ? wg + (long)(col0 + c) * Hd : nullptr, 1.f}; };
  auto rowU = [&](int c) { return RowRef{col0 + c < F ? wu + (long)(col0 + c) * Hd : nullptr, 1.f}; };
  if (plain) {
    tile_mac_mfma<WT>(g, rowX, rowG, Hd, Xs, Ws);
    tile_each<WT>(g, [&](int m, int n, float v) {
      const int r = r0 + m, c = col0 + n;
      if (r < rend && c < F) hmid[(long)r * F + c] = (bf16)apply_act(v, plain, 0.f, 0.f);
    });
    return;
  }
  if constexpr (WT == 2) {
    tile_mac_mfma2<WT>(g, u, rowX, rowG, rowU, Hd, Xs, Ws, Vs);
  } else {
    tile_mac_mfma<WT>(g, rowX, rowG, Hd, Xs, Ws);
    tile_mac_mfma<WT>(u, rowX, rowU, Hd, Xs, Ws);
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 16 * WT, wn = (wave & 1) * 16 * WT;
#pragma unroll
  for (int tn = 0; tn < WT; ++tn)
#pragma unroll
    for (int tm = 0; tm < WT; ++tm)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = r0 + wm + 16 * tm + (lane & 15), c = col0 + wn + 16 * tn + 4 * (lane >> 4) + i;
        if (r >= rend || c >= F) continue;
        const float gg = fminf(g[tn][tm][i], limit);
        const float uu = fminf(fmaxf(u[tn][tm][i], -limit), limit);
        hmid[(long)r * F + c] = (bf16)(gg / (1.f + expf(-alpha * gg)) * (uu + up_offset));
      }
}

template <int WT>
__global__ __launch_bounds__(256) void moe_down_mfma_kernel(const bf16* __restrict__ hmid, const int* __restrict__ perm,
                                                            const int* __restrict__ offsets_e,
                                                            const int* __restrict__ tiles,
                                                            const int* __restrict__ ntiles,
                                                            const bf16* __restrict__ down_w, float* __restrict__ y,
                                                            int Hd, int F) {
  if ((int)blockIdx.y >= ntiles[0]) return;
  constexpr int BT = 32 * WT;
  __shared__ __attribute__((aligned(16))) bf16 Xs[BT][MLD], Ws[BT][MLD];
  const int e = tiles[2 * blockIdx.y], r0 = tiles[2 * blockIdx.y + 1];
  const int rend = offsets_e[e + 1];
  const int col0 = blockIdx.x * BT;
  const bf16* wd = down_w + (long)e * Hd * F;
  BFLY_ZERO_ACC(acc);
  tile_mac_mfma<WT>(
      acc, [&](int r) { return RowRef{r0 + r < rend ? hmid + (long)(r0 + r) * F : nullptr, 1.f}; },
      [&](int c) { return RowRef{col0 + c < Hd ? wd + (long)(col0 + c) * F : nullptr, 1.f}; }, F, Xs, Ws);
  tile_each<WT>(acc, [&](int m, int n, float v) {
    const int r = r0 + m, c = col0 + n;
    if (r < rend && c < Hd) y[(long)perm[r] * Hd + c] = v;
  });
}

inline int ew_blocks(long n) { return (int)std::min<long>(4096, std::max<long>(1, (n + 255) / 256)); }

}  // namespace

void launch_gemm_any(const void* x, long ldx, const void* w, long ldw, const void* bias, void* out, long ldo,
                     int M, int N, int K, int act, float a0, float a1, bool f32, bool out_f32, hipStream_t s,
                     int batch, long bx, long bw, long bo) {
  if (M <= 0 || N <= 0 || batch <= 0) return;
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM, batch);
  if (!f32 && M >= 512 && N >= 128) {        // large row counts: the 128 x 128 workgroup tile
    dim3 g2((N + 127) / 128, (M + 127) / 128, batch);
    if (out_f32)
      gemm_any_mfma_kernel<float, 4><<<g2, 256, 0, s>>>((const bf16*)x, ldx, (const bf16*)w, ldw, (const bf16*)bias,
                                                        (float*)out, ldo, M, N, K, act, a0, a1, bx, bw, bo);
    else
      gemm_any_mfma_kernel<bf16, 4><<<g2, 256, 0, s>>>((const bf16*)x, ldx, (const bf16*)w, ldw, (const bf16*)bias,
                                                       (bf16*)out, ldo, M, N, K, act, a0, a1, bx, bw, bo);
    return;
  }
  if (f32)
    gemm_any_kernel<float, float><<<grid, 256, 0, s>>>((const float*)x, ldx, (const float*)w, ldw, (const float*)bias,
                                                       (float*)out, ldo, M, N, K, act, a0, a1, bx, bw, bo);
  else if (out_f32)
    gemm_any_mfma_kernel<float, 2><<<grid, 256, 0, s>>>((const bf16*)x, ldx, (const bf16*)w, ldw, (const bf16*)bias,
                                                     (float*)out, ldo, M, N, K, act, a0, a1, bx, bw, bo);
  else
    gemm_any_mfma_kernel<bf16, 2><<<grid, 256, 0, s>>>((const bf16*)x, ldx, (const bf16*)w, ldw, (const bf16*)bias,
                                                    (bf16*)out, ldo, M, N, K, act, a0, a1, bx, bw, bo);
}

void launch_act(void* x, long n, int act, float a0, float a1, bool f32, hipStream_t s) {
  if (n <= 0 || act == ACT_NONE) return;
  if (f32) act_kernel<float><<<ew_blocks(n), 256, 0, s>>>((float*)x, n, act, a0, a1);
  else act_kernel<bf16><<<ew_blocks(n), 256, 0, s>>>((bf16*)x, n, act, a0, a1);
}

void launch_router_logits(const void* x, long ldx, const void* wr, float* logits, int T, int E, int Hd, bool f32,
                          hipStream_t s) {
  if (T <= 0) return;
  dim3 grid(T, (E + 3) / 4);
  if (f32) router_logits_kernel<float><<<grid, 256, 0, s>>>((const float*)x, ldx, (const float*)wr, logits, E, Hd);
  else router_logits_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)x, ldx, (const bf16*)wr, logits, E, Hd);
}

void launch_moe_topk_scores(const float* logits, const float* bias, int top_k, int scoring, bool renorm, int* ids,
                            float* w, int T, int E, hipStream_t s, const float* select_bias) {
  if (T <= 0) return;
  moe_topk_scores_kernel<<<T, 64, 0, s>>>(logits, bias, top_k, scoring, renorm, ids, w, E, select_bias);
}

int moe_sort_max_tiles(int TKp, int E) { return (TKp + 63) / 64 + E; }

// 128-row tiles when the experts average at least 256 grouped rows (bf16 only), else 64
int moe_tile_rows(int TKp, int E, bool f32) { return (!f32 && TKp >= 256 * E) ? 128 : 64; }

void launch_moe_sort(const int* ids, int TKp, int E, int* perm, int* offsets, int* tiles, int* ntiles, int tile_rows,
                     hipStream_t s) {
  moe_sort_kernel<<<1, 1024, 0, s>>>(ids, TKp, E, perm, offsets, tiles, ntiles, tile_rows);
}

void launch_moe_glu_up(const void* x, long ldx, const float* topk_w, int K, const int* perm, const int* offsets,
                       const int* tiles, const int* ntiles, int max_tiles, const void* gate_up_w, float limit,
                       float alpha, float up_offset, void* hmid, int Hd, int F, bool f32, int tile_rows, hipStream_t s,
                       int plain_act) {
  if (tile_rows == 128) {
    dim3 g2((F + 127) / 128, max_tiles);
    moe_glu_up_mfma_kernel<4><<<g2, 256, 0, s>>>((const bf16*)x, ldx, topk_w, K, perm, offsets, tiles, ntiles,
                                                 (const bf16*)gate_up_w, limit, alpha, up_offset, (bf16*)hmid, Hd, F,
                                                 plain_act);
    return;
  }
  dim3 grid((F + TN - 1) / TN, max_tiles);
  if (f32)
    moe_glu_up_kernel<float><<<grid, 256, 0, s>>>((const float*)x, ldx, topk_w, K, perm, offsets, tiles, ntiles,
                                                  (const float*)gate_up_w, limit, alpha, up_offset, (float*)hmid, Hd, F,
                                                  plain_act);
  else
    moe_glu_up_mfma_kernel<2><<<grid, 256, 0, s>>>((const bf16*)x, ldx, topk_w, K, perm, offsets, tiles, ntiles,
                                                (const bf16*)gate_up_w, limit, alpha, up_offset, (bf16*)hmid, Hd, F,
                                                plain_act);
}

void launch_moe_down(const void* hmid, const int* perm, const int* offsets, const int* tiles, const int* ntiles,
                     int max_tiles, const void* down_w, float* y, int Hd, int F, bool f32, int tile_rows, hipStream_t s) {
  if (tile_rows == 128) {
    dim3 g2((Hd + 127) / 128, max_tiles);
    moe_down_mfma_kernel<4><<<g2, 256, 0, s>>>((const bf16*)hmid, perm, offsets, tiles, ntiles, (const bf16*)down_w, y,
                                               Hd, F);
    return;
  }
  dim3 grid((Hd + TN - 1) / TN, max_tiles);
  if (f32)
    moe_down_kernel<float><<<grid, 256, 0, s>>>((const float*)hmid, perm, offsets, tiles, ntiles,
                                                (const float*)down_w, y, Hd, F);
  else
    moe_down_mfma_kernel<2><<<grid, 256, 0, s>>>((const bf16*)hmid, perm, offsets, tiles, ntiles, (const bf16*)down_w, y,
                                              Hd, F);
}

void launch_moe_sum(const float* y, const float* wts, int K, void* out, int T, int Hd, bool f32, hipStream_t s) {
  const long n = (long)T * Hd;
  if (n <= 0) return;
  if (f32) moe_sum_kernel<float><<<ew_blocks(n), 256, 0, s>>>(y, wts, K, (float*)out, T, Hd);
  else moe_sum_kernel<bf16><<<ew_blocks(n), 256, 0, s>>>(y, wts, K, (bf16*)out, T, Hd);
}

}  // namespace bfly
