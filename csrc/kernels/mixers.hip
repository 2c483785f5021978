// Sequence mixers for heterogeneous layer stacks, generic in head count, head sizes and element
// type (bf16 or f32 activations / caches; scores, softmax, angles, decays and state are f32):
//   rope_partial_kv_kernel    interleaved-pair rotary on the first 2 * nrot dims of q / k heads,
//                             fused with the paged append of k and v
//                             (K [blocks, G, BS, D] rows, V [blocks, G, Dv, BS] transposed: a
//                             page's keys are contiguous for the P V operand)
//   attn_window_paged_kernel  attention of packed rows over the paged cache: causal sliding
//                             window plus the always-visible first `keep_first` positions, and a
//                             per-head sink logit that only enters the softmax denominator
//   gla_scan_kernel           gated linear attention S <- diag(a) S + k v^T, o = S^T q with the
//                             state pooled in per-sequence slots
//   gla_out_kernel            per-head RMS norm of o, times silu(gate)
// Rows of a step are packed: sequence s owns rows row_cu[s] .. row_cu[s+1] (one row for a
// decoded token, several for a prompt chunk), positions[] gives each row's position.
#include <algorithm>

#include "bfly_common.h"
#include "bfly_mixers.h"

namespace bfly {

namespace {

template <typename T>
__global__ __launch_bounds__(256) void rope_partial_kv_kernel(T* __restrict__ q, long q_ld, T* __restrict__ k, long k_ld,
                                                              const T* __restrict__ v, long v_ld,
                                                              const int* __restrict__ positions,
                                                              const float* __restrict__ inv_freq, int nrot,
                                                              const int* __restrict__ slots, T* __restrict__ k_cache,
                                                              T* __restrict__ v_cache, int H, int G, int D, int Dv,
                                                              int bs) {
  const long t = blockIdx.x;
  const float p = (float)positions[t];
  const int slot = (slots && k) ? slots[t] : -1;
  // rotated pairs of the q heads, then of the k heads
  const int nq = H * nrot, nk = k ? G * nrot : 0;
  for (int i = threadIdx.x; i < nq + nk; i += blockDim.x) {
    const bool isq = i < nq;
    const int j = isq ? i : i - nq;
    const int h = j / nrot, r = j % nrot;
    T* ptr = (isq ? q + t * q_ld : k + t * k_ld) + (long)h * D + 2 * r;
    const float a = p * inv_freq[r];
    double sd, cd;
    sincos((double)a, &sd, &cd);
    const float c = (float)cd, s = (float)sd;
    const float u = (float)ptr[0], w = (float)ptr[1];
    ptr[0] = (T)(u * c - w * s);
    ptr[1] = (T)(w * c + u * s);
  }
  if (slot < 0) return;
  __syncthreads();      // the rotated k is read back below
  const long blk = slot / bs, off = slot % bs;
  for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
    const int g = i / D, d = i % D;
    k_cache[((blk * G + g) * bs + off) * D + d] = k[t * k_ld + i];
  }
  for (int i = threadIdx.x; i < G * Dv; i += blockDim.x) {
    const int g = i / Dv, d = i % Dv;
    v_cache[((blk * G + g) * Dv + d) * bs + off] = v[t * v_ld + i];
  }
}

// One wave per (row, query head). Keys are visited 64 at a time (one per lane) with an online
// softmax seeded by the sink: m = sink, l = 1, acc = 0, so the sink counts once in the
// denominator and has no value (no sink: m very low, l = 0, an ordinary softmax). Lane `l` then
// owns output dims l, l + 64, ... (Dv <= 512). out_scale (nullable) [T, H] multiplies the output
// of every (row, head): an output gate.
constexpr int kMaxDvLane = 8;

// Score modifiers shared by the attention kernels (AttnMod): the lowest visible position of a row
// outside the kept prefix, the row's score scale, and the capped / distance-biased score.
__device__ __forceinline__ int attn_row_lo(int p, int window, int chunk) {
  return chunk > 0 ? p - p % chunk : max(0, p - window + 1);
}
__device__ __forceinline__ float attn_row_scale(int p, float scale, const AttnMod& md) {
  if (md.qt_coef == 0.f) return scale;
  return scale * (1.f + md.qt_coef * logf((float)((p + 1) / md.qt_every) + 1.f));
}
// FAST (the bf16 matrix-core form): hardware exp / log / reciprocal; the generic form, which also
// serves true-f32 runs, keeps the precise functions.
template <bool FAST>
__device__ __forceinline__ float attn_score(float dot, float rscale, int dist, float da, float db, const AttnMod& md) {
  float sc = dot * rscale;
  if (md.softcap > 0.f) {
    if (FAST) sc = md.softcap * (1.f - __fdividef(2.f, __expf(2.f * __fdividef(sc, md.softcap)) + 1.f));
    else sc = md.softcap * tanhf(sc / md.softcap);
  }
  if (md.dist_a) {      // no second vector: the linear form
    if (!md.dist_b) sc -= da * (float)dist;
    else sc -= da * (FAST ? __logf(1.f + db * (float)dist) : log1pf(db * (float)dist));
  }
  return sc;
}

template <typename T>
__global__ __launch_bounds__(64) void attn_window_paged_kernel(const T* __restrict__ q, long q_ld,
                                                               const T* __restrict__ k_cache,
                                                               const T* __restrict__ v_cache,
                                                               const int* __restrict__ tables, int max_blocks,
                                                               const int* __restrict__ row_seq,
                                                               const int* __restrict__ positions, float scale,
                                                               int window, int keep_first,
                                                               const float* __restrict__ sink,
                                                               const float* __restrict__ out_scale,
                                                               void* __restrict__ out_v, int H, int G, int D, int Dv,
                                                               int bs, AttnMod md) {
  extern __shared__ float smem[];      // q [D] | p [64] | key row base index [64] (as int)
  float* sq = smem;
  float* sp = smem + D;
  long* sj = reinterpret_cast<long*>(smem + D + 64 + ((D & 1) ? 1 : 0));
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  // G value heads; md.maps key heads per value head, query heads ordered (head, map)
  const int Gk = G * md.maps;
  const int gk = ((h / md.maps) / ((H / md.maps) / G)) * md.maps + h % md.maps;
  const int g = gk / md.maps;
  const int s = row_seq[t];
  T* out = reinterpret_cast<T*>(out_v);
  float* outf = reinterpret_cast<float*>(out_v);
  if (s < 0) {       // padding row of a fixed-shape step
    for (int d = lane; d < Dv; d += 64) {
      if (md.out_f32) outf[(t * H + h) * Dv + d] = 0.f;
      else out[(t * H + h) * Dv + d] = (T)0.f;
    }
    return;
  }
  const int p = positions[t];
  const float rscale = attn_row_scale(p, scale, md);
  const float da = md.dist_a ? md.dist_a[h] : 0.f, db = md.dist_b ? md.dist_b[h] : 0.f;
  const int* tab = tables + (long)s * max_blocks;
  for (int d = lane; d < D; d += 64) sq[d] = (float)q[t * q_ld + (long)h * D + d];
  __syncthreads();
  const int lo = attn_row_lo(p, window, md.chunk);
  const int n1 = min(keep_first, lo);          // kept first positions outside the window
  const int total = n1 + (p - lo + 1);
  float m = sink ? sink[h] : -1e30f, l = sink ? 1.f : 0.f;
  float acc[kMaxDvLane] = {};
  for (int i0 = 0; i0 < total; i0 += 64) {
    const int i = i0 + lane;
    float sc = -INFINITY;
    long kv_row = 0;      // index of V^T[0][key] of this lane's key
    if (i < total) {
      const int j = i < n1 ? i : lo + (i - n1);
      const long blk = tab[j / bs];
      kv_row = (blk * G + g) * Dv * bs + (j % bs);
      const T* kr = k_cache + ((blk * Gk + gk) * bs + (j % bs)) * D;
      float a = 0.f;
      for (int d = 0; d < D; ++d) a = fmaf(sq[d], (float)kr[d], a);
      sc = attn_score<false>(a, rscale, p - j, da, db, md);
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float pe = i < total ? expf(sc - mn) : 0.f;
    const float corr = expf(m - mn);
    l = l * corr + wave_sum(pe);
    m = mn;
    __syncthreads();
    sp[lane] = pe;
    sj[lane] = kv_row;
    __syncthreads();
    const int cnt = min(64, total - i0);
#pragma unroll
    for (int c = 0; c < kMaxDvLane; ++c) {
      const int d = lane + 64 * c;
      if (d >= Dv) break;
      float a = acc[c] * corr;
      for (int x = 0; x < cnt; ++x) a = fmaf(sp[x], (float)v_cache[sj[x] + (long)d * bs], a);
      acc[c] = a;
    }
  }
  const float inv = (out_scale ? out_scale[t * H + h] : 1.f) / l;
#pragma unroll
  for (int c = 0; c < kMaxDvLane; ++c) {
    const int d = lane + 64 * c;
    if (d < Dv) {
      if (md.out_f32) outf[(t * H + h) * Dv + d] = acc[c] * inv;
      else out[(t * H + h) * Dv + d] = (T)(acc[c] * inv);
    }
  }
}

// MFMA form for bf16 with 32-token pages, D = 32 DS, Dv = 16 DVT. A workgroup of 4 waves owns 16
// consecutive rows of a sequence and one query head; the visible pages (the kept prefix, then the
// window) are dealt round-robin to the waves, each wave keeps its own online softmax, and wave 0
// folds the other three in through LDS at the end (a decoded row's ~window / 32 pages are thus
// walked by four waves, a prompt tile's by four as well). Per page, no LDS: S^T = K Q^T
// (16x16x32 tiles, K rows read as 16-byte segments straight from the page), masks and softmax
// in f32 (the four lanes that share a query row combine by shuffles), then O^T += V^T P with the
// page's keys as the MFMA k index in the order the score tiles leave them (keys 4g..4g+3 and
// 16+4g..16+4g+3 in lane group g), which the transposed V page serves with two 8-byte reads.
// The next page's K and V fragments are loaded before the current page is multiplied. The sink
// seeds wave 0's softmax (m = sink, l = 1; without a sink m is very low and l = 0). The
// per-element mask settles the window edges. `fold` > 0 (one shared key / value head, G = 1,
// fold = H): the tile's 16 rows run over (token, head) pairs, row r = token * H + head, so the
// heads of a decoded token share one tile and a token's heads walk the cached pages once.
// `nsplit` > 1 (steps of few tiles, i.e. decoding): gridDim.z workgroups share a tile's pages,
// each leaves its unnormalised (o, m, l) per row in `part` and attn_split_merge_kernel folds them.
template <int DS, int DVT>
__global__ __launch_bounds__(256) void attn_window_mfma_kernel(const bf16* __restrict__ q, long q_ld,
                                                               const bf16* __restrict__ k_cache,
                                                               const bf16* __restrict__ v_cache,
                                                               const int* __restrict__ tables, int max_blocks,
                                                               const int* __restrict__ row_cu, int nseq,
                                                               const int* __restrict__ positions, float scale,
                                                               int window, int keep_first,
                                                               const float* __restrict__ sink,
                                                               const float* __restrict__ out_scale,
                                                               void* __restrict__ out_v, int H, int G, int fold,
                                                               int nsplit, float* __restrict__ part,
                                                               long part_rows, AttnMod md) {
  constexpr int D = 32 * DS, Dv = 16 * DVT, BS = 32;
  const int split = blockIdx.z;
  extern __shared__ float smem[];          // o of waves 1-3 [3][DVT][4][64] | m [3][16] | l [3][16]
  float* so = smem;
  float* sm = smem + 3 * DVT * 256;
  float* sl = sm + 48;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int tile = blockIdx.x;
  const int rf = fold > 0 ? fold : 1;       // tile rows per token
  int s = 0, row0 = 0, rend = 0;
  for (; s < nseq; ++s) {
    const int a = row_cu[s] * rf, b = row_cu[s + 1] * rf;
    const int nt = (b - a + 15) >> 4;
    if (tile < nt) { row0 = a + 16 * tile; rend = b; break; }
    tile -= nt;
  }
  if (s >= nseq) return;                   // (the whole workgroup: the tile is per workgroup)
  const int qr = lane & 15, gg = lane >> 4;
  const bool rv = row0 + qr < rend;
  const long frow = rv ? row0 + qr : row0;
  const long row = frow / rf;                                   // the token's row
  const int h = fold > 0 ? (int)(frow % rf) : (int)blockIdx.y;  // this lane's query head
  // G value heads; md.maps key heads per value head, query heads ordered (head, map)
  const int Gk = G * md.maps;
  const int gk = fold > 0 ? 0 : ((h / md.maps) / ((H / md.maps) / G)) * md.maps + h % md.maps;
  const int g = gk / md.maps;
  const int p = rv ? positions[row] : -1;
  const int plo = attn_row_lo(max(p, 0), window, md.chunk);
  const float rscale = attn_row_scale(max(p, 0), scale, md);
  const float da = md.dist_a ? md.dist_a[h] : 0.f, db = md.dist_b ? md.dist_b[h] : 0.f;
  int pmin = rv ? p : 0x7fffffff, pmax = p;
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) {
    pmin = min(pmin, __shfl_xor(pmin, o, 64));
    pmax = max(pmax, __shfl_xor(pmax, o, 64));
  }
  bf16x8 qf[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds)
    qf[ds] = *reinterpret_cast<const bf16x8*>(q + row * q_ld + (long)h * D + 32 * ds + 8 * gg);
  const int* tab = tables + (long)s * max_blocks;
  const bool seeded = wave == 0 && split == 0 && sink;
  float m = seeded ? sink[h] : -1e30f, l = seeded ? 1.f : 0.f;
  f32x4 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int kp = (min(keep_first, pmax + 1) + BS - 1) / BS;          // pages of the kept prefix
  const int wp0 = max(attn_row_lo(pmin, window, md.chunk) / BS, kp), wp1 = pmax / BS;
  const int npages = kp + max(0, wp1 - wp0 + 1);
  auto page_of = [&](int i) { return i < kp ? i : wp0 + (i - kp); };
  auto load_kv = [&](int pg, bf16x8 (&kf)[2][DS], bf16x8 (&vf)[DVT]) {
    const long blk = tab[pg];
    const bf16* Kp = k_cache + (blk * Gk + gk) * BS * D;
    const bf16* Vp = v_cache + (blk * G + g) * Dv * BS;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
      for (int ds = 0; ds < DS; ++ds)
        kf[kh][ds] = *reinterpret_cast<const bf16x8*>(Kp + (long)(16 * kh + qr) * D + 32 * ds + 8 * gg);
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
      const bf16* vr = Vp + (long)(16 * t + qr) * BS + 4 * gg;
      const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(vr);
      const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(vr + 16);
      vf[t] = bf16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
    }
  };
  bf16x8 kf[2][DS], vf[DVT];
  const int pstep = 4 * nsplit;
  int pi = wave + 4 * split;
  if (pi < npages) load_kv(page_of(pi), kf, vf);
  while (pi < npages) {
    const int pg = page_of(pi);
    const int ni = pi + pstep;
    bf16x8 nkf[2][DS], nvf[DVT];
    if (ni < npages) load_kv(page_of(ni), nkf, nvf);
    f32x4 st[2];
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      st[kh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) st[kh] = mfma16(kf[kh][ds], qf[ds], st[kh]);
    }
    float sc[8], mx = -INFINITY;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = pg * BS + 16 * kh + 4 * gg + i;
        const bool ok = j <= p && (j >= plo || j < keep_first);
        sc[4 * kh + i] = ok ? attn_score<true>(st[kh][i], rscale, p - j, da, db, md) : -INFINITY;
        mx = fmaxf(mx, sc[4 * kh + i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float corr = __expf(m - mn);
    float rs = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = __expf(sc[e] - mn);      // exp(-inf) = 0 for masked keys
      rs += pe;
      pb[e] = (bf16)pe;
    }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l = l * corr + rs;
    m = mn;
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= corr;
      o[t] = mfma16(vf[t], pb, o[t]);
    }
    if (ni < npages) {
#pragma unroll
      for (int kh = 0; kh < 2; ++kh)
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) kf[kh][ds] = nkf[kh][ds];
#pragma unroll
      for (int t = 0; t < DVT; ++t) vf[t] = nvf[t];
    }
    pi = ni;
  }
  if (wave > 0) {
    float* po = so + (long)(wave - 1) * DVT * 256;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) po[(t * 4 + i) * 64 + lane] = o[t][i];
    if (gg == 0) {
      sm[(wave - 1) * 16 + qr] = m;
      sl[(wave - 1) * 16 + qr] = l;
    }
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int u = 0; u < 3; ++u) {
    const float mu = sm[u * 16 + qr], lu = sl[u * 16 + qr];
    const float mn = fmaxf(m, mu);
    const float c0 = __expf(m - mn), cu = __expf(mu - mn);
    l = l * c0 + lu * cu;
    m = mn;
    const float* po = so + (long)u * DVT * 256;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] = o[t][i] * c0 + po[(t * 4 + i) * 64 + lane] * cu;
  }
  if (!rv) return;
  if (nsplit > 1) {
    float* pp = part + ((long)split * part_rows + (row * H + h)) * (Dv + 2);
#pragma unroll
    for (int t = 0; t < DVT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) pp[16 * t + 4 * gg + i] = o[t][i];
    if (gg == 0) { pp[Dv] = m; pp[Dv + 1] = l; }
    return;
  }
  const float inv = (out_scale ? out_scale[row * H + h] : 1.f) / l;
  if (md.out_f32) {
    float* orow = reinterpret_cast<float*>(out_v) + (row * H + h) * Dv;
#pragma unroll
    for (int t = 0; t < DVT; ++t)
      *reinterpret_cast<f32x4*>(orow + 16 * t + 4 * gg) =
          f32x4{o[t][0] * inv, o[t][1] * inv, o[t][2] * inv, o[t][3] * inv};
    return;
  }
  bf16* orow = reinterpret_cast<bf16*>(out_v) + (row * H + h) * Dv;
#pragma unroll
  for (int t = 0; t < DVT; ++t) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (bf16)(o[t][i] * inv);
    *reinterpret_cast<bf16x4*>(orow + 16 * t + 4 * gg) = w;
  }
}

// Folded form for steps of many rows (prompts), one shared key / value head: a workgroup owns 64
// consecutive (token, head) rows of a sequence, 16 per wave, and walks the union of their visible
// pages once. Each page's K rows and transposed V rows are staged in LDS by all four waves
// (double buffered: the next page travels to registers while the current one is multiplied, one
// barrier per page), so a page is read from memory once per 64 rows instead of once per 16, and
// every wave keeps its own rows' online softmax: no merge at the end. Rows pitch D + 8 (K) and
// 32 + 4 (V^T) elements keep the 16-byte / 8-byte fragment reads off a common bank.
template <int DS, int DVT>
__global__ __launch_bounds__(256) void attn_fold_tile_kernel(const bf16* __restrict__ q, long q_ld,
                                                             const bf16* __restrict__ k_cache,
                                                             const bf16* __restrict__ v_cache,
                                                             const int* __restrict__ tables, int max_blocks,
                                                             const int* __restrict__ row_cu, int nseq,
                                                             const int* __restrict__ positions, float scale,
                                                             int window, int keep_first,
                                                             const float* __restrict__ sink,
                                                             const float* __restrict__ out_scale,
                                                             bf16* __restrict__ out, int H) {
  constexpr int D = 32 * DS, Dv = 16 * DVT, BS = 32, KP = D + 8, VP = BS + 4;
  constexpr int NK = BS * D / 8, NV = Dv * BS / 8;            // 16-byte segments of a page
  constexpr int NKS = (NK + 255) / 256, NVS = (NV + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) unsigned char fold_smem[];
  bf16* Ks = reinterpret_cast<bf16*>(fold_smem);            // [2][BS][KP]
  bf16* Vs = Ks + 2 * BS * KP;                                // [2][Dv][VP]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int tile = blockIdx.x;
  int s = 0, row0 = 0, rend = 0;
  for (; s < nseq; ++s) {
    const int a = row_cu[s] * H, b = row_cu[s + 1] * H;
    const int nt = (b - a + 63) >> 6;
    if (tile < nt) { row0 = a + 64 * tile; rend = b; break; }
    tile -= nt;
  }
  if (s >= nseq) return;                   // (the whole workgroup)
  const int qr = lane & 15, gg = lane >> 4;
  const bool rv = row0 + 16 * wave + qr < rend;
  const long frow = rv ? row0 + 16 * wave + qr : row0;
  const long row = frow / H;
  const int h = (int)(frow % H);
  const int p = rv ? positions[row] : -1;
  // positions grow along a sequence's rows: the tile's first and last rows bound them
  const int pmin = positions[row0 / H], pmax = positions[(min(rend, row0 + 64) - 1) / H];
  bf16x8 qf[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds)
    qf[ds] = *reinterpret_cast<const bf16x8*>(q + row * q_ld + (long)h * D + 32 * ds + 8 * gg);
  const int* tab = tables + (long)s * max_blocks;
  float m = sink ? sink[h] : -1e30f, l = sink ? 1.f : 0.f;
  f32x4 o[DVT];
#pragma unroll
  for (int t = 0; t < DVT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int kp = (min(keep_first, pmax + 1) + BS - 1) / BS;          // pages of the kept prefix
  const int wp0 = max(max(0, pmin - window + 1) / BS, kp), wp1 = pmax / BS;
  const int npages = kp + max(0, wp1 - wp0 + 1);
  auto page_of = [&](int i) { return i < kp ? i : wp0 + (i - kp); };
  bf16x8 kreg[NKS], vreg[NVS];
  auto gload = [&](int pg) {
    const long blk = tab[pg];
    const bf16* Kp = k_cache + blk * BS * D;
    const bf16* Vp = v_cache + blk * Dv * BS;
#pragma unroll
    for (int i = 0; i < NKS; ++i) {
      const int idx = tid + 256 * i;
      if (idx < NK) kreg[i] = *reinterpret_cast<const bf16x8*>(Kp + (long)idx * 8);
    }
#pragma unroll
    for (int i = 0; i < NVS; ++i) {
      const int idx = tid + 256 * i;
      if (idx < NV) vreg[i] = *reinterpret_cast<const bf16x8*>(Vp + (long)idx * 8);
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NKS; ++i) {
      const int idx = tid + 256 * i;
      if (idx < NK) *reinterpret_cast<bf16x8*>(Ks + (long)(buf * BS + idx / (D / 8)) * KP + 8 * (idx % (D / 8))) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < NVS; ++i) {
      const int idx = tid + 256 * i;
      if (idx < NV) {
        bf16* dst = Vs + (long)(buf * Dv + idx / 4) * VP + 8 * (idx & 3);       // 8-byte aligned rows
        const bf16x8 v = vreg[i];
        *reinterpret_cast<bf16x4*>(dst) = bf16x4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<bf16x4*>(dst + 4) = bf16x4{v[4], v[5], v[6], v[7]};
      }
    }
  };
  if (npages > 0) gload(page_of(0));
  for (int pi = 0; pi < npages; ++pi) {
    const int buf = pi & 1;
    sstore(buf);
    __syncthreads();      // the page is in LDS; every wave has left the buffer written next
    if (pi + 1 < npages) gload(page_of(pi + 1));
    const int pg = page_of(pi);
    const bf16* Kb = Ks + (long)buf * BS * KP;
    const bf16* Vb = Vs + (long)buf * Dv * VP;
    f32x4 st[2];
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      st[kh] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ds = 0; ds < DS; ++ds)
        st[kh] = mfma16(*reinterpret_cast<const bf16x8*>(Kb + (16 * kh + qr) * KP + 32 * ds + 8 * gg), qf[ds], st[kh]);
    }
    float sc[8], mx = -INFINITY;
#pragma unroll
    for (int kh = 0; kh < 2; ++kh)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = pg * BS + 16 * kh + 4 * gg + i;
        const bool ok = j <= p && (p - j < window || j < keep_first);
        sc[4 * kh + i] = ok ? st[kh][i] * scale : -INFINITY;
        mx = fmaxf(mx, sc[4 * kh + i]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float corr = __expf(m - mn);
    float rs = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = __expf(sc[e] - mn);      // exp(-inf) = 0 for masked keys
      rs += pe;
      pb[e] = (bf16)pe;
    }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l = l * corr + rs;
    m = mn;
#pragma unroll
    for (int t = 0; t < DVT; ++t) {
      const bf16* vr = Vb + (16 * t + qr) * VP + 4 * gg;
      const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(vr);
      const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(vr + 16);
#pragma unroll
      for (int i = 0; i < 4; ++i) o[t][i] *= corr;
      o[t] = mfma16(bf16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]}, pb, o[t]);
    }
  }
  if (!rv) return;
  const float inv = (out_scale ? out_scale[row * H + h] : 1.f) / l;
  bf16* orow = out + (row * H + h) * Dv;
#pragma unroll
  for (int t = 0; t < DVT; ++t) {
    bf16x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (bf16)(o[t][i] * inv);
    *reinterpret_cast<bf16x4*>(orow + 16 * t + 4 * gg) = w;
  }
}

// One wave per (row, head): fold the nsplit partial results part[split][row][o (Dv) | m | l].
__global__ __launch_bounds__(64) void attn_split_merge_kernel(const float* __restrict__ part, long part_rows,
                                                              int nsplit, const float* __restrict__ out_scale,
                                                              void* __restrict__ out_v, int Dv, bool out_f32) {
  const long r = blockIdx.x;
  const int lane = threadIdx.x;
  float m = -1e30f;
  for (int s = 0; s < nsplit; ++s) m = fmaxf(m, part[((long)s * part_rows + r) * (Dv + 2) + Dv]);
  float l = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* pp = part + ((long)s * part_rows + r) * (Dv + 2);
    l += pp[Dv + 1] * __expf(pp[Dv] - m);
  }
  const float inv = (out_scale ? out_scale[r] : 1.f) / l;
  for (int d = lane; d < Dv; d += 64) {
    float a = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float* pp = part + ((long)s * part_rows + r) * (Dv + 2);
      a += pp[d] * __expf(pp[Dv] - m);
    }
    if (out_f32) reinterpret_cast<float*>(out_v)[r * Dv + d] = a * inv;
    else reinterpret_cast<bf16*>(out_v)[r * Dv + d] = (bf16)(a * inv);
  }
}

// row -> sequence map of a packed step (rows outside every sequence: -1)
__global__ void row_seq_kernel(const int* __restrict__ row_cu, int nseq, int* __restrict__ row_seq, int T) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  int s = -1;
  for (int i = 0; i < nseq; ++i)
    if (t >= row_cu[i] && t < row_cu[i + 1]) { s = i; break; }
  row_seq[t] = s;
}

// Workgroup = (sequence, head, 64-column slice of Dv), 8 waves; wave w owns 8 columns. A lane is
// (column c = lane & 7, row group gg = lane >> 3) and keeps the NR rows d = gg * NR .. + NR - 1 of
// its column's state in registers, so a token costs NR fused updates per lane and three shuffles to
// sum the eight row groups: no barrier inside the token loop. Tokens are staged 16 at a time:
// their decays (a = exp(log sigmoid(z) / tau), f32), keys, scaled queries and values go to LDS in
// one pass (rows past D are zero, so the row loop needs no bound), the outputs of the 16 tokens
// leave through LDS in another.
template <typename T, int NR>
__global__ __launch_bounds__(512) void gla_scan_kernel(const T* __restrict__ q, long q_ld, const T* __restrict__ k,
                                                       long k_ld, const T* __restrict__ v, long v_ld,
                                                       const T* __restrict__ z, long z_ld, float* __restrict__ state,
                                                       const int* __restrict__ state_slots,
                                                       const int* __restrict__ row_cu,
                                                       const int* __restrict__ positions, float inv_tau,
                                                       float q_scale, float* __restrict__ o, int H, int D, int Dv) {
  constexpr int TB = 16, DP = 8 * NR, NT = 512;
  __shared__ __attribute__((aligned(16))) float sa[TB * DP], sk[TB * DP], sq[TB * DP];
  __shared__ float sv[TB][64], so[TB][64];
  const int s = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * 64;
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int cl = 8 * w + (lane & 7), gg = lane >> 3;
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
  float* S = state + ((long)slot * H + h) * D * Dv;
  float st[NR];
  const bool fresh = positions[r0] == 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = gg * NR + i;
    st[i] = (!fresh && live && d < D) ? S[(long)d * Dv + col] : 0.f;
  }
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nb = min(TB, r1 - t0);
    for (int i = threadIdx.x; i < nb * DP; i += NT) {
      const int tt = i / DP, d = i - tt * DP;
      float a = 0.f, kk = 0.f, qq = 0.f;
      if (d < D) {
        const long t = t0 + tt;
        const float zz = (float)z[t * z_ld + (long)h * D + d];
        // log sigmoid(z) = -softplus(-z), stable on both sides
        float ls;
        if constexpr (sizeof(T) == 2) {   // bf16 inputs: hardware exp / log (f32, ~1 ulp)
          ls = zz < 0.f ? zz - __logf(1.f + __expf(zz)) : -__logf(1.f + __expf(-zz));
          a = __expf(ls * inv_tau);
        } else {
          ls = zz < 0.f ? zz - log1pf(expf(zz)) : -log1pf(expf(-zz));
          a = expf(ls * inv_tau);
        }
        kk = (float)k[t * k_ld + (long)h * D + d];
        qq = (float)q[t * q_ld + (long)h * D + d] * q_scale;
      }
      sa[i] = a;
      sk[i] = kk;
      sq[i] = qq;
    }
    for (int i = threadIdx.x; i < nb * 64; i += NT) {
      const int tt = i >> 6, c = i & 63;
      sv[tt][c] = (c0 + c < Dv) ? (float)v[(long)(t0 + tt) * v_ld + (long)h * Dv + c0 + c] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nb; ++tt) {
      const float vv = sv[tt][cl];
      const f32x4* pa = reinterpret_cast<const f32x4*>(sa + tt * DP + gg * NR);
      const f32x4* pk = reinterpret_cast<const f32x4*>(sk + tt * DP + gg * NR);
      const f32x4* pq = reinterpret_cast<const f32x4*>(sq + tt * DP + gg * NR);
      float po = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < NR / 4; ++i4) {
        const f32x4 a4 = pa[i4], k4 = pk[i4], q4 = pq[i4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          st[4 * i4 + j] = fmaf(a4[j], st[4 * i4 + j], k4[j] * vv);
          po = fmaf(q4[j], st[4 * i4 + j], po);
        }
      }
      po += __shfl_xor(po, 8, 64);
      po += __shfl_xor(po, 16, 64);
      po += __shfl_xor(po, 32, 64);
      if (gg == 0) so[tt][cl] = po;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nb * 64; i += NT) {
      const int tt = i >> 6, c = i & 63;
      if (c0 + c < Dv) o[((long)(t0 + tt) * H + h) * Dv + c0 + c] = so[tt][c];
    }
    // (the next block's staging overwrites sa / sk / sq / sv, which every wave finished reading
    // at the barrier above; so is rewritten only after the next block's first barrier)
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = gg * NR + i;
      if (d < D) S[(long)d * Dv + col] = st[i];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(const float* __restrict__ o, const T* __restrict__ g, long g_ld,
                                                     const float* __restrict__ norm_w, float eps, T* __restrict__ out,
                                                     int H, int Dv) {
  const long t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* row = o + (t * H + h) * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) ss = fmaf(row[d], row[d], ss);
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / (float)Dv + eps);
  for (int d = lane; d < Dv; d += 64) {
    const float gg = (float)g[t * g_ld + (long)h * Dv + d];
    const float y = row[d] * r * norm_w[d];
    out[(t * H + h) * Dv + d] = (T)(y * (gg / (1.f + expf(-gg))));
  }
}

}  // namespace

void launch_rope_partial_kv(void* q, long q_ld, void* k, long k_ld, const void* v, long v_ld, const int* positions,
                            const float* inv_freq, int nrot, const int* slots, void* k_cache, void* v_cache,
                            int T, int H, int G, int D, int Dv, int block_size, bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    rope_partial_kv_kernel<float><<<T, 256, 0, s>>>((float*)q, q_ld, (float*)k, k_ld, (const float*)v, v_ld, positions,
                                                    inv_freq, nrot, slots, (float*)k_cache, (float*)v_cache, H, G, D,
                                                    Dv, block_size);
  else
    rope_partial_kv_kernel<bf16><<<T, 256, 0, s>>>((bf16*)q, q_ld, (bf16*)k, k_ld, (const bf16*)v, v_ld, positions,
                                                   inv_freq, nrot, slots, (bf16*)k_cache, (bf16*)v_cache, H, G, D, Dv,
                                                   block_size);
}

void launch_row_seq(const int* row_cu, int nseq, int* row_seq, int T, hipStream_t s) {
  if (T <= 0) return;
  row_seq_kernel<<<(T + 255) / 256, 256, 0, s>>>(row_cu, nseq, row_seq, T);
}

template <int DS>
static bool attn_mfma_dv(const bf16* q, long q_ld, const bf16* kc, const bf16* vc, const int* tables, int max_blocks,
                         const int* row_cu, int nseq, const int* positions, float scale, int window, int keep_first,
                         const float* sink, const float* out_scale, void* out, int T, int H, int G, int Dv, bool fold,
                         int nsplit, float* part, hipStream_t s, const AttnMod& md) {
  if (fold && (long)T * H >= 2048 && (long)T * H >= 128L * nseq) {
    // many rows per sequence (prompts): 64-row tiles over pages staged in LDS
    const unsigned tiles = (unsigned)(((long)T * H + 63) / 64 + nseq);
#define BFLY_ATF(DVT)                                                                                         \
  {                                                                                                           \
    constexpr size_t lds = 2 * (32 * (32 * DS + 8) + 16 * DVT * 36) * sizeof(bf16);                           \
    static bool once = false;                                                                                 \
    if (!once) {                                                                                              \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fold_tile_kernel<DS, DVT>),               \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                        \
      once = true;                                                                                            \
    }                                                                                                         \
    attn_fold_tile_kernel<DS, DVT><<<tiles, 256, lds, s>>>(q, q_ld, kc, vc, tables, max_blocks, row_cu, nseq,   \
                                                          positions, scale, window, keep_first, sink, out_scale, \
                                                          (bf16*)out, H);                                            \
  }
    switch (Dv) {
      case 32: BFLY_ATF(2); return true;
      case 64: BFLY_ATF(4); return true;
      case 96: BFLY_ATF(6); return true;
      case 128: BFLY_ATF(8); return true;
      case 192: BFLY_ATF(12); return true;
      case 256: BFLY_ATF(16); return true;
      default: return false;
    }
#undef BFLY_ATF
  }
  // one workgroup per 16-row tile; every sequence adds at most one partly filled tile
  dim3 grid(((fold ? T * H : T) + 15) / 16 + nseq, fold ? 1 : H, nsplit);
  const int fd = fold ? H : 0;
  const long prow = (long)T * H;
#define BFLY_ATT(DVT)                                                                                          \
  attn_window_mfma_kernel<DS, DVT><<<grid, 256, (3 * DVT * 256 + 96) * sizeof(float), s>>>(                    \
      q, q_ld, kc, vc, tables, max_blocks, row_cu, nseq, positions, scale, window, keep_first, sink, out_scale, out, H, \
      G, fd, nsplit, part, prow, md)
  switch (Dv) {
    case 32: BFLY_ATT(2); break;
    case 64: BFLY_ATT(4); break;
    case 96: BFLY_ATT(6); break;
    case 128: BFLY_ATT(8); break;
    case 192: BFLY_ATT(12); break;
    case 256: BFLY_ATT(16); break;
    default: return false;
  }
  if (nsplit > 1)
    attn_split_merge_kernel<<<(unsigned)prow, 64, 0, s>>>(part, prow, nsplit, out_scale, out, Dv, md.out_f32);
  return true;
#undef BFLY_ATT
}

bool launch_attn_window_mfma(const void* q, long q_ld, const void* k_cache, const void* v_cache, const int* tables,
                             int max_blocks, const int* row_cu, int nseq, const int* positions, float scale, int window,
                             int keep_first, const float* sink, const float* out_scale, void* out, int T, int H, int G,
                             int D, int Dv, int block_size, bool fold, float* part, long part_floats, hipStream_t s,
                             const AttnMod& md) {
  if (block_size != 32 || (q_ld & 7) || (reinterpret_cast<uintptr_t>(q) & 15) || (fold && G != 1)) return false;
  const bool plain = md.chunk == 0 && md.softcap == 0.f && !md.dist_a && md.qt_coef == 0.f && md.maps == 1 && !md.out_f32;
  if (fold && !plain) return false;        // the folded tile has no score modifiers
  if (T <= 0) return true;
  // few tiles (decoding): several workgroups share a tile's pages, as many as fill the chip, the
  // pages of a row (window and table width bound them) and the scratch allow
  int nsplit = 1;
  {
    const long tiles = (long)(((fold ? T * H : T) + 15) / 16 + nseq) * (fold ? 1 : H);
    const long span = md.chunk > 0 ? md.chunk : window;
    const long pages = std::min<long>(span / 32 + 2 + (keep_first + 31) / 32, max_blocks);
    const long fit = part ? part_floats / ((long)T * H * (Dv + 2)) : 1;
    nsplit = (int)std::max<long>(1, std::min<long>(std::min<long>((256 + tiles - 1) / tiles, pages / 8),
                                                    std::min<long>(fit, 16)));
  }
#define BFLY_ATTD(DS)                                                                                          \
  return attn_mfma_dv<DS>((const bf16*)q, q_ld, (const bf16*)k_cache, (const bf16*)v_cache, tables, max_blocks, row_cu, \
                          nseq, positions, scale, window, keep_first, sink, out_scale, out, T, H, G, Dv, fold,           \
                          nsplit, part, s, md)
  switch (D) {
    case 32: BFLY_ATTD(1);
    case 64: BFLY_ATTD(2);
    case 96: BFLY_ATTD(3);
    case 128: BFLY_ATTD(4);
    case 192: BFLY_ATTD(6);
    case 256: BFLY_ATTD(8);
    default: return false;
  }
#undef BFLY_ATTD
}

void launch_attn_window_paged(const void* q, long q_ld, const void* k_cache, const void* v_cache, const int* tables,
                              int max_blocks, const int* row_seq, int nseq, const int* positions, float scale,
                              int window, int keep_first, const float* sink, const float* out_scale, void* out, int T,
                              int H, int G, int D, int Dv, int block_size, bool f32, hipStream_t s, const AttnMod& md) {
  if (T <= 0) return;
  (void)nseq;
  dim3 grid(T, H);
  const size_t sm = (size_t)(D + 64 + 2) * sizeof(float) + 64 * sizeof(long);
  if (f32)
    attn_window_paged_kernel<float><<<grid, 64, sm, s>>>((const float*)q, q_ld, (const float*)k_cache,
                                                         (const float*)v_cache, tables, max_blocks, row_seq, positions,
                                                         scale, window, keep_first, sink, out_scale, out, H, G,
                                                         D, Dv, block_size, md);
  else
    attn_window_paged_kernel<bf16><<<grid, 64, sm, s>>>((const bf16*)q, q_ld, (const bf16*)k_cache,
                                                        (const bf16*)v_cache, tables, max_blocks, row_seq, positions,
                                                        scale, window, keep_first, sink, out_scale, out, H, G, D,
                                                        Dv, block_size, md);
}

template <typename T>
static int gla_scan_t(const T* q, long q_ld, const T* k, long k_ld, const T* v, long v_ld, const T* z, long z_ld,
                      float* state, const int* state_slots, const int* row_cu, int nseq, const int* positions,
                      float tau, float q_scale, float* o, int H, int D, int Dv, hipStream_t s) {
  dim3 grid(nseq, H, (Dv + 63) / 64);
  const float it = 1.f / tau;
#define BFLY_GLA(NR)                                                                                              \
  gla_scan_kernel<T, NR><<<grid, 512, 0, s>>>(q, q_ld, k, k_ld, v, v_ld, z, z_ld, state, state_slots, row_cu, positions, \
                                              it, q_scale, o, H, D, Dv)
  if (D <= 32) BFLY_GLA(4);
  else if (D <= 64) BFLY_GLA(8);
  else if (D <= 128) BFLY_GLA(16);
  else if (D <= 256) BFLY_GLA(32);
  else return -1;
#undef BFLY_GLA
  return 0;
}

int launch_gla_scan(const void* q, long q_ld, const void* k, long k_ld, const void* v, long v_ld, const void* z,
                    long z_ld, float* state, const int* state_slots, const int* row_cu, int nseq,
                    const int* positions, float tau, float q_scale, float* o, int T, int H, int D, int Dv, bool f32,
                    hipStream_t s) {
  if (T <= 0 || nseq <= 0) return 0;
  if (f32)
    return gla_scan_t<float>((const float*)q, q_ld, (const float*)k, k_ld, (const float*)v, v_ld, (const float*)z, z_ld,
                             state, state_slots, row_cu, nseq, positions, tau, q_scale, o, H, D, Dv, s);
  return gla_scan_t<bf16>((const bf16*)q, q_ld, (const bf16*)k, k_ld, (const bf16*)v, v_ld, (const bf16*)z, z_ld, state,
                          state_slots, row_cu, nseq, positions, tau, q_scale, o, H, D, Dv, s);
}

void launch_gla_out(const float* o, const void* g, long g_ld, const float* norm_w, float eps, void* out, int T, int H,
                    int Dv, bool f32, hipStream_t s) {
  if (T <= 0) return;
  dim3 grid(T, H);
  if (f32) gla_out_kernel<float><<<grid, 64, 0, s>>>(o, (const float*)g, g_ld, norm_w, eps, (float*)out, H, Dv);
  else gla_out_kernel<bf16><<<grid, 64, 0, s>>>(o, (const bf16*)g, g_ld, norm_w, eps, (bf16*)out, H, Dv);
}

}  // namespace bfly
