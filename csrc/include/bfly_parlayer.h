// Host-side launch API of the kernels for parallel layers (mixer and feed-forward read two norms
// of the same residual) with a token shift, for attention whose queries and keys are normed and
// half-rotated per head, for the combination of differential attention maps, and for the dense
// clamped GLU. Every launcher is stream-ordered, allocation-free and synchronisation-free. `f32`:
// the activation element type is float (else bf16); the residual, norms, the shift state, angles
// and the combination are f32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bfly {

// x' = x + (ya + yb) (ya / yb nullable; x_out nullable when both are: x' = x), n = x' / rms(x'),
// ha = n (norm_a + offset), mixed with the previous token's unmixed ha when shift != nullptr:
// ha + (prev - ha) shift, prev = row t - 1 of the same sequence, else state[slot] (position > 0),
// else zero. hb = n (norm_b + offset) (nullable). state[slot] <- the unmixed ha of the sequence's
// last row. Rows with row_seq < 0 (padding) get zero outputs. x_out must not alias x.
void launch_par_norm_shift(const float* x, const void* ya, const void* yb, float* x_out, const float* norm_a,
                           const float* norm_b, float eps, float offset, const float* shift, float* state,
                           const int* state_slots, const int* row_seq, const int* row_cu, const int* positions,
                           void* ha, void* hb, int T, int W, bool f32, hipStream_t s);
// out[i] = rms(x[r] + (ya[r] + yb[r])) (w + offset), r = idx[i] (idx == nullptr: every row)
void launch_par_final(const float* x, const void* ya, const void* yb, const float* norm_w, float eps, float offset,
                      const long* idx, void* out, int R, int W, bool f32, hipStream_t s);
// cs [T, 2, nrot] f32 = cos | sin of positions[t] * inv_freq[f] (f64 product and evaluation)
void launch_rope_table(const int* positions, const float* inv_freq, int nrot, float* cs, int T, hipStream_t s);
// Per head: RMS norm over D with weight qn_w / kn_w (nullable: none), then the first 2 nrot dims
// rotate with dimension i paired with i + nrot by the angles of cs (launch_rope_table). q [T, Hq, D] ->
// q_out [T, Hq, Dp] (zero padded); k [T, Gk, D], v [T, Gv, Dv] -> K [blocks, Gk, BS, Dp],
// V [blocks, Gv, Dvp, BS] at slots[t] >= 0 (cache padding is left as it is). D <= 512. q_out == nullptr
// (allowed without query norm and rotation when Dp == D): the queries stay where they are.
void launch_qk_norm_rope_kv(const void* q, long q_ld, const void* k, long k_ld, const void* v, long v_ld,
                            const float* qn_w, const float* kn_w, float eps, const float* cs, int nrot,
                            const int* slots, void* q_out, void* k_cache,
                            void* v_cache, int T, int Hq, int Gk, int Gv, int D, int Dp, int Dv, int Dvp, int block_size,
                            bool f32, hipStream_t s);
// a [T, 2 H, Dvp] f32, heads ordered (head, map): o = a[2h] - lam a[2h + 1] over the first Dv values,
// o / rms(o) * out_mul * sigmoid(gate[t, h * Dv + d]) (gate nullable) -> out [T, H * Dv]. Dv <= 512.
void launch_diff_combine(const float* a, float lam, float eps, float out_mul, const void* gate, long gate_ld,
                         void* out, int T, int H, int Dv, int Dvp, bool f32, hipStream_t s);
// out[t, f] = g sigmoid(alpha g) (u + up_offset), g = min(gate, limit), u = clamp(up, +-limit); gate / up of
// column f are gu[t, f] and gu[t, F + f] (group == 0), or lie in alternating blocks of `group` columns
// (gate block, up block, ...: the row layout of the GEMMs' fused gate / up epilogues)
void launch_glu_clamp(const void* gu, long gu_ld, float limit, float alpha, float up_offset, void* out, int T, int F,
                      int group, bool f32, hipStream_t s);

}  // namespace bfly
