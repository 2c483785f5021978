// Host-side launch API of csrc/kernels/delta.hip: the step between two sublayers of a stack with
// layer norms on both sides of every sublayer, short causal convolutions with an activation on
// projected rows (history pooled per sequence), and the gated delta rule with pooled per-sequence
// state. Every launcher is stream-ordered, allocation-free and synchronisation-free. `f32`: the
// activation element type is float (else bf16); norms, decays, unit norms and the state are f32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bfly {

// x <- x + mult * (layer_norm(y) * nw + nb) (+ extra, nullable f32 [T, W]); h (nullable) = layer_norm(x) * nw2 + nb2
void launch_post_norm_add_norm(float* x, const void* y, const float* nw, const float* nb, float eps, float mult,
                               const float* extra, const float* nw2, const float* nb2, void* h, int T, int W, bool f32,
                               hipStream_t s);
// out[t, c] = act(sum_j w[c, j] z[t - (taps - 1 - j), c]) inside row t's sequence; rows before the step's
// first row of the sequence: state[slot][taps - 1 - k] is the input k steps before it, zero before
// position 0. z rows are z_ld elements apart; state f32 [slots, taps - 1, C]; act 0 none, 1 silu;
// out [T, C] float when out_f32 (or f32), else bf16.
void launch_short_conv_act(const void* z, long z_ld, const float* w, const float* state, const int* state_slots,
                           const int* row_cu, int nseq, const int* positions, void* out, int T, int C, int taps, int act,
                           bool f32, bool out_f32, hipStream_t s);
// state[slot] <- the last n rows of z of every sequence of the step (n = taps - 1; older entries shift)
void launch_short_conv_state_update(const void* z, long z_ld, float* state, const int* state_slots, const int* row_cu,
                                    int nseq, const int* positions, int C, int n, bool f32, hipStream_t s);
// Gated delta rule over packed rows (see ops.delta_scan): q, k f32 [T, G, D], v f32 [T, H, Dv] with row
// strides, b / a [T, H] logits of the activation type, state f32 [slots, H, Dv, D] (a head's state
// column by column), o f32 [T, H, Dv].
// Returns < 0 if D > 256.
int launch_delta_scan(const float* q, long q_ld, const float* k, long k_ld, const float* v, long v_ld, const void* b,
                      long b_ld, const void* a, long a_ld, const float* a_log, const float* dt_bias, float* state,
                      const int* state_slots, const int* row_cu, int nseq, const int* positions, float q_scale,
                      float unit_eps, float* o, int T, int H, int G, int D, int Dv, bool f32, hipStream_t s);

}  // namespace bfly
