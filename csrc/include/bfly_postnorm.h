// Host-side launch API of csrc/kernels/postnorm.hip: scaled embedding, causal per-channel
// convolution over a sequence's rows with a pooled per-sequence history, layer norm on a
// sublayer's output with a per-channel scale before the residual sum, a learned average over all
// layers' outputs, the preparation of latent attention (norms of the latents, shared rotated key
// part, output gates, paged append). Every launcher is stream-ordered, allocation-free and
// synchronisation-free. `f32`: the activation / weight / cache element type is float (else bf16);
// the residual, norm statistics, angles and gates are f32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bfly {

// out[t] = table[ids[t]] * scale (f32 [T, W])
void launch_embed_scaled(const int* ids, const void* table, float scale, float* out, int T, int W, int vocab, bool f32,
                         hipStream_t s);
// out[t, c] = x[t, c] + sum_j w[c, j] x[t - (taps - 1 - j), c] inside row t's sequence; rows before
// the step's first row of the sequence: state[slot][taps - 1 - k] is the input k steps before it,
// zero before position 0. w == nullptr: out = x. x f32 [T, W], state f32 [slots, taps - 1, W].
void launch_conv_mix(const float* x, const float* w, const float* state, const int* state_slots, const int* row_cu,
                     int nseq, const int* positions, void* out, int T, int W, int taps, bool f32, hipStream_t s);
// state[slot] <- the last n inputs of every sequence of the step (n = taps - 1; older entries shift)
void launch_conv_state_update(const float* x, float* state, const int* state_slots, const int* row_cu, int nseq,
                              const int* positions, int W, int n, hipStream_t s);
// out = x + scale * (layer_norm(y) * nw + nb); cast (nullable): out rounded to the activation type
void launch_post_norm_add(const float* x, const void* y, const float* nw, const float* nb, float eps,
                          const float* scale, float* out, void* cast, int T, int W, bool f32, hipStream_t s);
// X = x + scale * layer_norm(y) (y == nullptr: X = x); stack[index] = X; x = sum_{j <= index} avg[j] stack[j];
// stack planes are `plane` floats apart
void launch_post_norm_add_avg(float* x, const void* y, const float* nw, const float* nb, float eps, const float* scale,
                              float* stack, long plane, int index, const float* avg, int T, int W, bool f32,
                              hipStream_t s);
// z rows [Q query latent | R key/value latent | rd shared key part | H gate logits]: cq = rms(q latent) qn_w,
// gate = sigmoid; K cache row (width Dk >= R + rd) <- [rms(kv latent) kvn_w | key part with its first nrot
// pairs rotated], V cache (Dvc >= R rows per page, tokens contiguous) <- the normed latent; slots < 0: no append
void launch_latent_prep(const void* z, long z_ld, int Q, int R, int rd, int H, const float* qn_w, const float* kvn_w,
                        float eps, const int* positions, const float* inv_freq, int nrot, const int* slots,
                        void* k_cache, void* v_cache, int block_size, int Dk, int Dvc, void* cq, float* gate, int T,
                        bool f32, hipStream_t s);
// dst[t, h, :n] = src[t, h, :n] with the first nrot interleaved pairs rotated by positions[t] * inv_freq;
// dst[t, h, n:nd] = 0
void launch_rope_heads_copy(const void* src, long s_ld, long s_hd, void* dst, long d_ld, long d_hd,
                            const int* positions, const float* inv_freq, int nrot, int T, int H, int n, int nd, bool f32,
                            hipStream_t s);
// out[i] = layer_norm(x[idx[i]]) * nw + nb (idx == nullptr: every row)
void launch_layer_norm_rows(const float* x, const float* nw, const float* nb, float eps, const long* idx, void* out,
                            int R, int W, bool f32, hipStream_t s);

}  // namespace bfly
