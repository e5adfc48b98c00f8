// Parallel residual streams (hyper-connections) with offset-weight RMS norms. The residual is
// S f32 streams per token, xs [T, S, W]. A sublayer reads one mixed-in row
// u = sum_s w_in[s] xs[s], normalised as u / sqrt(mean(u^2) + eps) * (w + offset) (offset 1: the
// weight is stored around zero), and its output y updates every stream from the old ones:
// xs[r] <- sum_s mix[s, r] xs[s] + w_out[r] y. One workgroup per token row; sums, norms and the
// streams are f32 whatever the activation type.
#include "bfly_common.h"
#include "bfly_mixers.h"

namespace bfly {

namespace {

constexpr int kMaxStreams = 16;

template <typename T>
__global__ __launch_bounds__(256) void embed_norm_streams_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                                 const float* __restrict__ norm_w, float eps,
                                                                 float offset, float* __restrict__ xs, int S, int W,
                                                                 int vocab) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* row = table + (long)id * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = (float)row[c];
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = (float)row[c] * r * (norm_w[c] + offset);
    for (int s = 0; s < S; ++s) xs[((long)t * S + s) * W + c] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void hc_pre_kernel(const float* __restrict__ xs, const float* __restrict__ w_in,
                                                     const float* __restrict__ norm_w, float eps, float offset,
                                                     T* __restrict__ out, int S, int W) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  const float* x = xs + t * S * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(w_in[s], x[(long)s * W + c], u);
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(w_in[s], x[(long)s * W + c], u);
    out[t * W + c] = (T)(u * r * (norm_w[c] + offset));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void hc_post_kernel(float* __restrict__ xs, const T* __restrict__ y,
                                                      const float* __restrict__ mix, const float* __restrict__ w_out,
                                                      int S, int W) {
  const long t = blockIdx.x;
  float* x = xs + t * S * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float old[kMaxStreams];
    for (int s = 0; s < S; ++s) old[s] = x[(long)s * W + c];
    const float yv = (float)y[t * W + c];
    for (int r = 0; r < S; ++r) {
      float v = 0.f;
      for (int s = 0; s < S; ++s) v = fmaf(mix[s * S + r], old[s], v);
      x[(long)r * W + c] = fmaf(w_out[r], yv, v);
    }
  }
}

// hc_post followed by the next sublayer's hc_pre on the updated streams, one pass over the row's
// streams for both (the same thread owns a column in both halves, so it rereads what it wrote).
template <typename T>
__global__ __launch_bounds__(256) void hc_post_pre_kernel(float* __restrict__ xs, const T* __restrict__ y,
                                                          const float* __restrict__ mix,
                                                          const float* __restrict__ w_out,
                                                          const float* __restrict__ w_in2,
                                                          const float* __restrict__ norm_w2, float eps, float offset,
                                                          T* __restrict__ out, int S, int W) {
  __shared__ float red[16];
  const long t = blockIdx.x;
  float* x = xs + t * S * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float old[kMaxStreams];
    for (int s = 0; s < S; ++s) old[s] = x[(long)s * W + c];
    const float yv = (float)y[t * W + c];
    float u = 0.f;
    for (int r = 0; r < S; ++r) {
      float v = 0.f;
      for (int s = 0; s < S; ++s) v = fmaf(mix[s * S + r], old[s], v);
      v = fmaf(w_out[r], yv, v);
      x[(long)r * W + c] = v;
      u = fmaf(w_in2[r], v, u);
    }
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u = fmaf(w_in2[s], x[(long)s * W + c], u);
    out[t * W + c] = (T)(u * r * (norm_w2[c] + offset));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void hc_final_kernel(const float* __restrict__ xs, const float* __restrict__ norm_w,
                                                       float eps, float offset, const long* __restrict__ idx,
                                                       T* __restrict__ out, int S, int W) {
  __shared__ float red[16];
  const long i = blockIdx.x;
  const long t = idx ? idx[i] : i;
  const float* x = xs + t * S * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += x[(long)s * W + c];
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += x[(long)s * W + c];
    out[i * W + c] = (T)(u * r * (norm_w[c] + offset));
  }
}

}  // namespace

void launch_embed_norm_streams(const int* ids, const void* table, const float* norm_w, float eps, float offset,
                               float* xs, int T, int S, int W, int vocab, bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32) embed_norm_streams_kernel<float><<<T, 256, 0, s>>>(ids, (const float*)table, norm_w, eps, offset, xs, S, W, vocab);
  else embed_norm_streams_kernel<bf16><<<T, 256, 0, s>>>(ids, (const bf16*)table, norm_w, eps, offset, xs, S, W, vocab);
}

void launch_hc_pre(const float* xs, const float* w_in, const float* norm_w, float eps, float offset, void* out,
                   int T, int S, int W, bool f32, hipStream_t s) {
  if (T <= 0) return;
  if (f32) hc_pre_kernel<float><<<T, 256, 0, s>>>(xs, w_in, norm_w, eps, offset, (float*)out, S, W);
  else hc_pre_kernel<bf16><<<T, 256, 0, s>>>(xs, w_in, norm_w, eps, offset, (bf16*)out, S, W);
}

void launch_hc_post(float* xs, const void* y, const float* mix, const float* w_out, int T, int S, int W, bool f32,
                    hipStream_t s) {
  if (T <= 0) return;
  if (f32) hc_post_kernel<float><<<T, 256, 0, s>>>(xs, (const float*)y, mix, w_out, S, W);
  else hc_post_kernel<bf16><<<T, 256, 0, s>>>(xs, (const bf16*)y, mix, w_out, S, W);
}

void launch_hc_post_pre(float* xs, const void* y, const float* mix, const float* w_out, const float* w_in2,
                        const float* norm_w2, float eps, float offset, void* out, int T, int S, int W, bool f32,
                        hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    hc_post_pre_kernel<float><<<T, 256, 0, s>>>(xs, (const float*)y, mix, w_out, w_in2, norm_w2, eps, offset, (float*)out, S, W);
  else
    hc_post_pre_kernel<bf16><<<T, 256, 0, s>>>(xs, (const bf16*)y, mix, w_out, w_in2, norm_w2, eps, offset, (bf16*)out, S, W);
}

void launch_hc_final(const float* xs, const float* norm_w, float eps, float offset, const long* idx, void* out,
                     int R, int S, int W, bool f32, hipStream_t s) {
  if (R <= 0) return;
  if (f32) hc_final_kernel<float><<<R, 256, 0, s>>>(xs, norm_w, eps, offset, idx, (float*)out, S, W);
  else hc_final_kernel<bf16><<<R, 256, 0, s>>>(xs, norm_w, eps, offset, idx, (bf16*)out, S, W);
}

}  // namespace bfly
