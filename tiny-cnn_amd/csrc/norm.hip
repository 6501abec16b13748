// norm.hip — batch normalization and dropout: the two layers of the reference whose backward
// pass needs more than the layer's own output gradient (batch statistics, a mask).
//
// Both are bound by HBM: every kernel here reads or writes each element once. Tensors are
// [batch][channels][spatial] floats; a channel's elements are `batch` runs of `spatial`
// consecutive floats.
//
// Statistics follow tiny_dnn/util/math_functions.h:25-96: mean = sum / (batch*spatial), variance
// = sum (x - mean)^2 / max(1, batch*spatial - 1), two passes. The sums are taken in a fixed
// order that depends on the shape only: workgroup (channel, group) adds the runs of images
// g, g+G, ... (block-wide tree per image), one wave per channel then adds the group sums.
#include "common.h"

namespace tdh {

namespace {

constexpr int NT = 256;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float block_sum(float v, float *smem4) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) smem4[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = (smem4[0] + smem4[1]) + (smem4[2] + smem4[3]);
  __syncthreads();
  return r;
}

// MODE 0: sum a; MODE 1: sum (a - center[ch])^2; MODE 2: sum a and sum a*b (two partials)
template <int MODE>
__global__ void __launch_bounds__(NT)
bn_partial_kernel(const float *__restrict__ a, const float *__restrict__ b,
                  const float *__restrict__ center, const int batch, const int channels,
                  const int spatial, const int groups, float *__restrict__ partial) {
  __shared__ float smem4[4];
  const int ch = blockIdx.x, g = blockIdx.y;
  const float c = MODE == 1 ? center[ch] : 0.0f;
  float s0 = 0.0f, s1 = 0.0f;
  for (int o = g; o < batch; o += groups) {
    const size_t base = (static_cast<size_t>(o) * channels + ch) * spatial;
    for (int i = threadIdx.x; i < spatial; i += NT) {
      const float v = a[base + i];
      if (MODE == 0) s0 += v;
      if (MODE == 1) s0 += (v - c) * (v - c);
      if (MODE == 2) { s0 += v; s1 += v * b[base + i]; }
    }
  }
  s0 = block_sum(s0, smem4);
  if (MODE == 2) s1 = block_sum(s1, smem4);
  if (threadIdx.x == 0) {
    partial[ch * groups + g] = s0;
    if (MODE == 2) partial[(channels + ch) * groups + g] = s1;
  }
}

// One wave per row of partial sums: out0[r] = sum / denom. WHAT 1 also writes
// out1[r] = sqrt(out0[r] + eps) (the standard deviation next to the variance).
template <int WHAT>
__global__ void __launch_bounds__(NT)
bn_finish_kernel(const float *__restrict__ partial, const int rows, const int groups,
                 const float denom, const float eps, float *__restrict__ out0,
                 float *__restrict__ out1) {
  const int r = blockIdx.x * (NT / 64) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (r >= rows) return;
  float s = 0.0f;
  for (int g = lane; g < groups; g += 64) s += partial[r * groups + g];
  s = wave_sum(s);
  if (lane == 0) {
    const float v = s / denom;
    out0[r] = v;
    if (WHAT == 1) out1[r] = sqrtf(v + eps);
  }
}

__global__ void __launch_bounds__(NT)
bn_stddev_kernel(const float *__restrict__ variance, const int channels, const float eps,
                 float *__restrict__ stddev) {
  const int c = blockIdx.x * NT + threadIdx.x;
  if (c < channels) stddev[c] = sqrtf(variance[c] + eps);
}

// batch_normalization_layer.h:150-163: y = (x - mean[ch]) / stddev[ch]
__global__ void __launch_bounds__(NT)
bn_apply_kernel(const float *__restrict__ x, const float *__restrict__ mean,
                const float *__restrict__ stddev, const int channels, const FastDiv div_spatial,
                const size_t total, float *__restrict__ y) {
  const size_t i = static_cast<size_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= total) return;
  const int ch = div_spatial.div(static_cast<uint32_t>(i)) % channels;
  y[i] = (x[i] - mean[ch]) / stddev[ch];
}

// batch_normalization_layer.h:112-125:
//   dx = (dy - mean(dy)[ch] - mean(dy*y)[ch] * y) / stddev[ch];  means = [mean(dy), mean(dy*y)]
__global__ void __launch_bounds__(NT)
bn_bwd_apply_kernel(const float *__restrict__ y, const float *__restrict__ dy,
                    const float *__restrict__ means, const float *__restrict__ stddev,
                    const int channels, const FastDiv div_spatial, const size_t total,
                    float *__restrict__ dx) {
  const size_t i = static_cast<size_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= total) return;
  const int ch = div_spatial.div(static_cast<uint32_t>(i)) % channels;
  float v = dy[i] - means[ch] - means[channels + ch] * y[i];
  dx[i]   = v / stddev[ch];
}

// batch_normalization_layer.h:171-177 (post_update)
__global__ void __launch_bounds__(NT)
bn_moving_kernel(const float *__restrict__ mean_cur, const float *__restrict__ var_cur,
                 const int channels, const float momentum, float *__restrict__ mean,
                 float *__restrict__ var) {
  const int c = blockIdx.x * NT + threadIdx.x;
  if (c >= channels) return;
  mean[c] = momentum * mean[c] + (1 - momentum) * mean_cur[c];
  var[c]  = momentum * var[c] + (1 - momentum) * var_cur[c];
}

// dropout_layer.h:104-113: y = mask * scale * x in the train phase, y = x otherwise
__global__ void __launch_bounds__(NT)
dropout_fwd_kernel(const uint8_t *__restrict__ mask, const float scale, const float *__restrict__ x,
                   const size_t total, float *__restrict__ y) {
  const size_t i = static_cast<size_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= total) return;
  y[i] = mask ? (static_cast<float>(mask[i]) * scale) * x[i] : x[i];
}

// dropout_layer.h:74-82: dx = mask * dy (the scale is NOT applied on the way back)
__global__ void __launch_bounds__(NT)
dropout_bwd_kernel(const uint8_t *__restrict__ mask, const float *__restrict__ dy,
                   const size_t total, float *__restrict__ dx) {
  const size_t i = static_cast<size_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= total) return;
  dx[i] = static_cast<float>(mask[i]) * dy[i];
}

int bn_groups(int batch) { return batch < 64 ? batch : 64; }

}  // namespace

size_t batchnorm_workspace_bytes(int channels, int batch) {
  // partial sums of two quantities, then their two means
  return ws_align(sizeof(float) * 2 * static_cast<size_t>(channels) * bn_groups(batch)) +
         ws_align(sizeof(float) * 2 * static_cast<size_t>(channels));
}

int batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                  float *mean, float *variance, float *stddev, float *y) {
  const int groups   = bn_groups(batch);
  const size_t total = static_cast<size_t>(batch) * channels * spatial;
  if (train) {
    void *ws = nullptr;
    TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(channels) * groups, &ws));
    float *partial = static_cast<float *>(ws);
    const float n  = static_cast<float>(batch) * static_cast<float>(spatial);
    ProfScope prof("batchnorm_moments", 8.0 * total, WORK_BYTE);
    TDH_LAUNCH((bn_partial_kernel<0>), dim3(channels, groups), dim3(NT), 0, ctx().stream, x,
                       nullptr, nullptr, batch, channels, spatial, groups, partial);
    TDH_LAUNCH_CHECK();
    TDH_LAUNCH((bn_finish_kernel<0>), dim3(ceil_div(channels, NT / 64)), dim3(NT), 0,
                       ctx().stream, partial, channels, groups, n, 0.0f, mean, nullptr);
    TDH_LAUNCH_CHECK();
    TDH_LAUNCH((bn_partial_kernel<1>), dim3(channels, groups), dim3(NT), 0, ctx().stream, x,
                       nullptr, mean, batch, channels, spatial, groups, partial);
    TDH_LAUNCH_CHECK();
    TDH_LAUNCH((bn_finish_kernel<1>), dim3(ceil_div(channels, NT / 64)), dim3(NT), 0,
                       ctx().stream, partial, channels, groups, std::max(1.0f, n - 1.0f), eps,
                       variance, stddev);
    TDH_LAUNCH_CHECK();
  } else {
    TDH_LAUNCH(bn_stddev_kernel, dim3(ceil_div(channels, NT)), dim3(NT), 0, ctx().stream,
                       variance, channels, eps, stddev);
    TDH_LAUNCH_CHECK();
  }
  ProfScope prof("batchnorm_fwd", 8.0 * total, WORK_BYTE);
  TDH_LAUNCH(bn_apply_kernel, dim3(static_cast<unsigned>(ceil_div_sz(total, NT))), dim3(NT),
                     0, ctx().stream, x, mean, stddev, channels, FastDiv(spatial), total, y);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                  const float *stddev, float *dx) {
  const int groups   = bn_groups(batch);
  const size_t total = static_cast<size_t>(batch) * channels * spatial;
  void *ws = nullptr, *ws2 = nullptr;
  TDH_TRY(ws_take(sizeof(float) * 2 * static_cast<size_t>(channels) * groups, &ws));
  TDH_TRY(ws_take(sizeof(float) * 2 * static_cast<size_t>(channels), &ws2));
  float *partial = static_cast<float *>(ws), *means = static_cast<float *>(ws2);
  const float n  = static_cast<float>(batch) * static_cast<float>(spatial);
  {
    ProfScope prof("batchnorm_bwd_moments", 8.0 * total, WORK_BYTE);
    TDH_LAUNCH((bn_partial_kernel<2>), dim3(channels, groups), dim3(NT), 0, ctx().stream, dy,
                       y, nullptr, batch, channels, spatial, groups, partial);
    TDH_LAUNCH_CHECK();
    TDH_LAUNCH((bn_finish_kernel<0>), dim3(ceil_div(2 * channels, NT / 64)), dim3(NT), 0,
                       ctx().stream, partial, 2 * channels, groups, n, 0.0f, means, nullptr);
    TDH_LAUNCH_CHECK();
  }
  ProfScope prof("batchnorm_bwd", 12.0 * total, WORK_BYTE);
  TDH_LAUNCH(bn_bwd_apply_kernel, dim3(static_cast<unsigned>(ceil_div_sz(total, NT))),
                     dim3(NT), 0, ctx().stream, y, dy, means, stddev, channels, FastDiv(spatial),
                     total, dx);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                            const float *var_cur, float *mean, float *var) {
  TDH_LAUNCH(bn_moving_kernel, dim3(ceil_div(channels, NT)), dim3(NT), 0, ctx().stream,
                     mean_cur, var_cur, channels, momentum, mean, var);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int dropout_fwd(size_t total, int train, float scale, const uint8_t *mask, const float *x, float *y) {
  ProfScope prof("dropout_fwd", (train ? 9.0 : 8.0) * total, WORK_BYTE);
  TDH_LAUNCH(dropout_fwd_kernel, dim3(static_cast<unsigned>(ceil_div_sz(total, NT))),
                     dim3(NT), 0, ctx().stream, train ? mask : nullptr, scale, x, total, y);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int dropout_bwd(size_t total, const uint8_t *mask, const float *dy, float *dx) {
  ProfScope prof("dropout_bwd", 9.0 * total, WORK_BYTE);
  TDH_LAUNCH(dropout_bwd_kernel, dim3(static_cast<unsigned>(ceil_div_sz(total, NT))),
                     dim3(NT), 0, ctx().stream, mask, dy, total, dx);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace tdh
