// Weight maintenance between training steps on the matrix in HBM: decay, diffusion, clipping, column reset and the
// bookkeeping of externally accumulated updates (delta weights).  Elementwise and memory-bound: grid-stride
// kernels with unit-stride accesses; the random draws are Philox streams keyed like every other draw of the tile.
#include "kernels.h"

namespace rpu_amd {

namespace {

__device__ __forceinline__ float clip_to(float w, const float *w_min, const float *w_max, size_t i) {
  if (w_max) w = fminf(w, w_max[i]);
  if (w_min) w = fmaxf(w, w_min[i]);
  return w;
}

// PulsedRPUDevice::decayWeights (rpu_pulsed_device.cpp:392-420): towards the reset bias, then the device bounds
__global__ __launch_bounds__(256) void k_decay_device(float *w, const float *decay_scale, const float *reset_bias,
                                                       const float *w_min, const float *w_max, float alpha,
                                                       int bias_no_decay, int x_size, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float s = 1.0f + alpha * (decay_scale[i] - 1.0f);
    if (bias_no_decay && (int)(i % x_size) == x_size - 1) s = 1.0f;
    const float b = reset_bias[i];
    w[i] = clip_to((w[i] - b) * s + b, w_min, w_max, i);
  }
}

// RPUSimple::decayWeights (rpu.cpp:1556-1575)
__global__ __launch_bounds__(256) void k_decay_scalar(float *w, float scale, int bias_no_decay, int x_size, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    if (!(bias_no_decay && (int)(i % x_size) == x_size - 1)) w[i] *= scale;
  }
}

// w += rate * N(0, 1), then the bounds (rpu_pulsed_device.cpp:432-446, rpu.cpp:1609-1620); four elements per thread
__global__ __launch_bounds__(256) void k_diffuse(float *w, const float *rates, float rate, const float *w_min,
                                                  const float *w_max, PhiloxKey key, uint32_t call, size_t n) {
  const size_t quads = (n + 3) / 4;
  for (size_t q = blockIdx.x * (size_t)blockDim.x + threadIdx.x; q < quads; q += (size_t)gridDim.x * blockDim.x) {
    float z[4];
    philox_normal4((uint32_t)q, (uint32_t)(q >> 32), call, RNG_DIFFUSE, key, z);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const size_t i = 4 * q + e;
      if (i < n) w[i] = clip_to(w[i] + (rates ? rates[i] : rate) * z[e], w_min, w_max, i);
    }
  }
}

// clip to +- *clip_dev (when positive) or to +- clip, and to the device bounds when given
// (rpu_pulsed_device.cpp:448-467, rpu.cpp:1589-1599)
__global__ __launch_bounds__(256) void k_clip_value(float *w, const float *w_min, const float *w_max, float clip,
                                                     const float *clip_dev, size_t n) {
  if (clip_dev) clip = *clip_dev;
  const bool symmetric = clip >= 0.0f;
  if (clip_dev && !(clip > 0.0f)) return;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float v = w[i];
    if (symmetric) v = fminf(fmaxf(v, -clip), clip);
    w[i] = clip_to(v, w_min, w_max, i);
  }
}

__device__ __forceinline__ float block_sum(float v, float *sh) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.0f;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) r += sh[i];
  return r;
}

// LayerGaussian (weight_clipper.cpp:68-93): clip value = sigma * sample standard deviation, capped by fixed_value.
// One workgroup; the sums are accumulated in double so that the figure does not depend on the thread count.
__global__ __launch_bounds__(1024) void k_clip_value_gaussian(const float *w, size_t n, float sigma, float fixed_value,
                                                               float *clip_out) {
  __shared__ double sh[16];
  auto reduce = [&](double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    double r = 0.0;
    for (int i = 0; i < 16; ++i) r += sh[i];
    return r;
  };
  double s = 0.0;
  for (size_t i = threadIdx.x; i < n; i += blockDim.x) s += (double)w[i];
  const double mean = reduce(s) / (double)n;
  double q = 0.0;
  for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
    const double m = (double)w[i] - mean;
    q += m * m;
  }
  const double var = reduce(q) / (double)(n - 1);
  if (threadIdx.x == 0) {
    float clip = (float)sqrt(var) * sigma;
    if (fixed_value > 0.0f) clip = fminf(clip, fixed_value);
    *clip_out = clip;
  }
}

// AverageChannelMax (weight_clipper.cpp:38-66): mean over the rows of the largest absolute weight of a row
__global__ __launch_bounds__(256) void k_row_abs_max(const float *w, int x_size, float *row_max) {
  __shared__ float sh[4];
  const float *row = w + (size_t)blockIdx.x * x_size;
  float m = 0.0f;
  for (int j = threadIdx.x; j < x_size; j += blockDim.x) m = fmaxf(m, fabsf(row[j]));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) row_max[blockIdx.x] = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
}

__global__ __launch_bounds__(256) void k_clip_value_channel(const float *row_max, int d_size, float fixed_value,
                                                             float *clip_out) {
  __shared__ float sh[4];
  float s = 0.0f;
  for (int i = threadIdx.x; i < d_size; i += blockDim.x) s += row_max[i];
  s = block_sum(s, sh);
  if (threadIdx.x == 0) {
    float clip = fabsf(s / (float)d_size);
    if (fixed_value > 0.0f) clip = fminf(clip, fixed_value);
    *clip_out = clip;
  }
}

// resetCols (rpu_pulsed_device.cpp:469-494, rpu_simple_device.cpp:148-168): columns start .. start + n_cols - 1
// (wrapping around) are set to the reset bias plus noise, each element with probability reset_prob
__global__ __launch_bounds__(256) void k_reset_cols(float *w, const float *reset_bias, const float *w_min,
                                                     const float *w_max, float reset_std, int start_col, int n_cols,
                                                     float reset_prob, int x_size, int d_size, PhiloxKey key,
                                                     uint32_t call) {
  const size_t total = (size_t)d_size * n_cols;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int i = (int)(idx / n_cols);
    const int j = (start_col + (int)(idx % n_cols)) % x_size;
    const size_t k = (size_t)i * x_size + j;
    float z[4];
    philox_normal4((uint32_t)j, (uint32_t)i, call, RNG_RESET, key, z);
    if (reset_prob < 1.0f) {
      const Philox4 r = philox4x32_10((uint32_t)j, (uint32_t)i, call, RNG_RESET | (1u << 8), key.k0, key.k1);
      if (!(u32_to_uniform(r.v[0]) < reset_prob)) continue;
    }
    float v = reset_bias ? reset_bias[k] : 0.0f;
    if (reset_std > 0.0f) v += reset_std * z[0];
    w[k] = clip_to(v, w_min, w_max, k);
  }
}

// RPUSimple::getAndResetWeightUpdate (rpu.cpp:1432-1442)
__global__ __launch_bounds__(256) void k_delta_finish(float *w, float *prev_w_and_delta, float scale, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const float w_old = prev_w_and_delta[i];
    prev_w_and_delta[i] = scale * (w[i] - w_old);
    w[i] = w_old;
  }
}

int grid_for(size_t n) {
  const size_t blocks = (n + 255) / 256;
  return (int)(blocks > 8192 ? 8192 : (blocks ? blocks : 1));
}

} // namespace

void launch_decay_device(float *w, const float *decay_scale, const float *reset_bias, const float *w_min,
                         const float *w_max, float alpha, int bias_no_decay, int x_size, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_decay_device, dim3(grid_for(n)), dim3(256), 0, s, w, decay_scale, reset_bias, w_min, w_max, alpha,
                     bias_no_decay, x_size, n);
}

void launch_decay_scalar(float *w, float scale, int bias_no_decay, int x_size, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_decay_scalar, dim3(grid_for(n)), dim3(256), 0, s, w, scale, bias_no_decay, x_size, n);
}

void launch_diffuse(float *w, const float *rates, float rate, const float *w_min, const float *w_max, PhiloxKey key,
                    uint32_t call, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_diffuse, dim3(grid_for((n + 3) / 4)), dim3(256), 0, s, w, rates, rate, w_min, w_max, key, call, n);
}

void launch_clip_value(float *w, const float *w_min, const float *w_max, float clip, const float *clip_dev, size_t n,
                       hipStream_t s) {
  hipLaunchKernelGGL(k_clip_value, dim3(grid_for(n)), dim3(256), 0, s, w, w_min, w_max, clip, clip_dev, n);
}

void launch_clip_value_gaussian(const float *w, size_t n, float sigma, float fixed_value, float *clip_out, hipStream_t s) {
  hipLaunchKernelGGL(k_clip_value_gaussian, dim3(1), dim3(1024), 0, s, w, n, sigma, fixed_value, clip_out);
}

void launch_clip_value_channel(const float *w, int x_size, int d_size, float fixed_value, float *row_max, float *clip_out,
                               hipStream_t s) {
  hipLaunchKernelGGL(k_row_abs_max, dim3(d_size), dim3(256), 0, s, w, x_size, row_max);
  hipLaunchKernelGGL(k_clip_value_channel, dim3(1), dim3(256), 0, s, row_max, d_size, fixed_value, clip_out);
}

void launch_reset_cols(float *w, const float *reset_bias, const float *w_min, const float *w_max, float reset_std,
                       int start_col, int n_cols, float reset_prob, int x_size, int d_size, PhiloxKey key, uint32_t call,
                       hipStream_t s) {
  hipLaunchKernelGGL(k_reset_cols, dim3(grid_for((size_t)d_size * n_cols)), dim3(256), 0, s, w, reset_bias, w_min, w_max,
                     reset_std, start_col, n_cols, reset_prob, x_size, d_size, key, call);
}

void launch_delta_finish(float *w, float *prev_w_and_delta, float scale, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_delta_finish, dim3(grid_for(n)), dim3(256), 0, s, w, prev_w_and_delta, scale, n);
}

} // namespace rpu_amd
