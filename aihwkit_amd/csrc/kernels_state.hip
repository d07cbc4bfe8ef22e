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
                                                       int bias_no_decay, MatLayout lay, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float s = 1.0f + alpha * (decay_scale[i] - 1.0f);
    if (bias_no_decay && lay.col_of(i) == lay.x_size - 1) s = 1.0f;
    const float b = reset_bias[i];
    w[i] = clip_to((w[i] - b) * s + b, w_min, w_max, i);
  }
}

// RPUSimple::decayWeights (rpu.cpp:1556-1575)
__global__ __launch_bounds__(256) void k_decay_scalar(float *w, float scale, int bias_no_decay, MatLayout lay, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    if (!(bias_no_decay && lay.col_of(i) == lay.x_size - 1)) w[i] *= scale;
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
    if (symmetric) {
      // the reference's order: upper limits first, then the lower ones win (it matters for a device whose sampled
      // bounds lie beyond the clip value on the wrong side)
      const float hi = w_max ? fminf(w_max[i], clip) : clip;
      const float lo = w_min ? fmaxf(w_min[i], -clip) : -clip;
      v = fmaxf(fminf(v, hi), lo);
    } else {
      v = clip_to(v, w_min, w_max, i);
    }
    w[i] = v;
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
__global__ __launch_bounds__(256) void k_row_abs_max(const float *w, MatLayout lay, float *row_max) {
  __shared__ float sh[4];
  float m = 0.0f;
  for (int j = threadIdx.x; j < lay.x_size; j += blockDim.x) m = fmaxf(m, fabsf(w[lay.at((int)blockIdx.x, j)]));
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
                                                     float reset_prob, MatLayout lay, PhiloxKey key, uint32_t call) {
  const int x_size = lay.x_size;
  const size_t total = (size_t)lay.d_size * n_cols;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int i = (int)(idx / n_cols);
    const int j = (start_col + (int)(idx % n_cols)) % x_size;
    const size_t k = lay.at(i, j);
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

// PulsedRPUDevice::applyUpdateWriteNoise (rpu_pulsed_device.cpp:573-588): every shown weight is its persistent one
// plus fresh noise; four elements per thread
__global__ __launch_bounds__(256) void k_write_noise_all(float *w_apparent, const float *w_persistent, float noise_std,
                                                          PhiloxKey key, uint32_t call, size_t n) {
  const size_t quads = (n + 3) / 4;
  for (size_t q = blockIdx.x * (size_t)blockDim.x + threadIdx.x; q < quads; q += (size_t)gridDim.x * blockDim.x) {
    float z[4];
    philox_normal4((uint32_t)q, (uint32_t)(q >> 32), call, RNG_WRITE_NOISE | (1u << 8), key, z);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const size_t i = 4 * q + e;
      if (i < n) w_apparent[i] = w_persistent[i] + noise_std * z[e];
    }
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

// WeightDrifter::apply (weight_drifter.cpp:108-150) with the saturation of a pulsed device
// (weight_drifter.cpp:98-106) folded in; z[0] varies nu, z[1] is the read noise
__global__ __launch_bounds__(256) void k_device_drift(float *w, float *prev, float *w0, float *t, const float *nu,
                                                       const float *w_min, const float *w_max, DriftDev p,
                                                       float current_t, PhiloxKey key, uint32_t call, size_t n) {
  const bool random = p.nu_std > 0.0f || p.w_read_std > 0.0f;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (random) philox_normal4((uint32_t)i, (uint32_t)(i >> 32), call, RNG_DEVICE_DRIFT, key, z);
    float v = w[i];
    if (fabsf(prev[i] - v) > p.reset_tol) {
      // the weight has changed: its drift starts again from here
      t[i] = current_t;
      w0[i] = v;
    } else {
      float nu_i = nu ? nu[i] : p.nu0;
      if (p.nu_std > 0.0f) nu_i = nu_i + p.nu_std * nu_i * z[0];
      if (p.nu_k != 0.0f) nu_i = nu_i - p.nu_k * logf((v - p.w_offset) / p.wg_ratio + p.g_offset) + p.nu_k * p.log_g0;
      const float delta_t = fmaxf(current_t - t[i], 1.0f);
      const float nu_scale = powf(delta_t, -nu_i);
      v = w0[i] * nu_scale;
      if (p.a != 0.0f) v = v + p.a * (nu_scale - 1.0f);
    }
    if (p.w_read_std > 0.0f) v += p.w_read_std * z[1];
    // saturate (weight_drifter.cpp:98-106): the lower bound first, the upper one wins
    if (w_min) v = fmaxf(v, w_min[i]);
    if (w_max) v = fminf(v, w_max[i]);
    prev[i] = v;
    w[i] = v;
  }
}

// one workgroup per row: largest absolute value (0), sum of squares (1) or sum (2) of the first n_cols columns
__global__ __launch_bounds__(256) void k_row_stat(const float *w, MatLayout lay, int n_cols, int sum_squares,
                                                   float *row_out) {
  __shared__ float sh[4];
  const float *row = w + lay.at((int)blockIdx.x, 0);
  const size_t sj = lay.xd ? (size_t)lay.d_size : 1; // distance between the columns of a row
  float m = 0.0f;
  if (sum_squares == 2) {
    for (int j = threadIdx.x; j < n_cols; j += blockDim.x) m += row[j * sj];
    m = block_sum(m, sh);
  } else if (sum_squares) {
    for (int j = threadIdx.x; j < n_cols; j += blockDim.x) m = __builtin_fmaf(row[j * sj], row[j * sj], m);
    m = block_sum(m, sh);
  } else {
    for (int j = threadIdx.x; j < n_cols; j += blockDim.x) m = fmaxf(m, fabsf(row[j * sj]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
  }
  if (threadIdx.x == 0) row_out[blockIdx.x] = m;
}

__device__ __forceinline__ float block_max(float v, float *sh) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r = fmaxf(r, sh[i]);
  return r;
}

__global__ __launch_bounds__(256) void k_max_or_one(const float *v, int n, float *out) {
  __shared__ float sh[4];
  float m = 0.0f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) m = fmaxf(m, v[i]);
  m = block_max(m, sh);
  if (threadIdx.x == 0) *out = m > 0.0f ? m : 1.0f;
}

// One workgroup: the per-row factors of a remap and the new scales.  The weights then become w * mul / div, which
// is the reference's w / f with mul = 1, and its w * old_scale / new_scale under a bounded scale range.
__global__ __launch_bounds__(256) void k_remap_factors(float *scales, const float *row_stat, float *mul, float *div,
                                                        int d_size, RemapDev p) {
  __shared__ float sh[4];
  if (p.type == RPU_REMAP_LAYERWISE_SYMMETRIC) {
    float m = 0.0f;
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) m = fmaxf(m, row_stat[i]);
    float amax = block_max(m, sh) / p.remapped_wmax;
    if (!(amax > 0.0f)) amax = 1.0f;
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) {
      if (amax != 1.0f) scales[i] *= amax;
      mul[i] = 1.0f;
      div[i] = amax;
    }
  } else if (p.type == RPU_REMAP_CHANNELWISE_SYMMETRIC && !(p.max_scale_range > 0.0f)) {
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) {
      float amax = row_stat[i];
      if (p.remapped_wmax != 1.0f) amax /= p.remapped_wmax;
      const float f = amax > 0.0f ? amax : 1.0f;
      scales[i] *= f;
      mul[i] = 1.0f;
      div[i] = f;
    }
  } else if (p.type == RPU_REMAP_CHANNELWISE_SYMMETRIC) {
    // bounded spread of the scales: no scale may exceed max_scale_range times the smallest one
    float mn = 3.4028234664e38f;
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) mn = fminf(mn, scales[i]);
    float min_scale = fmaxf(-block_max(-mn, sh), 0.0f);
    if (min_scale > 0.0f && p.max_scale_ref != 0.0f) min_scale = fmaxf(min_scale, p.max_scale_ref);
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) {
      const float amax = row_stat[i];
      const float old_scale = scales[i];
      float new_scale = amax > 0.0f ? amax * old_scale : old_scale;
      if (min_scale > 0.0f && new_scale / min_scale > p.max_scale_range) new_scale = min_scale * p.max_scale_range;
      scales[i] = new_scale;
      mul[i] = old_scale;
      div[i] = new_scale;
    }
  } else { // RPU_REMAP_CHANNELWISE_NORM: row_stat holds the sums of squares
    for (int i = threadIdx.x; i < d_size; i += blockDim.x) {
      float nm = sqrtf(row_stat[i]);
      nm = nm > 0.0f ? nm : 1.0f;
      nm /= p.row_norm;
      nm = nm > 1.0f ? nm : 1.0f;
      if (!p.clip_if) scales[i] *= nm;
      mul[i] = 1.0f;
      div[i] = nm;
    }
  }
}

__global__ __launch_bounds__(256) void k_remap_apply(float *w, const float *mul, const float *div, MatLayout lay, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const int r = lay.row_of(i);
    w[i] = w[i] * mul[r] / div[r];
  }
}

// getDiscretizedValueRound (utility_functions.h:195-202)
__device__ __forceinline__ float discretize(float v, float res, int sto_round, float u) {
  if (res <= 0.0f) return v;
  return sto_round ? roundf(v / res + (u - 0.5f)) * res : roundf(v / res) * res;
}

// WeightModifier::apply (weight_modifier.cpp:28-224).  One Philox call per element: words 0, 1 give the normal
// draw, word 2 the stochastic rounding, word 3 the dropped connections.
__global__ __launch_bounds__(256) void k_modify(float *out, const float *w, ModifierDev p, const float *amax_dev,
                                                 PhiloxKey key, uint32_t call, MatLayout lay, size_t n) {
  const float amax = amax_dev ? *amax_dev : p.assumed_wmax;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float v = w[i];
    if (p.copy_last_column && lay.col_of(i) == lay.x_size - 1) {
      out[i] = v;
      continue;
    }
    const Philox4 r = philox4x32_10((uint32_t)i, (uint32_t)(i >> 32), call, RNG_MODIFIER, key.k0, key.k1);
    float z, z_unused;
    box_muller(r.v[0], r.v[1], z, z_unused);
    const float u = u32_to_uniform(r.v[2]);
    switch (p.type) {
    case RPU_MODIFIER_DISCRETIZE:
      if (p.res > 0.0f) v = amax * discretize(v / amax, p.res, p.sto_round, u);
      break;
    case RPU_MODIFIER_MULT_NORMAL:
      if (p.std_dev > 0.0f) v += v * (p.std_dev * amax) * z;
      break;
    case RPU_MODIFIER_ADD_NORMAL:
      if (p.std_dev > 0.0f) v += (p.std_dev * amax) * z;
      break;
    case RPU_MODIFIER_DISCRETIZE_ADD_NORMAL:
      if (p.res > 0.0f || p.std_dev * amax > 0.0f) {
        v = amax * discretize(v / amax, p.res, p.sto_round, u);
        v = v + (p.std_dev * amax) * z;
      }
      break;
    case RPU_MODIFIER_DOREFA:
      if (p.res > 0.0f) {
        const float scale = fabsf(p.dorefa_clip / tanhf(amax));
        v = discretize(tanhf(v) * scale, p.res, p.sto_round, u);
      }
      break;
    case RPU_MODIFIER_POLY:
    case RPU_MODIFIER_PROG_NOISE:
      if (p.std_dev > 0.0f && p.n_coeffs > 0) {
        const float aw = fabsf(v) / amax;
        float paw = 1.0f, sig = p.coeffs[0];
        for (int c = 1; c < p.n_coeffs; ++c) {
          paw *= aw;
          sig += p.coeffs[c] * paw;
        }
        if (p.type == RPU_MODIFIER_POLY) {
          sig *= p.std_dev;
          v += amax * sig * z;
        } else {
          // the noise never changes the sign of a weight
          sig *= p.std_dev / p.g_max;
          const float noisy = fabsf(v + amax * sig * z);
          v = v < 0.0f ? -noisy : noisy;
        }
      }
      break;
    default: // copy, drop connect
      break;
    }
    if (p.pdrop > 0.0f && u32_to_uniform(r.v[3]) < p.pdrop) v = 0.0f;
    out[i] = v;
  }
}

int grid_for(size_t n) {
  const size_t blocks = (n + 255) / 256;
  return (int)(blocks > 8192 ? 8192 : (blocks ? blocks : 1));
}

} // namespace

void launch_decay_device(float *w, const float *decay_scale, const float *reset_bias, const float *w_min,
                         const float *w_max, float alpha, int bias_no_decay, const MatLayout &lay, hipStream_t s) {
  const size_t n = lay.size();
  hipLaunchKernelGGL(k_decay_device, dim3(grid_for(n)), dim3(256), 0, s, w, decay_scale, reset_bias, w_min, w_max, alpha,
                     bias_no_decay, lay, n);
}

void launch_decay_scalar(float *w, float scale, int bias_no_decay, const MatLayout &lay, hipStream_t s) {
  const size_t n = lay.size();
  hipLaunchKernelGGL(k_decay_scalar, dim3(grid_for(n)), dim3(256), 0, s, w, scale, bias_no_decay, lay, n);
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

void launch_clip_value_channel(const float *w, const MatLayout &lay, float fixed_value, float *row_max, float *clip_out,
                               hipStream_t s) {
  hipLaunchKernelGGL(k_row_abs_max, dim3(lay.d_size), dim3(256), 0, s, w, lay, row_max);
  hipLaunchKernelGGL(k_clip_value_channel, dim3(1), dim3(256), 0, s, row_max, lay.d_size, fixed_value, clip_out);
}

void launch_reset_cols(float *w, const float *reset_bias, const float *w_min, const float *w_max, float reset_std,
                       int start_col, int n_cols, float reset_prob, const MatLayout &lay, PhiloxKey key, uint32_t call,
                       hipStream_t s) {
  hipLaunchKernelGGL(k_reset_cols, dim3(grid_for((size_t)lay.d_size * n_cols)), dim3(256), 0, s, w, reset_bias, w_min, w_max,
                     reset_std, start_col, n_cols, reset_prob, lay, key, call);
}

void launch_device_drift(float *w, float *prev, float *w0, float *t, const float *nu, const float *w_min,
                         const float *w_max, const DriftDev &p, float current_t, PhiloxKey key, uint32_t call, size_t n,
                         hipStream_t s) {
  hipLaunchKernelGGL(k_device_drift, dim3(grid_for(n)), dim3(256), 0, s, w, prev, w0, t, nu, w_min, w_max, p, current_t,
                     key, call, n);
}

void launch_row_stat(const float *w, const MatLayout &lay, int n_cols, int sum_squares, float *row_out, hipStream_t s) {
  hipLaunchKernelGGL(k_row_stat, dim3(lay.d_size), dim3(256), 0, s, w, lay, n_cols, sum_squares, row_out);
}

void launch_max_or_one(const float *v, int n, float *out, hipStream_t s) {
  hipLaunchKernelGGL(k_max_or_one, dim3(1), dim3(256), 0, s, v, n, out);
}

void launch_remap(float *w, float *scales, float *row_stat, float *mul, float *div, const MatLayout &lay,
                  const RemapDev &p, hipStream_t s) {
  launch_row_stat(w, lay, lay.x_size, p.type == RPU_REMAP_CHANNELWISE_NORM ? 1 : 0, row_stat, s);
  hipLaunchKernelGGL(k_remap_factors, dim3(1), dim3(256), 0, s, scales, row_stat, mul, div, lay.d_size, p);
  const size_t n = lay.size();
  hipLaunchKernelGGL(k_remap_apply, dim3(grid_for(n)), dim3(256), 0, s, w, mul, div, lay, n);
}

void launch_modify(float *out, const float *w, const ModifierDev &p, const float *amax_dev, PhiloxKey key, uint32_t call,
                   const MatLayout &lay, hipStream_t s) {
  const size_t n = lay.size();
  hipLaunchKernelGGL(k_modify, dim3(grid_for(n)), dim3(256), 0, s, out, w, p, amax_dev, key, call, lay, n);
}

void launch_write_noise_all(float *w_apparent, const float *w_persistent, float noise_std, PhiloxKey key, uint32_t call,
                            size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_write_noise_all, dim3(grid_for((n + 3) / 4)), dim3(256), 0, s, w_apparent, w_persistent, noise_std,
                     key, call, n);
}

// out[c][r] = in[r][c] for a row-major [rows][cols] matrix, 32 x 32 tiles through LDS
__global__ __launch_bounds__(256) void k_transpose(const float *__restrict__ in, float *__restrict__ out, int rows, int cols) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  for (int i = ty; i < 32; i += 8) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[i][tx] = in[(size_t)r * cols + c];
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols) out[(size_t)c * rows + r] = tile[tx][i];
  }
}

void launch_transpose(const float *in, float *out, int rows, int cols, hipStream_t s) {
  hipLaunchKernelGGL(k_transpose, dim3((cols + 31) / 32, (rows + 31) / 32), dim3(256), 0, s, in, out, rows, cols);
}

void launch_delta_finish(float *w, float *prev_w_and_delta, float scale, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_delta_finish, dim3(grid_for(n)), dim3(256), 0, s, w, prev_w_and_delta, scale, n);
}

} // namespace rpu_amd
