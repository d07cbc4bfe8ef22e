// Inference weight pipeline on gfx950: statistical PCM programming noise, conductance drift and accumulated
// 1/f read noise applied to the HBM-resident weight matrix (the reference does this in torch on the host side
// of its bindings: src/aihwkit/inference/noise/pcm.py:100-158 over
// src/aihwkit/inference/converter/conductance.py:51-82).  Element-wise kernels, one read and one write of each
// array: HBM-bound.  Every normal is a Philox draw keyed by (element, call), so a seed reproduces a run.
// The file also holds the gather / fold / permute kernels of the indexed (convolution) interface.
#include "kernels.h"

#include <algorithm>

namespace rpu_amd {

namespace {

constexpr float ZERO_CLIP = 1e-7f;

__global__ __launch_bounds__(256) void k_abs_max(const float *w, size_t n, uint32_t *out_bits) {
  __shared__ float sh[4];
  float m = 0.0f;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    m = fmaxf(m, fabsf(w[i]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    atomicMax(out_bits, __float_as_uint(m));
  }
}

__global__ void k_zero_u32(uint32_t *p) { p[0] = 0u; }

// weights -> (g_plus, g_minus): conductance.py:51-63
__device__ __forceinline__ void to_conductances(float w, float ratio, const PcmDev &p, float &gp, float &gm) {
  const float sw = w * ratio;
  gp = fminf(fmaxf(sw, 0.0f), p.g_max) + p.g_min;
  gm = fminf(fmaxf(-sw, 0.0f), p.g_max) + p.g_min;
}

// pcm.py:100-117
__device__ __forceinline__ float program_conductance(float g, const PcmDev &p, float normal) {
  const float rel = g / p.g_max;
  float mat = rel;
  float sig = p.c0 + mat * p.c1;
  mat *= rel;
  sig += mat * p.c2;
  sig *= p.sig_scale;
  return fmaxf(g + p.prog_noise_scale * sig * normal, 0.0f);
}

// pcm.py:119-131
__device__ __forceinline__ float drift_coefficient(float g, const PcmDev &p, float normal) {
  const float rel = fmaxf(fabsf(g / p.g_max), ZERO_CLIP);
  const float lg = logf(rel);
  const float mu = fminf(fmaxf(-0.0155f * lg + 0.0244f, 0.049f), 0.1f);
  const float sd = fminf(fmaxf(-0.0125f * lg - 0.0059f, 0.008f), 0.045f);
  return fmaxf(fabsf(mu + sd * normal), 0.0f) * p.drift_scale;
}

__global__ __launch_bounds__(256) void k_pcm_program(const float *w_ref, float *w_prog, float *nu_plus, float *nu_minus,
                                                      size_t n, const uint32_t *abs_max_bits, PcmDev p, PhiloxKey key,
                                                      uint32_t call) {
  const float abs_max = __uint_as_float(abs_max_bits[0]);
  const float ratio = (p.g_max - p.g_min) / fmaxf(abs_max, ZERO_CLIP);
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float gp, gm;
    to_conductances(w_ref[i], ratio, p, gp, gm);
    float nz[4];
    philox_normal4((uint32_t)i, (uint32_t)(i >> 32), call, RNG_PCM_PROGRAM, key, nz);
    const float gp_prog = program_conductance(gp, p, nz[0]);
    const float gm_prog = program_conductance(gm, p, nz[1]);
    nu_plus[i] = drift_coefficient(gp, p, nz[2]);
    nu_minus[i] = drift_coefficient(gm, p, nz[3]);
    w_prog[i] = ((gp_prog - p.g_min) - (gm_prog - p.g_min)) / ratio; // conductance.py:65-82
  }
}

// pcm.py:133-158
__device__ __forceinline__ float drift_conductance(float g, float nu, const PcmDev &p, float normal) {
  const float g_drift = p.drift_base_log2 > 0.0f ? g * exp2f(-nu * p.drift_base_log2) : g;
  if (p.read_sigma < 0.0f) return fmaxf(g, 0.0f);
  const float q = fminf(0.0088f / fmaxf(powf(fabsf(g) / p.g_max, 0.65f), 1e-3f), 0.2f);
  const float sig = q * p.read_sigma;
  return fmaxf(g_drift + fabsf(g_drift) * p.read_noise_scale * sig * normal, 0.0f);
}

__global__ __launch_bounds__(256) void k_pcm_drift(const float *w_prog, const float *nu_plus, const float *nu_minus,
                                                    float *w_out, size_t n, const uint32_t *abs_max_bits, PcmDev p,
                                                    PhiloxKey key, uint32_t call) {
  const float abs_max = __uint_as_float(abs_max_bits[0]);
  const float ratio = (p.g_max - p.g_min) / fmaxf(abs_max, ZERO_CLIP);
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float gp, gm;
    to_conductances(w_prog[i], ratio, p, gp, gm);
    float nz[4];
    philox_normal4((uint32_t)i, (uint32_t)(i >> 32), call, RNG_PCM_DRIFT, key, nz);
    const float gp_f = drift_conductance(gp, nu_plus[i], p, nz[0]);
    const float gm_f = drift_conductance(gm, nu_minus[i], p, nz[1]);
    w_out[i] = ((gp_f - p.g_min) - (gm_f - p.g_min)) / ratio;
  }
}

// One workgroup, so that the order of the sum is fixed; eight 16-byte loads per thread are in flight at a time (one
// load per trip made the kernel a chain of 256 memory latencies for a 512 x 512 tile).
__global__ __launch_bounds__(1024) void k_mean_abs(const float *v, size_t n, float *out) {
  __shared__ float sh[16];
  float acc = 0.0f;
  size_t done = 0;
  if ((((uintptr_t)v) & 15) == 0) {
    const size_t n4 = n >> 2;
    const float4 *v4 = reinterpret_cast<const float4 *>(v);
    float part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = 0.0f;
    for (size_t q0 = 0; q0 < n4; q0 += 8 * (size_t)blockDim.x) {
      float4 t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const size_t q = q0 + (size_t)u * blockDim.x + threadIdx.x;
        t[u] = q < n4 ? v4[q] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) part[u] += (fabsf(t[u].x) + fabsf(t[u].y)) + (fabsf(t[u].z) + fabsf(t[u].w));
    }
    acc = ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
    done = 4 * n4;
  }
  for (size_t i = done + threadIdx.x; i < n; i += blockDim.x) acc += fabsf(v[i]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.0f;
    for (int k = 0; k < 16; ++k) total += sh[k];
    out[0] = total / (float)n;
  }
}

// Patch matrix of the images: entry (p, k) of image n is the image element that the index names, 0 or 1 (bias row).
// A workgroup moves a block of 64 patches x 64 lines through LDS: it reads with lanes along the patches, the order
// of the index matrix [x_size][patches] and, for a convolution, of the image rows (neighbouring patches read
// neighbouring elements), and writes with lanes along the lines, the order of the rows of x_mat.
__global__ __launch_bounds__(256) void k_gather_indexed(float *x_mat, const float *images, const int *indices, int x_size,
                                                         int x_ld, int patches, int n_images, long image_size) {
  __shared__ float tile[64][65];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int blocks_p = (patches + 63) / 64;
  const int p0 = (int)(blockIdx.x % blocks_p) * 64, k0 = (int)(blockIdx.x / blocks_p) * 64;
  for (int n = blockIdx.y; n < n_images; n += gridDim.y) {
    const float *image = images + (size_t)n * image_size;
    int j[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int k = k0 + wave * 16 + i, p = p0 + lane;
      j[i] = (k < x_size && p < patches) ? indices[(size_t)k * patches + p] : 0;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) tile[lane][wave * 16 + i] = (j[i] <= 1) ? (float)j[i] : image[j[i] - 2];
    __syncthreads();
    float *dst = x_mat + ((size_t)n * patches + p0) * x_ld + k0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = i * 4 + wave;
      if (p0 + row < patches && k0 + lane < x_size) dst[(size_t)row * x_ld + lane] = tile[row][lane];
    }
    __syncthreads();
  }
}

// [image][line][patch] -> [(image, patch)][line]: the gradient rows of the samples of an indexed update
__global__ __launch_bounds__(256) void k_ndp_bd(float *dst, const float *src, int n_images, int d_size, int patches) {
  const size_t total = (size_t)n_images * d_size * patches;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    // idx walks the destination with unit stride
    const int d = (int)(idx % d_size);
    const size_t b = idx / d_size;
    const int p = (int)(b % patches);
    const size_t n = b / patches;
    dst[idx] = src[(n * d_size + d) * patches + p];
  }
}

// [image][line][patch] <-> [line][image][patch]: runs of `patches` elements move as they are
__global__ __launch_bounds__(256) void k_images_lines(float *dst, const float *src, int n_images, int lines, int patches,
                                                       int to_lines) {
  const size_t total = (size_t)n_images * lines * patches;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int p = (int)(idx % patches);
    const size_t r = idx / patches;
    // idx walks the destination with unit stride
    if (to_lines) {
      const int n = (int)(r % n_images), l = (int)(r / n_images);
      dst[idx] = src[((size_t)n * lines + l) * patches + p];
    } else {
      const int l = (int)(r % lines), n = (int)(r / lines);
      dst[idx] = src[((size_t)l * n_images + n) * patches + p];
    }
  }
}

__global__ void k_fill(float *p, float value, size_t n) {
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) p[idx] = value;
}

int grid_of(size_t n) {
  size_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

} // namespace

void launch_abs_max(const float *w, size_t n, uint32_t *abs_max_bits, hipStream_t s) {
  hipLaunchKernelGGL(k_zero_u32, dim3(1), dim3(1), 0, s, abs_max_bits);
  hipLaunchKernelGGL(k_abs_max, dim3(grid_of(n)), dim3(256), 0, s, w, n, abs_max_bits);
}

void launch_pcm_program(const float *w_ref, float *w_prog, float *nu_plus, float *nu_minus, size_t n,
                        const uint32_t *abs_max_bits, const PcmDev &p, PhiloxKey key, uint32_t call, hipStream_t s) {
  hipLaunchKernelGGL(k_pcm_program, dim3(grid_of(n)), dim3(256), 0, s, w_ref, w_prog, nu_plus, nu_minus, n, abs_max_bits,
                     p, key, call);
}

void launch_pcm_drift(const float *w_prog, const float *nu_plus, const float *nu_minus, float *w_out, size_t n,
                      const uint32_t *abs_max_bits, const PcmDev &p, PhiloxKey key, uint32_t call, hipStream_t s) {
  hipLaunchKernelGGL(k_pcm_drift, dim3(grid_of(n)), dim3(256), 0, s, w_prog, nu_plus, nu_minus, w_out, n, abs_max_bits, p,
                     key, call);
}

void launch_gather_indexed(float *x_mat, const float *images, const int *indices, int x_size, int x_ld, int patches,
                           int n_images, long image_size, hipStream_t s) {
  const unsigned blocks = (unsigned)(((patches + 63) / 64) * ((x_size + 63) / 64));
  hipLaunchKernelGGL(k_gather_indexed, dim3(blocks, (unsigned)std::min(n_images, 65535)), dim3(256), 0, s, x_mat, images,
                     indices, x_size, x_ld, patches, n_images, image_size);
}

// Fold of the patch matrix back into the images without atomics: image element e of image n is the sum of the patch
// entries that were gathered from it, listed per element (ptr[e] .. ptr[e + 1] into kp: pairs (k, p) of line and
// patch) in the order of the reference's loop (math_util / rpu.cpp:1130-1141 walks k, then p), added one after the
// other from zero: the same bits on every run, and the reference's.  x_mat is line-major, [x_size][n_images * patches]:
// neighbouring image elements meet the same lines at neighbouring patches, so a wave reads runs of a row.
__global__ __launch_bounds__(256) void k_fold_indexed(float *images, const float *x_mat, const int *ptr, const int2 *kp,
                                                      int patches, int n_images, long image_size) {
  // a thread adds up one image element of four images: the list entries are read once for the four
  constexpr int NI = 4;
  const int groups = (n_images + NI - 1) / NI;
  const size_t total = (size_t)groups * image_size;
  const long row = (long)n_images * patches;
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const int n0 = (int)(idx / image_size) * NI;
    const long e = (long)(idx - (size_t)(n0 / NI) * image_size);
    const float *src = x_mat + (long)n0 * patches;
    const int live = min(NI, n_images - n0);
    float acc[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) acc[i] = 0.0f;
    const int t_end = ptr[e + 1];
    for (int t0 = ptr[e]; t0 < t_end; t0 += 4) { // sixteen loads in flight, added in list order
      float v[4][NI];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        long at = 0;
        if (t0 + u < t_end) {
          const int2 q = kp[t0 + u];
          at = (long)q.x * row + q.y;
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) v[u][i] = (t0 + u < t_end && i < live) ? src[at + (long)i * patches] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (t0 + u < t_end) {
#pragma unroll
          for (int i = 0; i < NI; ++i) acc[i] += v[u][i];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      if (i < live) images[(size_t)(n0 + i) * image_size + e] = acc[i];
    }
  }
}

void launch_fold_indexed(float *images, const float *x_mat, const int *ptr, const int *kp, int x_size, int patches,
                         int n_images, long image_size, hipStream_t s) {
  (void)x_size;
  const size_t total = (size_t)((n_images + 3) / 4) * image_size;
  hipLaunchKernelGGL(k_fold_indexed, dim3(grid_of(total)), dim3(256), 0, s, images, x_mat, ptr,
                     reinterpret_cast<const int2 *>(kp), patches, n_images, image_size);
}

void launch_images_to_lines(float *lines_major, const float *images, int n_images, int lines, int patches, hipStream_t s) {
  const size_t total = (size_t)n_images * lines * patches;
  hipLaunchKernelGGL(k_images_lines, dim3(grid_of(total)), dim3(256), 0, s, lines_major, images, n_images, lines, patches, 1);
}

void launch_lines_to_images(float *images, const float *lines_major, int n_images, int lines, int patches, hipStream_t s) {
  const size_t total = (size_t)n_images * lines * patches;
  hipLaunchKernelGGL(k_images_lines, dim3(grid_of(total)), dim3(256), 0, s, images, lines_major, n_images, lines, patches, 0);
}

void launch_ndp_to_bd(float *bd, const float *ndp, int n_images, int d_size, int patches, hipStream_t s) {
  const size_t total = (size_t)n_images * d_size * patches;
  hipLaunchKernelGGL(k_ndp_bd, dim3(grid_of(total)), dim3(256), 0, s, bd, ndp, n_images, d_size, patches);
}

void launch_fill(float *p, float value, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_fill, dim3(grid_of(n)), dim3(256), 0, s, p, value, n);
}

void launch_mean_abs(const float *v, size_t n, float *out, hipStream_t s) {
  hipLaunchKernelGGL(k_mean_abs, dim3(1), dim3(1024), 0, s, v, n, out);
}

} // namespace rpu_amd
