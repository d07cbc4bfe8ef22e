// Analog non-idealities of the MVM that act on the sums before the ADC stage: output-referred weight noise
// (ForwardBackwardPassIOManaged::applyOutputWeightNoise, rpu_forward_backward_pass.cpp:325-385) and IR drop
// (applyIrDrop, :387-433, with computeTotalCurrent, :508-530).  Each of them needs one or two more contractions of
// the same shape as the MVM itself, over transformed operands (|W| with x^2 or |x|, W with position-weighted x);
// those run on the MFMA round kernel.  The kernels here make the transformed operands and combine the results
// into the one addend per output that the ADC stage of the round kernel reads.
#include "kernels.h"

namespace rpu_amd {

namespace {

int grid_for(size_t n) {
  const size_t blocks = (n + 255) / 256;
  return (int)(blocks > 8192 ? 8192 : (blocks ? blocks : 1));
}

__global__ __launch_bounds__(256) void k_side_rows(const float *xq, float *out, size_t total, int k_pad, int K, int mode,
                                                    int part, const int *skip_if_zero) {
  if (skip_if_zero && *skip_if_zero == 0) return;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const int j = (int)(i % k_pad);
    float x = xq[i];
    if (part < 0) x = fminf(x, 0.0f);
    if (part > 0) x = fmaxf(x, 0.0f);
    float v;
    if (mode == 0) {
      v = x * x;
    } else if (mode == 1) {
      v = fabsf(x);
    } else if (mode == 2) {
      // lines far from the output see the largest drop: x_j (1 - (1 - j / n)^2)
      const float p = 1.0f - (float)j / (float)K;
      v = x * (1.0f - p * p);
    } else {
      v = x;
    }
    out[i] = j < K ? v : 0.0f;
  }
}

__global__ __launch_bounds__(256) void k_abs_copy(const float *w, float *out, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    out[i] = fabsf(w[i]);
  }
}

__global__ __launch_bounds__(256) void k_mul_copy(const float *w, const float *f, float *out, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    out[i] = w[i] * f[i];
  }
}

// four outputs per thread (one Philox call)
__global__ __launch_bounds__(256) void k_side_combine(float *pre, const float *s_noise, const float *row_sumsq,
                                                       const float *s_cur, const float *s_ir, SideDev p, int rows, int O,
                                                       PhiloxKey key, uint32_t call, int round, const int *skip_if_zero) {
  if (skip_if_zero && *skip_if_zero == 0) return;
  const int quads = (O + 3) / 4;
  const size_t total = (size_t)rows * quads;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const int row = (int)(i / quads);
    const int o0 = (int)(i % quads) * 4;
    const uint32_t sample = p.row_sample ? (uint32_t)p.row_sample[row] : (uint32_t)row; // keys the random draws
    float z[4] = {0.f, 0.f, 0.f, 0.f}, zo[4] = {0.f, 0.f, 0.f, 0.f};
    int hit_u = 0, hit_l = 0;
    const bool noisy = p.w_noise_type != 0 && p.w_noise > 0.0f;
    if (noisy) philox_normal4((uint32_t)(o0 >> 2), sample, call, RNG_W_NOISE | ((uint32_t)round << 8), key, z);
    const bool total = p.s_y != nullptr;
    const bool out_noisy = total && (p.out_noise != nullptr || p.out_noise_all > 0.0f);
    if (out_noisy) philox_normal4((uint32_t)(o0 >> 2), sample, call, RNG_OUT_NOISE | ((uint32_t)round << 8), key, zo);
    const float x_norm = (noisy && p.w_noise_type == 1) ? sqrtf(row_sumsq[row]) : 0.0f;
    const float y_ref = (total && p.v_offset && p.v_offset_w_min != 0.0f) ? -p.v_offset_w_min * p.x_accum[row] : 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int o = o0 + q;
      if (o >= O) break;
      const size_t k = (size_t)row * O + o;
      float v = total ? p.s_y[k] : 0.0f;
      if (p.ir_drop > 0.0f) {
        // a_i = sum_j |w_ij| |x_j| n / (Gw / g_max); c_i = a_i (a_i (0.05 a_i - 0.2) + 0.5)
        const float a = p.a_scale * s_cur[k];
        const float c = a * (a * (0.05f * a - 0.2f) + 0.5f);
        v -= c * (p.ir_drop * s_ir[k]);
      }
      if (total && p.v_offset) {
        const float vo = p.v_offset[o];
        const float rs = fmaxf(p.r_series, 0.0f);
        if (p.v_offset_w_min == 0.0f) {
          v = rs <= 0.0f ? v * (1.0f - vo) : (1.0f - vo) * v / (1.0f + fminf(rs * fabsf(v), p.r_series_max_total));
        } else if (rs <= 0.0f) {
          v = v * (1.0f - vo) - vo * (y_ref * 2.0f);
        } else {
          // the positive and the reference line see their own series resistance
          const float y_pos = v + y_ref;
          const float p_nom = 1.0f + fminf(rs * fabsf(y_pos), p.r_series_max_total);
          const float n_nom = 1.0f + fminf(rs * fabsf(y_ref), p.r_series_max_total);
          v = (1.0f - vo) * y_pos / p_nom - (1.0f + vo) * y_ref / n_nom;
        }
      }
      if (noisy) {
        if (p.w_noise_type == 1) v += (p.w_noise * x_norm) * z[q];
        else v += p.w_noise * sqrtf(s_noise[k]) * z[q];
      }
      if (p.add_ni) v += p.add_ni[k];
      if (total && !p.ni_only) {
        if (p.out_nl) v = p.nl_factor * v / (1.0f + fabsf(p.out_nl[o] * v));
        if (p.out_asym > 0.0f) v = v < 0.0f ? v * (1.0f - p.out_asym) : v;
        if (out_noisy) v += (p.out_noise ? p.out_noise[o] : p.out_noise_all) * zo[q];
      }
      if (p.adc_here) {
        // this pass's own ADC (finalizeOutput, rpu_forward_backward_pass.cpp:666-719)
        if (p.adc_res > 0.0f) {
          float qq = v / p.adc_res;
          if (p.adc_sto_round) {
            const Philox4 rr = philox4x32_10((uint32_t)o, sample, call, RNG_OUT_SR | ((uint32_t)round << 8), key.k0, key.k1);
            qq = qq + (u32_to_uniform(rr.v[0]) - 0.5f);
          }
          v = rintf(qq) * p.adc_res;
        }
        const bool over = v > p.adc_bound, under = v < -p.adc_bound;
        v = over ? p.adc_bound : (under ? -p.adc_bound : v);
        if (over) hit_u = o + 1;
        if (under) hit_l = o + 1;
      }
      pre[k] = v;
    }
    if (p.hit_up) {
      if (hit_u) atomicMax(&p.hit_up[row], hit_u);
      if (hit_l) atomicMax(&p.hit_lo[row], hit_l);
    }
  }
}

__global__ __launch_bounds__(256) void k_side_row_samples(int *row_sample, const int *list, const int *row, const int *count,
                                                           int rows) {
  const int n = min(*count, rows);
  for (int pos = blockIdx.x * blockDim.x + threadIdx.x; pos < n; pos += gridDim.x * blockDim.x) {
    const int r = row[pos];
    if (r >= 0 && r < rows) row_sample[r] = list[pos];
  }
}

} // namespace

void launch_side_row_samples(int *row_sample, const int *list, const int *row, const int *count, int rows, hipStream_t s) {
  hipLaunchKernelGGL(k_side_row_samples, dim3(grid_for((size_t)rows)), dim3(256), 0, s, row_sample, list, row, count, rows);
}

void launch_side_rows(const float *xq, float *out, int rows, int k_pad, int K, int mode, int part, const int *skip_if_zero,
                      hipStream_t s) {
  const size_t total = (size_t)rows * k_pad;
  hipLaunchKernelGGL(k_side_rows, dim3(grid_for(total)), dim3(256), 0, s, xq, out, total, k_pad, K, mode, part,
                     skip_if_zero);
}

void launch_abs_copy(const float *w, float *out, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_abs_copy, dim3(grid_for(n)), dim3(256), 0, s, w, out, n);
}

void launch_mul_copy(const float *w, const float *factors, float *out, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_mul_copy, dim3(grid_for(n)), dim3(256), 0, s, w, factors, out, n);
}

void launch_side_combine(float *pre, const float *s_noise, const float *row_sumsq, const float *s_cur, const float *s_ir,
                         const SideDev &p, int rows, int O, PhiloxKey key, uint32_t call, int round,
                         const int *skip_if_zero, hipStream_t s) {
  const size_t total = (size_t)rows * ((O + 3) / 4);
  hipLaunchKernelGGL(k_side_combine, dim3(grid_for(total)), dim3(256), 0, s, pre, s_noise, row_sumsq, s_cur, s_ir, p,
                     rows, O, key, call, round, skip_if_zero);
}

} // namespace rpu_amd
