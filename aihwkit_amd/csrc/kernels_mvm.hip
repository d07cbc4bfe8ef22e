// Noisy quantized matrix-vector products of the analog tile on gfx950 (CDNA4, wave64).
//
// One "round" is  DAC(in) -> fp32 MFMA contraction with the weights -> ADC(out)  for a batch of
// samples, following the per-sample semantics of the reference CPU path
// (src/rpucuda/rpu_forward_backward_pass.cpp:571-604 DAC, :666-719 ADC, :900-1027 drivers).
// Iterative bound management re-runs only the samples whose ADC saturated, with a halved input
// range, through per-sample state kept in HBM; the host never waits for a round.
//
// Work decomposition of a round: one workgroup (4 waves) owns a 32 (outputs) x 32 (samples) tile of
// the result.  The 4 waves split the contraction length K in four contiguous quarters, each wave
// runs v_mfma_f32_32x32x2_f32 over its quarter straight from global memory (operands are read as
// one float4 per lane and 8 k-values, quantized in registers), the four partial tiles are summed in
// a fixed order through LDS and each wave finishes 8 output rows: noise, quantize, clip, bound
// bookkeeping, rescale, store.  A 1024 x 1024 tile at batch 256 gives 256 workgroups = 1024 waves,
// one per SIMD of the chip.
#include "kernels.h"

namespace rpu_amd {

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int TILE = 32;
constexpr int WAVES = 4;

__device__ __forceinline__ float dac_value(float x, float scale, const IoDev &io, PhiloxKey key,
                                           uint32_t call, int round, int b, int k) {
  // value *= scale; discretize; clip; (+ noise); (asymmetry)      rpu_forward_backward_pass.cpp:583-602
  float v = x * scale;
  if (io.inp_res > 0.0f) {
    float q = v / io.inp_res;
    if (io.inp_sto_round) {
      const Philox4 r = philox4x32_10((uint32_t)k, (uint32_t)b, call, RNG_INP_SR | ((uint32_t)round << 8), key.k0, key.k1);
      q = q + (u32_to_uniform(r.v[0]) - 0.5f);
    }
    v = rintf(q) * io.inp_res;
  }
  v = (v > io.inp_bound) ? io.inp_bound : v;
  v = (v < -io.inp_bound) ? -io.inp_bound : v;
  if (io.inp_noise > 0.0f) {
    float n[4];
    philox_normal4((uint32_t)k, (uint32_t)b, call, RNG_INP_NOISE | ((uint32_t)round << 8), key, n);
    v += io.inp_noise * n[0];
  }
  if (io.inp_asym != 0.0f) {
    v = v < 0.0f ? v * (1.0f - io.inp_asym) : v;
  }
  return v;
}

__global__ __launch_bounds__(256) void k_mvm_round(MvmArgs a) {
  __shared__ float red[WAVES][16][64];

  const int n_act = (a.round > 0) ? a.st.count[a.round] : a.m_batch;
  const int tile_b = blockIdx.y;
  if (tile_b * TILE >= n_act) {
    return; // whole workgroup leaves: no barrier is reached by anyone
  }
  const int tile_o = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;

  // operand rows owned by this lane
  const int o_in = tile_o * TILE + r;
  const bool o_ok = o_in < a.O;
  const int slot_in = tile_b * TILE + r;
  const bool b_ok = slot_in < n_act;
  int b_in = 0;
  if (b_ok) {
    b_in = (a.round > 0) ? a.st.list[a.round & 1][slot_in] : slot_in;
  }
  const float scale_in = (b_ok && !a.io.perfect) ? a.st.scale[b_in] : 1.0f;

  const long w_so = a.transposed ? 1 : a.x_size;
  const long w_sk = a.transposed ? a.x_size : 1;
  const float *w_row = a.w + (long)(o_ok ? o_in : 0) * w_so;
  const float *in_row = a.in + (long)b_in * a.in_sb;

  const int K = a.K;
  const int kq = ((K + 31) / 32) * 8; // per-wave share, a multiple of 8
  const int k_begin = wave * kq;
  const int k_end = min(K, k_begin + kq);

  const bool full8 = (K % 8) == 0;
  const bool vec_w = full8 && (w_sk == 1) && ((a.x_size & 3) == 0) && ((((uintptr_t)a.w) & 15) == 0);
  const bool vec_in = full8 && (a.in_sk == 1) && ((a.in_sb & 3) == 0) && ((((uintptr_t)a.in) & 15) == 0);
  const bool plain_dac = a.io.perfect || (!a.io.inp_sto_round && !(a.io.inp_noise > 0.0f) && a.io.inp_asym == 0.0f);
  const float inp_res = a.io.inp_res;
  const float inp_bound = a.io.inp_bound;

  floatx16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

#pragma unroll 2
  for (int k = k_begin; k < k_end; k += 8) {
    const int kk = k + h * 4;
    float wv[4], xv[4];
    if (vec_w) {
      const float4 t = o_ok ? *reinterpret_cast<const float4 *>(w_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
      wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w;
    } else {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        wv[m] = (o_ok && (kk + m) < k_end) ? w_row[(long)(kk + m) * w_sk] : 0.0f;
      }
    }
    if (vec_in) {
      const float4 t = b_ok ? *reinterpret_cast<const float4 *>(in_row + kk) : make_float4(0.f, 0.f, 0.f, 0.f);
      xv[0] = t.x; xv[1] = t.y; xv[2] = t.z; xv[3] = t.w;
    } else {
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        xv[m] = (b_ok && (kk + m) < k_end) ? in_row[(long)(kk + m) * a.in_sk] : 0.0f;
      }
    }
    if (!a.io.perfect) {
      if (plain_dac) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          float v = xv[m] * scale_in;
          if (inp_res > 0.0f) v = rintf(v / inp_res) * inp_res;
          v = (v > inp_bound) ? inp_bound : v;
          v = (v < -inp_bound) ? -inp_bound : v;
          xv[m] = v;
        }
      } else {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const bool ok = b_ok && (kk + m) < k_end;
          xv[m] = ok ? dac_value(xv[m], scale_in, a.io, a.key, a.call, a.round, b_in, kk + m) : 0.0f;
        }
      }
    }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[m], xv[m], acc, 0, 0, 0);
    }
  }

  // sum the four K-quarters in a fixed order
#pragma unroll
  for (int i = 0; i < 16; ++i) red[wave][i][lane] = acc[i];
  __syncthreads();

  // this wave finishes accumulator group `wave`: rows wave*8 + h*4 + m, column r
  float v[4];
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    const int i = wave * 4 + m;
    v[m] = ((red[0][i][lane] + red[1][i][lane]) + red[2][i][lane]) + red[3][i][lane];
  }
  if (!b_ok) return;
  const int b = b_in;
  const int o0 = tile_o * TILE + wave * 8 + h * 4;
  if (o0 >= a.O) return;

  float *out_p = a.out + (long)b * a.out_sb + (long)o0 * a.out_so;
  if (a.io.perfect) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      if (o0 + m < a.O) {
        float res = a.alpha * v[m];
        if (a.beta != 0.0f) res += a.beta * out_p[(long)m * a.out_so];
        out_p[(long)m * a.out_so] = res;
      }
    }
    return;
  }

  const float fin = a.st.fin[b];
  if (fin == 0.0f) { // zero input: the reference short-cuts to a zero output
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      if (o0 + m < a.O) out_p[(long)m * a.out_so] = 0.0f;
    }
    return;
  }

  float nz[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.io.out_noise > 0.0f) {
    philox_normal4((uint32_t)(o0 >> 2), (uint32_t)b, a.call, RNG_OUT_NOISE | ((uint32_t)a.round << 8), a.key, nz);
  }
  const bool with_bm = a.io.bound_management != RPU_BM_NONE;
  const float bound = a.io.out_bound;
  int up = 0, lo = 0;
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    float y = v[m];
    if (a.io.out_asym > 0.0f) y = y < 0.0f ? y * (1.0f - a.io.out_asym) : y;
    if (a.io.out_noise > 0.0f) y += a.io.out_noise * nz[m];
    if (a.io.out_res > 0.0f) {
      float q = y / a.io.out_res;
      if (a.io.out_sto_round) {
        const Philox4 rr = philox4x32_10((uint32_t)(o0 + m), (uint32_t)b, a.call, RNG_OUT_SR | ((uint32_t)a.round << 8), a.key.k0, a.key.k1);
        q = q + (u32_to_uniform(rr.v[0]) - 0.5f);
      }
      y = rintf(q) * a.io.out_res;
    }
    if (y > bound) {
      y = bound;
      if (o0 + m < a.O) up = o0 + m + 1;
    } else if (y < -bound) {
      y = -bound;
      if (o0 + m < a.O) lo = o0 + m + 1;
    }
    v[m] = y * fin;
  }
  if (with_bm) {
    if (up) atomicMax(&a.st.hit_up[b], up);
    if (lo) atomicMax(&a.st.hit_lo[b], lo);
  }
  if (a.out_so == 1 && (o0 + 3) < a.O && ((((uintptr_t)out_p) & 15) == 0)) {
    *reinterpret_cast<float4 *>(out_p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      if (o0 + m < a.O) out_p[(long)m * a.out_so] = v[m];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// per-sample noise management and state of round 0.  One workgroup per sample.
// rpu_forward_backward_pass.cpp:112-178 (scales), :919-969 (forward), :1003-1022 (backward)

__device__ __forceinline__ float block_reduce_max(float v, float *sh) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r = fmaxf(r, sh[i]);
  __syncthreads();
  return r;
}

__device__ __forceinline__ float block_reduce_sum(float v, float *sh) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = sh[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) r += sh[i];
  __syncthreads();
  return r;
}

__device__ __forceinline__ void set_round_scales(const MvmArgs &a, int b, float nm, float red) {
  const IoDev &io = a.io;
  const bool use_nm = io.noise_management != RPU_NM_NONE;
  const bool bm = io.bound_management != RPU_BM_NONE;
  if (a.transposed) {
    // backward: scale = 1 / nm ; result *= out_scale * nm
    if (use_nm && nm <= 0.0f) {
      a.st.scale[b] = 0.0f;
      a.st.fin[b] = 0.0f;
      return;
    }
    a.st.scale[b] = use_nm ? 1.0f / nm : 1.0f;
    a.st.fin[b] = use_nm ? io.out_scale * nm : io.out_scale;
    return;
  }
  if (use_nm && nm <= 0.0f && io.inp_noise <= 0.0f) {
    a.st.scale[b] = 0.0f;
    a.st.fin[b] = 0.0f;
    return;
  }
  float scale = 1.0f;
  if (use_nm && nm > 0.0f) scale /= nm;
  if (bm) scale /= red;
  a.st.scale[b] = scale;
  a.st.fin[b] = io.out_scale / scale;
}

__global__ __launch_bounds__(256) void k_mvm_init(MvmArgs a) {
  __shared__ float sh[8];
  const int b = blockIdx.x;
  const IoDev &io = a.io;
  const float *row = a.in + (long)b * a.in_sb;
  float nm = 1.0f;
  if (io.noise_management == RPU_NM_ABS_MAX || io.noise_management == RPU_NM_ABS_MAX_NP_SUM ||
      io.bound_management == RPU_BM_ITERATIVE_WORST_CASE || io.noise_management == RPU_NM_MAX) {
    float amax = 0.0f, vmax = -INFINITY, ps = 0.0f, ns = 0.0f;
    for (int k = threadIdx.x; k < a.K; k += blockDim.x) {
      const float x = row[(long)k * a.in_sk];
      amax = fmaxf(amax, fabsf(x));
      vmax = fmaxf(vmax, x);
      ps += x > 0.0f ? x : 0.0f;
      ns += x < 0.0f ? x : 0.0f;
    }
    amax = block_reduce_max(amax, sh);
    if (io.noise_management == RPU_NM_MAX) {
      vmax = block_reduce_max(vmax, sh);
      nm = io.nm_thres > 0.0f ? fminf(vmax, io.nm_thres) : vmax;
    } else {
      nm = io.nm_thres > 0.0f ? fminf(amax, io.nm_thres) : amax;
    }
    if (io.noise_management == RPU_NM_ABS_MAX_NP_SUM || io.bound_management == RPU_BM_ITERATIVE_WORST_CASE) {
      ps = block_reduce_sum(ps, sh);
      ns = block_reduce_sum(ns, sh);
      const float bound = isinf(io.out_bound) ? 1.0f : io.out_bound;
      const float sum = fmaxf(ps, -ns);
      const float am = io.nm_thres > 0.0f ? fminf(amax, io.nm_thres) : amax;
      float np = sum * io.nm_assumed_wmax / bound;
      if (io.inp_res > 0.0f) np = fminf(am / io.inp_res * io.max_bm_res, np);
      np = fmaxf(am, np);
      if (io.noise_management == RPU_NM_ABS_MAX_NP_SUM) nm = np;
      if (threadIdx.x == 0) a.st.nm_np[b] = np;
    }
  } else if (io.noise_management == RPU_NM_CONSTANT) {
    nm = io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
  }
  if (threadIdx.x == 0) {
    a.st.nm[b] = nm;
    a.st.red[b] = 1.0f;
    a.st.hit_up[b] = 0;
    a.st.hit_lo[b] = 0;
    set_round_scales(a, b, nm, 1.0f);
    a.st.rounds[b] = (a.st.fin[b] == 0.0f) ? 0 : 1;
  }
  if (b == 0 && threadIdx.x < 40) a.st.count[threadIdx.x] = 0;
}

// After round a.round: samples whose ADC saturated get another round unless the reduction limit is
// reached (rpu_forward_backward_pass.cpp:944-983).
__global__ __launch_bounds__(256) void k_mvm_advance(MvmArgs a) {
  const int n_act = (a.round > 0) ? a.st.count[a.round] : a.m_batch;
  const int slot = blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= n_act) return;
  const int b = (a.round > 0) ? a.st.list[a.round & 1][slot] : slot;
  const IoDev &io = a.io;
  const int up = a.st.hit_up[b], lo = a.st.hit_lo[b];
  a.st.hit_up[b] = 0;
  a.st.hit_lo[b] = 0;
  if (a.st.fin[b] == 0.0f) return;
  // the CPU loop sets "failed" on an upper hit and *assigns* !bm_test_negative_bound on a lower hit,
  // walking the outputs in index order: the last hit decides
  const bool failed = io.bm_test_negative_bound ? (up > 0 || lo > 0) : (up > lo);
  if (!failed) return;
  float red = a.st.red[b];
  const bool stop = ((int)red > io.max_bm_factor) || ((io.inp_res > 0.0f) && (red > io.max_bm_res / io.inp_res));
  if (stop) return;
  red *= 2.0f;
  float nm = a.st.nm[b];
  if (a.round == 0 && io.bound_management == RPU_BM_ITERATIVE_WORST_CASE &&
      io.noise_management != RPU_NM_ABS_MAX_NP_SUM) {
    nm = a.st.nm_np[b];
    a.st.nm[b] = nm;
    red = 1.0f;
  }
  a.st.red[b] = red;
  a.st.rounds[b] += 1;
  set_round_scales(a, b, nm, red);
  const int pos = atomicAdd(&a.st.count[a.round + 1], 1);
  a.st.list[(a.round + 1) & 1][pos] = b;
}

__global__ void k_make_bias(const float *in, float *out, int m_batch, int x_size, int in_trans) {
  const long n = (long)m_batch * x_size;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n; idx += (long)gridDim.x * blockDim.x) {
    const int b = (int)(idx / x_size);
    const int j = (int)(idx % x_size);
    float v = 1.0f;
    if (j < x_size - 1) v = in_trans ? in[(long)j * m_batch + b] : in[(long)b * (x_size - 1) + j];
    out[idx] = v;
  }
}

__global__ void k_drop_bias(const float *in, float *out, int m_batch, int x_size, int out_trans) {
  const long n = (long)m_batch * (x_size - 1);
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n; idx += (long)gridDim.x * blockDim.x) {
    const int b = (int)(idx / (x_size - 1));
    const int j = (int)(idx % (x_size - 1));
    const float v = in[(long)b * x_size + j];
    if (out_trans) out[(long)j * m_batch + b] = v;
    else out[idx] = v;
  }
}

} // namespace

int mvm_max_rounds(const IoDev &io) {
  if (io.perfect || io.bound_management == RPU_BM_NONE) return 1;
  // round r (0-based) runs with reduction 2^r; it is the last one when the stop test holds for it.
  // IterativeWorstCase restarts the reduction at 1 in its second round: one more round at most.
  int rounds = 0;
  float red = 1.0f;
  while (rounds < 31) {
    ++rounds;
    const bool stop = ((int)red > io.max_bm_factor) || ((io.inp_res > 0.0f) && (red > io.max_bm_res / io.inp_res));
    if (stop) break;
    red *= 2.0f;
  }
  if (io.bound_management == RPU_BM_ITERATIVE_WORST_CASE) ++rounds;
  return rounds > 32 ? 32 : rounds;
}

void launch_mvm_init(const MvmArgs &a, hipStream_t s) {
  hipLaunchKernelGGL(k_mvm_init, dim3(a.m_batch), dim3(256), 0, s, a);
}

void launch_mvm_round(const MvmArgs &a, hipStream_t s) {
  dim3 grid((a.O + TILE - 1) / TILE, (a.m_batch + TILE - 1) / TILE);
  hipLaunchKernelGGL(k_mvm_round, grid, dim3(256), 0, s, a);
}

void launch_mvm_advance(const MvmArgs &a, hipStream_t s) {
  hipLaunchKernelGGL(k_mvm_advance, dim3((a.m_batch + 255) / 256), dim3(256), 0, s, a);
}

void launch_make_bias(const float *in, float *out, int m_batch, int x_size, int in_trans, hipStream_t s) {
  const long n = (long)m_batch * x_size;
  const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
  hipLaunchKernelGGL(k_make_bias, dim3(blocks), dim3(256), 0, s, in, out, m_batch, x_size, in_trans);
}

void launch_drop_bias(const float *in, float *out, int m_batch, int x_size, int out_trans, hipStream_t s) {
  const long n = (long)m_batch * (x_size - 1);
  const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
  hipLaunchKernelGGL(k_drop_bias, dim3(blocks), dim3(256), 0, s, in, out, m_batch, x_size, out_trans);
}

} // namespace rpu_amd
