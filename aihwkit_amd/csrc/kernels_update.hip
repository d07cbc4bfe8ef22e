// Pulsed weight update of the analog tile on gfx950.
//
// Stages of one update call over a batch (all on one stream, no host round trip):
//   1. per sample: abs-max of x and d -> bit-line length BL and probability scales A (for d), B (for x)
//      (src/rpucuda/rpu_pulsed_meta_parameter.cpp:152-236),
//   2. per line element and sample: one packed 32-bit pulse word, bit 0 = sign, bits 1..BL = pulses
//      drawn with probability |v| * scale (src/rpucuda/sparse_bit_line_maker.cpp:199-238; word format
//      src/rpucuda/rpu_weight_updater.cpp:297-324),
//   3. per cross-point: walk the samples in batch order, n = popcount(x_word & d_word) coincidences of
//      one sample all have the sign sign(x) * sign(d), apply n device steps
//      (src/rpucuda/rpu_weight_updater.cpp:263-283, rpu_pulsed_device.h:450-459; device steps
//      rpu_constantstep_device.cpp:27-55, rpu_linearstep_device.cpp:112-164).
// The weight matrix and the per-device parameter arrays are row-major [d_size][x_size]; a wavefront
// covers 64 consecutive x of one d row, so the d word of a sample is wave-uniform (scalar load) and
// the x words, weights and parameters are read with unit stride.
#include "kernels.h"
#include "rpu_host.h"

#include <algorithm>
#include <cmath>
#include <mutex>
#include <vector>

namespace rpu_amd {

namespace {

// rpu_pulsed_meta_parameter.cpp:152-181
__device__ __forceinline__ void calc_bl_ab(const UpdateDev &up, int &BL, float &A, float &B, float lr, float dw_min) {
  if (lr == 0.0f) {
    A = 0.0f;
    B = 0.0f;
    BL = 0;
    return;
  }
  if (up.fixed_bl || up.update_bl_management) {
    BL = up.desired_bl;
    A = sqrtf(lr / (dw_min * (float)BL));
    B = A;
  } else {
    if ((dw_min * (float)up.desired_bl) < lr) {
      A = 1.0f;
      B = 1.0f;
      BL = max((int)ceilf(lr / dw_min), 1);
    } else {
      BL = up.desired_bl;
      A = sqrtf(lr / (dw_min * (float)BL));
      B = A;
    }
  }
}

// x and d values of a sample wherever the call keeps them: plain strided matrices, or the image tensors of the indexed
// interface read in place (UpdateArgs::x_index, d_group)
__device__ __forceinline__ float update_x_value(const UpdateArgs &a, int b, int j) {
  if (a.x_index) {
    const int n = b / a.x_group;
    const int idx = a.x_index[(long)(b - n * a.x_group) * a.x_size + j];
    return idx <= 1 ? (float)idx : a.x[(long)n * a.x_gs + (idx - 2)];
  }
  return a.x[(long)b * a.x_sb + (long)j * a.x_sj];
}
__device__ __forceinline__ const float *update_d_row(const UpdateArgs &a, int b) {
  if (a.d_group) {
    const int n = b / a.d_group;
    return a.d + (long)n * a.d_gs + (long)(b - n * a.d_group) * a.d_sb;
  }
  return a.d + (long)b * a.d_sb;
}

// largest absolute value of a line of n elements (element j at v[j * stride]) over the part that thread `t` of `width`
// takes; rows that are contiguous and 16-byte aligned are read four elements at a time
__device__ __forceinline__ float part_abs_max(const float *v, int n, long stride, int t, int width) {
  float m = 0.0f;
  if (stride == 1 && ((((uintptr_t)v) & 15) == 0)) {
    const int n4 = n >> 2;
    const float4 *v4 = reinterpret_cast<const float4 *>(v);
    for (int q = t; q < n4; q += width) {
      const float4 x = v4[q];
      m = fmaxf(fmaxf(m, fmaxf(fabsf(x.x), fabsf(x.y))), fmaxf(fabsf(x.z), fabsf(x.w)));
    }
    for (int j = 4 * n4 + t; j < n; j += width) m = fmaxf(m, fabsf(v[j]));
  } else {
    for (int j = t; j < n; j += width) m = fmaxf(m, fabsf(v[(long)j * stride]));
  }
  return m;
}

// BL, A and B of sample b from the largest |x| and |d| of its lines (rpu_pulsed_meta_parameter.cpp:183-236), by one thread
__device__ __forceinline__ void update_prepare_finish(const UpdateArgs &a, const int b, const float xm, const float dm) {
  const float lr = fabsf(a.lr);
  const float dw_min = a.dev.dw_min;
  int BL;
  float A, B;
  calc_bl_ab(a.up, BL, A, B, lr, dw_min);
  if ((a.up.update_management || a.up.update_bl_management) && lr > 0.0f) {
    if (dm == 0.0f || xm == 0.0f) {
      A = 1.0f;
      B = 1.0f;
      BL = 0;
    } else {
      const float x_val = xm;
      float d_val = a.up.um_grad_scale * dm;
      const float k_val = lr * x_val * d_val / dw_min;
      if (a.up.update_bl_management) {
        BL = (int)ceilf(k_val);
        if (BL > a.up.desired_bl) BL = a.up.desired_bl;
        A = sqrtf(lr / (dw_min * (float)BL));
        B = A;
      }
      if (a.up.update_management) {
        if (k_val > (float)a.up.desired_bl) d_val *= (float)a.up.desired_bl / k_val;
        A *= sqrtf(x_val / d_val);
        B *= sqrtf(d_val / x_val);
      }
    }
  }
  a.bl[b] = BL;
  // largest number of pulse slots in a row of words (a longer bit line takes several rows of 31): this call's slot
  // was zeroed by the previous call, which used the other one
  if (a.kmax) {
    // a running maximum of at most 31: a sample only sends its value when what it reads is still smaller (with
    // hundreds of thousands of samples the atomics on the one word were most of this kernel's time)
    const int mine = min(BL, 31);
    if (mine > 0 && __hip_atomic_load(&a.kmax[a.kmax_slot], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < mine) {
      atomicMax(&a.kmax[a.kmax_slot], mine);
    }
    if (b == 0) a.kmax[a.kmax_slot ^ 1] = 0;
  }
  a.prob_a[b] = A;
  a.prob_b[b] = B;
}

// One workgroup per sample: the loads of both lines are in flight together (a line of 1024 elements is one 16-byte load
// per thread), then one exchange through LDS gives the first thread both maxima and it sets the sample's BL, A, B.
// SUB threads share a sample: the whole workgroup (long lines), a wave, or 16 lanes (the short patch rows of a
// convolution come by the hundred thousand: a workgroup per sample would spend its time being launched)
template <int SUB>
__device__ __forceinline__ void update_prepare_sample(const UpdateArgs &a, const int b, float (*sh)[4]) {
  const int t = threadIdx.x % SUB;
  const bool leader = t == 0;
  float xm = 0.0f, dm = 0.0f;
  if (a.up.update_management || a.up.update_bl_management) {
    if (a.x_index) {
      for (int j = t; j < a.x_size; j += SUB) xm = fmaxf(xm, fabsf(update_x_value(a, b, j)));
    } else {
      xm = part_abs_max(a.x + (long)b * a.x_sb, a.x_size, a.x_sj, t, SUB);
    }
    dm = part_abs_max(update_d_row(a, b), a.d_size, a.d_si, t, SUB);
#pragma unroll
    for (int off = (SUB < 64 ? SUB : 64) / 2; off > 0; off >>= 1) {
      xm = fmaxf(xm, __shfl_xor(xm, off));
      dm = fmaxf(dm, __shfl_xor(dm, off));
    }
    if constexpr (SUB == 256) {
      if ((threadIdx.x & 63) == 0) {
        sh[0][threadIdx.x >> 6] = xm;
        sh[1][threadIdx.x >> 6] = dm;
      }
      __syncthreads();
      if (!leader) return;
      xm = fmaxf(fmaxf(sh[0][0], sh[0][1]), fmaxf(sh[0][2], sh[0][3]));
      dm = fmaxf(fmaxf(sh[1][0], sh[1][1]), fmaxf(sh[1][2], sh[1][3]));
    }
  }
  if (!leader) return;
  update_prepare_finish(a, b, xm, dm);
}

// The lines of the indexed interface read in place, for long batches: one thread per sample, so that neighbouring
// lanes read neighbouring patches -- the line-major index, the gradient tensor and (mostly) the image elements are
// then runs of a row for every load of a wave.
__global__ __launch_bounds__(64) void k_update_prepare_in_place(UpdateArgs a) {
  if (a.row_cost) {
    for (int i = (int)(blockIdx.x * 64u + threadIdx.x); i < a.d_size; i += (int)(gridDim.x * 64u)) a.row_cost[i] = 0;
  }
  const int b = (int)blockIdx.x * 64 + (int)threadIdx.x;
  if (b >= a.m_batch) return;
  float xm = 0.0f, dm = 0.0f;
  if (a.up.update_management || a.up.update_bl_management) {
    const int n = b / a.x_group;
    const int *idx = a.x_index_lines + (b - n * a.x_group);
    const float *image = a.x + (long)n * a.x_gs - 2;
    // eight entries of the index, then the eight elements they name, in flight together
    for (int j0 = 0; j0 < a.x_size; j0 += 8) {
      int at[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) at[u] = (j0 + u < a.x_size) ? idx[(long)(j0 + u) * a.x_group] : 0;
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = at[u] <= 1 ? (float)at[u] : image[at[u]];
#pragma unroll
      for (int u = 0; u < 8; ++u) xm = fmaxf(xm, fabsf(v[u]));
    }
    const float *row = update_d_row(a, b);
    for (int i0 = 0; i0 < a.d_size; i0 += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = (i0 + u < a.d_size) ? row[(long)(i0 + u) * a.d_si] : 0.0f;
#pragma unroll
      for (int u = 0; u < 8; ++u) dm = fmaxf(dm, fabsf(v[u]));
    }
  }
  update_prepare_finish(a, b, xm, dm);
}

template <int SUB>
__global__ __launch_bounds__(256) void k_update_prepare(UpdateArgs a) {
  __shared__ float sh[2][4];
  if (a.row_cost) {
    for (int i = (int)(blockIdx.x * 256u + threadIdx.x); i < a.d_size; i += (int)(gridDim.x * 256u)) a.row_cost[i] = 0;
  }
  const int b = (int)blockIdx.x * (256 / SUB) + (int)threadIdx.x / SUB;
  if (b >= a.m_batch) return; // all SUB threads of a sample leave together
  update_prepare_sample<SUB>(a, b, sh);
}

// The same for several tiles in one launch (all with the same batch): workgroup n works on sample n % m_batch of tile
// n / m_batch.  A tile's arguments are copied out of HBM once, by scalar loads (the tile index is uniform).
__global__ __launch_bounds__(256) void k_update_prepare_group(UpdateGroup g) {
  __shared__ float sh[2][4];
  const int t = (int)blockIdx.x / g.m_batch;
  const UpdateArgs a = g.args[t];
  update_prepare_sample<256>(a, (int)blockIdx.x - t * g.m_batch, sh);
}

__device__ __forceinline__ float discretize_prob(float pp, float res, int sto_round, uint32_t rnd) {
  if (res <= 0.0f) return pp;
  float q = pp / res;
  if (sto_round) q = q + (u32_to_uniform(rnd) - 0.5f);
  return rintf(q) * res;
}

// packed pulse word of line element j (an x line or a d line) for sample b: bit 0 = sign, bits 1..K = pulses;
// `row` numbers the sample's rows of words (pulse slots 31 row + 1 ..), each with its own uniforms
__device__ __forceinline__ uint32_t pulse_word(const UpdateArgs &a, bool is_x, int j, int b, float v, float P, int K,
                                               int row = 0) {
  uint32_t sr = 0;
  if (a.up.res > 0.0f && a.up.sto_round) {
    sr = philox4x32_10((uint32_t)j, (uint32_t)b, a.call, RNG_UPDATE_SR | ((uint32_t)is_x << 8), a.key.k0, a.key.k1).v[0];
  }
  const float PP = discretize_prob(fabsf(v) * P, a.up.res, a.up.sto_round, sr);
  const uint32_t purpose = is_x ? RNG_PULSE_X : RNG_PULSE_D;
  uint32_t word = 0;
  if (PP != 0.0f && K > 0) {
    for (int k0 = 0; k0 < K; k0 += 4) {
      const Philox4 r = philox4x32_10((uint32_t)j, (uint32_t)b, a.call, purpose | ((uint32_t)(8 * row + (k0 >> 2)) << 8), a.key.k0, a.key.k1);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (k0 + q < K && PP > u32_to_uniform(r.v[q])) word |= (2u << (k0 + q));
      }
    }
    word |= (v > 0.0f) ? 0u : 1u;
  }
  return word;
}

// Pulse words and their sample-transposed bit planes in one pass.  A workgroup owns 64 samples x LINES_E line elements
// (x lines first, then d lines): the values are read 4 LINES_E bytes per sample row into LDS, then each wave takes every
// fourth element with its lanes on the 64 samples, so that a ballot over the wave is a plane word; the packed words
// go back through LDS and are written 4 LINES_E bytes per sample row.
// LINES_E = 16 moves whole 64-byte row segments; small launches take 4 elements per workgroup (one per wave) so that
// there are four times as many workgroups.
// bx: number of the workgroup's block of line elements (x blocks first, then d blocks), by: its block of 64 rows of words
// IN_PLACE: the call may read its lines from the tensors of the indexed interface (UpdateArgs::x_index, d_group)
template <int LINES_E, bool IN_PLACE = false>
__device__ __forceinline__ void update_lines_block(const UpdateArgs &a, const int bx, const int by,
                                                   float (*vals)[LINES_E + 1], uint32_t (*wt)[LINES_E + 1]) {
  const int tiles_x = (a.x_size + LINES_E - 1) / LINES_E;
  const bool is_x = bx < tiles_x;
  const int e0 = (is_x ? bx : bx - tiles_x) * LINES_E;
  const int size = is_x ? a.x_size : a.d_size;
  const int b0 = by * 64;
  const float *src = is_x ? a.x : a.d;
  const long s_b = is_x ? a.x_sb : a.d_sb, s_e = is_x ? a.x_sj : a.d_si;
  constexpr int ROWS_PER_PASS = 256 / LINES_E;
  const int col = threadIdx.x % LINES_E, row0 = threadIdx.x / LINES_E;
  const int wps = max(a.words_per_sample, 1);
  if (IN_PLACE && is_x && a.x_index) {
    // patches read in place, a wave on one element of 64 samples: the entries of the line-major index are one run, and
    // so are the image elements they name wherever neighbouring patches are neighbours in the image
    const int rb = threadIdx.x & 63;
    const int b = b0 + rb;
    const int sample = wps > 1 ? b / wps : b;
    const int n = sample / a.x_group;
    const int *idx = a.x_index_lines + (sample - n * a.x_group);
    const float *image = a.x + (long)n * a.x_gs - 2;
    int at[LINES_E / 4];
#pragma unroll
    for (int i = 0; i < LINES_E / 4; ++i) {
      const int e = e0 + (threadIdx.x >> 6) + 4 * i;
      at[i] = (b < a.m_batch && e < size) ? idx[(long)e * a.x_group] : 0;
    }
#pragma unroll
    for (int i = 0; i < LINES_E / 4; ++i) {
      vals[rb][(threadIdx.x >> 6) + 4 * i] = at[i] <= 1 ? (float)at[i] : image[at[i]];
    }
  } else if (IN_PLACE && !is_x && a.d_group) {
    // the [image][output][patch] tensor in place: neighbouring samples are neighbours in memory, so a wave takes one
    // element of 64 samples
    const int rb = threadIdx.x & 63;
    const int b = b0 + rb;
    const int sample = wps > 1 ? b / wps : b;
    const float *row = b < a.m_batch ? update_d_row(a, sample) : a.d;
#pragma unroll
    for (int i = 0; i < LINES_E / 4; ++i) {
      const int c = (threadIdx.x >> 6) + 4 * i;
      const int e = e0 + c;
      vals[rb][c] = (b < a.m_batch && e < size) ? row[(long)e * s_e] : 0.0f;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 64 / ROWS_PER_PASS; ++i) {
      const int rb = row0 + ROWS_PER_PASS * i;
      const int b = b0 + rb, e = e0 + col;
      const int sample = wps > 1 ? b / wps : b;
      vals[rb][col] = (b < a.m_batch && e < size) ? src[(long)sample * s_b + (long)e * s_e] : 0.0f;
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int b = b0 + lane; // row of words
  const bool b_ok = b < a.m_batch;
  const int sample = wps > 1 ? b / wps : b, wrow = wps > 1 ? b - sample * wps : 0;
  const float P = b_ok ? (is_x ? a.prob_b[sample] : a.prob_a[sample]) : 0.0f;
  const int K = b_ok ? min(max(a.bl[sample] - 31 * wrow, 0), 31) : 0;
  const int kmax = a.kmax[a.kmax_slot];
  uint32_t *planes = is_x ? a.x_planes : a.d_planes;
  const int c0 = 2 * by;
  for (int el = wave; el < LINES_E; el += 4) {
    const int e = e0 + el;
    if (e >= size) break; // wave-uniform
    const uint32_t word = b_ok ? pulse_word(a, is_x, e, sample, vals[lane][el], P, K, wrow) : 0u;
    wt[lane][el] = word;
    unsigned long long any = 0ull;
    int passes = 0;
    for (int k = 0; k < kmax; ++k) {
      const unsigned long long m = __ballot((word >> (k + 1)) & 1u);
      any |= m;
      passes += __popcll(m);
      if (lane == 0) {
        planes[((long)c0 * a.plane_slots + k) * size + e] = (uint32_t)m;
        if (c0 + 1 < a.n_chunks) planes[((long)(c0 + 1) * a.plane_slots + k) * size + e] = (uint32_t)(m >> 32);
      }
    }
    // what the pulse loop will spend on this d row for these samples: a pass per pulse, a set-up per sample with pulses
    if (!is_x && a.row_cost && lane == 0 && passes) atomicAdd(&a.row_cost[e], 9 * passes + 4 * __popcll(any));
    const unsigned long long sg = __ballot(word & 1u); // the last slot of a chunk holds the sign bits
    if (lane == 0) {
      const int ks = a.plane_slots - 1;
      planes[((long)c0 * a.plane_slots + ks) * size + e] = (uint32_t)sg;
      if (c0 + 1 < a.n_chunks) planes[((long)(c0 + 1) * a.plane_slots + ks) * size + e] = (uint32_t)(sg >> 32);
    }
  }
  __syncthreads();
  uint32_t *words = is_x ? a.x_words : a.d_words;
#pragma unroll
  for (int i = 0; i < 64 / ROWS_PER_PASS; ++i) {
    const int rb = row0 + ROWS_PER_PASS * i;
    const int bb = b0 + rb, ee = e0 + col;
    if (bb < a.m_batch && ee < size) words[(long)bb * size + ee] = wt[rb][col];
  }
}

// Row-major copy a.w of the [x_size][d_size] matrix a.wt_src for the pulse loop, 32 x 32 tiles through LDS: made by
// workgroups that the launch of the pulse trains carries beyond its own (`first` .. of blockIdx.x), so that it costs no
// launch of its own and runs beside that kernel's work.
__device__ __forceinline__ void update_copy_weights(const UpdateArgs &a, int first, float (*tile)[33]) {
  const int tiles_j = (a.x_size + 31) / 32, tiles_i = (a.d_size + 31) / 32;
  const int workers = ((int)gridDim.x - first) * (int)gridDim.y;
  const int me = ((int)blockIdx.x - first) * (int)gridDim.y + (int)blockIdx.y;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 8 rows of 32 per pass
  for (int t = me; t < tiles_j * tiles_i; t += workers) {
    const int j0 = (t / tiles_i) * 32, i0 = (t % tiles_i) * 32;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = j0 + ty + 8 * r, i = i0 + tx;
      tile[ty + 8 * r][tx] = (j < a.x_size && i < a.d_size) ? a.wt_src[(size_t)j * a.d_size + i] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int i = i0 + ty + 8 * r, j = j0 + tx;
      if (i < a.d_size && j < a.x_size) a.w[(size_t)i * a.x_size + j] = tile[tx][ty + 8 * r];
    }
    __syncthreads();
  }
}

template <int LINES_E, bool IN_PLACE = false>
__global__ __launch_bounds__(256) void k_update_lines(UpdateArgs a) {
  __shared__ float vals[64][LINES_E + 1];
  __shared__ uint32_t wt[64][LINES_E + 1];
  const int own = (a.x_size + LINES_E - 1) / LINES_E + (a.d_size + LINES_E - 1) / LINES_E;
  if ((int)blockIdx.x >= own) { // only launched with a.wt_src set
    __shared__ float tile[32][33];
    update_copy_weights(a, own, tile);
    return;
  }
  update_lines_block<LINES_E, IN_PLACE>(a, (int)blockIdx.x, (int)blockIdx.y, vals, wt);
}

// Several tiles in one launch: start[t] .. start[t + 1] are the element blocks of tile t.
template <int LINES_E>
__global__ __launch_bounds__(256) void k_update_lines_group(UpdateGroup g) {
  __shared__ float vals[64][LINES_E + 1];
  __shared__ uint32_t wt[64][LINES_E + 1];
  int t = 0;
  while (t + 1 < g.n && (int)blockIdx.x >= g.start[t + 1]) ++t;
  const UpdateArgs a = g.args[t];
  update_lines_block<LINES_E>(a, (int)blockIdx.x - g.start[t], (int)blockIdx.y, vals, wt);
}

// deterministic implicit line values (src/rpucuda/dense_bit_line_maker.cpp:209-235)
__global__ __launch_bounds__(256) void k_update_implicit_lines(UpdateArgs a) {
  const long per_sample = (long)a.x_size + a.d_size;
  const long total = per_sample * a.m_batch;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int b = (int)(idx / per_sample);
    const int e = (int)(idx % per_sample);
    const bool is_x = e < a.x_size;
    const int j = is_x ? e : e - a.x_size;
    float v = is_x ? update_x_value(a, b, j) : update_d_row(a, b)[(long)j * a.d_si];
    if (a.lr < 0.0f) v = -v;
    const float P = is_x ? a.prob_b[b] : a.prob_a[b];
    const bool mean_count = a.up.pulse_type == RPU_PULSE_MEAN_COUNT;
    const float res = mean_count ? a.up.res : (is_x ? a.up.x_res_implicit : a.up.d_res_implicit);
    uint32_t sr = 0;
    if (res > 0.0f && a.up.sto_round) {
      sr = philox4x32_10((uint32_t)j, (uint32_t)b, a.call, RNG_UPDATE_SR | ((uint32_t)is_x << 8), a.key.k0, a.key.k1).v[0];
    }
    float pp = discretize_prob(fabsf(v) * P, res, a.up.sto_round, sr);
    float val;
    if (mean_count) {
      // generateCountsMean (dense_bit_line_maker.cpp:140-170): the expected number of pulses, no fluctuation; the d line
      // stores its count over BL as generateCoincidences (:176-201) divides it
      const int BL = a.bl[b];
      const int ntimes = pp == 0.0f ? 0 : max(min((int)rintf((float)BL * pp), BL), 0);
      const float count = (v >= 0.0f) ? (float)ntimes : -(float)ntimes;
      val = (is_x || ntimes == 0) ? count : count / (float)BL;
    } else {
      pp = fmaxf(fminf(pp, 1.0f), 0.0f);
      val = (v >= 0.0f) ? pp : -pp;
    }
    if (is_x) a.x_val[(long)b * a.x_size + j] = val;
    else a.d_val[(long)b * a.d_size + j] = val;
  }
}

// signed coincidence count of cross-point (i, j) for sample b from the stored line values:
// rintf((dv * BL) * xv) (generateCoincidencesDetI, dense_bit_line_maker.cpp:237-264), or with mean counts
// rintf((d_count / BL) * x_count) (generateCoincidences, :176-201)
// (i, j) are the row and column of the stored matrix: with the swapped view, row i is an x line of the tile and the
// arrays named d hold the x values, and the product keeps the reference's operand order
__device__ __forceinline__ int implicit_count(const UpdateArgs &a, int b, int i, int j) {
  const float row_val = a.d_val[(long)b * a.d_size + i], col_val = a.x_val[(long)b * a.x_size + j];
  float dc = a.swapped ? col_val : row_val;
  if (dc == 0.0f) return 0;
  if (a.up.pulse_type != RPU_PULSE_MEAN_COUNT) dc *= (float)a.bl[b];
  return (int)rintf(dc * (a.swapped ? row_val : col_val));
}

// ---- device steps ------------------------------------------------------------------------------

struct CtocStream {
  // four N(0,1) per Philox call, keyed by (cross-point, refill index, call)
  float n0, n1, n2, n3;
  int left;
  uint32_t refill;
  uint32_t cell;
  __device__ __forceinline__ float next(PhiloxKey key, uint32_t call) {
    if (left == 0) {
      float t[4];
      philox_normal4(cell, refill, call, RNG_CTOC, key, t);
      n0 = t[0]; n1 = t[1]; n2 = t[2]; n3 = t[3];
      left = 4;
      ++refill;
    }
    const float g = n0;
    n0 = n1; n1 = n2; n2 = n3;
    --left;
    return g;
  }
};

struct CellParams {
  float w_max, w_min, scale_up, scale_down, slope_up, slope_down;
};

template <int KIND, bool MULT>
__device__ __forceinline__ float device_step(float w, int sign_down, const CellParams &c, float std_, CtocStream &rng,
                                             PhiloxKey key, uint32_t call) {
  if (KIND == RPU_DEVICE_CONSTANT_STEP) {
    if (std_ > 0.0f) {
      const float f = 1.0f + std_ * rng.next(key, call);
      if (sign_down) w -= f * c.scale_down;
      else w += f * c.scale_up;
    } else {
      if (sign_down) w -= c.scale_down;
      else w += c.scale_up;
    }
    w = fminf(w, c.w_max);
    w = fmaxf(w, c.w_min);
  } else {
    const float f = (std_ > 0.0f) ? 1.0f + std_ * rng.next(key, call) : 1.0f;
    if (MULT) {
      if (sign_down) w -= (c.slope_down * w + c.scale_down) * f;
      else w += (c.slope_up * w + c.scale_up) * f;
    } else {
      if (sign_down) w -= c.slope_down * w + c.scale_down * f;
      else w += c.slope_up * w + c.scale_up * f;
    }
    w = fmaxf(w, c.w_min);
    w = fminf(w, c.w_max);
  }
  return w;
}

// one device pulse with the normal already drawn
template <int KIND, bool MULT>
__device__ __forceinline__ float device_step_g(float w, int sign_down, const CellParams &c, float std_, float g) {
  if (KIND == RPU_DEVICE_CONSTANT_STEP) {
    if (std_ > 0.0f) {
      const float f = 1.0f + std_ * g;
      if (sign_down) w -= f * c.scale_down;
      else w += f * c.scale_up;
    } else {
      if (sign_down) w -= c.scale_down;
      else w += c.scale_up;
    }
    w = fminf(w, c.w_max);
    w = fmaxf(w, c.w_min);
  } else {
    const float f = (std_ > 0.0f) ? 1.0f + std_ * g : 1.0f;
    if (MULT) {
      if (sign_down) w -= (c.slope_down * w + c.scale_down) * f;
      else w += (c.slope_up * w + c.scale_up) * f;
    } else {
      if (sign_down) w -= c.slope_down * w + c.scale_down * f;
      else w += c.slope_up * w + c.scale_up * f;
    }
    w = fmaxf(w, c.w_min);
    w = fminf(w, c.w_max);
  }
  return w;
}

template <int KIND>
__device__ __forceinline__ CellParams load_cell(const DeviceDev &d, long k) {
  CellParams c;
  c.w_max = d.w_max[k];
  c.w_min = d.w_min[k];
  c.scale_up = d.scale_up[k];
  c.scale_down = d.scale_down[k];
  if (KIND != RPU_DEVICE_CONSTANT_STEP) {
    c.slope_up = d.slope_up[k];
    c.slope_down = d.slope_down[k];
  } else {
    c.slope_up = 0.0f;
    c.slope_down = 0.0f;
  }
  return c;
}

// Pulse words -> bit planes.  One wave per (line element, block of 64 samples): lane q holds the word of
// sample 64 sb + q, a 64-bit ballot per pulse slot is the plane word of two 32-sample chunks.
__global__ __launch_bounds__(256) void k_update_planes(UpdateArgs a) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int sb = blockIdx.y;
  const int total = a.x_size + a.d_size;
  if (e >= total) return;
  const bool is_x = e < a.x_size;
  const int el = is_x ? e : e - a.x_size;
  const int size = is_x ? a.x_size : a.d_size;
  const uint32_t *words = is_x ? a.x_words : a.d_words;
  uint32_t *planes = is_x ? a.x_planes : a.d_planes;
  const int b = sb * 64 + lane;
  const uint32_t word = (b < a.m_batch) ? words[(long)b * size + el] : 0u;
  const int kmax = a.kmax[a.kmax_slot];
  const int c0 = 2 * sb;
  for (int k = 0; k < kmax; ++k) {
    const unsigned long long m = __ballot((word >> (k + 1)) & 1u);
    if (lane == 0) {
      planes[((long)c0 * a.plane_slots + k) * size + el] = (uint32_t)m;
      if (c0 + 1 < a.n_chunks) planes[((long)(c0 + 1) * a.plane_slots + k) * size + el] = (uint32_t)(m >> 32);
    }
  }
  // the last slot of a chunk holds the sign bits of its samples
  const unsigned long long sg = __ballot(word & 1u);
  if (lane == 0) {
    const int ks = a.plane_slots - 1;
    planes[((long)c0 * a.plane_slots + ks) * size + el] = (uint32_t)sg;
    if (c0 + 1 < a.n_chunks) planes[((long)(c0 + 1) * a.plane_slots + ks) * size + el] = (uint32_t)(sg >> 32);
  }
}

// Longest bit line among packed pulse words made elsewhere: the highest pulse slot set in any word of the batch
// (bit 0 is the sign).  out[0] must be zero before; every workgroup sends its own maximum.
__global__ __launch_bounds__(256) void k_words_kmax(const uint32_t *xw, size_t nx, const uint32_t *dw, size_t nd, int *out) {
  __shared__ uint32_t sh[4];
  uint32_t acc = 0u;
  const size_t stride = (size_t)gridDim.x * 256u, first = (size_t)blockIdx.x * 256u + threadIdx.x;
  for (size_t i = first; i < nx; i += stride) acc |= xw[i];
  for (size_t i = first; i < nd; i += stride) acc |= dw[i];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc |= (uint32_t)__shfl_xor((int)acc, off);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t pulses = (sh[0] | sh[1] | sh[2] | sh[3]) >> 1;
    if (pulses) atomicMax(out, 32 - __clz((int)pulses));
  }
}

__global__ void k_zero_word(int *p) {
  if (threadIdx.x == 0) *p = 0;
}

// Cross-point parameters of the pulse loop.  A step down subtracts (slope_down * w + scale_down) * f; with
// the down parameters negated every pulse is the same "w += (slope * w + scale) * f", and negation is
// exact in floating point.  The two clips of the reference (rpu_constantstep_device.cpp:48-53:
// min(w_max) then max(w_min); rpu_linearstep_device.cpp:155-160: max(w_min) then min(w_max)) are a
// median of three for bounds chosen so that crossed bounds give what the reference's order gives.
template <int KIND>
struct PulseCell {
  float scale_up, scale_dn, slope_up, slope_dn, lo, hi;
  __device__ __forceinline__ void load(const DeviceDev &d, unsigned cell) {
    const float w_max = d.w_max[cell], w_min = d.w_min[cell];
    scale_up = d.scale_up[cell];
    scale_dn = -d.scale_down[cell];
    if (KIND != RPU_DEVICE_CONSTANT_STEP) {
      slope_up = d.slope_up[cell];
      slope_dn = -d.slope_down[cell];
      lo = fminf(w_min, w_max); // crossed bounds: always w_max
      hi = w_max;
    } else {
      slope_up = slope_dn = 0.0f;
      lo = w_min;
      hi = fmaxf(w_min, w_max); // crossed bounds: always w_min
    }
  }
};

// one pulse with the noise factor f = 1 + std * N(0,1) (1 without cycle-to-cycle noise)
template <int KIND, bool MULT>
__device__ __forceinline__ float pulse(float w, float slope, float scale, float f, float lo, float hi) {
  // fused multiply-adds: one rounding less per operation than the reference's separate multiply and add, a
  // difference of at most half an ulp of w per pulse
  float wn;
  if (KIND == RPU_DEVICE_CONSTANT_STEP) wn = __builtin_fmaf(scale, f, w);
  else if (MULT) wn = __builtin_fmaf(__builtin_fmaf(slope, w, scale), f, w);
  else wn = __builtin_fmaf(scale, f, __builtin_fmaf(slope, w, w));
  return __builtin_amdgcn_fmed3f(wn, lo, hi);
}

// eight noise factors of one cross-point, keyed by (cross-point, refill index)
__device__ __forceinline__ void noise_factors(float (&f)[8], float std_, unsigned cell, uint32_t refill,
                                              const UpdateArgs &a) {
  if (std_ > 0.0f) {
    philox_factor8(cell, refill, a.call, RNG_CTOC, a.key, std_, f);
  } else {
#pragma unroll
    for (int q = 0; q < 8; ++q) f[q] = 1.0f;
  }
}

// Normal quantiles of the cycle-to-cycle noise: xi[q] = Phi^-1((q + 0.5) / CTOC_LEVELS) scaled to unit variance,
// exactly antisymmetric (zero mean).  Filled once per GPU by ensure_update_tables(); the update kernel turns it into
// the factors 1 + std * xi in LDS.
constexpr int CTOC_LEVELS = 256;
__device__ float g_ctoc_xi[CTOC_LEVELS];

// bitwise m ? a : b for a mask of all ones or all zeros (v_bfi_b32)
__device__ __forceinline__ float select_bits(uint32_t m, float a, float b) {
  return __uint_as_float((__float_as_uint(a) & m) | (__float_as_uint(b) & ~m));
}

// x bit planes of one 32-sample chunk for the C columns of a lane: NK pulse slots and the sign plane
template <int NK, int C> struct ChunkPlanes {
  uint32_t k[C][NK], sg[C];
  __device__ __forceinline__ void load(const UpdateArgs &a, const int (&j)[C], unsigned chunk) {
    const unsigned xs = (unsigned)a.x_size, slots = (unsigned)a.plane_slots;
    const unsigned base = chunk * slots;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const uint32_t *xpl = a.x_planes + j[c];
#pragma unroll
      for (int s = 0; s < NK; ++s) k[c][s] = xpl[(base + (unsigned)s) * xs]; // slots beyond the batch's longest line are never tested
      sg[c] = xpl[(base + slots - 1u) * xs];
    }
  }
};

// Pulse loop for short bit lines (at most NK pulse slots in use).  The lanes of a wave hold cross-points of one d
// row (C columns per lane, 256 apart), so the d pulses are wave-uniform: the wave walks the 32 samples of a chunk in
// batch order and, per sample, the pulse slots in which its d line fired -- scalar bit tests and branches, nothing
// for samples without a d pulse -- and in such a (sample, slot) pass every cross-point whose x line fired in that
// slot takes one device step.  All coincidences of a sample have one direction per cross-point, sign(x) * sign(d),
// picked once per sample.  Several columns per lane share the scalar work of a pass and give the vector pipeline
// independent chains.  The x planes of the next chunk are fetched while the current one is walked (two register
// sets in turn).  Lanes beyond the row end compute on the last column's data and never store.
// Cycle-to-cycle noise: a step takes its factor 1 + std * xi from a table of 256 normal quantiles in LDS (unit
// variance, kurtosis 2.92, |xi| <= 2.9), indexed by one byte of a per-lane xoroshiro64 stream (four factors per 32-bit
// output, fetched one pass ahead) whose state is one Philox4x32-10 output keyed by (first cross-point of the lane,
// call): reproducible from the tile seed.
template <int KIND, bool MULT, int NK, bool NOISE, int C> struct PulsedRows {
  const UpdateArgs &a;
  float (&w)[C];
  const PulseCell<KIND> (&cp)[C];
  const float *tbl;
  uint32_t s0 = 1u, s1 = 0u;
  float fnext[C];

  __device__ __forceinline__ PulsedRows(const UpdateArgs &a_, float (&w_)[C], const PulseCell<KIND> (&cp_)[C], const float *tbl_)
      : a(a_), w(w_), cp(cp_), tbl(tbl_) {}

  __device__ __forceinline__ void draw() {
    if (!NOISE) return;
#pragma unroll
    for (int c = 0; c < C; c += 4) {
      const uint32_t r = s0 + s1;
      s1 ^= s0;
      s0 = __builtin_amdgcn_bitop3_b32(__builtin_rotateleft32(s0, 26), s1, s1 << 9, 0x96); // three-input xor
      s1 = __builtin_rotateleft32(s1, 13);
      // one byte of the output per factor: the table offset is the byte times four
      fnext[c] = *(const float *)((const char *)tbl + ((r & 0xffu) << 2));
      if (c + 1 < C) fnext[c + 1] = *(const float *)((const char *)tbl + (((r >> 8) & 0xffu) << 2));
      if (c + 2 < C) fnext[c + 2] = *(const float *)((const char *)tbl + (((r >> 16) & 0xffu) << 2));
      if (c + 3 < C) fnext[c + 3] = *(const float *)((const char *)tbl + ((r >> 24) << 2));
    }
  }

  __device__ __forceinline__ void chunk(const ChunkPlanes<NK, C> &x, unsigned ch, int i, int kmax, uint32_t lr_mask) {
    const unsigned ds = (unsigned)a.d_size, slots = (unsigned)a.plane_slots;
    const uint32_t *dpl = a.d_planes + i;
    const unsigned base = ch * slots;
    uint32_t dk[NK], any = 0u; // wave-uniform
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      dk[k] = (k < kmax) ? dpl[(base + (unsigned)k) * ds] : 0u;
      any |= dk[k];
    }
    if (!any) return;
    // bit set: x and d have the same sign, which steps down when lr > 0
    walk(x, dk, any, ~dpl[(base + slots - 1u) * ds] ^ lr_mask);
  }

  // the passes of one chunk: dk the row's d pulses per slot (wave-uniform), any their union, dflip the direction bits
  __device__ __forceinline__ void walk(const ChunkPlanes<NK, C> &x, const uint32_t (&dk)[NK], uint32_t any, const uint32_t dflip) {
    uint32_t same[C];
#pragma unroll
    for (int c = 0; c < C; ++c) same[c] = x.sg[c] ^ dflip;
    while (any) {
      const int q = __builtin_ctz(any);
      any &= any - 1u;
      float slope[C], scale[C];
#pragma unroll
      for (int c = 0; c < C; ++c) {
        const uint32_t dm = (uint32_t)__builtin_amdgcn_sbfe((int)same[c], (uint32_t)q, 1u);
        slope[c] = select_bits(dm, cp[c].slope_dn, cp[c].slope_up);
        scale[c] = select_bits(dm, cp[c].scale_dn, cp[c].scale_up);
      }
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        if ((dk[k] >> q) & 1u) {
          float f[C];
#pragma unroll
          for (int c = 0; c < C; ++c) f[c] = NOISE ? fnext[c] : 1.0f;
          draw(); // the factors of the next pass are on their way while this one computes
#pragma unroll
          for (int c = 0; c < C; ++c) {
            const uint32_t pm = (uint32_t)__builtin_amdgcn_sbfe((int)x.k[c][k], (uint32_t)q, 1u);
            const float wn = pulse<KIND, MULT>(w[c], slope[c], scale[c], f[c], cp[c].lo, cp[c].hi);
            w[c] = select_bits(pm, wn, w[c]);
          }
        }
      }
    }
  }

  // Long batches on small tiles (the patches of a convolution): a chunk with few d pulses is walked in a fraction of a
  // memory latency, so fetching one chunk ahead leaves the wave waiting on every chunk.  Here the planes of PB chunks
  // are fetched at a time, two such blocks in turn: the x planes per lane, the row's d planes with lane l fetching those
  // of the block's chunk l (read back with v_readlane, which also keeps them out of the scalar cache's latency).
  static constexpr int PB = 8;
  struct Block {
    ChunkPlanes<NK, C> x[PB];
    uint32_t dk[NK], dsg; // of chunk (first chunk of the block + lane)
  };
  __device__ __forceinline__ void load_block(Block &b, const int (&j)[C], unsigned ch0, int i, int kmax) {
    const unsigned n_chunks = (unsigned)a.n_chunks, ds = (unsigned)a.d_size, slots = (unsigned)a.plane_slots;
#pragma unroll
    for (int p = 0; p < PB; ++p) b.x[p].load(a, j, min(ch0 + (unsigned)p, n_chunks - 1u));
    const unsigned chl = min(ch0 + (threadIdx.x & 63u), n_chunks - 1u);
    const uint32_t *dpl = a.d_planes + i;
#pragma unroll
    for (int k = 0; k < NK; ++k) b.dk[k] = (k < kmax) ? dpl[(chl * slots + (unsigned)k) * ds] : 0u;
    b.dsg = dpl[(chl * slots + slots - 1u) * ds];
  }
  __device__ __forceinline__ void walk_block(const Block &b, unsigned ch0, uint32_t lr_mask) {
    const unsigned n_chunks = (unsigned)a.n_chunks;
#pragma unroll
    for (int p = 0; p < PB; ++p) {
      if (ch0 + (unsigned)p >= n_chunks) break; // wave-uniform
      uint32_t dk[NK], any = 0u;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        dk[k] = (uint32_t)__builtin_amdgcn_readlane((int)b.dk[k], p);
        any |= dk[k];
      }
      if (!any) continue;
      walk(b.x[p], dk, any, ~(uint32_t)__builtin_amdgcn_readlane((int)b.dsg, p) ^ lr_mask);
    }
  }
  __device__ __forceinline__ void run_blocks(int i, const int (&j)[C], int kmax, uint32_t lr_mask) {
    const unsigned n_chunks = (unsigned)a.n_chunks;
    Block ba, bb;
    load_block(ba, j, 0u, i, kmax);
    for (unsigned ch = 0; ch < n_chunks; ch += 2u * PB) {
      if (ch + PB < n_chunks) load_block(bb, j, ch + PB, i, kmax);
      walk_block(ba, ch, lr_mask);
      if (ch + PB < n_chunks) {
        if (ch + 2u * PB < n_chunks) load_block(ba, j, ch + 2u * PB, i, kmax);
        walk_block(bb, ch + PB, lr_mask);
      }
    }
  }

  template <bool DEEP = false>
  __device__ __forceinline__ void run(unsigned cell, int i, const int (&j)[C], int kmax) {
    const uint32_t lr_mask = a.lr < 0.0f ? 0xffffffffu : 0u;
    const unsigned n_chunks = (unsigned)a.n_chunks;
    if (NOISE) {
      const Philox4 r = philox4x32_10(cell, 0u, a.call, RNG_CTOC, a.key.k0, a.key.k1);
      s0 = r.v[0] | 1u; // the all-zero state is the one fixed point of the generator
      s1 = r.v[1];
      draw();
    }
    if constexpr (DEEP) {
      run_blocks(i, j, kmax, lr_mask);
      return;
    }
    if (NK > 3) { // one register set: the longer lines are the rarer case, and two sets would not fit
      ChunkPlanes<NK, C> p;
      for (unsigned ch = 0; ch < n_chunks; ++ch) {
        p.load(a, j, ch);
        chunk(p, ch, i, kmax, lr_mask);
      }
      return;
    }
    ChunkPlanes<NK, C> pa, pb;
    pa.load(a, j, 0u);
    for (unsigned ch = 0; ch < n_chunks; ch += 2u) {
      const bool second = ch + 1u < n_chunks;
      if (second) pb.load(a, j, ch + 1u);
      chunk(pa, ch, i, kmax, lr_mask);
      if (second) {
        if (ch + 2u < n_chunks) pa.load(a, j, ch + 2u);
        chunk(pb, ch + 1u, i, kmax, lr_mask);
      }
    }
  }
};

// Pulse loop for any bit-line length.  The batch is walked in blocks of 128 samples.  For a block every lane
// first builds the 128-bit set of samples in which its cross-point has a coincidence: OR over the pulse
// slots of (x_plane & d_plane).  Then every lane walks its own set in batch order; the count and
// direction of an event come from the two packed words of that sample.  The wave loop applies at most
// one pulse per lane and pass and ends when the lane with the most pulses is done.
template <int KIND, bool MULT>
__device__ __forceinline__ float pulsed_gather(const UpdateArgs &a, float w, const PulseCell<KIND> &cp, unsigned cell,
                                               int i, int j, bool valid, int kmax) {
  const float std_ = a.dev.dw_min_std;
  const uint32_t lr_neg = a.lr < 0.0f ? 1u : 0u;
  const int n_chunks = a.n_chunks;
  const uint32_t *xpl = a.x_planes + j;
  const uint32_t *dpl = a.d_planes + i;
  const uint32_t *xwp = a.x_words + j;
  const uint32_t *dwp = a.d_words + i;
  const unsigned xs = (unsigned)a.x_size, ds = (unsigned)a.d_size;
  const int slots = a.plane_slots;

  uint32_t refill = 0;
  for (int c0 = 0; c0 < n_chunks; c0 += 4) {
    // event sets of the next 128 samples
    uint32_t ev[4];
#pragma unroll
    for (int cc = 0; cc < 4; ++cc) {
      const int c = c0 + cc;
      uint32_t e = 0u;
      if (c < n_chunks) {
        const unsigned base = (unsigned)c * (unsigned)slots;
        for (int k = 0; k < kmax; ++k) {
          const uint32_t dk = dpl[(base + k) * ds]; // wave-uniform
          if (dk) e |= dk & xpl[(base + k) * xs];
        }
      }
      ev[cc] = valid ? e : 0u;
    }
    unsigned long long cur = ((unsigned long long)ev[1] << 32) | ev[0];
    unsigned long long nxt = ((unsigned long long)ev[3] << 32) | ev[2];
    unsigned sample0 = (unsigned)c0 * 32u; // sample index of bit 0 of cur
    int left = 0;                          // pulses left in the current event
    float slope = 0.0f, scale = 0.0f;
    bool block_done = !__any((cur | nxt) != 0ull);
    while (!block_done) {
      float f[8];
      noise_factors(f, std_, cell, refill, a);
      ++refill;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        if (left == 0) {
          if (cur == 0ull) {
            cur = nxt;
            nxt = 0ull;
            sample0 += 64u;
          }
          if (cur != 0ull) {
            const int bit = __ffsll((long long)cur) - 1;
            cur &= cur - 1ull;
            const unsigned b = sample0 + (unsigned)bit;
            const uint32_t xw = xwp[__umul24(b, xs)];
            const uint32_t dw = dwp[__umul24(b, ds)];
            left = __popc(xw & dw & ~1u);
            // step down when x and d have the same sign and lr > 0
            const bool down = (((xw ^ dw) & 1u) ^ lr_neg) == 0u;
            slope = down ? cp.slope_dn : cp.slope_up;
            scale = down ? cp.scale_dn : cp.scale_up;
          }
        }
        if (!__any(left > 0)) {
          block_done = true;
          break;
        }
        if (left > 0) {
          w = pulse<KIND, MULT>(w, slope, scale, f[q], cp.lo, cp.hi);
          --left;
        }
      }
    }
  }
  return w;
}

// grid: x = ceil(x_size / (256 C)), y = d_size.  A thread holds C cross-points of one d row, 256 columns apart; a
// wave covers 64 consecutive x per column group, so everything that belongs to the d line is wave-uniform and the x
// planes, weights and parameters are read with unit stride.  The pulse loop is chosen by the longest bit line of
// the batch.
// bx: the workgroup's block of 256 C columns, i: its row; tbl: the noise factors 1 + std * quantile in LDS
// DEEP: the planes of eight chunks are fetched at a time (PulsedRows::run_blocks; short bit lines, one column per lane)
// tid: number of the thread among the 256 that share the row
template <int KIND, bool MULT, bool NOISE, int C, bool DEEP>
__device__ __forceinline__ void update_pulsed_row(const UpdateArgs &a, const int bx, const int i, float *tbl,
                                                  const int tid = (int)threadIdx.x) {
  if (NOISE) {
    static_assert(CTOC_LEVELS == 256, "one table entry per thread");
    if (threadIdx.x < CTOC_LEVELS) tbl[threadIdx.x] = __builtin_fmaf(a.dev.dw_min_std, g_ctoc_xi[threadIdx.x], 1.0f);
    __syncthreads();
  }
  int j[C];
  bool valid[C];
  unsigned cell[C];
  PulseCell<KIND> cp[C];
  float w[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int jt = (bx * C + c) * 256 + tid;
    valid[c] = jt < a.x_size;
    j[c] = valid[c] ? jt : a.x_size - 1;
    cell[c] = (unsigned)i * (unsigned)a.x_size + (unsigned)j[c];
    cp[c].load(a.dev, cell[c]);
    w[c] = a.w[cell[c]];
  }
  const int kmax = a.kmax[a.kmax_slot];
  if (DEEP && kmax <= 1) {
    // bit lines of one pulse (small gradients under update-BL management, the rule for the patches of a convolution):
    // every sample with a d pulse is one pass, no slots to test
    PulsedRows<KIND, MULT, 1, NOISE, C>(a, w, cp, tbl).template run<DEEP>(cell[0], i, j, kmax);
  } else if (kmax <= 3) {
    PulsedRows<KIND, MULT, 3, NOISE, C>(a, w, cp, tbl).template run<DEEP>(cell[0], i, j, kmax);
  } else if (kmax <= 7) {
    PulsedRows<KIND, MULT, 7, NOISE, C>(a, w, cp, tbl).run(cell[0], i, j, kmax);
  } else {
#pragma unroll
    for (int c = 0; c < C; ++c) w[c] = pulsed_gather<KIND, MULT>(a, w[c], cp[c], cell[c], i, j[c], valid[c], kmax);
  }
  if (a.w_out) { // the tile's own matrix is laid out another way (UpdateArgs::w_out)
#pragma unroll
    for (int c = 0; c < C; ++c) {
      if (valid[c]) a.w_out[(long)i * a.wo_si + (long)j[c] * a.wo_sj] = w[c];
    }
    return;
  }
#pragma unroll
  for (int c = 0; c < C; ++c) {
    if (valid[c]) a.w[cell[c]] = w[c];
  }
}

template <int KIND, bool MULT, bool NOISE, int C, bool DEEP = false>
__global__ __launch_bounds__(256, ((C > 1 || DEEP) ? 4 : 8)) void k_update_pulsed(UpdateArgs a) {
  __shared__ float tbl[CTOC_LEVELS];
  int row = (int)blockIdx.y;
  if (a.w_out && (a.d_size & 7) == 0 && gridDim.x == 1) {
    // Stores along a column of a matrix whose rows run the other way: consecutive workgroups go to different XCDs, so
    // each XCD is given a band of consecutive rows and the cache lines of the target are put together in one L2.
    const int band = a.d_size >> 3;
    row = (row & 7) * band + (row >> 3);
  }
  update_pulsed_row<KIND, MULT, NOISE, C, DEEP>(a, (int)blockIdx.x, row, tbl);
}

// The same pulse loop with the rows dealt out by their work.  The time a row takes follows its number of d pulses, which
// varies by several percent between rows, and a CU holds four rows at a time: whichever CU draws four long ones sets
// the kernel's time.  Here a workgroup of 1024 threads fills a CU and takes four rows, one per 256 threads, chosen so
// that every workgroup has the same work: workgroup n (on XCD n % 8) belongs to the band of d_size / 8 consecutive rows
// of its XCD, ranks the band's rows by a.row_cost (ties by row number: every workgroup of the band finds the same
// order) and takes, as number s of the band's S = d_size / 32 workgroups, the ranks s, 2 S - 1 - s, 2 S + s and
// 4 S - 1 - s.  Rows of a band in one L2 also keep the strided stores of UpdateArgs::w_out together.
// For four columns per lane, rows of at most 1024 columns, d_size a multiple of 256 (bands of whole groups of 32 rows).  Which row a group of threads works
// on changes nothing in the result of the row.
constexpr int BALANCED_MAX_BAND = 1024;
template <int KIND, bool MULT, bool NOISE>
__global__ __launch_bounds__(1024) void k_update_pulsed_balanced(UpdateArgs a) {
  __shared__ float tbl[CTOC_LEVELS];
  __shared__ int cost[BALANCED_MAX_BAND];
  __shared__ int order[BALANCED_MAX_BAND];
  const int band = a.d_size >> 3, per_band = band >> 2;
  const int xcd = (int)blockIdx.x & 7, s = (int)blockIdx.x >> 3;
  const int row0 = xcd * band;
  for (int t = (int)threadIdx.x; t < band; t += 1024) {
    cost[t] = a.row_cost[row0 + t];
    order[t] = 0; // first the rank of row t, summed from the parts below
  }
  __syncthreads();
  // rank of a row = rows of the band that come before it; the threads split the comparisons, 32 rows each
  for (int idx = (int)threadIdx.x; idx < band * (band >> 5); idx += 1024) {
    const int t = idx % band, u0 = (idx / band) << 5;
    const int mine = cost[t];
    int before = 0;
#pragma unroll 8
    for (int u = u0; u < u0 + 32; ++u) {
      const int c = cost[u];
      before += (c < mine || (c == mine && u < t)) ? 1 : 0;
    }
    atomicAdd(&order[t], before);
  }
  __syncthreads();
  int rank_of[BALANCED_MAX_BAND / 1024];
#pragma unroll
  for (int q = 0; q < BALANCED_MAX_BAND / 1024; ++q) {
    const int t = (int)threadIdx.x + 1024 * q;
    rank_of[q] = t < band ? order[t] : 0;
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < BALANCED_MAX_BAND / 1024; ++q) {
    const int t = (int)threadIdx.x + 1024 * q;
    if (t < band) order[rank_of[q]] = t;
  }
  __syncthreads();
  const int g = (int)threadIdx.x >> 8;
  const int rank = (g & 1) ? (g + 1) * per_band - 1 - s : g * per_band + s;
  // the same for the 256 threads of a row: kept in a scalar register, like a row number taken from the grid
  const int row = __builtin_amdgcn_readfirstlane(row0 + order[rank]);
  update_pulsed_row<KIND, MULT, NOISE, 4, false>(a, 0, row, tbl, (int)threadIdx.x & 255);
}

// Several tiles in one launch (same device kind, noise and columns per lane): start[t] .. start[t + 1] are the
// workgroups of tile t, column blocks of a row next to each other.
template <int KIND, bool MULT, bool NOISE, int C, bool DEEP = false>
__global__ __launch_bounds__(256, ((C > 1 || DEEP) ? 4 : 8)) void k_update_pulsed_group(UpdateGroup g) {
  __shared__ float tbl[CTOC_LEVELS];
  int t = 0;
  while (t + 1 < g.n && (int)blockIdx.x >= g.start[t + 1]) ++t;
  const UpdateArgs a = g.args[t];
  const int blocks = (a.x_size + 256 * C - 1) / (256 * C);
  const int local = (int)blockIdx.x - g.start[t];
  update_pulsed_row<KIND, MULT, NOISE, C, DEEP>(a, local % blocks, local / blocks, tbl);
}

// ---- opt-in variant: aggregated steps -----------------------------------------------------------------------
// NOT the reference's per-pulse arithmetic: a statistically equivalent short-cut for LinearStep / SoftBounds devices
// with multiplicative cycle-to-cycle noise, chosen per tile (rpu_tile_set_update_variant).  The batch is cut into
// groups of `agg_chunks` 32-sample chunks.  Per group a cross-point only counts its coincidences by direction
// (population counts on the bit planes) and then takes n_up up-steps and n_dn down-steps in closed form: n noise-free
// steps w <- w + (slope w + scale) move w to w + (slope w + scale) (a^n - 1) / slope with a = 1 + slope (n steps of
// the geometric approach to -scale / slope; n (slope w + scale) when slope is zero), the up-steps split in two halves
// around the down-steps (symmetric splitting: the error of ignoring the order inside a group is third order in
// n * slope).  The cycle-to-cycle noise of the group's pulses is added as ONE normal draw per group with the summed
// variance std^2 (n_up step_up^2 + n_dn step_dn^2), step sizes taken at the end of the group, then the device bounds are
// applied once.  Mean and variance of
// the weight change agree with the per-pulse update to first order in n * slope (about 1 % of the change per 32
// samples at benchmark configuration 2); the pulse trains, their counts and their directions are exactly the same.
struct AggCell {
  float slope_up, scale_up, slope_dn, scale_dn, lo, hi;
  float log_up, inv_up, lin_up, log_dn, inv_dn, lin_dn;
  __device__ __forceinline__ void load(const DeviceDev &d, unsigned cell) {
    PulseCell<RPU_DEVICE_LINEAR_STEP> p;
    p.load(d, cell);
    slope_up = p.slope_up; scale_up = p.scale_up; slope_dn = p.slope_dn; scale_dn = p.scale_dn; lo = p.lo; hi = p.hi;
    prepare(slope_up, log_up, inv_up, lin_up);
    prepare(slope_dn, log_dn, inv_dn, lin_dn);
  }
  // (a^n - 1) / slope = (exp2(n log2 a) - 1) * inv + n * lin, with lin = 1 and inv = 0 where the slope vanishes (or
  // where 1 + slope is not positive, which no sensible device has: such a cross-point then takes linear steps)
  static __device__ __forceinline__ void prepare(float slope, float &lg, float &inv, float &lin) {
    const bool geometric = fabsf(slope) > 1e-7f;
    // 1 + slope <= 0 (a bound closer than one step): the first step overshoots the fixed point and is cut back by the
    // bounds, the following ones do not move: a^n is taken as 0 for every n >= 1
    lg = !geometric ? 0.0f : (slope > -1.0f ? __builtin_amdgcn_logf(1.0f + slope) : -126.0f);
    inv = geometric ? 1.0f / slope : 0.0f;
    lin = geometric ? 0.0f : 1.0f;
  }
};

__device__ __forceinline__ float agg_steps(float w, float n, float slope, float scale, float lg, float inv, float lin) {
  const float first_step = __builtin_fmaf(slope, w, scale);
  const float e = __builtin_amdgcn_exp2f(n * lg);
  const float g = __builtin_fmaf(e - 1.0f, inv, n * lin);
  return __builtin_fmaf(first_step, g, w);
}

// A lane holds R cross-points of one column (rows i0 .. i0 + R - 1): the x planes of a chunk are fetched once (the
// next chunk's while this one is counted) and serve R rows, whose d planes are scalar loads.
template <bool NOISE, int R> struct AggregatedRows {
  const UpdateArgs &a;
  const float *tbl;
  AggCell cp[R];
  float w[R];
  unsigned n_all[R], n_dn[R];
  int i0, rows; // rows: how many of the R rows exist
  uint32_t s0 = 1u, s1 = 0u, lr_mask;

  __device__ __forceinline__ AggregatedRows(const UpdateArgs &a_, const float *tbl_) : a(a_), tbl(tbl_) {}

  // d planes of four chunks for the R rows, one word per lane: lane ((chunk & 3) * R + row) * 4 + kk holds pulse slot
  // kk < 3, or the sign plane for kk = 3.  One gather per four chunks instead of a scalar load (and its latency) per
  // row, chunk and slot; the counting loop reads the words back with v_readlane.
  __device__ __forceinline__ uint32_t gather_d(unsigned block, int kmax) const {
    static_assert(R == 4, "lane layout of the d-plane gather");
    const unsigned lane = threadIdx.x & 63u;
    const unsigned ch = 4u * block + (lane >> 4), r = (lane >> 2) & 3u, kk = lane & 3u;
    const unsigned slots = (unsigned)a.plane_slots;
    const unsigned slot = kk < 3u ? kk : slots - 1u;
    const unsigned row = min((unsigned)i0 + r, (unsigned)a.d_size - 1u);
    const bool wanted = ch < (unsigned)a.n_chunks && (kk == 3u || (int)kk < kmax);
    const unsigned chc = min(ch, (unsigned)a.n_chunks - 1u);
    const uint32_t v = a.d_planes[(size_t)(chc * slots + slot) * (unsigned)a.d_size + row];
    return wanted ? v : 0u;
  }

  // counts of one chunk (q = chunk & 3) from its x planes and the gathered d planes
  __device__ __forceinline__ void count(const ChunkPlanes<3, 1> &x, uint32_t dvec, int q) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r >= rows) continue; // wave-uniform
      uint32_t dk[3], any = 0u;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        dk[k] = (uint32_t)__builtin_amdgcn_readlane((int)dvec, (q * R + r) * 4 + k);
        any |= dk[k];
      }
      if (!any) continue;
      const uint32_t dsg = (uint32_t)__builtin_amdgcn_readlane((int)dvec, (q * R + r) * 4 + 3);
      const uint32_t same = x.sg[0] ^ (~dsg ^ lr_mask); // bit set: step down
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        if (!dk[k]) continue;
        const uint32_t hit = dk[k] & x.k[0][k];
        n_all[r] += __popc(hit);
        n_dn[r] += __popc(hit & same);
      }
    }
  }

  // any bit-line length: planes read where they are used
  __device__ __forceinline__ void count_generic(int j, unsigned ch, int kmax) {
    const unsigned xs = (unsigned)a.x_size, ds = (unsigned)a.d_size, slots = (unsigned)a.plane_slots, base = ch * slots;
    const uint32_t *xpl = a.x_planes + j;
    const uint32_t xsg = xpl[(base + slots - 1u) * xs];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r >= rows) continue;
      const uint32_t *dpl = a.d_planes + (i0 + r);
      const uint32_t same = xsg ^ (~dpl[(base + slots - 1u) * ds] ^ lr_mask);
      for (int k = 0; k < kmax; ++k) {
        const uint32_t dk = dpl[(base + (unsigned)k) * ds];
        if (!dk) continue;
        const uint32_t hit = dk & xpl[(base + (unsigned)k) * xs];
        n_all[r] += __popc(hit);
        n_dn[r] += __popc(hit & same);
      }
    }
  }

  __device__ __forceinline__ void apply() {
    uint32_t rnd = 0u;
    if (NOISE) {
      rnd = s0 + s1;
      s1 ^= s0;
      s0 = __builtin_amdgcn_bitop3_b32(__builtin_rotateleft32(s0, 26), s1, s1 << 9, 0x96);
      s1 = __builtin_rotateleft32(s1, 13);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float nd = (float)n_dn[r], nu = (float)(n_all[r] - n_dn[r]);
      n_all[r] = n_dn[r] = 0u;
      // half of the up-steps, all down-steps, the other half of the up-steps (symmetric splitting)
      float wn = w[r];
      wn = agg_steps(wn, 0.5f * nu, cp[r].slope_up, cp[r].scale_up, cp[r].log_up, cp[r].inv_up, cp[r].lin_up);
      wn = agg_steps(wn, nd, cp[r].slope_dn, cp[r].scale_dn, cp[r].log_dn, cp[r].inv_dn, cp[r].lin_dn);
      wn = agg_steps(wn, 0.5f * nu, cp[r].slope_up, cp[r].scale_up, cp[r].log_up, cp[r].inv_up, cp[r].lin_up);
      if (NOISE) {
        // The noise of a pulse is scaled by every later step of the group: n steps of one direction leave
        // n * (last step)^2 * std^2, so the step sizes are taken where the group ends.
        const float su = __builtin_fmaf(cp[r].slope_up, wn, cp[r].scale_up);
        const float sd = __builtin_fmaf(cp[r].slope_dn, wn, cp[r].scale_dn);
        const float var = __builtin_fmaf(nu * su, su, (nd * sd) * sd);
        const float xi = *(const float *)((const char *)tbl + (((rnd >> (8 * (r & 3))) & 0xffu) << 2));
        wn = __builtin_fmaf(__builtin_amdgcn_sqrtf(var), xi, wn);
      }
      w[r] = __builtin_amdgcn_fmed3f(wn, cp[r].lo, cp[r].hi);
    }
  }

  __device__ __forceinline__ void run(int j, int kmax, int agg_chunks) {
    const int n_chunks = a.n_chunks;
    int in_group = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) n_all[r] = n_dn[r] = 0u;
    if (kmax <= 3) {
      // blocks of four chunks: the x planes and the d-plane gather of the next block are in flight while this one
      // is counted
      const int jj[1] = {j};
      const int n_blocks = (n_chunks + 3) / 4;
      ChunkPlanes<3, 1> cur[4], nxt[4];
      uint32_t dcur = gather_d(0u, kmax), dnxt = 0u;
#pragma unroll
      for (int q = 0; q < 4; ++q) cur[q].load(a, jj, (unsigned)min(q, n_chunks - 1));
      for (int b = 0; b < n_blocks; ++b) {
        if (b + 1 < n_blocks) {
          dnxt = gather_d((unsigned)b + 1u, kmax);
#pragma unroll
          for (int q = 0; q < 4; ++q) nxt[q].load(a, jj, (unsigned)min(4 * b + 4 + q, n_chunks - 1));
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = 4 * b + q;
          if (ch < n_chunks) {
            count(cur[q], dcur, q);
            if (++in_group == agg_chunks || ch + 1 == n_chunks) { apply(); in_group = 0; }
          }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) cur[q] = nxt[q];
        dcur = dnxt;
      }
    } else {
      for (int ch = 0; ch < n_chunks; ++ch) {
        count_generic(j, (unsigned)ch, kmax);
        if (++in_group == agg_chunks || ch + 1 == n_chunks) { apply(); in_group = 0; }
      }
    }
  }
};

// grid: x = ceil(x_size / 256), y = ceil(d_size / R)
template <bool NOISE, int R>
__global__ __launch_bounds__(256) void k_update_aggregated(UpdateArgs a, int agg_chunks) {
  __shared__ float tbl[CTOC_LEVELS]; // std * quantile
  if (NOISE) {
    tbl[threadIdx.x] = a.dev.dw_min_std * g_ctoc_xi[threadIdx.x];
    __syncthreads();
  }
  AggregatedRows<NOISE, R> rows(a, tbl);
  rows.i0 = blockIdx.y * R;
  rows.rows = min(R, a.d_size - rows.i0);
  rows.lr_mask = a.lr < 0.0f ? 0xffffffffu : 0u;
  const int jt = blockIdx.x * 256 + threadIdx.x;
  const bool valid = jt < a.x_size;
  const int j = valid ? jt : a.x_size - 1;
  unsigned cell[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(rows.i0 + r, a.d_size - 1);
    cell[r] = (unsigned)i * (unsigned)a.x_size + (unsigned)j;
    rows.cp[r].load(a.dev, cell[r]);
    rows.w[r] = a.w[cell[r]];
  }
  if (NOISE) {
    const Philox4 p = philox4x32_10(cell[0], 1u, a.call, RNG_CTOC, a.key.k0, a.key.k1);
    rows.s0 = p.v[0] | 1u;
    rows.s1 = p.v[1];
  }
  rows.run(j, a.kmax[a.kmax_slot], agg_chunks);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (valid && r < rows.rows) a.w[cell[r]] = rows.w[r];
  }
}

// deterministic implicit: n = (int) rintf((dv * BL) * xv) per sample (dense_bit_line_maker.cpp:237-264),
// |n| steps, n > 0 steps down (rpu_pulsed_device.h:461-474)
template <int KIND, bool MULT>
__global__ __launch_bounds__(256) void k_update_implicit(UpdateArgs a) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.x_size) return;
  const long k = (long)i * a.x_size + j;
  const CellParams c = load_cell<KIND>(a.dev, k);
  float w = a.w[k];
  CtocStream rng;
  rng.left = 0;
  rng.refill = 0;
  // the noise stream of a cross-point is keyed by its row-major number in the tile, however the matrix is stored
  rng.cell = a.swapped ? (uint32_t)((long)j * a.d_size + i) : (uint32_t)k;
  rng.n0 = rng.n1 = rng.n2 = rng.n3 = 0.0f;
  const float std_ = a.dev.dw_min_std;
  for (int b = 0; b < a.m_batch; ++b) {
    const int cn = implicit_count(a, b, i, j);
    if (cn == 0) continue;
    const int sign_down = cn > 0;
    for (int n = abs(cn); n > 0; --n) w = device_step<KIND, MULT>(w, sign_down, c, std_, rng, a.key, a.call);
  }
  a.w[k] = w;
}

__global__ __launch_bounds__(256) void k_implicit_counts(UpdateArgs a, int32_t *counts) {
  const long per = (long)a.x_size * a.d_size;
  const long total = per * a.m_batch;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int b = (int)(idx / per);
    const long rem = idx % per;
    const int i = (int)(rem / a.x_size);
    const int j = (int)(rem % a.x_size);
    counts[idx] = implicit_count(a, b, i, j);
  }
}

// kernelPulseCounter (cuda/pwu_kernel.h:1523-1627) on the bit planes: one thread per cross-point
__global__ __launch_bounds__(256) void k_count_pulses(UpdateArgs a, unsigned long long *pos, unsigned long long *neg) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.x_size) return;
  const int kmax = a.kmax[a.kmax_slot];
  const unsigned xs = (unsigned)a.x_size, ds = (unsigned)a.d_size, slots = (unsigned)a.plane_slots;
  const uint32_t *xpl = a.x_planes + j;
  const uint32_t *dpl = a.d_planes + i;
  unsigned n_same = 0, n_diff = 0;
  for (int c = 0; c < a.n_chunks; ++c) {
    const unsigned base = (unsigned)c * slots;
    const uint32_t same = ~(xpl[(base + slots - 1) * xs] ^ dpl[(base + slots - 1) * ds]);
    for (int k = 0; k < kmax; ++k) {
      const uint32_t dk = dpl[(base + k) * ds]; // wave-uniform
      if (!dk) continue;
      const uint32_t m = dk & xpl[(base + k) * xs];
      n_same += __popc(m & same);
      n_diff += __popc(m & ~same);
    }
  }
  const size_t cell = (size_t)i * a.x_size + j;
  pos[cell] += n_same;
  neg[cell] += n_diff;
}

// the same for the deterministic implicit pulses: n > 0 are coincidences of equal sign
__global__ __launch_bounds__(256) void k_count_pulses_implicit(UpdateArgs a, unsigned long long *pos,
                                                                unsigned long long *neg) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.x_size) return;
  unsigned long long n_same = 0, n_diff = 0;
  for (int b = 0; b < a.m_batch; ++b) {
    const int cn = implicit_count(a, b, i, j);
    if (cn > 0) n_same += (unsigned)cn;
    else n_diff += (unsigned)(-cn);
  }
  const size_t cell = (size_t)i * a.x_size + j;
  pos[cell] += n_same;
  neg[cell] += n_diff;
}

// Write noise (rpu_linearstep_device.cpp:112-164): the pulses act on the persistent weights; a cross-point that took at
// least one pulse in this update shows its persistent weight plus fresh noise, the others keep what they showed.
// Runs after the update kernel, on the same bit planes (or line values): one thread per cross-point.
__global__ __launch_bounds__(256) void k_write_noise_touched(UpdateArgs a, float *w_apparent, const float *w_persistent,
                                                              float noise_std, int implicit) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.x_size) return;
  bool touched = false;
  if (implicit) {
    for (int b = 0; b < a.m_batch && !touched; ++b) touched = implicit_count(a, b, i, j) != 0;
  } else {
    const int kmax = a.kmax[a.kmax_slot];
    const unsigned xs = (unsigned)a.x_size, ds = (unsigned)a.d_size, slots = (unsigned)a.plane_slots;
    const uint32_t *xpl = a.x_planes + j;
    const uint32_t *dpl = a.d_planes + i;
    uint32_t any = 0u;
    for (int c = 0; c < a.n_chunks; ++c) {
      const unsigned base = (unsigned)c * slots;
      for (int k = 0; k < kmax; ++k) {
        const uint32_t dk = dpl[(base + k) * ds]; // wave-uniform
        if (dk) any |= dk & xpl[(base + k) * xs];
      }
    }
    touched = any != 0u;
  }
  if (!touched) return;
  const size_t cell = (size_t)i * a.x_size + j;
  float z[4];
  philox_normal4((uint32_t)cell, (uint32_t)(cell >> 32), a.call, RNG_WRITE_NOISE, a.key, z);
  w_apparent[cell] = w_persistent[cell] + noise_std * z[0];
}

// PulseType NoneWithDevice (rpu_weight_updater.cpp:216-224): per sample the floating-point outer product
// w_ij += (-lr d_i) x_j, then the device bounds; the clipping makes the samples a sequence, one thread per cross-point
// walks it
__global__ __launch_bounds__(256) void k_update_fp_clipped(UpdateArgs a) {
  const int i = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= a.x_size) return;
  const size_t cell = (size_t)i * a.x_size + j;
  float w = a.w[cell];
  const float lo = a.dev.w_min[cell], hi = a.dev.w_max[cell];
  for (int b = 0; b < a.m_batch; ++b) {
    const float row_val = a.d[(long)b * a.d_sb + (long)i * a.d_si]; // wave-uniform
    const float col_val = a.x[(long)b * a.x_sb + (long)j * a.x_sj];
    const float di = -a.lr * (a.swapped ? col_val : row_val); // the tile's d value, whichever side holds it
    w = w + di * (a.swapped ? row_val : col_val);
    w = fmaxf(fminf(w, hi), lo);
  }
  a.w[cell] = w;
}

__global__ void k_clip(float *w, const float *w_min, const float *w_max, size_t n) {
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
    float v = w[idx];
    v = fminf(v, w_max[idx]);
    v = fmaxf(v, w_min[idx]);
    w[idx] = v;
  }
}

__global__ void k_unit_vectors(float *out, int n_vec, int size, int start) {
  const long n = (long)n_vec * size;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < n; idx += (long)gridDim.x * blockDim.x) {
    const int v = (int)(idx / size);
    const int j = (int)(idx % size);
    out[idx] = (j == (start + v) % size) ? 1.0f : 0.0f;
  }
}

__global__ void k_reduce_weights(float *out, ReduceArgs r, size_t n) {
  for (size_t idx = blockIdx.x * (size_t)blockDim.x + threadIdx.x; idx < n; idx += (size_t)gridDim.x * blockDim.x) {
    float acc = 0.0f;
    for (int k = 0; k < r.n; ++k) acc += r.gamma[k] * r.w[k][idx];
    out[idx] = acc;
  }
}

int grid_for(long total) {
  long blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
  return (int)blocks;
}

} // namespace

void launch_update_prepare(const UpdateArgs &a, hipStream_t s) {
  const int longest = a.x_size > a.d_size ? a.x_size : a.d_size;
  if (a.x_index_lines && a.d_group && a.m_batch >= 4096) {
    hipLaunchKernelGGL(k_update_prepare_in_place, dim3((a.m_batch + 63) / 64), dim3(64), 0, s, a);
    return;
  }
  if (longest > 1024 || a.m_batch <= 1024) {
    hipLaunchKernelGGL(k_update_prepare<256>, dim3(a.m_batch), dim3(256), 0, s, a);
  } else if (longest > 64) {
    hipLaunchKernelGGL(k_update_prepare<64>, dim3((a.m_batch + 3) / 4), dim3(256), 0, s, a);
  } else {
    hipLaunchKernelGGL(k_update_prepare<16>, dim3((a.m_batch + 15) / 16), dim3(256), 0, s, a);
  }
}

void launch_update_lines(const UpdateArgs &a, hipStream_t s) {
  const unsigned sample_tiles = (a.m_batch + 63) / 64;
  const unsigned wide = (a.x_size + 15) / 16 + (a.d_size + 15) / 16;
  // workgroups beyond the kernel's own make the row-major copy of the weights (update_copy_weights): about four
  // 32 x 32 tiles each, at most 256 of them
  unsigned extra = 0;
  if (a.wt_src) {
    const unsigned tiles = ((a.x_size + 31) / 32) * ((a.d_size + 31) / 32);
    extra = std::min(256u, (tiles + 3) / 4);
    extra = (extra + sample_tiles - 1) / sample_tiles;
  }
  const bool in_place = a.x_index || a.d_group;
  const dim3 narrow((a.x_size + 3) / 4 + (a.d_size + 3) / 4 + extra, sample_tiles);
  if (wide * sample_tiles >= 256) {
    if (in_place) hipLaunchKernelGGL((k_update_lines<16, true>), dim3(wide + extra, sample_tiles), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(k_update_lines<16>, dim3(wide + extra, sample_tiles), dim3(256), 0, s, a);
  } else {
    if (in_place) hipLaunchKernelGGL((k_update_lines<4, true>), narrow, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(k_update_lines<4>, narrow, dim3(256), 0, s, a);
  }
}

void launch_update_implicit_lines(const UpdateArgs &a, hipStream_t s) {
  const long total = ((long)a.x_size + a.d_size) * a.m_batch;
  hipLaunchKernelGGL(k_update_implicit_lines, dim3(grid_for(total)), dim3(256), 0, s, a);
}

#define RPU_DISPATCH_DEVICE(KERNEL, grid, s, a)                                                     \
  do {                                                                                              \
    if ((a).dev.kind == RPU_DEVICE_CONSTANT_STEP) {                                                 \
      hipLaunchKernelGGL((KERNEL<RPU_DEVICE_CONSTANT_STEP, true>), grid, dim3(256), 0, s, a);       \
    } else if ((a).dev.ls_mult_noise) {                                                             \
      hipLaunchKernelGGL((KERNEL<RPU_DEVICE_LINEAR_STEP, true>), grid, dim3(256), 0, s, a);         \
    } else {                                                                                        \
      hipLaunchKernelGGL((KERNEL<RPU_DEVICE_LINEAR_STEP, false>), grid, dim3(256), 0, s, a);        \
    }                                                                                               \
  } while (0)

void launch_words_kmax(const UpdateArgs &a, hipStream_t s) {
  const size_t nx = (size_t)a.m_batch * a.x_size, nd = (size_t)a.m_batch * a.d_size;
  const size_t blocks = std::min<size_t>(256, (nx + nd + 4095) / 4096);
  hipLaunchKernelGGL(k_zero_word, dim3(1), dim3(64), 0, s, a.kmax + a.kmax_slot);
  hipLaunchKernelGGL(k_words_kmax, dim3((unsigned)std::max<size_t>(blocks, 1)), dim3(256), 0, s, a.x_words, nx, a.d_words, nd,
                     a.kmax + a.kmax_slot);
}

void launch_update_planes(const UpdateArgs &a, hipStream_t s) {
  dim3 grid((a.x_size + a.d_size + 3) / 4, (a.m_batch + 63) / 64);
  hipLaunchKernelGGL(k_update_planes, grid, dim3(256), 0, s, a);
}

// whether the launch that deals the rows out by their work serves this call (see k_update_pulsed_balanced): only
// where its workgroups, a quarter as many as rows, still fill the chip
static bool balanced_shape(const UpdateArgs &a, int columns) {
  return columns == 4 && a.x_size <= 1024 && a.d_size >= 1024 && a.d_size % 256 == 0 && a.d_size / 8 <= BALANCED_MAX_BAND;
}
bool update_pulsed_balanced(const UpdateArgs &a, int columns) { return a.row_cost && balanced_shape(a, columns); }

static int update_pulsed_columns(const UpdateArgs &a);

// whether a call of this shape reads UpdateArgs::row_cost at all: elsewhere the tile leaves it null, and the kernel that
// makes the pulse trains sends no sums (on a tile of few rows and very many samples those were thousands of atomics per
// address)
bool update_reads_row_cost(const UpdateArgs &a) { return balanced_shape(a, update_pulsed_columns(a)); }

template <bool NOISE, int C, bool DEEP = false> static void launch_update_pulsed_t(const UpdateArgs &a, hipStream_t s) {
  if (C == 4 && !DEEP && update_pulsed_balanced(a, C)) {
    const dim3 grid(a.d_size / 4);
    if (a.dev.kind == RPU_DEVICE_CONSTANT_STEP) {
      hipLaunchKernelGGL((k_update_pulsed_balanced<RPU_DEVICE_CONSTANT_STEP, true, NOISE>), grid, dim3(1024), 0, s, a);
    } else if (a.dev.ls_mult_noise) {
      hipLaunchKernelGGL((k_update_pulsed_balanced<RPU_DEVICE_LINEAR_STEP, true, NOISE>), grid, dim3(1024), 0, s, a);
    } else {
      hipLaunchKernelGGL((k_update_pulsed_balanced<RPU_DEVICE_LINEAR_STEP, false, NOISE>), grid, dim3(1024), 0, s, a);
    }
    return;
  }
  dim3 grid((a.x_size + 256 * C - 1) / (256 * C), a.d_size);
  if (a.dev.kind == RPU_DEVICE_CONSTANT_STEP) {
    hipLaunchKernelGGL((k_update_pulsed<RPU_DEVICE_CONSTANT_STEP, true, NOISE, C, DEEP>), grid, dim3(256), 0, s, a);
  } else if (a.dev.ls_mult_noise) {
    hipLaunchKernelGGL((k_update_pulsed<RPU_DEVICE_LINEAR_STEP, true, NOISE, C, DEEP>), grid, dim3(256), 0, s, a);
  } else {
    hipLaunchKernelGGL((k_update_pulsed<RPU_DEVICE_LINEAR_STEP, false, NOISE, C, DEEP>), grid, dim3(256), 0, s, a);
  }
}

// many chunks on one column per lane: the block-wise fetch of the planes (same results)
static bool update_pulsed_deep(const UpdateArgs &a) { return a.n_chunks >= 32; }

// Columns per lane: several once a row is long enough to keep every lane busy with them (they share the scalar work of a
// pass) and the tile has enough rows to fill the chip with such workgroups.  A function of the tile alone: the noise
// streams are laid out per lane, so a tile must take the same variant on its own and in a group.  Two columns are
// neutral for a single tile of 512 x 512 and 25 .. 30 % faster for a group of twelve tiles of 384 x 512 or 512 x 384.
static int update_pulsed_columns(const UpdateArgs &a) {
  if (a.x_size >= 1024 && (long)a.x_size * a.d_size >= (1L << 19)) return 4;
  if (a.x_size > 256 && (long)a.x_size * a.d_size >= (1L << 17)) return 2;
  return 1;
}

void launch_update_pulsed(const UpdateArgs &a, hipStream_t s) {
  const int cols = update_pulsed_columns(a);
  if (a.dev.dw_min_std > 0.0f) {
    if (cols == 4) launch_update_pulsed_t<true, 4>(a, s);
    else if (cols == 2) launch_update_pulsed_t<true, 2>(a, s);
    else if (update_pulsed_deep(a)) launch_update_pulsed_t<true, 1, true>(a, s);
    else launch_update_pulsed_t<true, 1>(a, s);
  } else {
    if (cols == 4) launch_update_pulsed_t<false, 4>(a, s);
    else if (cols == 2) launch_update_pulsed_t<false, 2>(a, s);
    else if (update_pulsed_deep(a)) launch_update_pulsed_t<false, 1, true>(a, s);
    else launch_update_pulsed_t<false, 1>(a, s);
  }
}

// device step (0 ConstantStep, 1 LinearStep with multiplicative noise, 2 with additive noise), cycle-to-cycle noise on,
// columns per lane (two bits: 1, 2 or 4)
int update_pulsed_variant(const UpdateArgs &a) {
  const int step = a.dev.kind == RPU_DEVICE_CONSTANT_STEP ? 0 : (a.dev.ls_mult_noise ? 1 : 2);
  const int cols = update_pulsed_columns(a);
  const int deep = (cols == 1 && update_pulsed_deep(a)) ? 1 : 0; // block-wise fetch of the planes (long batches)
  return ((step * 2 + (a.dev.dw_min_std > 0.0f ? 1 : 0)) * 2 + deep) * 4 + cols / 2;
}

int update_pulsed_workgroups(const UpdateArgs &a) {
  const int c = update_pulsed_columns(a);
  return ((a.x_size + 256 * c - 1) / (256 * c)) * a.d_size;
}

template <bool NOISE, int C, bool DEEP = false>
static void launch_update_pulsed_group_t(const UpdateGroup &g, int step, dim3 grid, hipStream_t s) {
  if (step == 0) {
    hipLaunchKernelGGL((k_update_pulsed_group<RPU_DEVICE_CONSTANT_STEP, true, NOISE, C, DEEP>), grid, dim3(256), 0, s, g);
  } else if (step == 1) {
    hipLaunchKernelGGL((k_update_pulsed_group<RPU_DEVICE_LINEAR_STEP, true, NOISE, C, DEEP>), grid, dim3(256), 0, s, g);
  } else {
    hipLaunchKernelGGL((k_update_pulsed_group<RPU_DEVICE_LINEAR_STEP, false, NOISE, C, DEEP>), grid, dim3(256), 0, s, g);
  }
}

void launch_update_pulsed_group(const UpdateGroup &g, int variant, int total_workgroups, hipStream_t s) {
  const dim3 grid(total_workgroups);
  const int step = variant >> 4, cols = 1 << (variant & 3); // 1, 2, 4 columns per lane were stored as 0, 1, 2
  const bool deep = (variant >> 2) & 1, noise = (variant >> 3) & 1;
  if (noise) {
    if (cols == 4) launch_update_pulsed_group_t<true, 4>(g, step, grid, s);
    else if (cols == 2) launch_update_pulsed_group_t<true, 2>(g, step, grid, s);
    else if (deep) launch_update_pulsed_group_t<true, 1, true>(g, step, grid, s);
    else launch_update_pulsed_group_t<true, 1>(g, step, grid, s);
  } else {
    if (cols == 4) launch_update_pulsed_group_t<false, 4>(g, step, grid, s);
    else if (cols == 2) launch_update_pulsed_group_t<false, 2>(g, step, grid, s);
    else if (deep) launch_update_pulsed_group_t<false, 1, true>(g, step, grid, s);
    else launch_update_pulsed_group_t<false, 1>(g, step, grid, s);
  }
}

void launch_update_prepare_group(const UpdateGroup &g, hipStream_t s) {
  hipLaunchKernelGGL(k_update_prepare_group, dim3((unsigned)g.n * (unsigned)g.m_batch), dim3(256), 0, s, g);
}

int update_lines_blocks(const UpdateArgs &a, bool wide) {
  const int e = wide ? 16 : 4;
  return (a.x_size + e - 1) / e + (a.d_size + e - 1) / e;
}

void launch_update_lines_group(const UpdateGroup &g, bool wide, int total_blocks, hipStream_t s) {
  const dim3 grid(total_blocks, (g.m_batch + 63) / 64);
  if (wide) hipLaunchKernelGGL(k_update_lines_group<16>, grid, dim3(256), 0, s, g);
  else hipLaunchKernelGGL(k_update_lines_group<4>, grid, dim3(256), 0, s, g);
}

void launch_update_aggregated(const UpdateArgs &a, int samples_per_step, hipStream_t s) {
  const int agg_chunks = std::max(1, samples_per_step / 32);
  constexpr int R = 4;
  const dim3 grid((a.x_size + 255) / 256, (a.d_size + R - 1) / R);
  if (a.dev.dw_min_std > 0.0f) hipLaunchKernelGGL((k_update_aggregated<true, R>), grid, dim3(256), 0, s, a, agg_chunks);
  else hipLaunchKernelGGL((k_update_aggregated<false, R>), grid, dim3(256), 0, s, a, agg_chunks);
}

void ensure_update_tables() {
  static std::mutex m;
  static bool done[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) throw RpuError("No current HIP device.");
  std::lock_guard<std::mutex> lock(m);
  if (done[device]) return;
  // quantile mid-points of the standard normal by bisection on erfc, lower half mirrored, scaled to unit variance
  const int n = CTOC_LEVELS;
  std::vector<double> xi(n);
  double sum2 = 0.0;
  for (int q = 0; q < n / 2; ++q) {
    const double p = (q + 0.5) / n;
    double lo = -10.0, hi = 0.0;
    for (int it = 0; it < 80; ++it) {
      const double mid = 0.5 * (lo + hi);
      if (0.5 * std::erfc(-mid / std::sqrt(2.0)) < p) lo = mid;
      else hi = mid;
    }
    xi[q] = 0.5 * (lo + hi);
    xi[n - 1 - q] = -xi[q];
    sum2 += 2.0 * xi[q] * xi[q];
  }
  const double norm = std::sqrt((double)n / sum2);
  std::vector<float> table(n);
  for (int q = 0; q < n; ++q) table[q] = (float)(xi[q] * norm);
  if (hipMemcpyToSymbol(HIP_SYMBOL(g_ctoc_xi), table.data(), sizeof(float) * n) != hipSuccess) {
    throw RpuError("Upload of the noise quantile table failed.");
  }
  done[device] = true;
}

UpdateArgs update_swapped_view(const UpdateArgs &a) {
  UpdateArgs v = a;
  v.swapped = a.swapped ? 0 : 1;
  std::swap(v.x_size, v.d_size);
  std::swap(v.x, v.d);
  std::swap(v.x_sb, v.d_sb);
  std::swap(v.x_sj, v.d_si);
  std::swap(v.x_words, v.d_words);
  std::swap(v.x_planes, v.d_planes);
  std::swap(v.x_val, v.d_val);
  return v;
}

void launch_update_implicit(const UpdateArgs &a, hipStream_t s) {
  dim3 grid((a.x_size + 255) / 256, a.d_size);
  RPU_DISPATCH_DEVICE(k_update_implicit, grid, s, a);
}

void launch_count_pulses(const UpdateArgs &a, unsigned long long *pos, unsigned long long *neg, bool implicit,
                         hipStream_t s) {
  dim3 grid((a.x_size + 255) / 256, a.d_size);
  if (implicit) hipLaunchKernelGGL(k_count_pulses_implicit, grid, dim3(256), 0, s, a, pos, neg);
  else hipLaunchKernelGGL(k_count_pulses, grid, dim3(256), 0, s, a, pos, neg);
}

void launch_write_noise_touched(const UpdateArgs &a, float *w_apparent, const float *w_persistent, float noise_std,
                                bool implicit, hipStream_t s) {
  dim3 grid((a.x_size + 255) / 256, a.d_size);
  hipLaunchKernelGGL(k_write_noise_touched, grid, dim3(256), 0, s, a, w_apparent, w_persistent, noise_std, implicit ? 1 : 0);
}

void launch_update_fp_clipped(const UpdateArgs &a, hipStream_t s) {
  dim3 grid((a.x_size + 255) / 256, a.d_size);
  hipLaunchKernelGGL(k_update_fp_clipped, grid, dim3(256), 0, s, a);
}

void launch_implicit_counts(const UpdateArgs &a, int32_t *counts, hipStream_t s) {
  const long total = (long)a.x_size * a.d_size * a.m_batch;
  hipLaunchKernelGGL(k_implicit_counts, dim3(grid_for(total)), dim3(256), 0, s, a, counts);
}

void launch_unit_vectors(float *out, int n_vec, int size, int start, hipStream_t s) {
  hipLaunchKernelGGL(k_unit_vectors, dim3(grid_for((long)n_vec * size)), dim3(256), 0, s, out, n_vec, size, start);
}

void launch_reduce_weights(float *out, const ReduceArgs &r, size_t size, hipStream_t s) {
  hipLaunchKernelGGL(k_reduce_weights, dim3(grid_for((long)size)), dim3(256), 0, s, out, r, size);
}

void launch_clip(float *w, const float *w_min, const float *w_max, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_clip, dim3(grid_for((long)n)), dim3(256), 0, s, w, w_min, w_max, n);
}

} // namespace rpu_amd
