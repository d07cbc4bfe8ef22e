// Noisy quantized matrix-vector products of the analog tile on gfx950 (CDNA4, wave64).
//
// One "round" is  DAC(in) -> fp32 MFMA contraction with the weights -> ADC(out)  for a batch of
// samples, following the per-sample semantics of the reference CPU path
// (src/rpucuda/rpu_forward_backward_pass.cpp:571-604 DAC, :666-719 ADC, :900-1027 drivers).
// Iterative bound management re-runs only the samples whose ADC saturated, with a halved input
// range, through per-sample state kept in HBM; the host never waits for a round.
//
// Kernels of a call:
//   k_mvm_init     one workgroup per sample: noise-management scale, per-sample state of round 0 and the
//                  DAC-quantized input row, written k-contiguous and zero padded into a scratch matrix.
//   k_mvm_round    the contraction + ADC epilogue.  One workgroup (4 waves) owns a 32 (outputs) x 32
//                  (samples) tile; the 4 waves split the contraction length in four contiguous parts, each
//                  runs v_mfma_f32_32x32x2_f32 over its part in steps of 32 k-values: unit-stride global
//                  loads -> wave-private LDS tile -> MFMA operand registers, software pipelined.  The four
//                  partial tiles are summed in a fixed order through LDS and each wave finishes 8 output
//                  rows: noise, quantize, clip, bound bookkeeping, rescale, store.  Workgroups are numbered
//                  so that the 8 XCDs each work on a contiguous band of output rows (own L2 slice of W).
//                  With bound management a workgroup first writes its share of the tile's input rows as the
//                  next round would quantize them (halved input range) into the other scratch matrix, and the
//                  last workgroup to finish a sample tile (a device-scope counter per tile and round) decides
//                  which of its 32 samples need that round and appends them to its list; no kernel sits
//                  between two rounds.
//   k_mvm_round_tail   later rounds of a launch whose full grid would be large: a fixed number of workgroups walk
//                  the tiles of the samples that are listed (usually few).
//   k_mvm_big      large batches on wide tiles: 128 x 128 workgroup tiles, both operands staged through LDS and
//                  shared by the four waves (64 x 64 per wave), same state / epilogue / random streams; a round is
//                  run by this or by the 32 x 32 kernel, by the number of samples it lists.
//   k_conv_forward convolution forward of a narrow tile (at most 32 outputs): unfold by the index matrix, noise
//                  management, DAC, contraction, ADC and the bound-management rounds in one kernel.
//   *_group        the same kernels over the tiles of a group in one launch.
#include "kernels.h"

#include <mutex>

namespace rpu_amd {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_unaligned __attribute__((ext_vector_type(4), aligned(4))); // a 16-byte load from any float address

namespace {

// Element i (0 or 1) of a two-pointer array of the argument block.  Both pointers are read with constant indices and
// the choice is made on their bits: an index computed at run time (which is also what a plain conditional is
// folded to) would force a kernel's copy of the whole block into indexed (scratch) memory.
template <typename T> __device__ __forceinline__ T *pick2(T *const (&p)[2], int i) {
  const uintptr_t p0 = (uintptr_t)p[0], p1 = (uintptr_t)p[1];
  return (T *)(p0 ^ ((p0 ^ p1) & (uintptr_t)(-(intptr_t)(i & 1))));
}

// quantized input rows read by round `round`: the rows shared within a group for rounds 0 and 1, else the tile's own
__device__ __forceinline__ const float *round_rows(const MvmArgs &a, int round) {
  return (a.xq_first[0] && round < 2) ? (round ? a.xq_first[1] : a.xq_first[0]) : pick2(a.xq, round & 1);
}

constexpr int TILE = 32;
constexpr int WAVES = 4;
constexpr int KSTEP = 32; // k-values per wave step: 128 bytes per operand row

// STOCH = false: for callers that have checked that the DAC draws no random numbers (no stochastic rounding, no input
// noise): the draws are then not even compiled in, which the fully unrolled callers pay for in registers
template <bool STOCH = true>
__device__ __forceinline__ float dac_value(float x, float scale, const IoDev &io, PhiloxKey key,
                                           uint32_t call, int round, int b, int k) {
  // value *= scale; discretize; clip; (+ noise); (asymmetry)      rpu_forward_backward_pass.cpp:583-602
  float v = x * scale;
  if (io.inp_res > 0.0f) {
    float q = v / io.inp_res;
    if (STOCH && io.inp_sto_round) {
      const Philox4 r = philox4x32_10((uint32_t)k, (uint32_t)b, call, RNG_INP_SR | ((uint32_t)round << 8), key.k0, key.k1);
      q = q + (u32_to_uniform(r.v[0]) - 0.5f);
    }
    v = rintf(q) * io.inp_res;
  }
  v = (v > io.inp_bound) ? io.inp_bound : v;
  v = (v < -io.inp_bound) ? -io.inp_bound : v;
  if (STOCH && io.inp_noise > 0.0f) {
    float n[4];
    philox_normal4((uint32_t)k, (uint32_t)b, call, RNG_INP_NOISE | ((uint32_t)round << 8), key, n);
    v += io.inp_noise * n[0];
  }
  if (io.inp_asym != 0.0f) {
    v = v < 0.0f ? v * (1.0f - io.inp_asym) : v;
  }
  return v;
}

// a sample's input row when the call gathers its input through an index (a.in_index)
struct MvmGatherRow {
  const float *image; // element j - 2 at image[j]
  const int *idx;
  __device__ __forceinline__ float at(int k) const {
    const int j = idx[k];
    return j <= 1 ? (float)j : image[j];
  }
};
__device__ __forceinline__ MvmGatherRow mvm_gather_row(const MvmArgs &a, int b) {
  const int n = b / a.in_group;
  return MvmGatherRow{a.in + (long)n * a.in_gs - 2, a.in_index + (long)(b - n * a.in_group) * a.K};
}

// quantized copy of sample b's input row into row `slot` of a scratch matrix, by `width` threads of which
// this one is number t
__device__ __forceinline__ void write_dac_row(const MvmArgs &a, int b, int slot, float scale, int round, float *dst,
                                              int t, int width) {
  float *out = dst + (long)slot * a.k_pad;
  if (a.in_sk == 0) return; // gathered input: the round that reads the rows writes them (mvm_gather_tile_rows)
  const float *row = a.in + (long)b * a.in_sb;
  for (int k = t; k < a.k_pad; k += width) {
    float v = 0.0f;
    if (k < a.K) {
      v = row[(long)k * a.in_sk];
      if (!a.io.perfect) v = dac_value(v, scale, a.io, a.key, a.call, round, b, k);
    }
    out[k] = v;
  }
}

constexpr int LDS_ROW = KSTEP + 4; // floats per staged row: 16-byte aligned, conflict-free 128-bit reads

// workgroup number n -> (output tile, sample tile).  With 8 or more output tiles workgroup n runs on XCD n % 8 and
// XCD x owns the output-row tiles [x * per, (x + 1) * per): each L2 holds a band of W.  A matrix of fewer output
// tiles fits every L2, and consecutive workgroups (hence all XCDs) simply walk the tiles in order.
template <int EDGE = 32>
__device__ __forceinline__ bool tile_of(const MvmArgs &a, int n, int n_act, int &tile_o, int &tile_b) {
  const int tiles_o = (a.O + EDGE - 1) / EDGE;
  if (tiles_o < 8) {
    tile_o = n % tiles_o;
    tile_b = n / tiles_o;
    return tile_b * EDGE < n_act;
  }
  const int per = (tiles_o + 7) / 8;
  const int xcd = n & 7;
  const int m = n >> 3;
  tile_o = xcd * per + (m % per);
  tile_b = m / per;
  return tile_o < tiles_o && tile_b * EDGE < n_act;
}

// workgroups that cover n_act samples with tiles of edge x edge (a multiple of 8)
__host__ __device__ __forceinline__ int workgroups_for(int O, int n_act, int edge = 32) {
  const int tiles_o = (O + edge - 1) / edge;
  const int tiles_b = (n_act + edge - 1) / edge;
  if (tiles_o < 8) return (tiles_o * tiles_b + 7) & ~7;
  return 8 * ((tiles_o + 7) / 8) * tiles_b;
}

// ADC of the four analog sums v of outputs o0 .. o0 + 3 of sample b: asymmetry, noise, quantization, clipping, output
// factor; up / lo return 1 + the largest output index that hit the upper / lower bound (0: none)
// STOCH = false: for callers that have checked that the ADC does not round stochastically
template <bool STOCH = true>
__device__ __forceinline__ void mvm_adc_values(const MvmArgs &a, int round, int b, float fin, int o0, float (&v)[4],
                                               int &up, int &lo, const float *pre = nullptr, const float *post = nullptr) {
  float nz[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.io.out_noise > 0.0f) {
    philox_normal4((uint32_t)(o0 >> 2), (uint32_t)b, a.call, RNG_OUT_NOISE | ((uint32_t)round << 8), a.key, nz);
  }
  const float bound = a.io.out_bound;
  int hit_u = 0, hit_l = 0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float y = v[q];
    // weight noise, IR drop (rpu_forward_backward_pass.cpp:535-560); with the per-line terms the whole value
    if (pre && o0 + q < a.O) y = a.pre_is_total ? pre[o0 + q] : y + pre[o0 + q];
    if (a.io.out_asym > 0.0f) y = y < 0.0f ? y * (1.0f - a.io.out_asym) : y;
    if (a.io.out_noise > 0.0f) y += a.io.out_noise * nz[q];
    if (a.io.out_res > 0.0f) {
      float qq = y / a.io.out_res;
      if (STOCH && a.io.out_sto_round) {
        const Philox4 rr = philox4x32_10((uint32_t)(o0 + q), (uint32_t)b, a.call, RNG_OUT_SR | ((uint32_t)round << 8), a.key.k0, a.key.k1);
        qq = qq + (u32_to_uniform(rr.v[0]) - 0.5f);
      }
      y = rintf(qq) * a.io.out_res;
    }
    const bool over = y > bound, under = y < -bound;
    y = over ? bound : (under ? -bound : y);
    const bool counts = o0 + q < a.O;
    hit_u = (over && counts) ? o0 + q + 1 : hit_u;
    hit_l = (under && counts) ? o0 + q + 1 : hit_l;
    if (post && counts) y += post[o0 + q]; // the other pass, through its own ADC already
    v[q] = y * fin;
  }
  up = hit_u;
  lo = hit_l;
}

// ADC stage for outputs o0 .. o0 + 3 of sample b: v holds the analog sums (rpu_forward_backward_pass.cpp:666-719)
// up / lo return 1 + the largest output index that hit the upper / lower ADC bound (0: none).
__device__ __forceinline__ void mvm_finish_outputs(const MvmArgs &a, int round, int b, float fin, int o0, float (&v)[4],
                                                   int &up, int &lo, const float *pre = nullptr,
                                                   const float *post = nullptr, float *out_rows = nullptr) {
  up = 0;
  lo = 0;
  float *out_p = a.out + (long)b * a.out_sb + (long)o0 * a.out_so;
  long out_so = a.out_so;
  if (out_rows) { // results kept aside, sample-major: [m_batch][O]
    out_p = out_rows + (long)b * a.O + o0;
    out_so = 1;
  }
  if (a.io.perfect) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (o0 + q < a.O) {
        float res = a.alpha * v[q];
        if (a.beta != 0.0f) res += a.beta * out_p[(long)q * out_so];
        out_p[(long)q * out_so] = res;
      }
    }
    return;
  }

  if (fin == 0.0f) { // zero input: the reference short-cuts to a zero output
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (o0 + q < a.O) out_p[(long)q * out_so] = 0.0f;
    }
    return;
  }

  mvm_adc_values(a, round, b, fin, o0, v, up, lo, pre, post);
  if (out_so == 1 && (o0 + 3) < a.O && ((((uintptr_t)out_p) & 15) == 0)) {
    *reinterpret_cast<float4 *>(out_p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (o0 + q < a.O) out_p[(long)q * out_so] = v[q];
    }
  }
}

// input scale of a round and the factor applied to its ADC output
__device__ __forceinline__ float round_scales(const MvmArgs &a, float nm, float red, float &fin) {
  const IoDev &io = a.io;
  const bool use_nm = io.noise_management != RPU_NM_NONE;
  const bool bm = io.bound_management != RPU_BM_NONE;
  float scale;
  if (a.transposed) {
    // backward: scale = 1 / nm ; result *= out_scale * nm
    if (use_nm && nm <= 0.0f) {
      scale = 0.0f;
      fin = 0.0f;
    } else {
      scale = use_nm ? 1.0f / nm : 1.0f;
      fin = use_nm ? io.out_scale * nm : io.out_scale;
    }
  } else if (use_nm && nm <= 0.0f && io.inp_noise <= 0.0f) {
    scale = 0.0f;
    fin = 0.0f;
  } else {
    scale = 1.0f;
    if (use_nm && nm > 0.0f) scale /= nm;
    if (bm) scale /= red;
    fin = io.out_scale / scale;
  }
  return scale;
}

__device__ __forceinline__ float set_round_scales(const MvmArgs &a, int b, float nm, float red) {
  float fin;
  const float scale = round_scales(a, nm, red, fin);
  a.st.scale[b] = scale;
  a.st.fin[b] = fin;
  return scale;
}

// Noise-management value and reduction that sample b, now at (nm, red) with output factor fin, would use in
// the round after `round`; false when the reduction limit is reached or the sample is short-cut to zero
// (rpu_forward_backward_pass.cpp:944-983).
// np_known: the sample's AbsMaxNPSum scale where the caller has just computed it (the init kernel, whose other
// threads must not read back what its first thread is storing); null: read from the per-sample state.
__device__ __forceinline__ bool next_round_params(const MvmArgs &a, int round, int b, float fin, float &nm, float &red,
                                                  const float *np_known = nullptr) {
  const IoDev &io = a.io;
  if (fin == 0.0f) return false;
  const bool stop = ((int)red > io.max_bm_factor) || ((io.inp_res > 0.0f) && (red > io.max_bm_res / io.inp_res));
  if (stop) return false;
  red *= 2.0f;
  if (round == 0 && io.bound_management == RPU_BM_ITERATIVE_WORST_CASE && io.noise_management != RPU_NM_ABS_MAX_NP_SUM) {
    nm = np_known ? *np_known : a.st.nm_np[b];
    red = 1.0f;
  }
  return true;
}

// input scale of the round after `round` for such a sample, 0 when there is none
__device__ __forceinline__ float next_round_scale(const MvmArgs &a, int round, int b, float fin, float nm, float red,
                                                  const float *np_known = nullptr) {
  if (!next_round_params(a, round, b, fin, nm, red, np_known)) return 0.0f;
  float fin_next;
  return round_scales(a, nm, red, fin_next);
}

// Instruction order of one pipelined step (a hint to the scheduler): the 16 MFMAs are spread over the step with
// the LDS writes of the next step's tiles between the first ones and its global loads and LDS reads
// between the others, so that the LDS and memory pipes work underneath the matrix pipe of the same wave.
template <int WMODE, int NACC = 1>
__device__ __forceinline__ void mvm_step_schedule() {
#define RPU_SG(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define RPU_SG_MFMA 0x008
#define RPU_SG_VMEM 0x020
#define RPU_SG_DSR 0x100
#define RPU_SG_DSW 0x200
  // per step: 16 NACC MFMAs; 4 (NACC + 1) LDS writes and as many global loads (a tile of the weights and NACC tiles of
  // quantized rows); LDS reads: 4 per tile of rows, 4 for the weights staged along k or 16 (one per k) for the weights
  // staged along the outputs
  constexpr int mfmas = 16 * NACC, tiles = NACC + 1;
  constexpr int reads = 4 * NACC + (WMODE == 1 ? 16 : 4);
  constexpr int reads_per_slot = (reads + 4 * tiles - 1) / (4 * tiles);
#pragma unroll
  for (int i = 0; i < 4 * tiles; ++i) {
    RPU_SG(RPU_SG_MFMA, 1);
    RPU_SG(RPU_SG_DSW, 1);
  }
#pragma unroll
  for (int i = 0; i < 4 * tiles; ++i) {
    RPU_SG(RPU_SG_MFMA, 1);
    RPU_SG(RPU_SG_VMEM, 1);
    RPU_SG(RPU_SG_DSR, reads_per_slot);
  }
  if (mfmas > 8 * tiles) RPU_SG(RPU_SG_MFMA, mfmas - 8 * tiles);
#undef RPU_SG
#undef RPU_SG_MFMA
#undef RPU_SG_VMEM
#undef RPU_SG_DSR
#undef RPU_SG_DSW
  __builtin_amdgcn_sched_barrier(0);
}

// WMODE = how the weight operand is addressed:
//   0  contraction index contiguous (forward), rows 16-byte aligned, K a multiple of 16
//   1  output index contiguous (backward: W is read transposed in place)
//   2  contraction index contiguous, any row length and alignment (a tile with a bias column has an odd row
//      length): 16-byte loads from 4-byte aligned addresses, the last 1 .. 3 elements of a row one by one
// Operand tiles with a contiguous contraction index (the quantized inputs always, the weights in modes 0, 2) are
// fetched with unit-stride 16-byte loads, 8 lanes per 128-byte row segment, staged in a wave-private LDS
// tile and read back in the MFMA operand layout (lane (r, h) holds row r, k = 16 h .. 16 h + 15).  Reading
// them straight into that layout would make every lane of a load touch a different cache line, which is
// address-bound in the vector L1.  Mode 1 fetches its weight tile the same way, along the outputs (a tile row is the
// 32 outputs of one k: 16-byte loads from 4-byte aligned addresses, nothing read past a row's end), and transposes it
// on the way through LDS: staged as [k][o], read back with one 4-byte read per k (sixteen instead of four 16-byte
// reads; the two half-waves meet in the same banks, which costs little beside a step's matrix work).  Loading the
// sixteen values straight into the operand layout, one 4-byte load each, was the slower way (backward round at
// configuration 2: 11.9 -> 10.8 us, at batch 1024 51.6 -> 43.5 us).  Out-of-range rows / k are clamped to valid
// addresses: their products meet the zero padding of the quantized inputs or are never stored.
// PD = 2, 4: software pipeline with the global loads of PD steps in flight, k_pad a multiple of
// PD * KSTEP * WAVES; PD = 1: one register set, for short contractions, k_pad a multiple of KSTEP.
// NACC = 2 (round 0 only, PD = 2): the same weights also multiply the rows that round 1 would use (written by the init
// kernel into the other scratch matrix), into a second accumulator; both rounds go through the ADC stage, round r
// into a.dual.buf[r], with their own saturation marks.  Which of the two is a sample's output is decided when its
// tile is finished (mvm_tile_finished_dual) and copied out at the start of the next launch.  NACC = 3: the rows of
// round 2 as well (a.dual.xq2, also written by the init kernel), into a third accumulator.
template <int PD, int WMODE, int NACC = 1>
__device__ __forceinline__ void mvm_round_tile(const MvmArgs &a, int round, int tile_o, int tile_b, int n_act,
                                               float (*red)[16][64], float *stage) {
  constexpr bool DUAL = NACC >= 2;
  constexpr bool TRI = NACC == 3;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;

  // operand rows owned by this lane in the MFMA layout
  const int slot_in = tile_b * TILE + r;
  const bool b_ok = slot_in < n_act;

  const int K = a.K;
  // steps of 32 k-values, dealt to the waves in contiguous parts (equal parts, a multiple of PD, when PD >= 2;
  // a short contraction may leave the last waves without a step)
  const int steps = a.k_pad / KSTEP;
  const int per_wave = (steps + WAVES - 1) / WAVES;
  const int s_begin = min(wave * per_wave, steps);
  const int s_end = min(s_begin + per_wave, steps);

  float *stage_x = stage + wave * ((NACC + 1) * TILE * LDS_ROW);
  float *stage_w = stage_x + TILE * LDS_ROW;
  float *stage_x1 = stage_w + TILE * LDS_ROW;  // DUAL only
  float *stage_x2 = stage_x1 + TILE * LDS_ROW; // TRI only

  // staging layout of this lane: pass t covers rows 8 t .. 8 t + 7, lane = (row in pass) * 8 + 16-byte chunk
  const int st_row = lane >> 3;
  const int st_chunk = (lane & 7) * 4;
  const float *xq = round_rows(a, round);
  const float *x_src[4];
  const float *x1_src[4];
  const float *x2_src[4];
  const float *w_src[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = t * 8 + st_row;
    const int slot = min(tile_b * TILE + row, n_act - 1);
    const int xrow = (round > 0) ? pick2(a.st.row, round & 1)[slot] : slot;
    x_src[t] = xq + (long)xrow * a.k_pad + st_chunk;
    x1_src[t] = DUAL ? a.xq[1] + (long)xrow * a.k_pad + st_chunk : nullptr;
    x2_src[t] = TRI ? a.dual.xq2 + (long)xrow * a.k_pad + st_chunk : nullptr;
    const int o = min(tile_o * TILE + row, a.O - 1);
    w_src[t] = a.w + (long)o * a.w_ld;
  }

  floatx16 acc, acc1, acc2;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc[i] = 0.0f;
    acc1[i] = 0.0f;
    acc2[i] = 0.0f;
  }

  // sample of this lane's output column and its output factor: fetched now, used by the ADC stage
  int b_out = slot_in;
  float fin_out = 1.0f;
  if (!a.io.perfect && b_ok) {
    if (round > 0) b_out = pick2(a.st.list, round & 1)[slot_in];
    fin_out = a.st.fin[b_out];
  }

  auto gload = [&](int s, f32x4 (&gx)[4], f32x4 (&gw)[4], float (&wd)[16], f32x4 (&gx1)[4], f32x4 (&gx2)[4]) {
    const int k0 = s * KSTEP;
#pragma unroll
    for (int t = 0; t < 4; ++t) gx[t] = *reinterpret_cast<const f32x4 *>(x_src[t] + k0);
    if constexpr (DUAL) {
#pragma unroll
      for (int t = 0; t < 4; ++t) gx1[t] = *reinterpret_cast<const f32x4 *>(x1_src[t] + k0);
    }
    if constexpr (TRI) {
#pragma unroll
      for (int t = 0; t < 4; ++t) gx2[t] = *reinterpret_cast<const f32x4 *>(x2_src[t] + k0);
    }
    if (WMODE == 0) {
      const int kc = min(k0 + st_chunk, K - 4); // K % 16 == 0: past K the inputs are zero padding
#pragma unroll
      for (int t = 0; t < 4; ++t) gw[t] = *reinterpret_cast<const f32x4 *>(w_src[t] + kc);
    } else if (WMODE == 1) {
      // rows of the stored matrix run along the outputs: 16-byte loads along o (eight lanes per 128-byte row of the
      // tile), transposed on the way through LDS
      const int o_base = tile_o * TILE + st_chunk;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int kc = min(k0 + t * 8 + st_row, K - 1);
        const float *p = a.w + (long)kc * a.w_ld + o_base;
        if (o_base + 4 <= a.O) {
          gw[t] = *reinterpret_cast<const f32x4_unaligned *>(p);
        } else { // the end of a row: nothing is read past it
          f32x4 z;
          z.x = (o_base < a.O) ? p[0] : 0.0f;
          z.y = (o_base + 1 < a.O) ? p[1] : 0.0f;
          z.z = (o_base + 2 < a.O) ? p[2] : 0.0f;
          z.w = 0.0f;
          gw[t] = z;
        }
      }
    } else {
      const int kc = k0 + st_chunk;
      if (kc + 4 <= K) {
#pragma unroll
        for (int t = 0; t < 4; ++t) gw[t] = *reinterpret_cast<const f32x4_unaligned *>(w_src[t] + kc);
      } else { // the end of a row: nothing is read past it
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          f32x4 z;
          z.x = (kc < K) ? w_src[t][kc] : 0.0f;
          z.y = (kc + 1 < K) ? w_src[t][kc + 1] : 0.0f;
          z.z = (kc + 2 < K) ? w_src[t][kc + 2] : 0.0f;
          z.w = 0.0f;
          gw[t] = z;
        }
      }
    }
  };
  auto lds_store = [&](const f32x4 (&gx)[4], const f32x4 (&gw)[4], const f32x4 (&gx1)[4], const f32x4 (&gx2)[4]) {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int off = (t * 8 + st_row) * LDS_ROW + st_chunk;
      *reinterpret_cast<f32x4 *>(stage_x + off) = gx[t];
      *reinterpret_cast<f32x4 *>(stage_w + off) = gw[t];
      if constexpr (DUAL) *reinterpret_cast<f32x4 *>(stage_x1 + off) = gx1[t];
      if constexpr (TRI) *reinterpret_cast<f32x4 *>(stage_x2 + off) = gx2[t];
    }
  };
  auto lds_read = [&](float (&xd)[16], float (&wd)[16], float (&xd1)[16], float (&xd2)[16]) {
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int off = r * LDS_ROW + h * 16 + v4 * 4;
      const f32x4 tx = *reinterpret_cast<const f32x4 *>(stage_x + off);
      xd[v4 * 4 + 0] = tx.x; xd[v4 * 4 + 1] = tx.y; xd[v4 * 4 + 2] = tx.z; xd[v4 * 4 + 3] = tx.w;
      if constexpr (DUAL) {
        const f32x4 t1 = *reinterpret_cast<const f32x4 *>(stage_x1 + off);
        xd1[v4 * 4 + 0] = t1.x; xd1[v4 * 4 + 1] = t1.y; xd1[v4 * 4 + 2] = t1.z; xd1[v4 * 4 + 3] = t1.w;
      }
      if constexpr (TRI) {
        const f32x4 t2 = *reinterpret_cast<const f32x4 *>(stage_x2 + off);
        xd2[v4 * 4 + 0] = t2.x; xd2[v4 * 4 + 1] = t2.y; xd2[v4 * 4 + 2] = t2.z; xd2[v4 * 4 + 3] = t2.w;
      }
      if (WMODE != 1) {
        const f32x4 tw = *reinterpret_cast<const f32x4 *>(stage_w + off);
        wd[v4 * 4 + 0] = tw.x; wd[v4 * 4 + 1] = tw.y; wd[v4 * 4 + 2] = tw.z; wd[v4 * 4 + 3] = tw.w;
      }
    }
    if (WMODE == 1) { // the staged tile is [k][o]: this lane's output column, k = 16 h .. 16 h + 15
#pragma unroll
      for (int i = 0; i < 16; ++i) wd[i] = stage_w[(h * 16 + i) * LDS_ROW + r];
    }
  };
  auto mfma16 = [&](const float (&wd)[16], const float (&xd)[16], const float (&xd1)[16], const float (&xd2)[16]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wd[i], xd[i], acc, 0, 0, 0);
      if constexpr (DUAL) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(wd[i], xd1[i], acc1, 0, 0, 0);
      if constexpr (TRI) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(wd[i], xd2[i], acc2, 0, 0, 0);
    }
  };

  if constexpr (PD >= 2) {
    // PD register sets hold the global loads of the next PD steps; the operand registers are double
    // buffered, so the LDS round trip of step t + 1 and the loads of step t + 1 + PD are issued ahead
    // of the 16 MFMAs of step t and complete underneath them.
    f32x4 gx0[4], gw0[4], gx1[4], gw1[4], gx2[4], gw2[4], gx3[4], gw3[4];
    f32x4 hx0[4], hx1[4], hx2[4], hx3[4]; // DUAL: the rows of round 1
    f32x4 ix0[4], ix1[4], ix2[4], ix3[4]; // TRI: the rows of round 2
    float wr0[16], wr1[16], wr2[16], wr3[16];
    float xc0[16], wc0[16], xc1[16], wc1[16];
    float yc0[16], yc1[16]; // DUAL: operands of round 1
    float zc0[16], zc1[16]; // TRI: operands of round 2
    // step T runs from the operand registers (XC, WC); step T + 1 moves from register set (GX, GW, WR)
    // through LDS into (XN, WN) and the set is refilled with step T + 1 + PD
#define RPU_MVM_STEP(T, GX, GW, WR, HX, IX, XC, WC, YC, ZC, XN, WN, YN, ZN) \
  {                                                                         \
    lds_store(GX, GW, HX, IX);                                              \
    gload(min((T) + 1 + PD, s_end - 1), GX, GW, WR, HX, IX);                \
    lds_read(XN, WN, YN, ZN);                                               \
    mfma16(WC, XC, YC, ZC);                                                 \
    mvm_step_schedule<WMODE, NACC>();                                       \
  }
    gload(s_begin, gx0, gw0, wr0, hx0, ix0);
    gload(min(s_begin + 1, s_end - 1), gx1, gw1, wr1, hx1, ix1);
    if constexpr (PD == 4) {
      gload(min(s_begin + 2, s_end - 1), gx2, gw2, wr2, hx2, ix2);
      gload(min(s_begin + 3, s_end - 1), gx3, gw3, wr3, hx3, ix3);
    }
    lds_store(gx0, gw0, hx0, ix0);
    lds_read(xc0, wc0, yc0, zc0);
    gload(min(s_begin + PD, s_end - 1), gx0, gw0, wr0, hx0, ix0);
    for (int s = s_begin; s < s_end; s += PD) {
      if constexpr (PD == 4) {
        RPU_MVM_STEP(s, gx1, gw1, wr1, hx1, ix1, xc0, wc0, yc0, zc0, xc1, wc1, yc1, zc1)
        RPU_MVM_STEP(s + 1, gx2, gw2, wr2, hx2, ix2, xc1, wc1, yc1, zc1, xc0, wc0, yc0, zc0)
        RPU_MVM_STEP(s + 2, gx3, gw3, wr3, hx3, ix3, xc0, wc0, yc0, zc0, xc1, wc1, yc1, zc1)
        RPU_MVM_STEP(s + 3, gx0, gw0, wr0, hx0, ix0, xc1, wc1, yc1, zc1, xc0, wc0, yc0, zc0)
      } else {
        RPU_MVM_STEP(s, gx1, gw1, wr1, hx1, ix1, xc0, wc0, yc0, zc0, xc1, wc1, yc1, zc1)
        RPU_MVM_STEP(s + 1, gx0, gw0, wr0, hx0, ix0, xc1, wc1, yc1, zc1, xc0, wc0, yc0, zc0)
      }
    }
#undef RPU_MVM_STEP
  } else {
    f32x4 gx[4], gw[4], hx[4], ix[4];
    float wn[16], xc[16], wc[16], yc[16], zc[16];
    if (s_begin < s_end) gload(s_begin, gx, gw, wn, hx, ix);
    for (int s = s_begin; s < s_end; ++s) {
      lds_store(gx, gw, hx, ix);
      lds_read(xc, wc, yc, zc);
      gload(min(s + 1, s_end - 1), gx, gw, wn, hx, ix);
      mfma16(wc, xc, yc, zc);
    }
  }

  // sum the four parts of the contraction in a fixed order
#pragma unroll
  for (int i = 0; i < 16; ++i) red[wave][i][lane] = acc[i];
  __syncthreads();

  // this wave finishes accumulator group `wave`: rows wave*8 + h*4 + m, column r
  float v[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int i = wave * 4 + q;
    v[q] = ((red[0][i][lane] + red[1][i][lane]) + red[2][i][lane]) + red[3][i][lane];
  }
  const int o0 = tile_o * TILE + wave * 8 + h * 4;
  int up = 0, lo = 0;
  if (b_ok && o0 < a.O) {
    const float *pre = nullptr, *post = nullptr;
    if (a.pre_add) {
      const int xrow = (round > 0) ? pick2(a.st.row, round & 1)[slot_in] : slot_in;
      pre = a.pre_add + (long)xrow * a.O;
      if (a.post_add) post = a.post_add + (long)xrow * a.O;
    }
    mvm_finish_outputs(a, round, b_out, fin_out, o0, v, up, lo, pre, post, DUAL ? a.dual.buf[0] : nullptr);
  }
  int up1 = 0, lo1 = 0, up2 = 0, lo2 = 0;
  if constexpr (DUAL) {
    // scale and output factor of the later rounds, as the sample's state will hold them if it gets there
    bool goes_on = b_ok && o0 < a.O;
    float nm = 0.0f, rd = 0.0f, fin_r = fin_out;
    if (goes_on) {
      nm = a.st.nm[b_out];
      rd = a.st.red[b_out];
    }
    auto later_round = [&](const floatx16 &acc_r, int r, float *rows, int &up_r, int &lo_r) {
      __syncthreads(); // the partial sums of the round before have been read
#pragma unroll
      for (int i = 0; i < 16; ++i) red[wave][i][lane] = acc_r[i];
      __syncthreads();
      float vr[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = wave * 4 + q;
        vr[q] = ((red[0][i][lane] + red[1][i][lane]) + red[2][i][lane]) + red[3][i][lane];
      }
      if (goes_on) goes_on = next_round_params(a, r - 1, b_out, fin_r, nm, rd);
      if (goes_on) {
        round_scales(a, nm, rd, fin_r);
        mvm_finish_outputs(a, r, b_out, fin_r, o0, vr, up_r, lo_r, nullptr, nullptr, rows);
      }
    };
    later_round(acc1, 1, a.dual.buf[1], up1, lo1);
    if constexpr (TRI) later_round(acc2, 2, a.dual.buf[2], up2, lo2);
  }
  if (!a.io.perfect && a.io.bound_management != RPU_BM_NONE) {
    // saturation flags of the tile's 32 samples: combined in LDS, then one device-scope atomic per sample
    // and bound.  The returned values are consumed so that the wave waits until the atomics have been
    // performed before the workgroup signals its tile as finished (mvm_tile_finished).  A fused launch sends the
    // marks of all its rounds together (thread 64 rr + t: round rr), so that it waits for one round trip, not one
    // per round; round 0 of a fused launch lists sample b at position b.
    int *hits = reinterpret_cast<int *>(&red[0][0][0]); // the partial sums have been consumed ...
    __syncthreads();                                      // ... by every wave
    if (threadIdx.x < NACC * 2 * TILE) hits[threadIdx.x] = 0;
    __syncthreads();
    if (up) atomicMax(&hits[r], up);
    if (lo) atomicMax(&hits[TILE + r], lo);
    if constexpr (DUAL) {
      if (up1) atomicMax(&hits[2 * TILE + r], up1);
      if (lo1) atomicMax(&hits[3 * TILE + r], lo1);
    }
    if constexpr (TRI) {
      if (up2) atomicMax(&hits[4 * TILE + r], up2);
      if (lo2) atomicMax(&hits[5 * TILE + r], lo2);
    }
    __syncthreads();
    if (threadIdx.x < NACC * 2 * TILE) {
      const int rr = (int)threadIdx.x / (2 * TILE);       // round of the fused launch (0 otherwise)
      const bool upper = ((int)threadIdx.x & (2 * TILE - 1)) < TILE;
      const int t = threadIdx.x & (TILE - 1);
      const int hit = hits[threadIdx.x];
      const int slot = tile_b * TILE + t;
      if (hit && slot < n_act) {
        int *target;
        if (rr == 0) {
          const int bs = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
          target = upper ? &a.st.hit_up[bs] : &a.st.hit_lo[bs];
        } else {
          target = (rr == 1 ? a.dual.hit1 : a.dual.hit2) + (upper ? 0 : a.m_batch) + slot;
        }
        const int old = atomicMax(target, hit);
        asm volatile("" ::"v"(old));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// per-sample noise management and state of round 0.  One workgroup per sample.
// rpu_forward_backward_pass.cpp:112-178 (scales), :919-969 (forward), :1003-1022 (backward)

// Reductions over the SUB threads that share a sample: SUB = 256 is the whole workgroup (through LDS), smaller
// values are aligned lane groups of a wave (shuffles).  Every thread of the group gets the result.
template <int SUB>
__device__ __forceinline__ float group_max(float v, float *sh) {
  if constexpr (SUB == 256) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    const float r = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    __syncthreads();
    return r;
  } else {
#pragma unroll
    for (int off = SUB / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
  }
}

template <int SUB>
__device__ __forceinline__ float group_sum(float v, float *sh) {
  if constexpr (SUB == 256) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    const float r = ((sh[0] + sh[1]) + sh[2]) + sh[3];
    __syncthreads();
    return r;
  } else {
#pragma unroll
    for (int off = SUB / 2; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
  }
}

// State of round 0 and quantized input row of sample b, by the SUB threads that share the sample (this one is
// number t of them); gid / gstride number the threads that work on this tile's call, for clearing its counters.
template <int SUB>
__device__ __forceinline__ void mvm_init_sample(const MvmArgs &a, int b, int t, long gid, long gstride, float *sh) {
  const IoDev &io = a.io;
  // rows shared with other tiles of a group are written by one of them
  float *const rows0 = a.xq_first[0] ? a.xq_first[0] : a.xq[0];
  float *const rows1 = a.xq_first[0] ? a.xq_first[1] : a.xq[1];
  const bool writes = !a.xq_first[0] || a.xq_first_writer;
  if (io.perfect) { // plain copy into the k-contiguous scratch
    if (writes) write_dac_row(a, b, b, 1.0f, 0, rows0, t, SUB);
    return;
  }
  const float *row = a.in + (long)b * a.in_sb;
  // a row of up to 8 elements per thread is read once and kept for the statistics and the quantized rows
  constexpr int KEEP = 8;
  const bool kept = a.k_pad <= KEEP * SUB;
  float xk[KEEP];
  if (kept) {
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int k = t + i * SUB;
      xk[i] = (k < a.K) ? row[(long)k * a.in_sk] : 0.0f;
    }
  }
  float nm = 1.0f;
  float np_scale = 0.0f; // the AbsMaxNPSum scale, known to every thread of the group once it is computed
  const bool worst_case = io.bound_management == RPU_BM_ITERATIVE_WORST_CASE;
  const bool need_np = io.noise_management == RPU_NM_ABS_MAX_NP_SUM || worst_case;
  const bool running = io.noise_management == RPU_NM_AVERAGE_ABS_MAX ||
                       io.noise_management == RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE;
  if (io.noise_management == RPU_NM_ABS_MAX || io.noise_management == RPU_NM_MAX || need_np || (running && a.nm_phase == 1)) {
    float amax = 0.0f, vmax = -INFINITY, ps = 0.0f, ns = 0.0f;
    if (kept) {
#pragma unroll
      for (int i = 0; i < KEEP; ++i) {
        if (t + i * SUB < a.K) {
          const float x = xk[i];
          amax = fmaxf(amax, fabsf(x));
          vmax = fmaxf(vmax, x);
          ps += x > 0.0f ? x : 0.0f;
          ns += x < 0.0f ? x : 0.0f;
        }
      }
    } else {
      for (int k = t; k < a.K; k += SUB) {
        const float x = row[(long)k * a.in_sk];
        amax = fmaxf(amax, fabsf(x));
        vmax = fmaxf(vmax, x);
        ps += x > 0.0f ? x : 0.0f;
        ns += x < 0.0f ? x : 0.0f;
      }
    }
    amax = group_max<SUB>(amax, sh);
    if (running && a.nm_phase == 1) { // first pass of the running average: the scan over the batch comes next
      if (t == 0) a.st.nm[b] = amax;
      return;
    }
    if (io.noise_management == RPU_NM_MAX) {
      vmax = group_max<SUB>(vmax, sh);
      nm = io.nm_thres > 0.0f ? fminf(vmax, io.nm_thres) : vmax;
    } else if (io.noise_management == RPU_NM_ABS_MAX) {
      nm = io.nm_thres > 0.0f ? fminf(amax, io.nm_thres) : amax;
    }
    if (need_np) {
      ps = group_sum<SUB>(ps, sh);
      ns = group_sum<SUB>(ns, sh);
      const float bound = isinf(io.out_bound) ? 1.0f : io.out_bound;
      const float sum = fmaxf(ps, -ns);
      const float am = io.nm_thres > 0.0f ? fminf(amax, io.nm_thres) : amax;
      float np = sum * io.nm_assumed_wmax / bound;
      if (io.inp_res > 0.0f) np = fminf(am / io.inp_res * io.max_bm_res, np);
      np = fmaxf(am, np);
      if (io.noise_management == RPU_NM_ABS_MAX_NP_SUM) nm = np;
      if (t == 0) a.st.nm_np[b] = np;
      np_scale = np;
    }
  }
  if (io.noise_management == RPU_NM_CONSTANT) {
    nm = io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
  }
  if (running) nm = a.st.nm[b]; // second pass: the averaged scale of this sample
  // every thread of the group knows nm: the scales need no exchange
  float fin;
  const float scale = round_scales(a, nm, 1.0f, fin);
  if (t == 0) {
    a.st.nm[b] = nm;
    a.st.red[b] = 1.0f;
    a.st.hit_up[b] = 0;
    a.st.hit_lo[b] = 0;
    a.st.scale[b] = scale;
    a.st.fin[b] = fin;
    a.st.rounds[b] = (fin == 0.0f) ? 0 : 1;
    if (io.bound_management != RPU_BM_NONE) a.st.next_scale[0][b] = next_round_scale(a, 0, b, fin, nm, 1.0f, &np_scale);
  }
  if (gid < MVM_COUNT_WORDS) a.st.count[gid] = 0; // per-round counts and the arrival counters of k_mvm_rounds_rest
  {
    const long n_done = 32L * ((a.m_batch + TILE - 1) / TILE);
    for (long idx = gid; idx < n_done; idx += gstride) a.st.tile_done[idx] = 0;
  }
  // the input range of a second round is known as well: its row is quantized now, while the input is at hand,
  // so that the first round has nothing to prepare
  float next = 0.0f, next2 = 0.0f;
  // (the scale of a worst-case second round is the one just computed: the threads of the other waves must not read it
  // back from memory, where the group's first thread may not have stored it yet)
  if (a.rows_ahead_in_init && io.bound_management != RPU_BM_NONE) next = next_round_scale(a, 0, b, fin, nm, 1.0f, &np_scale);
  if (a.dual.rounds == 3 && next != 0.0f) { // the fused launch of three rounds reads the rows of round 2 as well
    float nm1 = nm, red1 = 1.0f, fin1 = fin;
    if (next_round_params(a, 0, b, fin1, nm1, red1, &np_scale)) {
      round_scales(a, nm1, red1, fin1);
      next2 = next_round_scale(a, 1, b, fin1, nm1, red1);
    }
  }
  if (!writes) return;
  if (kept) {
    float *out0 = rows0 + (long)b * a.k_pad;
    float *out1 = rows1 + (long)b * a.k_pad;
    float *out2 = a.dual.xq2 + (long)b * a.k_pad;
#pragma unroll
    for (int i = 0; i < KEEP; ++i) {
      const int k = t + i * SUB;
      if (k < a.k_pad) {
        out0[k] = (k < a.K) ? dac_value(xk[i], scale, io, a.key, a.call, 0, b, k) : 0.0f;
        if (next != 0.0f) out1[k] = (k < a.K) ? dac_value(xk[i], next, io, a.key, a.call, 1, b, k) : 0.0f;
        if (next2 != 0.0f) out2[k] = (k < a.K) ? dac_value(xk[i], next2, io, a.key, a.call, 2, b, k) : 0.0f;
      }
    }
  } else {
    write_dac_row(a, b, b, scale, 0, rows0, t, SUB);
    if (next != 0.0f) write_dac_row(a, b, b, next, 1, rows1, t, SUB);
    if (next2 != 0.0f) write_dac_row(a, b, b, next2, 2, a.dual.xq2, t, SUB);
  }
}

// SUB threads per sample: a workgroup holds 256 / SUB samples
template <int SUB>
__global__ __launch_bounds__(256) void k_mvm_init(MvmArgs a) {
  __shared__ float sh[8];
  const int b = blockIdx.x * (256 / SUB) + threadIdx.x / SUB;
  if (b >= a.m_batch) return; // a whole group of SUB threads leaves together
  mvm_init_sample<SUB>(a, b, threadIdx.x % SUB, blockIdx.x * 256L + threadIdx.x, gridDim.x * 256L, sh);
}

// Init kernels of a call whose samples are patches gathered from images (MvmArgs::in_index).  Both read with lanes
// along the patches: that follows the index matrix as it is set ([K][patches]) and, for a convolution, the image rows
// (neighbouring patches read neighbouring elements).  Same per-sample state and the same DAC draws (keyed by sample
// and element) as mvm_init_sample on the materialized patch matrix.  For noise management none / constant / abs-max /
// max; the other kinds run mvm_init_sample, which gathers row by row.
//
// First kernel (abs-max / max only): a workgroup of 16 waves owns 64 patches, one per lane, of four images; wave w
// takes the elements k = w (mod 16), so a patch's largest input is a running maximum of its lane and the waves meet in
// LDS.  The noise-management value goes to st.nm.
__global__ __launch_bounds__(1024) void k_mvm_gather_max(MvmArgs a) {
  constexpr int NI = 4; // images per workgroup: an index entry is read once for the four
  __shared__ float sh_max[2][NI][16][64];
  const IoDev &io = a.io;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int P = a.in_group;
  const int blocks_p = (P + 63) / 64;
  const int n_images = a.m_batch / P;
  const int n0 = (int)(blockIdx.x / blocks_p) * NI, p0 = (int)(blockIdx.x % blocks_p) * 64;
  const bool live = p0 + lane < P;
  const int images = min(NI, n_images - n0);
  const float *image = a.in + (long)n0 * a.in_gs - 2;
  const int *idx = a.in_index_lines + p0 + lane; // + k * P
  float amax[NI], vmax[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    amax[i] = 0.0f;
    vmax[i] = -INFINITY;
  }
  for (int k0 = wave; k0 < a.K; k0 += 64) { // sixteen loads in flight
    int j[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 16 * u;
      j[u] = (live && k < a.K) ? idx[(long)k * P] : -1;
    }
    float x[4][NI];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int i = 0; i < NI; ++i) x[u][i] = (j[u] > 1 && i < images) ? image[j[u] + (long)i * a.in_gs] : (float)j[u];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j[u] >= 0) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          amax[i] = fmaxf(amax[i], fabsf(x[u][i]));
          vmax[i] = fmaxf(vmax[i], x[u][i]);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    sh_max[0][i][wave][lane] = amax[i];
    sh_max[1][i][wave][lane] = vmax[i];
  }
  __syncthreads();
  if (wave >= images || !live) return; // wave i finishes image n0 + i
  float am = 0.0f, vm = -INFINITY;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    am = fmaxf(am, sh_max[0][wave][w][lane]);
    vm = fmaxf(vm, sh_max[1][wave][w][lane]);
  }
  float nm;
  if (io.noise_management == RPU_NM_MAX) nm = io.nm_thres > 0.0f ? fminf(vm, io.nm_thres) : vm;
  else nm = io.nm_thres > 0.0f ? fminf(am, io.nm_thres) : am;
  a.st.nm[(n0 + wave) * P + p0 + lane] = nm;
}

// Second kernel: a workgroup quantizes a block of 64 patches x 64 elements with each patch's input scale and stores it
// through LDS with lanes along a row; the workgroups of the first 64 elements also set up the per-sample state.
__global__ __launch_bounds__(256) void k_mvm_init_gather(MvmArgs a) {
  __shared__ float tile[64][65];
  const IoDev &io = a.io;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int P = a.in_group;
  const int blocks_p = (P + 63) / 64, blocks_k = a.k_pad / 64 + ((a.k_pad & 63) ? 1 : 0);
  const int k0 = (int)(blockIdx.x % blocks_k) * 64;
  const int pb = (int)(blockIdx.x / blocks_k);
  const int n = pb / blocks_p, p0 = (pb % blocks_p) * 64;
  const bool live = p0 + lane < P;
  const int b = n * P + p0 + lane;
  const float *image = a.in + (long)n * a.in_gs - 2;
  const int *idx = a.in_index_lines + p0 + lane; // + k * P
  int j[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int k = k0 + wave * 16 + i;
    j[i] = (live && k < a.K) ? idx[(long)k * P] : -1;
  }
  float scale = 1.0f;
  if (!io.perfect) {
    float nm = 1.0f;
    if (io.noise_management == RPU_NM_ABS_MAX || io.noise_management == RPU_NM_MAX) nm = live ? a.st.nm[b] : 1.0f;
    else if (io.noise_management == RPU_NM_CONSTANT) nm = io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
    float fin;
    scale = round_scales(a, nm, 1.0f, fin);
    if (k0 == 0 && wave == 0 && live) {
      a.st.nm[b] = nm;
      a.st.red[b] = 1.0f;
      a.st.hit_up[b] = 0;
      a.st.hit_lo[b] = 0;
      a.st.scale[b] = scale;
      a.st.fin[b] = fin;
      a.st.rounds[b] = (fin == 0.0f) ? 0 : 1;
      if (io.bound_management != RPU_BM_NONE) a.st.next_scale[0][b] = next_round_scale(a, 0, b, fin, nm, 1.0f);
    }
    const long gid = blockIdx.x * 256L + threadIdx.x, gstride = gridDim.x * 256L;
    if (gid < MVM_COUNT_WORDS) a.st.count[gid] = 0;
    const long n_done = 32L * ((a.m_batch + TILE - 1) / TILE);
    for (long i = gid; i < n_done; i += gstride) a.st.tile_done[i] = 0;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int k = k0 + wave * 16 + i;
    float v = 0.0f;
    if (j[i] >= 0) {
      v = (j[i] <= 1) ? (float)j[i] : image[j[i]];
      if (!io.perfect) v = dac_value(v, scale, io, a.key, a.call, 0, b, k);
    }
    tile[lane][wave * 16 + i] = v;
  }
  __syncthreads();
  float *rows = a.xq[0] + ((long)n * P + p0) * a.k_pad + k0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = i * 4 + wave;
    if (p0 + row < P && k0 + lane < a.k_pad) rows[(long)row * a.k_pad + lane] = tile[row][lane];
  }
}

// At the start of round `round`, the workgroups of a sample tile (one per output tile) each quantize a
// 1 / tiles_o share of the tile's input rows with the input range the *next* round would use (next_scale),
// into the other scratch matrix at the rows of this round's list positions.  Whether a sample needs that
// round is only known when all of its outputs are done; writing the rows ahead costs a few elements per
// thread and takes the re-quantization off the path between two rounds.
// FUSED: called by the fused launch of rounds 0 and 1 for the rows of round 2 (as `round` = 1 with every sample
// listed at its own number); the scale is derived from the sample's state of round 0 and the rows go to a.dual.xq2.
template <bool FUSED = false>
__device__ __forceinline__ void mvm_prepare_next_rows(const MvmArgs &a, int round, int tile_o, int tile_b, int n_act) {
  __shared__ float sh_next_scale[TILE];
  __shared__ int sh_next_b[TILE];
  if (threadIdx.x < TILE) {
    const int slot = tile_b * TILE + threadIdx.x;
    int b = 0;
    float scale = 0.0f; // 0: the sample can have no further round
    if (slot < n_act) {
      if constexpr (FUSED) {
        b = slot;
        float nm = a.st.nm[b], red = a.st.red[b], fin = a.st.fin[b];
        if (next_round_params(a, 0, b, fin, nm, red)) {
          round_scales(a, nm, red, fin);
          scale = next_round_scale(a, 1, b, fin, nm, red);
        }
      } else {
        b = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
        scale = pick2(a.st.next_scale, round & 1)[slot];
      }
    }
    sh_next_b[threadIdx.x] = b;
    sh_next_scale[threadIdx.x] = scale;
  }
  __syncthreads();
  const int tiles_o = (a.O + TILE - 1) / TILE;
  const int chunk = (a.k_pad + tiles_o - 1) / tiles_o;
  const int k_lo = tile_o * chunk;
  const int k_hi = min(k_lo + chunk, a.k_pad);
  float *__restrict__ dst = FUSED ? a.dual.xq2 : pick2(a.xq, (round + 1) & 1);
  const float *__restrict__ in = a.in;
  // a trip covers 32 k-values of all 32 rows: 8 thread-rows x 4 rows each.  The loads of four trips are issued
  // together: a narrow tile has few workgroups per sample tile and each walks a long piece of the rows.
  const int kq = threadIdx.x & 31, rq = threadIdx.x >> 5;
  float sc[4];
  int bt[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bt[i] = sh_next_b[4 * rq + i];
    sc[i] = sh_next_scale[4 * rq + i];
  }
  for (int k0 = k_lo; k0 < k_hi; k0 += 128) {
    float xv[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 32 * u + kq;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xv[u][i] = (k < k_hi && sc[i] != 0.0f && k < a.K) ? in[(long)bt[i] * a.in_sb + (long)k * a.in_sk] : 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + 32 * u + kq;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (k < k_hi && sc[i] != 0.0f) {
          const float v = (k < a.K) ? dac_value(xv[u][i], sc[i], a.io, a.key, a.call, round + 1, bt[i], k) : 0.0f;
          dst[(long)(tile_b * TILE + 4 * rq + i) * a.k_pad + k] = v;
        }
      }
    }
  }
}

// After round `round`, for sample b at position `slot` of that round's list: a sample whose ADC saturated
// gets another round unless the reduction limit is reached (rpu_forward_backward_pass.cpp:944-983); its
// quantized row for that round was written ahead at the row of its list position (rows_ahead), or is written by
// the caller into row `pos` of the other scratch matrix.  One thread per sample; returns the sample's position in
// the next round's list, -1 when it has no further round.
__device__ __forceinline__ int mvm_advance_sample(const MvmArgs &a, int round, int b, int slot, bool rows_ahead,
                                                  float &scale) {
  const IoDev &io = a.io;
  // the flags were raised with device-scope atomics by workgroups on any XCD: read and clear them the same way
  const int up = atomicExch(&a.st.hit_up[b], 0);
  const int lo = atomicExch(&a.st.hit_lo[b], 0);
  // the CPU loop sets "failed" on an upper hit and *assigns* !bm_test_negative_bound on a lower hit,
  // walking the outputs in index order: the last hit decides
  bool failed = io.bm_test_negative_bound ? (up > 0 || lo > 0) : (up > lo);
  if (a.post_hit_up) {
    // the negative pass went through the ADC stage on its own: either pass can fail the bound test
    // (rpu_forward_backward_pass.cpp:861-877); a sample short-cut to zero has no passes
    const int xrow = (round > 0) ? pick2(a.st.row, round & 1)[slot] : slot;
    const int nu = atomicExch(&a.post_hit_up[xrow], 0);
    const int nl = atomicExch(&a.post_hit_lo[xrow], 0);
    if (a.st.fin[b] != 0.0f) failed = failed || (io.bm_test_negative_bound ? (nu > 0 || nl > 0) : (nu > nl));
  }
  if (!failed) return -1;
  float nm = a.st.nm[b], red = a.st.red[b];
  if (!next_round_params(a, round, b, a.st.fin[b], nm, red)) return -1;
  a.st.nm[b] = nm;
  a.st.red[b] = red;
  a.st.rounds[b] += 1;
  scale = set_round_scales(a, b, nm, red);
  const int pos = atomicAdd(&a.st.count[round + 1], 1);
  pick2(a.st.list, (round + 1) & 1)[pos] = b;
  pick2(a.st.row, (round + 1) & 1)[pos] = rows_ahead ? slot : pos;
  pick2(a.st.next_scale, (round + 1) & 1)[pos] = next_round_scale(a, round + 1, b, a.st.fin[b], nm, red);
  return pos;
}

// Called by every workgroup of a round once its outputs are stored and its saturation flags are raised.  The
// workgroups of a sample tile (one per output tile, spread over the XCDs) count themselves off; the last one
// decides for the 32 samples of the tile whether they need another round, so that the next round's kernel
// can follow directly.
__device__ __forceinline__ void mvm_tile_finished(const MvmArgs &a, int round, int tile_b, int n_act) {
  __shared__ int sh_last;
  const int tiles_o = (a.O + TILE - 1) / TILE;
  const int tiles_b = (a.m_batch + TILE - 1) / TILE;
  __syncthreads(); // all flag atomics of this workgroup have been performed
  if (threadIdx.x == 0) {
    const int prev = atomicAdd(&a.st.tile_done[round * tiles_b + tile_b], 1);
    sh_last = (prev == tiles_o - 1) ? 1 : 0;
  }
  __syncthreads();
  if (!sh_last) return;
  __shared__ int sh_more, sh_more_b[TILE], sh_more_pos[TILE];
  __shared__ float sh_more_scale[TILE];
  if (threadIdx.x == 0) sh_more = 0;
  __syncthreads();
  if (threadIdx.x < TILE) {
    const int slot = tile_b * TILE + threadIdx.x;
    if (slot < n_act) {
      const int b = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
      float scale = 0.0f;
      const int pos = mvm_advance_sample(a, round, b, slot, a.speculate != 0, scale);
      if (pos >= 0 && !a.speculate) {
        const int i = atomicAdd(&sh_more, 1);
        sh_more_b[i] = b;
        sh_more_pos[i] = pos;
        sh_more_scale[i] = scale;
      }
    }
  }
  if (a.speculate) return;
  // a large batch does not quantize rows ahead (few samples go on, and twice the input traffic would be paid for
  // them): the rows of the samples that do go on are written now
  __syncthreads();
  for (int i = 0; i < sh_more; ++i) {
    write_dac_row(a, sh_more_b[i], sh_more_pos[i], sh_more_scale[i], round + 1, pick2(a.xq, (round + 1) & 1), threadIdx.x, 256);
  }
}

// The fused launch of rounds 0 and 1 (and 2): the last workgroup of a sample tile decides for its 32 samples which
// result stands (rpu_forward_backward_pass.cpp:944-983 walked once per fused round): round 0 unless its ADC saturated
// and the reduction may still grow, else round 1, unless that saturated too and may go on, and so on; a sample whose
// last fused round saturated as well is listed for the round after the launch.  With two fused rounds the workgroups of
// the launch have written the rows of round 2 ahead (into a.dual.xq2: round 0's rows are still being read); with three
// (the init kernel wrote those rows) a sample listed for round 3 is rare, and this workgroup writes its row now, over
// the sample's row of round 1, which every workgroup of the sample tile has finished reading.
template <int NACC>
__device__ __forceinline__ void mvm_tile_finished_dual(const MvmArgs &a, int tile_b) {
  __shared__ int sh_last;
  const int tiles_o = (a.O + TILE - 1) / TILE;
  __syncthreads(); // all flag atomics of this workgroup have been performed
  if (threadIdx.x == 0) {
    const int prev = atomicAdd(&a.st.tile_done[tile_b], 1);
    sh_last = (prev == tiles_o - 1) ? 1 : 0;
  }
  __syncthreads();
  if (!sh_last) return;
  __shared__ int sh_more, sh_more_b[TILE];
  __shared__ float sh_more_scale[TILE];
  if (threadIdx.x == 0) sh_more = 0;
  __syncthreads();
  const IoDev &io = a.io;
  constexpr int next_launch = NACC; // the first round after the fused ones
  if (threadIdx.x < TILE) {
    const int b = tile_b * TILE + threadIdx.x;
    if (b < a.m_batch) {
      const int up0 = atomicExch(&a.st.hit_up[b], 0), lo0 = atomicExch(&a.st.hit_lo[b], 0);
      const int up1 = atomicExch(&a.dual.hit1[b], 0), lo1 = atomicExch(&a.dual.hit1[a.m_batch + b], 0);
      int up2 = 0, lo2 = 0;
      if (NACC == 3) {
        up2 = atomicExch(&a.dual.hit2[b], 0);
        lo2 = atomicExch(&a.dual.hit2[a.m_batch + b], 0);
      }
      auto failed = [&](int up, int lo) { return io.bm_test_negative_bound ? (up > 0 || lo > 0) : (up > lo); };
      int sel = 0;
      float nm = a.st.nm[b], red = a.st.red[b];
      bool more = failed(up0, lo0) && next_round_params(a, 0, b, a.st.fin[b], nm, red);
      if (more) {
        // the sample has run round 1
        sel = 1;
        atomicAdd(&a.st.count[1], 1); // how many did: read by the host for its choice of launches
        a.st.rounds[b] += 1;
        set_round_scales(a, b, nm, red);
        more = failed(up1, lo1) && next_round_params(a, 1, b, a.st.fin[b], nm, red);
        if (NACC == 3 && more) { // and round 2
          sel = 2;
          atomicAdd(&a.st.count[2], 1);
          a.st.rounds[b] += 1;
          set_round_scales(a, b, nm, red);
          more = failed(up2, lo2) && next_round_params(a, 2, b, a.st.fin[b], nm, red);
        }
        if (more) {
          sel = next_launch;
          a.st.rounds[b] += 1;
          const float scale = set_round_scales(a, b, nm, red);
          const int pos = atomicAdd(&a.st.count[next_launch], 1);
          pick2(a.st.list, next_launch & 1)[pos] = b;
          pick2(a.st.row, next_launch & 1)[pos] = b; // at the sample's own row
          pick2(a.st.next_scale, next_launch & 1)[pos] = next_round_scale(a, next_launch, b, a.st.fin[b], nm, red);
          if (NACC == 3) {
            const int i = atomicAdd(&sh_more, 1);
            sh_more_b[i] = b;
            sh_more_scale[i] = scale;
          }
        }
        a.st.nm[b] = nm;
        a.st.red[b] = red;
      }
      a.dual.sel[b] = sel;
    }
  }
  if (NACC != 3) return;
  __syncthreads();
  for (int i = 0; i < sh_more; ++i) {
    write_dac_row(a, sh_more_b[i], sh_more_b[i], sh_more_scale[i], next_launch, pick2(a.xq, next_launch & 1), threadIdx.x, 256);
  }
}

// At the start of the launch after the fused one: workgroup n copies the 32 x 32 block of outputs it would own in a
// round over all samples from the kept results to the caller's output, per sample by a.dual.sel (samples listed for
// this round are written by it).
__device__ __forceinline__ void mvm_dual_select(const MvmArgs &a, int n) {
  int tile_o, tile_b;
  if (!tile_of(a, n, a.m_batch, tile_o, tile_b)) return;
  // four elements per thread (workgroups of 256): the choices first, then the kept values, then the stores, so that
  // the loads of a step are in flight together
  int sel[4];
  float v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = (int)threadIdx.x + 256 * i;
    const int b = tile_b * TILE + (idx >> 5), o = tile_o * TILE + (idx & 31);
    sel[i] = (b < a.m_batch && o < a.O) ? a.dual.sel[b] : a.dual.rounds;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = (int)threadIdx.x + 256 * i;
    const int b = tile_b * TILE + (idx >> 5), o = tile_o * TILE + (idx & 31);
    v[i] = 0.0f;
    if (sel[i] < a.dual.rounds) {
      const float *kept = sel[i] == 2 ? a.dual.buf[2] : (sel[i] == 1 ? a.dual.buf[1] : a.dual.buf[0]);
      v[i] = kept[(long)b * a.O + o];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = (int)threadIdx.x + 256 * i;
    const int b = tile_b * TILE + (idx >> 5), o = tile_o * TILE + (idx & 31);
    if (sel[i] < a.dual.rounds) a.out[(long)b * a.out_sb + (long)o * a.out_so] = v[i];
  }
}

// NACC rounds in one launch, from round 0
template <int WMODE, int NACC>
__global__ __launch_bounds__(256) void k_mvm_dual(MvmArgs a) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * (NACC + 1) * TILE * LDS_ROW];
  int tile_o, tile_b;
  if (!tile_of(a, blockIdx.x, a.m_batch, tile_o, tile_b)) return;
  if (NACC == 2) mvm_prepare_next_rows<true>(a, 1, tile_o, tile_b, a.m_batch);
  mvm_round_tile<2, WMODE, NACC>(a, 0, tile_o, tile_b, a.m_batch, red, stage);
  mvm_tile_finished_dual<NACC>(a, tile_b);
}

// work of workgroup number n of a round launch of one tile
template <int PD, int WMODE>
__device__ __forceinline__ void mvm_round_workgroup(const MvmArgs &a, int round, int n, int n_act, float (*red)[16][64],
                                                    float *stage) {
  int tile_o, tile_b;
  if (!tile_of(a, n, n_act, tile_o, tile_b)) return;
  const bool more_rounds = round + 1 < a.max_rounds;
  if (more_rounds && a.speculate && !(round == 0 && a.rows_ahead_in_init)) {
    mvm_prepare_next_rows(a, round, tile_o, tile_b, n_act);
  }
  mvm_round_tile<PD, WMODE>(a, round, tile_o, tile_b, n_act, red, stage);
  if (more_rounds) mvm_tile_finished(a, round, tile_b, n_act);
}

// Waits between the workgroups of one launch.  They are bounded, and a wait that runs out is reported, not passed
// over: the thread that gives up raises the launch's abort word (every other waiting workgroup sees it and gives up
// too), writes 1 + the round into the host-visible word `failed`, and every workgroup leaves the kernel -- the rounds
// that were still to run would read stale lists.  The host finds the word at its next call on the tile, reports that
// call's results as invalid and goes back to one launch per round.
struct RoundWait {
  int *abort;   // device memory, zero at the start of the call
  int *failed;  // host-visible, may be null
  int limit;    // polls before giving up
  int extra;    // arrivals expected beyond the launch's own workgroups (0; a test of the give-up path asks for one more)
};
constexpr int REST_SPIN_LIMIT = 1 << 15; // about 1 us per poll: some tens of milliseconds

__device__ __forceinline__ RoundWait round_wait_of(int *count, int *seen, int spins, int extra) {
  return RoundWait{count + MVM_ABORT_WORD, seen ? seen + 3 : nullptr, spins > 0 ? spins : REST_SPIN_LIMIT, extra};
}

// thread 0: polls until *word reaches `target`; false when the wait ran out or another workgroup gave up
__device__ __forceinline__ bool round_wait_poll(const RoundWait &wt, int *word, int target, int round) {
  int spins = 0;
  while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
    const bool gave_up = ++spins >= wt.limit;
    if (gave_up || ((spins & 15) == 0 && __hip_atomic_load(wt.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
      if (gave_up) {
        __hip_atomic_store(wt.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (wt.failed) __hip_atomic_store(wt.failed, round + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      return false;
    }
    __builtin_amdgcn_s_sleep(8);
  }
  return true;
}

// All workgroups of a launch wait for each other, and what they wrote before is visible to all of them after (the
// launch must fit on the GPU at once).  Returns false when the wait gave up: the caller leaves the kernel.
__device__ __forceinline__ bool mvm_device_barrier(int *counter, int total, const RoundWait &wt, int round) {
  __shared__ int sh_ok;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  __syncthreads();
  if (threadIdx.x == 0) {
    __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sh_ok = round_wait_poll(wt, counter, total + wt.extra, round) ? 1 : 0;
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return sh_ok != 0;
}

// All workgroups of a launch wait until each has arrived, which it does once the atomics of its threads have been
// performed (their results were consumed before the barrier): after the wait, what those atomics built up -- the number
// of samples listed for the next round -- is final and can be read with a device-scope load.  Nothing else the
// workgroups wrote is made visible: a launch that goes on to read such data calls mvm_device_barrier as well.  A few
// microseconds, against tens for that one; bounded and reported in the same way.
// counter[0] counts the arrivals; the last one raises counter[1], which the others poll (so that the polls do not
// queue up in front of the arrivals at the one address).
__device__ __forceinline__ bool mvm_arrive(int *counter, int total, const RoundWait &wt, int round) {
  __shared__ int sh_ok;
  __syncthreads();
  if (threadIdx.x == 0) {
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before == total + wt.extra - 1) {
      __hip_atomic_store(counter + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sh_ok = 1;
    } else {
      sh_ok = round_wait_poll(wt, counter + 1, 1, round) ? 1 : 0;
    }
  }
  __syncthreads();
  return sh_ok != 0;
}

// Host-visible summary of a call for the choice of the next call's launches (a.dual.seen), kept by the first thread of
// a launch of round r that lists n_act samples; first_after_fused: the launch that follows the fused one.
__device__ __forceinline__ void mvm_note_round(const MvmArgs &a, int r, int n_act, bool first_after_fused) {
  if (!a.dual.seen || blockIdx.x != 0 || threadIdx.x != 0) return;
  if (r == 1 || first_after_fused) {
    const int needed = (r == 1) ? n_act : a.st.count[1];
    a.dual.seen[0] = needed;
    a.dual.seen[1] = a.m_batch;
    // (after three fused rounds count[2] is the number of samples whose round 2 was used)
    a.dual.seen[2] = n_act > 0 ? r : ((r == 3 && a.st.count[2] > 0) ? 2 : (needed > 0 ? 1 : 0));
  } else if (n_act > 0) {
    a.dual.seen[2] = r;
  }
}

// big_from > 0: the large-tile kernel runs the rounds that list at least that many samples; < 0: it runs round 0
__device__ __forceinline__ bool runs_on_large_tiles(const MvmArgs &a, int round, int n_act) {
  return (a.big_from > 0 && n_act >= a.big_from) || (a.big_from < 0 && round == 0);
}

// Rounds after the first usually list few samples, but their launch is sized before that is known.  When the
// full grid would be large, this variant runs them instead: a fixed number of workgroups walk the tiles of the
// listed samples, with one register set (k_pad only needs to be a multiple of 32).
// Calls on gathered patches (MvmArgs::in_index) write no rows for the samples that go on to a further round
// (write_dac_row has no patch matrix to read): the workgroup that is about to run sample tile tile_b of round `round`
// gathers the quantized rows of that tile's listed samples itself, through the patch-major index and with the scale
// that the round before has set.  The workgroups of the other output tiles of the same samples write the same values.
__device__ __forceinline__ void mvm_gather_tile_rows(const MvmArgs &a, int round, int tile_b, int n_act) {
  float *rows = pick2(a.xq, round & 1);
  const int *list = pick2(a.st.list, round & 1);
  const int first = tile_b * TILE, count = min(TILE, n_act - first);
  for (int i = threadIdx.x >> 3; i < count; i += 32) { // eight threads per row
    const int b = list[first + i];
    const float scale = a.st.scale[b];
    const MvmGatherRow row = mvm_gather_row(a, b);
    float *out = rows + (long)(first + i) * a.k_pad;
    for (int k = threadIdx.x & 7; k < a.k_pad; k += 8) {
      out[k] = (k < a.K) ? dac_value(row.at(k), scale, a.io, a.key, a.call, round, b, k) : 0.0f;
    }
  }
  __threadfence_block();
  __syncthreads();
}

template <int WMODE>
__global__ __launch_bounds__(256) void k_mvm_round_tail(MvmArgs a) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  if (a.dual.on == 2) { // the launch after the fused one: the kept results of every tile go to the caller's output
    const int all = workgroups_for(a.O, a.m_batch);
    for (int n = blockIdx.x; n < all; n += gridDim.x) mvm_dual_select(a, n);
  }
  const int n_act = (a.round > 0) ? a.st.count[a.round] : a.m_batch;
  if (a.round > 0) mvm_note_round(a, a.round, n_act, a.dual.on == 2);
  if (runs_on_large_tiles(a, a.round, n_act)) return;
  const int total = workgroups_for(a.O, n_act);
  for (int n = blockIdx.x; n < total; n += gridDim.x) {
    if (a.in_index && a.round > 0) {
      int tile_o, tile_b;
      if (tile_of(a, n, n_act, tile_o, tile_b)) mvm_gather_tile_rows(a, a.round, tile_b, n_act);
    }
    mvm_round_workgroup<1, WMODE>(a, a.round, n, n_act, red, stage);
    __syncthreads(); // LDS is reused by the next tile
  }
}

// Whether any tile of the group lists a sample for round 1: written to host-visible memory for the host's choice of
// launches at its next call (seen[0]: 1 / 0, seen[1]: the batch).  Called by the first workgroup of a round-1 launch.
__device__ __forceinline__ void group_seen_update(const MvmGroup &g, int *seen) {
  __shared__ int sh_any;
  if (threadIdx.x == 0) sh_any = 0;
  __syncthreads();
  for (int t = threadIdx.x; t < g.n; t += blockDim.x) {
    const MvmArgs &a = g.args[t];
    if (a.max_rounds > 1 && __hip_atomic_load(&a.st.count[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) > 0) sh_any = 1;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    seen[0] = sh_any;
    seen[1] = g.m_batch;
  }
}

// The same for a group: the workgroups first find out, one thread per tile, how many 32 x 32 tiles each member has
// listed for this round (usually none), then walk the concatenation of those.
constexpr int MAX_GROUP = 1024;

template <int WMODE>
__global__ __launch_bounds__(256) void k_mvm_round_tail_group(MvmGroup g, int round, int *seen) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  __shared__ int sh_first[MAX_GROUP + 1]; // first workgroup number of member t; [g.n] = total
  if (seen && round == 1 && blockIdx.x == 0) group_seen_update(g, seen);
  for (int t = threadIdx.x; t < g.n; t += blockDim.x) {
    const MvmArgs &a = g.args[t];
    int wg = 0;
    if (round < a.max_rounds) {
      const int n_act = (round > 0) ? a.st.count[round] : a.m_batch;
      if (!runs_on_large_tiles(a, round, n_act) && n_act > 0) wg = workgroups_for(a.O, n_act);
    }
    sh_first[t + 1] = wg;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0;
    sh_first[0] = 0;
    for (int t = 0; t < g.n; ++t) {
      sum += sh_first[t + 1];
      sh_first[t + 1] = sum;
    }
  }
  __syncthreads();
  const int total = sh_first[g.n];
  int t = 0;
  for (int n = blockIdx.x; n < total; n += gridDim.x) {
    while (n >= sh_first[t + 1]) ++t;
    const MvmArgs &a = g.args[t];
    const int n_act = (round > 0) ? a.st.count[round] : a.m_batch;
    mvm_round_workgroup<1, WMODE>(a, round, n - sh_first[t], n_act, red, stage);
    __syncthreads();
  }
}

// The rounds from round_first on of all tiles of a group in one launch (see k_mvm_rounds_rest): a fixed number of
// workgroups, all resident at once, walk the tiles that the members list for a round; after a round they wait for each
// other's arrival and leave if the next round lists nothing (else a full device-wide wait comes first).  The arrival
// counters are those of the group's first tile.
template <int WMODE>
__global__ __launch_bounds__(256) void k_mvm_rest_group(MvmGroup g, int round_first, int rounds, int *seen) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  __shared__ int sh_first[MAX_GROUP + 1]; // first workgroup number of member t; [g.n] = total
  const RoundWait wt{g.args[0].st.count + MVM_ABORT_WORD, g.wait_failed, g.wait_spins > 0 ? g.wait_spins : REST_SPIN_LIMIT,
                     g.wait_extra};
  for (int round = round_first; round < rounds; ++round) {
    for (int t = threadIdx.x; t < g.n; t += blockDim.x) {
      const MvmArgs &a = g.args[t];
      int wg = 0;
      if (round < a.max_rounds) {
        const int n_act = __hip_atomic_load(&a.st.count[round], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (!runs_on_large_tiles(a, round, n_act) && n_act > 0) wg = workgroups_for(a.O, n_act);
      }
      sh_first[t + 1] = wg;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int sum = 0;
      sh_first[0] = 0;
      for (int t = 0; t < g.n; ++t) {
        sum += sh_first[t + 1];
        sh_first[t + 1] = sum;
      }
    }
    __syncthreads();
    const int total = sh_first[g.n];
    if (seen && round == 1 && blockIdx.x == 0) group_seen_update(g, seen);
    if (total == 0) return; // the same for every workgroup
    // the rows and lists that the round before left must be visible on every XCD
    if (round > round_first &&
        !mvm_device_barrier(&g.args[0].st.count[MVM_ARRIVE_BASE + 4 * round + 2], (int)gridDim.x, wt, round)) {
      return;
    }
    int t = 0;
    for (int n = blockIdx.x; n < total; n += gridDim.x) {
      while (n >= sh_first[t + 1]) ++t;
      const MvmArgs &a = g.args[t];
      const int n_act = __hip_atomic_load(&a.st.count[round], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      mvm_round_workgroup<1, WMODE>(a, round, n - sh_first[t], n_act, red, stage);
      __syncthreads();
    }
    if (round + 1 == rounds) return;
    // the counts of the next round are final once every workgroup has arrived
    if (!mvm_arrive(&g.args[0].st.count[MVM_ARRIVE_BASE + 4 * round], (int)gridDim.x, wt, round)) return;
  }
}

// Every round from a.round on in ONE launch, for calls whose samples are expected to be done by the end of round
// a.round (as in the tile's last calls): after that round the workgroups wait for each other's arrival, find the next
// list empty and leave, where separate launches would cost a few microseconds each for nothing.  Where the expectation
// fails the rounds still run, one after the other, each behind a wait that also makes the rows and lists of the round
// before visible on every XCD (mvm_device_barrier: tens of microseconds, which is why this launch is only chosen by
// expectation).  With a.dual.on = 2 it is the launch after the fused one and starts with that launch's selection.
template <int PD, int WMODE>
__global__ __launch_bounds__(256) void k_mvm_rounds_rest(MvmArgs a) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  if (a.dual.on == 2) mvm_dual_select(a, blockIdx.x);
  const RoundWait wt = round_wait_of(a.st.count, a.dual.seen, a.wait_spins, a.wait_extra);
  for (int r = a.round; r < a.max_rounds; ++r) {
    // final since the launch before (first round) or since every workgroup arrived after the round before
    const int n_act = __hip_atomic_load(&a.st.count[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    mvm_note_round(a, r, n_act, r == a.round && a.dual.on == 2);
    if (n_act == 0) return; // the same for every workgroup
    if (r > a.round && !mvm_device_barrier(&a.st.count[MVM_ARRIVE_BASE + 4 * r + 2], (int)gridDim.x, wt, r)) return;
    mvm_round_workgroup<PD, WMODE>(a, r, blockIdx.x, n_act, red, stage);
    if (r + 1 == a.max_rounds) return;
    if (!mvm_arrive(&a.st.count[MVM_ARRIVE_BASE + 4 * r], (int)gridDim.x, wt, r)) return;
  }
}

template <int PD, int WMODE>
__global__ __launch_bounds__(256) void k_mvm_round(MvmArgs a) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  if (a.skip_if_zero && *a.skip_if_zero == 0) return;
  if (a.dual.on == 2) mvm_dual_select(a, blockIdx.x);
  const int n_act = (a.round > 0) ? a.st.count[a.round] : a.m_batch;
  // how many samples needed a second round, and the last round that listed any: the host reads it (whenever it next
  // looks) to choose its launches
  if (a.round > 0) mvm_note_round(a, a.round, n_act, a.dual.on == 2);
  if (runs_on_large_tiles(a, a.round, n_act)) return;
  mvm_round_workgroup<PD, WMODE>(a, a.round, blockIdx.x, n_act, red, stage);
}

// ---------------------------------------------------------------------------------------------
// Large-batch round: one workgroup (4 waves as 2 x 2) owns 128 outputs x 128 samples, each wave a 64 x 64 block as
// 2 x 2 MFMA tiles.  Both operands go through LDS stages of 32 k-values shared by the four waves (a stage is
// fetched into registers while the previous one is multiplied, then written to the other LDS buffer: one barrier
// per stage), so a byte fetched from L2 feeds 64 multiply-adds instead of 16 and the matrix pipe, not the memory
// path, sets the pace.  Same per-sample state, lists, epilogue and random streams as the 32 x 32 kernel: a round
// may be run by either (the launcher picks by the number of samples in the round).
// WT = 0: weights contiguous along k (forward), 1: contiguous along the outputs (backward, W read in place).

constexpr int BT = 128;        // outputs of a workgroup tile; its samples: BB = 128, or 64 (each wave 64 x 32: twice the
                               // workgroups, for launches that would put fewer than about three of the square tiles on a CU)
constexpr int BKS = 32;        // k-values per stage
constexpr int BROW = 32;       // floats per staged row of a k-contiguous operand, no padding.  LDS has 64 banks: two rows
                               // fill the 16 chunk slots (of 16 bytes) of a 256-byte line, and chunk c of row `row` sits in
                               // slot (8 (row % 2) + c + row / 2) % 16 of its line: 16 rows that read the same chunk, and the 16
                               // threads that store two rows, each touch all 64 banks once
__device__ __forceinline__ int big_lds_offset(int row, int chunk) {
  return (row >> 1) * (2 * BROW) + ((((row & 1) << 3) + chunk + (row >> 1)) & 15) * 4;
}
constexpr int BPITCH_T = 132;  // floats per staged k-row of an output-contiguous weight tile

template <int BB>
__device__ __forceinline__ void big_prepare_next_rows(const MvmArgs &a, int round, int tile_o, int tile_b, int n_act,
                                                      int *sh_b, float *sh_scale) {
  if (threadIdx.x < BB) {
    const int slot = tile_b * BB + threadIdx.x;
    int b = 0;
    float scale = 0.0f;
    if (slot < n_act) {
      b = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
      scale = pick2(a.st.next_scale, round & 1)[slot];
    }
    sh_b[threadIdx.x] = b;
    sh_scale[threadIdx.x] = scale;
  }
  __syncthreads();
  const int tiles_o = (a.O + BT - 1) / BT;
  const int chunk = (((a.k_pad + tiles_o - 1) / tiles_o) + 31) & ~31;
  const int k_lo = tile_o * chunk;
  const int k_hi = min(k_lo + chunk, a.k_pad);
  float *__restrict__ dst = pick2(a.xq, (round + 1) & 1);
  const float *__restrict__ in = a.in;
  constexpr int RPT = BB / 8; // 8 thread-rows of RPT rows each
  const int kq = threadIdx.x & 31, rq = threadIdx.x >> 5;
  for (int k0 = k_lo; k0 < k_hi; k0 += 32) {
    const int k = k0 + kq;
    float xv[RPT]; // all loads of a trip are in flight together
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = rq * RPT + i;
      xv[i] = (sh_scale[row] != 0.0f && k < a.K) ? in[(long)sh_b[row] * a.in_sb + (long)k * a.in_sk] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int row = rq * RPT + i;
      const float sc = sh_scale[row];
      if (sc != 0.0f) {
        const float v = (k < a.K) ? dac_value(xv[i], sc, a.io, a.key, a.call, round + 1, sh_b[row], k) : 0.0f;
        dst[(long)(tile_b * BB + row) * a.k_pad + k] = v;
      }
    }
  }
}

// Instruction order of 16 MFMAs and the LDS reads of the operands that follow them (a hint to the scheduler): the
// reads are spread behind the first MFMAs so that they complete underneath the rest.
template <int WT, int NB>
__device__ __forceinline__ void mvm_big_schedule() {
  // NB sample blocks per wave: 8 NB MFMAs.  WT = 0: 2 + NB wide LDS reads; WT = 1: NB wide reads and the 8 single
  // reads of the transposed weight tile
  constexpr int mfmas = 8 * NB;
  constexpr int paired = WT == 0 ? 2 + NB : (NB == 2 ? 6 : 5);
  constexpr int doubled = (WT == 1 && NB == 1) ? 4 : 0; // pairs that carry two LDS reads
#pragma unroll
  for (int i = 0; i < doubled; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); // two LDS reads
  }
#pragma unroll
  for (int i = doubled; i < paired; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one MFMA
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // one LDS read
  }
  __builtin_amdgcn_sched_group_barrier(0x008, mfmas - paired, 0);
}

// work of workgroup number n of a large-tile round launch of one tile; BB: samples of a workgroup tile (128 or 64)
// NARROW (tiles of at most 64 outputs, BB = 128): every wave takes outputs 0 .. 63 and one of the four 32-sample
// blocks, instead of two waves on outputs that do not exist: half of the MFMAs, spread over all four SIMDs; the
// k order of every sum is the same.
// NBUF = 1 (contractions of one or two stages): a single staging buffer, half of the LDS, so that a third workgroup
// fits a CU and covers the ADC stage of the other two, which is all such a call consists of.
// LAZY (calls with speculate = 0): nothing is quantized ahead; the last workgroup of a sample tile writes the rows of
// the samples that go on.  The other instantiations always quantize ahead, as their callers ask for.
template <int WT, int BB, bool NARROW = false, int NBUF = 2, bool LAZY = false>
__device__ __forceinline__ void mvm_big_workgroup(const MvmArgs &a, const int round, const int n, const int min_active) {
  static_assert(BB == 128 || BB == 64, "sample tile of 128 or 64");
  static_assert(!NARROW || BB == 128, "the narrow wave layout covers four sample blocks");
  constexpr int NB = NARROW ? 1 : BB / 64; // 32-sample blocks per wave
  constexpr int XJ = BB / 32; // staged sample rows per thread
  __shared__ __attribute__((aligned(16))) float lds_x[NBUF][BB * BROW];
  __shared__ __attribute__((aligned(16))) float lds_w[NBUF][WT ? BKS * BPITCH_T : BT * BROW];
  __shared__ int sh_hits[2 * BB];
  __shared__ int sh_b[BB];
  __shared__ float sh_scale[BB];
  __shared__ int sh_last;

  const int n_act = (round > 0) ? a.st.count[round] : a.m_batch;
  if (n_act < min_active) return; // this round is run by the 32 x 32 kernel
  // workgroup n runs on XCD n % 8: an XCD walks the output tiles of one sample tile after the other, so a tile of
  // quantized inputs (the large operand) enters one L2 only and the small weight matrix is what every XCD streams
  const int tile_o = (n >> 3) % ((a.O + BT - 1) / BT);
  const int tile_b = ((n >> 3) / ((a.O + BT - 1) / BT)) * 8 + (n & 7);
  if (tile_b * BB >= n_act) return;
  const bool more_rounds = round + 1 < a.max_rounds;
  if (more_rounds && !LAZY && !(round == 0 && a.rows_ahead_in_init)) {
    big_prepare_next_rows<BB>(a, round, tile_o, tile_b, n_act, sh_b, sh_scale);
  }

  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int wy = NARROW ? 0 : wave >> 1, wx = wave & 1;
  const int blk = NARROW ? wave >> 1 : 0; // NARROW: this wave's sample block within its half
  const int K = a.K;

  // global -> LDS assignment.  k-contiguous operand: chunk c = t + 256 j covers row c / 8, floats 4 (c % 8) ..;
  // output-contiguous weights: chunk c covers k-row c / 32, outputs 4 (c % 32) ..
  const float *xq = round_rows(a, round);
  const float *x_src[XJ];
  const float *w_src[4];
  const int st_col = (t & 7) * 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = (t >> 3) + 32 * j;
    if (j < XJ) {
      const int slot = min(tile_b * BB + row, n_act - 1);
      const int xrow = (round > 0) ? pick2(a.st.row, round & 1)[slot] : slot;
      x_src[j] = xq + (long)xrow * a.k_pad + st_col;
    }
    if (WT == 0) w_src[j] = a.w + (long)min(tile_o * BT + row, a.O - 1) * a.w_ld;
  }
  const int wt_o = tile_o * BT + (t & 31) * 4; // WT = 1: first of this thread's four outputs

  auto gload = [&](int s, f32x4 (&gx)[XJ], f32x4 (&gw)[4]) {
    const int k0 = s * BKS;
#pragma unroll
    for (int j = 0; j < XJ; ++j) gx[j] = *reinterpret_cast<const f32x4 *>(x_src[j] + k0);
    if (WT == 0) {
      const int kc = k0 + st_col;
      if (kc + 4 <= K) {
#pragma unroll
        for (int j = 0; j < 4; ++j) gw[j] = *reinterpret_cast<const f32x4_unaligned *>(w_src[j] + kc);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          f32x4 z;
          z.x = (kc < K) ? w_src[j][kc] : 0.0f;
          z.y = (kc + 1 < K) ? w_src[j][kc + 1] : 0.0f;
          z.z = (kc + 2 < K) ? w_src[j][kc + 2] : 0.0f;
          z.w = 0.0f;
          gw[j] = z;
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = min(k0 + (t >> 5) + 8 * j, K - 1); // rows past K meet the zero padding of the inputs
        const float *row = a.w + (long)k * a.w_ld;
        if (wt_o + 4 <= a.O) {
          gw[j] = *reinterpret_cast<const f32x4_unaligned *>(row + wt_o);
        } else {
          f32x4 z;
          z.x = (wt_o < a.O) ? row[wt_o] : 0.0f;
          z.y = (wt_o + 1 < a.O) ? row[wt_o + 1] : 0.0f;
          z.z = (wt_o + 2 < a.O) ? row[wt_o + 2] : 0.0f;
          z.w = 0.0f;
          gw[j] = z;
        }
      }
    }
  };
  auto lds_store = [&](int buf, const f32x4 (&gx)[XJ], const f32x4 (&gw)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = (t >> 3) + 32 * j;
      if (j < XJ) *reinterpret_cast<f32x4 *>(&lds_x[buf][big_lds_offset(row, t & 7)]) = gx[j < XJ ? j : 0];
      if (WT == 0) {
        *reinterpret_cast<f32x4 *>(&lds_w[buf][big_lds_offset(row, t & 7)]) = gw[j];
      } else {
        const int krow = (t >> 5) + 8 * j;
        *reinterpret_cast<f32x4 *>(&lds_w[buf][krow * BPITCH_T + (t & 31) * 4]) = gw[j];
      }
    }
  };

  // accumulators of the 2 x 2 MFMA tiles (output block, sample block), named one by one so that they stay in
  // registers whatever the inlining order
  floatx16 acc00, acc01, acc10, acc11;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    acc00[i] = 0.0f;
    acc01[i] = 0.0f;
    acc10[i] = 0.0f;
    acc11[i] = 0.0f;
  }

  // lane (r, h) multiplies k = 16 h .. 16 h + 15 of a stage, four values at a time; the operands of the next four
  // are read from LDS before the 16 MFMAs of the current four are issued, so that the reads complete underneath them
  struct Operands {
    f32x4 xb0, xb1, wa0, wa1;
  };
  // staged offsets of this lane's four operand chunks (rows 32 further on: 32 * BROW floats further on)
  int x_off[4], w_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    x_off[q] = big_lds_offset(wx * (BB / 2) + blk * 32 + r, h * 4 + q);
    w_off[q] = big_lds_offset(wy * 64 + r, h * 4 + q);
  }
  auto read_operands = [&](int buf, int q, Operands &o) __attribute__((always_inline)) {
    const int kk = h * 16 + q * 4;
    o.xb0 = *reinterpret_cast<const f32x4 *>(&lds_x[buf][x_off[q]]);
    if (NB == 2) o.xb1 = *reinterpret_cast<const f32x4 *>(&lds_x[buf][x_off[q] + 32 * BROW]);
    if (WT == 0) {
      o.wa0 = *reinterpret_cast<const f32x4 *>(&lds_w[buf][w_off[q]]);
      o.wa1 = *reinterpret_cast<const f32x4 *>(&lds_w[buf][w_off[q] + 32 * BROW]);
    } else {
      const float *col = &lds_w[buf][kk * BPITCH_T + wy * 64 + r];
      o.wa0.x = col[0];
      o.wa0.y = col[BPITCH_T];
      o.wa0.z = col[2 * BPITCH_T];
      o.wa0.w = col[3 * BPITCH_T];
      o.wa1.x = col[32];
      o.wa1.y = col[BPITCH_T + 32];
      o.wa1.z = col[2 * BPITCH_T + 32];
      o.wa1.w = col[3 * BPITCH_T + 32];
    }
  };
  auto multiply = [&](const Operands &o) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc00 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.wa0[e], o.xb0[e], acc00, 0, 0, 0);
      if (NB == 2) acc01 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.wa0[e], o.xb1[e], acc01, 0, 0, 0);
      acc10 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.wa1[e], o.xb0[e], acc10, 0, 0, 0);
      if (NB == 2) acc11 = __builtin_amdgcn_mfma_f32_32x32x2f32(o.wa1[e], o.xb1[e], acc11, 0, 0, 0);
    }
  };
  auto compute = [&](int buf) __attribute__((always_inline)) {
    Operands even, odd;
    read_operands(buf, 0, even);
    read_operands(buf, 1, odd);
    multiply(even);
    mvm_big_schedule<WT, NB>();
    read_operands(buf, 2, even);
    multiply(odd);
    mvm_big_schedule<WT, NB>();
    read_operands(buf, 3, odd);
    multiply(even);
    mvm_big_schedule<WT, NB>();
    multiply(odd);
  };

  const int stages = a.k_pad / BKS;
  {
    f32x4 gx[XJ], gw[4];
    gload(0, gx, gw);
    lds_store(0, gx, gw);
    __syncthreads();
    for (int s = 0; s < stages; ++s) {
      const bool next = s + 1 < stages;
      if (next) gload(s + 1, gx, gw);
      compute(NBUF == 1 ? 0 : s & 1);
      if (NBUF == 1 && next) __syncthreads(); // every wave is done with the one buffer
      if (next) lds_store(NBUF == 1 ? 0 : (s + 1) & 1, gx, gw);
      __syncthreads();
    }
  }

  // ADC stage: lane (r, h) of wave (wy, wx) holds, for its 2 x 2 tiles, sample column r and output rows
  // g * 8 + h * 4 + q of each tile
  if (t < 2 * BB) sh_hits[t] = 0;
  __syncthreads();
  const bool flags = !a.io.perfect && a.io.bound_management != RPU_BM_NONE;
  // sample block bi of this wave: its two output blocks
  auto finish_block = [&](const int bi, const floatx16 &acc_o0, const floatx16 &acc_o1) __attribute__((always_inline)) {
    const int local_b = wx * (BB / 2) + bi * 32 + r;
    const int slot = tile_b * BB + local_b;
    if (slot >= n_act) return;
    int b_out = slot;
    float fin_out = 1.0f;
    if (!a.io.perfect) {
      if (round > 0) b_out = pick2(a.st.list, round & 1)[slot];
      fin_out = a.st.fin[b_out];
    }
    int up_max = 0, lo_max = 0;
#pragma unroll
    for (int oi = 0; oi < 2; ++oi) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int o0 = tile_o * BT + wy * 64 + oi * 32 + g * 8 + h * 4;
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = oi ? acc_o1[4 * g + q] : acc_o0[4 * g + q];
        int up = 0, lo = 0;
        if (o0 < a.O) mvm_finish_outputs(a, round, b_out, fin_out, o0, v, up, lo);
        up_max = max(up_max, up);
        lo_max = max(lo_max, lo);
      }
    }
    if (flags) {
      if (up_max) atomicMax(&sh_hits[local_b], up_max);
      if (lo_max) atomicMax(&sh_hits[BB + local_b], lo_max);
    }
  };
  finish_block(blk, acc00, acc10);
  if (NB == 2) finish_block(1, acc01, acc11);
  if (!flags) return;
  __syncthreads();
  if (t < 2 * BB) {
    const int local_b = t & (BB - 1);
    const int hit = sh_hits[t];
    const int slot = tile_b * BB + local_b;
    if (hit && slot < n_act) {
      const int bs = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
      const int old = atomicMax(t < BB ? &a.st.hit_up[bs] : &a.st.hit_lo[bs], hit);
      asm volatile("" ::"v"(old));
    }
  }
  if (!more_rounds) return;
  // the last workgroup of this sample tile decides which of its samples go on (see mvm_tile_finished)
  __syncthreads();
  if (t == 0) {
    const int tiles_o = (a.O + BT - 1) / BT;
    const int tiles_b = (a.m_batch + BB - 1) / BB;
    const int prev = atomicAdd(&a.st.tile_done[round * tiles_b + tile_b], 1);
    sh_last = (prev == tiles_o - 1) ? 1 : 0;
  }
  __syncthreads();
  if (!sh_last) return;
  constexpr bool ahead = !LAZY;
  if (!ahead) { // sh_last becomes the number of samples of this tile that go on
    __syncthreads();
    if (t == 0) sh_last = 0;
    __syncthreads();
  }
  if (t < BB) {
    const int slot = tile_b * BB + t;
    if (slot < n_act) {
      float scale = 0.0f;
      const int b = (round > 0) ? pick2(a.st.list, round & 1)[slot] : slot;
      const int pos = mvm_advance_sample(a, round, b, slot, ahead, scale);
      if (pos >= 0 && !ahead) {
        const int i = atomicAdd(&sh_last, 1);
        sh_b[i] = b;
        sh_hits[i] = pos;
        sh_scale[i] = scale;
      }
    }
  }
  if (ahead) return;
  // nothing was quantized ahead (a long batch on a narrow tile: few samples go on, and every row written ahead
  // would be paid for): the rows of the samples that do go on are written now
  __syncthreads();
  for (int i = 0; i < sh_last; ++i) {
    write_dac_row(a, sh_b[i], sh_hits[i], sh_scale[i], round + 1, pick2(a.xq, (round + 1) & 1), t, 256);
  }
}

template <int WT, int BB>
__global__ __launch_bounds__(256, 2) void k_mvm_big(MvmArgs a, int min_active) {
  mvm_big_workgroup<WT, BB>(a, a.round, (int)blockIdx.x, min_active);
}
template <int BB>
__global__ __launch_bounds__(256, 3) void k_mvm_big_short(MvmArgs a, int min_active) {
  mvm_big_workgroup<1, BB, false, 1>(a, a.round, (int)blockIdx.x, min_active);
}
__global__ __launch_bounds__(256, 2) void k_mvm_big_narrow(MvmArgs a, int min_active) {
  mvm_big_workgroup<0, 128, true, 2, true>(a, a.round, (int)blockIdx.x, min_active);
}
template <int WT, int BB>
__global__ __launch_bounds__(256, 2) void k_mvm_big_lazy(MvmArgs a, int min_active) {
  mvm_big_workgroup<WT, BB, false, 2, true>(a, a.round, (int)blockIdx.x, min_active);
}

// several tiles in one launch (round 0): a tile that is not run by this kernel has no workgroups in the table
template <int WT, int BB>
__global__ __launch_bounds__(256, 2) void k_mvm_big_group(MvmGroup g, int round) {
  int t = 0;
  while (t + 1 < g.n && (int)blockIdx.x >= g.start[t + 1]) ++t;
  const MvmArgs &a = g.args[t];
  if (round > 0 && round >= a.max_rounds) return;
  mvm_big_workgroup<WT, BB>(a, round, (int)blockIdx.x - g.start[t], 0);
}

// ---------------------------------------------------------------------------------------------
// Convolution forward for a tile of at most 32 outputs, fused: unfold by the index matrix, noise management, DAC,
// contraction, ADC and the bound-management rounds in one kernel, the result written in the image layout
// [n][output][patch].  A wave owns 32 consecutive patches; it has all outputs of its patches, so whether a patch
// needs another round (and that round) stays inside the wave: no lists, no scratch matrices, no further launch.
// The unfolded matrix is never written: element k of patch (n, p) is gathered from the image through the
// transposed index matrix idx_t[p][k] (0: padding, 1: the bias input, j >= 2: image element j - 2) where it is needed.
// Random streams, per-patch state and results are those of the unfolded path (same counters: element k, patch number).

typedef int i32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));

// ONE_STEP: the patch row fits one contraction step (K <= 32, a first convolution layer): the gathered values stay
// in registers between noise management and the rounds.
// STOCH: the DAC or the ADC draws random numbers beyond the output noise (see dac_value, mvm_adc_values).
// WOC: the stored matrix holds the outputs of one k per row (MvmArgs::w_oc); a kernel instance per addressing, so that
// neither carries the other's registers.
template <bool ONE_STEP, bool STOCH, bool WOC = false>
__global__ __launch_bounds__(256, STOCH ? 2 : 3) void k_conv_forward(MvmArgs a, ConvArgs c) {
  const int lane = threadIdx.x & 63;
  const int r = lane & 31, h = lane >> 5;
  const long tile = blockIdx.x * 4L + (threadIdx.x >> 6);
  const long total = (long)c.n_images * c.patches;
  if (tile * 32 >= total) return;
  const long s_raw = tile * 32 + r;
  const bool s_ok = s_raw < total;
  const long sample = s_ok ? s_raw : total - 1;
  const int n = (int)(sample / c.patches);
  const int p = (int)(sample - (long)n * c.patches);
  const float *image = c.images + (long)n * c.image_size;
  const int *idx_row = c.idx_t + (long)p * a.K;
  const float *w_row = a.w + (long)min(r, a.O - 1) * (WOC ? 1 : a.w_ld); // WOC: the lane's output column
  const int K = a.K, O = a.O;
  const int steps = ONE_STEP ? 1 : (K + 31) / 32;
  const IoDev &io = a.io;
  const int b = (int)sample; // the patch number keys the random streams

  // the 16 elements k0 .. k0 + 15 of this lane's patch row (zero past K)
  auto gather16 = [&](int k0, float (&x)[16]) __attribute__((always_inline)) {
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int k = k0 + 4 * v4;
      int j[4];
      if (k + 4 <= K) {
        const i32x4_unaligned t = *reinterpret_cast<const i32x4_unaligned *>(idx_row + k);
        j[0] = t.x; j[1] = t.y; j[2] = t.z; j[3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) j[e] = (k + e < K) ? idx_row[k + e] : 0;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * v4 + e] = (j[e] <= 1) ? (float)j[e] : image[j[e] - 2];
    }
  };
  auto weights16 = [&](int k0, float (&w)[16]) __attribute__((always_inline)) {
    if constexpr (WOC) { // rows of the stored matrix hold the outputs of one k: a uniform row address + the lane's column
      const unsigned col = (unsigned)min(r, O - 1);
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = (a.w + (long)min(k0 + i, K - 1) * a.w_ld)[col];
      if (k0 + 16 > K) {
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i] = (k0 + i < K) ? w[i] : 0.0f;
      }
    } else
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int k = k0 + 4 * v4;
      if (k + 4 <= K) {
        const f32x4_unaligned t = *reinterpret_cast<const f32x4_unaligned *>(w_row + k);
        w[4 * v4] = t.x; w[4 * v4 + 1] = t.y; w[4 * v4 + 2] = t.z; w[4 * v4 + 3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) w[4 * v4 + e] = (k + e < K) ? w_row[k + e] : 0.0f;
      }
    }
    if (r >= O) {
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = 0.0f;
    }
  };

  float x_keep[16];
  if (ONE_STEP) gather16(h * 16, x_keep);

  // noise management over the patch row (rpu_forward_backward_pass.cpp:112-178)
  float nm = 1.0f;
  if (!io.perfect && (io.noise_management == RPU_NM_ABS_MAX || io.noise_management == RPU_NM_MAX)) {
    float amax = 0.0f, vmax = -INFINITY;
    for (int st = 0; st < steps; ++st) {
      float x[16];
      if (!ONE_STEP) gather16(st * 32 + h * 16, x);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float xv = ONE_STEP ? x_keep[i] : x[i];
        if (st * 32 + h * 16 + i < K) {
          amax = fmaxf(amax, fabsf(xv));
          vmax = fmaxf(vmax, xv);
        }
      }
    }
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    vmax = fmaxf(vmax, __shfl_xor(vmax, 32));
    const float m = io.noise_management == RPU_NM_MAX ? vmax : amax;
    nm = io.nm_thres > 0.0f ? fminf(m, io.nm_thres) : m;
  } else if (!io.perfect && io.noise_management == RPU_NM_CONSTANT) {
    nm = io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
  }
  float red = 1.0f, fin = 1.0f, scale = 1.0f;
  if (!io.perfect) scale = round_scales(a, nm, red, fin);
  bool active = s_ok;
  int rounds_run = 0;
  float *out = c.out + (long)n * O * c.patches + p;

  const int max_rounds = io.perfect ? 1 : a.max_rounds;
  for (int round = 0; round < max_rounds; ++round) {
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    // wave-uniform: the lanes also carry the weight rows of the contraction, whatever their own patch holds (a zero
    // patch has scale 0 and contributes zeros)
    if (__any(fin != 0.0f) || io.perfect) {
      for (int st = 0; st < steps; ++st) {
        const int k0 = st * 32 + h * 16;
        float xd[16], wd[16];
        if (!ONE_STEP) gather16(k0, xd);
        weights16(k0, wd);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float x = ONE_STEP ? x_keep[i] : xd[i];
          if (!io.perfect && k0 + i < K) x = dac_value<STOCH>(x, scale, io, a.key, a.call, round, b, k0 + i);
          xd[i] = x;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wd[i], xd[i], acc, 0, 0, 0);
      }
    }
    // ADC: lane (r, h) holds, of patch r, the outputs g * 8 + h * 4 + q
    int up_max = 0, lo_max = 0;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int o0 = g * 8 + h * 4;
      if (o0 >= O) continue;
      float v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = acc[4 * g + q];
      int up = 0, lo = 0;
      if (io.perfect) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] *= a.alpha;
      } else if (fin == 0.0f) { // zero input: the reference short-cuts to a zero output
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = 0.0f;
      } else {
        mvm_adc_values<STOCH>(a, round, b, fin, o0, v, up, lo);
      }
      if (active) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (o0 + q < O) out[(long)(o0 + q) * c.patches] = v[q];
        }
      }
      up_max = max(up_max, up);
      lo_max = max(lo_max, lo);
    }
    if (active && (io.perfect || fin != 0.0f)) rounds_run = round + 1;
    if (io.perfect || io.bound_management == RPU_BM_NONE) break;
    // both halves of the wave hold outputs of patch r
    up_max = max(up_max, __shfl_xor(up_max, 32));
    lo_max = max(lo_max, __shfl_xor(lo_max, 32));
    const bool failed = io.bm_test_negative_bound ? (up_max > 0 || lo_max > 0) : (up_max > lo_max);
    bool more = false;
    if (active && failed) {
      float nm_next = nm, red_next = red;
      if (next_round_params(a, round, b, fin, nm_next, red_next)) {
        nm = nm_next;
        red = red_next;
        scale = round_scales(a, nm, red, fin);
        more = true;
      }
    }
    active = more;
    if (!__any(active)) break;
  }
  if (s_ok && !io.perfect && h == 0) a.st.rounds[b] = rounds_run;
}

// Long patch rows (more than two contraction steps): one workgroup per 32 patches, its four waves share the patches
// and deal the contraction steps among themselves (partial sums added through LDS in a fixed order, each wave then
// finishes 8 of the 32 output rows).  Every wave keeps the per-patch state, so the round loop is workgroup-uniform.
template <bool STOCH, bool WOC = false>
__global__ __launch_bounds__(256, 4) void k_conv_forward_split(MvmArgs a, ConvArgs c) {
  __shared__ float red[WAVES][16][64];
  __shared__ float sh_max[2][WAVES][32];
  __shared__ int sh_hits[2][32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  const long tile = blockIdx.x;
  const long total = (long)c.n_images * c.patches;
  const long s_raw = tile * 32 + r;
  const bool s_ok = s_raw < total;
  const long sample = s_ok ? s_raw : total - 1;
  const int n = (int)(sample / c.patches);
  const int p = (int)(sample - (long)n * c.patches);
  const float *image = c.images + (long)n * c.image_size;
  const int *idx_row = c.idx_t + (long)p * a.K;
  const float *w_row = a.w + (long)min(r, a.O - 1) * (WOC ? 1 : a.w_ld); // WOC: the lane's output column
  const int K = a.K, O = a.O;
  const int steps = (K + 31) / 32;
  const IoDev &io = a.io;
  const int b = (int)sample;

  auto gather16 = [&](int k0, float (&x)[16]) __attribute__((always_inline)) {
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int k = k0 + 4 * v4;
      int j[4];
      if (k + 4 <= K) {
        const i32x4_unaligned t = *reinterpret_cast<const i32x4_unaligned *>(idx_row + k);
        j[0] = t.x; j[1] = t.y; j[2] = t.z; j[3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) j[e] = (k + e < K) ? idx_row[k + e] : 0;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * v4 + e] = (j[e] <= 1) ? (float)j[e] : image[j[e] - 2];
    }
  };
  auto weights16 = [&](int k0, float (&w)[16]) __attribute__((always_inline)) {
    if constexpr (WOC) { // rows of the stored matrix hold the outputs of one k: a uniform row address + the lane's column
      const unsigned col = (unsigned)min(r, O - 1);
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = (a.w + (long)min(k0 + i, K - 1) * a.w_ld)[col];
      if (k0 + 16 > K) {
#pragma unroll
        for (int i = 0; i < 16; ++i) w[i] = (k0 + i < K) ? w[i] : 0.0f;
      }
    } else
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int k = k0 + 4 * v4;
      if (k + 4 <= K) {
        const f32x4_unaligned t = *reinterpret_cast<const f32x4_unaligned *>(w_row + k);
        w[4 * v4] = t.x; w[4 * v4 + 1] = t.y; w[4 * v4 + 2] = t.z; w[4 * v4 + 3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) w[4 * v4 + e] = (k + e < K) ? w_row[k + e] : 0.0f;
      }
    }
    if (r >= O) {
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = 0.0f;
    }
  };

  float nm = 1.0f;
  if (!io.perfect && (io.noise_management == RPU_NM_ABS_MAX || io.noise_management == RPU_NM_MAX)) {
    float amax = 0.0f, vmax = -INFINITY;
    for (int st = wave; st < steps; st += WAVES) {
      float x[16];
      gather16(st * 32 + h * 16, x);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (st * 32 + h * 16 + i < K) {
          amax = fmaxf(amax, fabsf(x[i]));
          vmax = fmaxf(vmax, x[i]);
        }
      }
    }
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    vmax = fmaxf(vmax, __shfl_xor(vmax, 32));
    if (h == 0) {
      sh_max[0][wave][r] = amax;
      sh_max[1][wave][r] = vmax;
    }
    __syncthreads();
    amax = fmaxf(fmaxf(sh_max[0][0][r], sh_max[0][1][r]), fmaxf(sh_max[0][2][r], sh_max[0][3][r]));
    vmax = fmaxf(fmaxf(sh_max[1][0][r], sh_max[1][1][r]), fmaxf(sh_max[1][2][r], sh_max[1][3][r]));
    const float m = io.noise_management == RPU_NM_MAX ? vmax : amax;
    nm = io.nm_thres > 0.0f ? fminf(m, io.nm_thres) : m;
  } else if (!io.perfect && io.noise_management == RPU_NM_CONSTANT) {
    nm = io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
  }
  float red_f = 1.0f, fin = 1.0f, scale = 1.0f;
  if (!io.perfect) scale = round_scales(a, nm, red_f, fin);
  bool active = s_ok;
  int rounds_run = 0;
  float *out = c.out + (long)n * O * c.patches + p;

  const int max_rounds = io.perfect ? 1 : a.max_rounds;
  for (int round = 0; round < max_rounds; ++round) {
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    // wave-uniform: the lanes also carry the weight rows of the contraction, whatever their own patch holds (a zero
    // patch has scale 0 and contributes zeros)
    if (__any(fin != 0.0f) || io.perfect) {
      for (int st = wave; st < steps; st += WAVES) {
        const int k0 = st * 32 + h * 16;
        float xd[16], wd[16];
        gather16(k0, xd);
        weights16(k0, wd);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (!io.perfect && k0 + i < K) xd[i] = dac_value<STOCH>(xd[i], scale, io, a.key, a.call, round, b, k0 + i);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wd[i], xd[i], acc, 0, 0, 0);
      }
    }
    if (threadIdx.x < 64) sh_hits[threadIdx.x >> 5][threadIdx.x & 31] = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) red[wave][i][lane] = acc[i];
    __syncthreads();
    // this wave finishes the output rows wave * 8 + h * 4 + q of patch r
    {
      const int o0 = wave * 8 + h * 4;
      float v[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = wave * 4 + q;
        v[q] = ((red[0][i][lane] + red[1][i][lane]) + red[2][i][lane]) + red[3][i][lane];
      }
      int up = 0, lo = 0;
      if (o0 < O) {
        if (io.perfect) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] *= a.alpha;
        } else if (fin == 0.0f) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = 0.0f;
        } else {
          mvm_adc_values<STOCH>(a, round, b, fin, o0, v, up, lo);
        }
        if (active) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (o0 + q < O) out[(long)(o0 + q) * c.patches] = v[q];
          }
        }
      }
      if (up) atomicMax(&sh_hits[0][r], up);
      if (lo) atomicMax(&sh_hits[1][r], lo);
    }
    if (active && (io.perfect || fin != 0.0f)) rounds_run = round + 1;
    if (io.perfect || io.bound_management == RPU_BM_NONE) break;
    __syncthreads();
    const int up_max = sh_hits[0][r], lo_max = sh_hits[1][r];
    const bool failed = io.bm_test_negative_bound ? (up_max > 0 || lo_max > 0) : (up_max > lo_max);
    bool more = false;
    if (active && failed) {
      float nm_next = nm, red_next = red_f;
      if (next_round_params(a, round, b, fin, nm_next, red_next)) {
        nm = nm_next;
        red_f = red_next;
        scale = round_scales(a, nm, red_f, fin);
        more = true;
      }
    }
    active = more;
    if (!__syncthreads_or(active ? 1 : 0)) break; // also keeps red / sh_hits until every wave has read them
  }
  if (s_ok && !io.perfect && wave == 0 && h == 0) a.st.rounds[b] = rounds_run;
}

// The same for several tiles in one launch: a workgroup finds its tile in the table of first workgroup numbers
// (a multiple of 8 per tile, so the XCD of a workgroup is the one its tile-local number implies).
template <int PD, int WMODE>
__global__ __launch_bounds__(256) void k_mvm_round_group(MvmGroup g, int round, int *seen) {
  __shared__ float red[WAVES][16][64];
  __shared__ __attribute__((aligned(16))) float stage[WAVES * 2 * TILE * LDS_ROW];
  if (seen && round == 1 && blockIdx.x == 0) group_seen_update(g, seen);
  int t = 0;
  while (t + 1 < g.n && (int)blockIdx.x >= g.start[t + 1]) ++t;
  const MvmArgs &a = g.args[t];
  if (round > 0 && round >= a.max_rounds) return;
  const int n_act = (round > 0) ? a.st.count[round] : a.m_batch;
  if (runs_on_large_tiles(a, round, n_act)) return;
  mvm_round_workgroup<PD, WMODE>(a, round, (int)blockIdx.x - g.start[t], n_act, red, stage);
}

template <int SUB>
__global__ __launch_bounds__(256) void k_mvm_init_group(MvmGroup g) {
  __shared__ float sh[8];
  static_assert(SUB % 64 == 0, "a wave works on one sample");
  const long sample = blockIdx.x * (long)(256 / SUB) + threadIdx.x / SUB; // m_batch is a multiple of 256 / SUB
  // the tile is the same for the whole wave: its arguments are fetched once, by scalar loads, into a copy that the
  // stores of the per-sample state cannot alias (through the pointer, every store would be followed by reloads)
  const int t = __builtin_amdgcn_readfirstlane((int)(sample / g.m_batch));
  if (t >= g.n) return;
  const int b = (int)(sample - (long)t * g.m_batch);
  const int lane = threadIdx.x % SUB;
  const MvmArgs a = g.args[t];
  mvm_init_sample<SUB>(a, b, lane, (long)b * SUB + lane, (long)g.m_batch * SUB, sh);
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

// prefetch depth used for a contraction length: deep for long contractions, where each of the few
// resident waves must cover the memory latency alone
static int mvm_prefetch_depth(int K, int k_pad) {
  if (K >= 512 && k_pad % (KSTEP * WAVES * 4) == 0) return 4;
  if (K >= 256 && k_pad % (KSTEP * WAVES * 2) == 0) return 2;
  return 1;
}

// tight: a multiple of 32 (what the large-tile kernel and the single-register-set variants need); otherwise K is
// rounded up so that the prefetch depth that suits its length can be used
int mvm_k_pad(int K, bool tight) {
  const int depth = tight ? 1 : (K >= 512 ? 4 : (K >= 256 ? 2 : 1));
  const int unit = depth == 1 ? KSTEP : KSTEP * WAVES * depth;
  return ((K + unit - 1) / unit) * unit;
}

// addressing mode of the weight operand (see k_mvm_round)
static int weight_mode(const MvmArgs &a) {
  if (!a.w_oc && (a.w_ld & 3) == 0 && (a.K & 15) == 0 && a.K >= 16 && ((((uintptr_t)a.w) & 15) == 0)) return 0;
  if (a.w_oc) return 1;
  return 2;
}

// A small batch gets a workgroup per sample (most workgroups in flight, shortest latency); a large one gets as
// many threads per sample as its rows can keep busy.
void launch_mvm_init(const MvmArgs &a, hipStream_t s) {
  if (a.in_index_lines) { // gathered input; the caller has checked that the noise management is one of these kernels'
    const long blocks = (long)(a.m_batch / a.in_group) * ((a.in_group + 63) / 64);
    if (!a.io.perfect && (a.io.noise_management == RPU_NM_ABS_MAX || a.io.noise_management == RPU_NM_MAX)) {
      const long max_blocks = (long)((a.m_batch / a.in_group + 3) / 4) * ((a.in_group + 63) / 64);
      hipLaunchKernelGGL(k_mvm_gather_max, dim3((unsigned)max_blocks), dim3(1024), 0, s, a);
    }
    hipLaunchKernelGGL(k_mvm_init_gather, dim3((unsigned)(blocks * ((a.k_pad + 63) / 64))), dim3(256), 0, s, a);
    return;
  }
  if (a.m_batch <= 1024 || a.K > 512) {
    hipLaunchKernelGGL(k_mvm_init<256>, dim3(a.m_batch), dim3(256), 0, s, a);
  } else if (a.K > 64) {
    hipLaunchKernelGGL(k_mvm_init<64>, dim3((a.m_batch + 3) / 4), dim3(256), 0, s, a);
  } else {
    hipLaunchKernelGGL(k_mvm_init<16>, dim3((a.m_batch + 15) / 16), dim3(256), 0, s, a);
  }
}

// a linear recurrence over the batch, evaluated in the reference's order and rounding by one thread
__global__ void k_nm_running_average(float *nm, int m_batch, float decay, float *aux) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  float v = *aux;
  for (int b = 0; b < m_batch; ++b) {
    const float amax = nm[b];
    v = v < 0.0f ? amax : v * (1.0f - decay) + decay * amax;
    nm[b] = v;
  }
  *aux = v;
}

void launch_nm_running_average(float *nm, int m_batch, float decay, float *aux, hipStream_t s) {
  hipLaunchKernelGGL(k_nm_running_average, dim3(1), dim3(64), 0, s, nm, m_batch, decay, aux);
}

int mvm_round_workgroups(const MvmArgs &a) { return workgroups_for(a.O, a.m_batch); }

void mvm_round_variant(const MvmArgs &a, int &prefetch_depth, int &mode) {
  prefetch_depth = mvm_prefetch_depth(a.K, a.k_pad);
  mode = weight_mode(a);
}

// max_k: the longest input row of the group
void launch_mvm_init_group(const MvmGroup &g, int max_k, hipStream_t s) {
  const long samples = (long)g.n * g.m_batch;
  if (samples > 2048 && max_k <= 512 && g.m_batch % 4 == 0) {
    hipLaunchKernelGGL(k_mvm_init_group<64>, dim3((unsigned)(samples / 4)), dim3(256), 0, s, g);
  } else {
    hipLaunchKernelGGL(k_mvm_init_group<256>, dim3((unsigned)samples), dim3(256), 0, s, g);
  }
}

constexpr int TAIL_GRID = 1024; // workgroups of a later-round launch when the full grid would be larger

// workgroups of a large-tile launch with sample tiles of `bb` samples
static int big_workgroups(const MvmArgs &a, int bb) {
  const int tiles_o = (a.O + 127) / 128, tiles_b = (a.m_batch + bb - 1) / bb;
  return 8 * tiles_o * ((tiles_b + 7) / 8);
}

int mvm_big_workgroups(const MvmArgs &a, int bb) { return a.O >= 128 ? big_workgroups(a, bb) : 0; }

// Sample-tile edge for a launch that would have `workgroups_128` workgroups with square tiles.  A CU holds two of
// those, so they run in rounds of 2 n_cus: where the last round is (nearly) full they are the better choice (more
// multiply-adds per byte staged), otherwise its idle CUs cost more than that (384 workgroups occupy half of the CUs
// twice as long as the other half) and tiles of 64 samples, three to a CU, fill the chip more evenly.  Measured on
// the 1024 x 1024 tile: batch 8192 and 16384 (exactly one and two rounds) are 7 .. 12 % faster with 128, every other
// batch between 2048 and 20480 with 64 (up to 35 % at 2048, 18 % at 10240).
int mvm_big_sample_tile(int workgroups_128, int n_cus) {
  const int slots = 2 * n_cus;
  const int rounds = (workgroups_128 + slots - 1) / slots;
  const int idle = rounds * slots - workgroups_128;
  return 10 * idle <= rounds * slots ? 128 : 64;
}

void launch_mvm_big_group(const MvmGroup &g, int total_workgroups, int bb, bool w_oc, hipStream_t s) {
  const dim3 grid(total_workgroups);
  if (bb == 128) {
    if (w_oc) hipLaunchKernelGGL((k_mvm_big_group<1, 128>), grid, dim3(256), 0, s, g, 0);
    else hipLaunchKernelGGL((k_mvm_big_group<0, 128>), grid, dim3(256), 0, s, g, 0);
  } else {
    if (w_oc) hipLaunchKernelGGL((k_mvm_big_group<1, 64>), grid, dim3(256), 0, s, g, 0);
    else hipLaunchKernelGGL((k_mvm_big_group<0, 64>), grid, dim3(256), 0, s, g, 0);
  }
}

// samples of a round from which the large-tile kernel takes over, 0 when a call of this shape never uses it: it
// needs outputs for a whole 128-wide tile and enough half tiles for every second CU
static int big_threshold(int m_batch, int O) {
  // measured on the 1024 x 1024 tile: the half tiles overtake the 32 x 32 kernel at about 1500 samples (backward 70
  // against 88 us at 1536, 74 against 113 us at 2000; at 1024 the 32 x 32 kernel still leads, 63 against 68 us)
  constexpr int big_min = 1536;
  // narrower tiles (the patches of a convolution): part of the 128 outputs of a tile are idle, but a staged operand
  // byte still meets four times the multiply-adds of the 32 x 32 kernel
  constexpr int narrow_min_batch = 16384, narrow_min_outputs = 33;
  if (m_batch < big_min || O < narrow_min_outputs || (O < 128 && m_batch < narrow_min_batch)) return 0;
  const int tiles_o = (O + 127) / 128, tiles_b = (m_batch + 63) / 64;
  if (8 * tiles_o * ((tiles_b + 7) / 8) < 128) return 0;
  return big_min;
}

static int current_device_cus() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

bool mvm_uses_large_tiles(int m_batch, int O) { return big_threshold(m_batch, O) > 0; }

void launch_mvm_round_group(const MvmGroup &g, int depth, int mode, int total_workgroups, int round, hipStream_t s,
                            int *seen) {
  if (round > 0 && total_workgroups > TAIL_GRID && g.n <= MAX_GROUP) {
    const dim3 tail(TAIL_GRID);
    if (mode == 0) hipLaunchKernelGGL(k_mvm_round_tail_group<0>, tail, dim3(256), 0, s, g, round, seen);
    else if (mode == 1) hipLaunchKernelGGL(k_mvm_round_tail_group<1>, tail, dim3(256), 0, s, g, round, seen);
    else hipLaunchKernelGGL(k_mvm_round_tail_group<2>, tail, dim3(256), 0, s, g, round, seen);
    return;
  }
  const dim3 grid(total_workgroups);
  if (mode == 1 && depth == 4 && total_workgroups > current_device_cus()) depth = 2; // as in launch_mvm_round
#define RPU_LAUNCH_ROUND(PD, WMODE) hipLaunchKernelGGL((k_mvm_round_group<PD, WMODE>), grid, dim3(256), 0, s, g, round, seen)
  if (mode == 0) {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 0);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 0);
    else RPU_LAUNCH_ROUND(1, 0);
  } else if (mode == 1) {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 1);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 1);
    else RPU_LAUNCH_ROUND(1, 1);
  } else {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 2);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 2);
    else RPU_LAUNCH_ROUND(1, 2);
  }
#undef RPU_LAUNCH_ROUND
}

// all rounds from round_first on in one launch of `workgroups` workgroups (at most one per CU: they wait for each other
// between rounds); for groups of at most MAX_GROUP tiles whose weights are not read transposed
bool mvm_group_can_merge_rest(const MvmGroup &g, int) { return g.n <= MAX_GROUP; }

void launch_mvm_rest_group(const MvmGroup &g, int mode, int round_first, int rounds, int workgroups, int *seen,
                           hipStream_t s) {
  const dim3 grid(workgroups);
  if (mode == 0) hipLaunchKernelGGL(k_mvm_rest_group<0>, grid, dim3(256), 0, s, g, round_first, rounds, seen);
  else if (mode == 1) hipLaunchKernelGGL(k_mvm_rest_group<1>, grid, dim3(256), 0, s, g, round_first, rounds, seen);
  else hipLaunchKernelGGL(k_mvm_rest_group<2>, grid, dim3(256), 0, s, g, round_first, rounds, seen);
}

// whether rounds 0 and 1 of this call can run as one launch (the caller decides whether they should)
bool mvm_can_fuse_rounds(const MvmArgs &a) {
  if (a.io.perfect || a.io.bound_management == RPU_BM_NONE || a.max_rounds < 3 || a.transposed) return false;
  if (a.pre_add || a.skip_if_zero || a.nm_phase || !a.speculate || !a.rows_ahead_in_init || a.in_index) return false;
  if (!a.small_tiles_only && big_threshold(a.m_batch, a.O) > 0) return false;
  return mvm_prefetch_depth(a.K, a.k_pad) >= 2;
}

// Workgroups of `kernel` (256 threads, static LDS only) that a launch may count on being resident together: one per CU,
// and none where the occupancy query finds no room for the kernel at all.  What the query reports beyond one per CU is
// not relied on: for k_mvm_rounds_rest<1, 0> (54 KB of LDS) it reports three, and a launch of 560 workgroups, 70 per
// XCD of 32 CUs, then ran into the limit of its wait -- not all of them had been placed.  The launches whose workgroups
// wait for each other are sized by this.
template <typename K> static int resident_workgroups(K kernel) {
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess || per_cu < 1) return 0;
  return current_device_cus();
}

// prefetch depth of the launch that runs several rounds: with the weights addressed along the outputs the deepest
// variant takes more than half of a SIMD's registers, and these launches mostly walk empty rounds
static int mvm_rest_depth(const MvmArgs &a) {
  const int depth = mvm_prefetch_depth(a.K, a.k_pad);
  return (weight_mode(a) == 1 && depth == 4) ? 2 : depth;
}

int mvm_rest_resident_limit(const MvmArgs &a) {
  static std::mutex m;
  static int limit[64][3][3] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  const int mode = weight_mode(a);
  const int depth = mvm_rest_depth(a);
  const int di = depth == 4 ? 2 : (depth == 2 ? 1 : 0);
  std::lock_guard<std::mutex> lock(m);
  int &v = limit[dev][di][mode];
  if (v == 0) {
    if (mode == 0) {
      v = depth == 4 ? resident_workgroups(k_mvm_rounds_rest<4, 0>)
                     : (depth == 2 ? resident_workgroups(k_mvm_rounds_rest<2, 0>) : resident_workgroups(k_mvm_rounds_rest<1, 0>));
    } else if (mode == 1) { // the deepest prefetch is not built for this addressing (mvm_rest_depth)
      v = depth == 2 ? resident_workgroups(k_mvm_rounds_rest<2, 1>) : resident_workgroups(k_mvm_rounds_rest<1, 1>);
    } else {
      v = depth == 4 ? resident_workgroups(k_mvm_rounds_rest<4, 2>)
                     : (depth == 2 ? resident_workgroups(k_mvm_rounds_rest<2, 2>) : resident_workgroups(k_mvm_rounds_rest<1, 2>));
    }
    if (v == 0) v = -1; // the query failed: never merge
  }
  return v > 0 ? v : 0;
}

int mvm_group_rest_resident_limit(int mode) {
  static std::mutex m;
  static int limit[64][3] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  std::lock_guard<std::mutex> lock(m);
  int &v = limit[dev][mode];
  if (v == 0) {
    v = mode == 0 ? resident_workgroups(k_mvm_rest_group<0>)
                  : (mode == 1 ? resident_workgroups(k_mvm_rest_group<1>) : resident_workgroups(k_mvm_rest_group<2>));
    if (v == 0) v = -1;
  }
  return v > 0 ? v : 0;
}

// whether the rounds after round 0 of this call can share one launch (mvm_can_fuse_rounds without the conditions of
// the two-accumulator kernel).  Its workgroups wait for each other between rounds, so all of them must be resident at
// once: resident_limit is what the GPU holds of that kernel when nothing else runs on it.  Another launch that holds
// CUs at that moment (a second stream) can make a wait run out; that is reported (see RoundWait), never passed over.
bool mvm_can_merge_rest(const MvmArgs &a, int resident_limit) {
  if (a.io.perfect || a.io.bound_management == RPU_BM_NONE || a.max_rounds < 3 || a.transposed) return false;
  // gathered input: the rows of a further round are written by k_mvm_round_tail alone, one launch per round
  if (a.pre_add || a.skip_if_zero || a.nm_phase || a.in_index) return false;
  if (!a.small_tiles_only && big_threshold(a.m_batch, a.O) > 0) return false;
  return mvm_round_workgroups(a) <= resident_limit;
}

void launch_mvm_dual(const MvmArgs &a_in, hipStream_t s) {
  MvmArgs a = a_in;
  a.big_from = 0;
  a.round = 0;
  a.dual.on = 1;
  const dim3 grid(mvm_round_workgroups(a));
  const int mode = weight_mode(a);
  if (a.dual.rounds == 3) {
    if (mode == 0) hipLaunchKernelGGL((k_mvm_dual<0, 3>), grid, dim3(256), 0, s, a);
    else if (mode == 1) hipLaunchKernelGGL((k_mvm_dual<1, 3>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((k_mvm_dual<2, 3>), grid, dim3(256), 0, s, a);
    return;
  }
  if (mode == 0) hipLaunchKernelGGL((k_mvm_dual<0, 2>), grid, dim3(256), 0, s, a);
  else if (mode == 1) hipLaunchKernelGGL((k_mvm_dual<1, 2>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((k_mvm_dual<2, 2>), grid, dim3(256), 0, s, a);
}

void launch_mvm_round(const MvmArgs &a_in, hipStream_t s) {
  MvmArgs a = a_in;
  a.big_from = a.small_tiles_only ? 0 : big_threshold(a.m_batch, a.O);
  // calls that quantize nothing ahead expect few samples in a further round: the 32 x 32 kernels take them all, and
  // the round is one launch
  if (a.round > 0 && !a.speculate) a.big_from = 0;
  if (a.big_from > 0) {
    // the variants below exist for the way a tile that stores [d_size][x_size] addresses its weights (forward: rows
    // along k, backward: rows along the outputs); the other storage takes the general kernels where its case has none
    const bool lazy = !a.transposed && !a.speculate && a.max_rounds > 1;
    const bool narrow = !a.transposed && !a.w_oc && a.O <= 64; // see mvm_big_workgroup
    const int bb = narrow ? 128 : mvm_big_sample_tile(big_workgroups(a, 128), current_device_cus());
    const dim3 big_grid(big_workgroups(a, bb));
    const int min_active = a.round > 0 ? a.big_from : 0;
    if (narrow) {
      hipLaunchKernelGGL(k_mvm_big_narrow, big_grid, dim3(256), 0, s, a, min_active);
    } else if (lazy && !a.w_oc) {
      if (bb == 128) hipLaunchKernelGGL((k_mvm_big_lazy<0, 128>), big_grid, dim3(256), 0, s, a, min_active);
      else hipLaunchKernelGGL((k_mvm_big_lazy<0, 64>), big_grid, dim3(256), 0, s, a, min_active);
    } else if (lazy) {
      if (bb == 128) hipLaunchKernelGGL((k_mvm_big_lazy<1, 128>), big_grid, dim3(256), 0, s, a, min_active);
      else hipLaunchKernelGGL((k_mvm_big_lazy<1, 64>), big_grid, dim3(256), 0, s, a, min_active);
    } else if (a.transposed && a.w_oc && a.k_pad <= 2 * BKS) { // see mvm_big_workgroup, NBUF
      if (bb == 128) hipLaunchKernelGGL((k_mvm_big_short<128>), big_grid, dim3(256), 0, s, a, min_active);
      else hipLaunchKernelGGL((k_mvm_big_short<64>), big_grid, dim3(256), 0, s, a, min_active);
    } else if (bb == 128) {
      if (a.w_oc) hipLaunchKernelGGL((k_mvm_big<1, 128>), big_grid, dim3(256), 0, s, a, min_active);
      else hipLaunchKernelGGL((k_mvm_big<0, 128>), big_grid, dim3(256), 0, s, a, min_active);
    } else {
      if (a.w_oc) hipLaunchKernelGGL((k_mvm_big<1, 64>), big_grid, dim3(256), 0, s, a, min_active);
      else hipLaunchKernelGGL((k_mvm_big<0, 64>), big_grid, dim3(256), 0, s, a, min_active);
    }
    if (a.round == 0) return; // later rounds: whichever kernel the number of listed samples calls for
  }
  const int all = mvm_round_workgroups(a);
  const int mode = weight_mode(a);
  if (a.round > 0 && (all > TAIL_GRID || a.in_index)) { // gathered input: only this kernel writes the rows it reads
    const dim3 grid(TAIL_GRID);
    if (mode == 0) hipLaunchKernelGGL(k_mvm_round_tail<0>, grid, dim3(256), 0, s, a);
    else if (mode == 1) hipLaunchKernelGGL(k_mvm_round_tail<1>, grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(k_mvm_round_tail<2>, grid, dim3(256), 0, s, a);
    return;
  }
  const dim3 grid(all);
  int depth = mvm_prefetch_depth(a.K, a.k_pad);
  // With more workgroups than CUs the output-contiguous variant is a little faster with two stages of loads in flight
  // than with four (backward on the 1024 x 1024 tile at batch 512 / 1024: 25.9 / 43.5 us against 26.7 / 44.9; same sums,
  // the waves split K the same way).
  if (mode == 1 && depth == 4 && all > current_device_cus()) depth = 2;
  if (a.rest_in_one) {
#define RPU_LAUNCH_REST(PD, WMODE) hipLaunchKernelGGL((k_mvm_rounds_rest<PD, WMODE>), grid, dim3(256), 0, s, a)
    if (mode == 0) {
      if (depth == 4) RPU_LAUNCH_REST(4, 0);
      else if (depth == 2) RPU_LAUNCH_REST(2, 0);
      else RPU_LAUNCH_REST(1, 0);
    } else if (mode == 1) {
      if (mvm_rest_depth(a) == 2) RPU_LAUNCH_REST(2, 1);
      else RPU_LAUNCH_REST(1, 1);
    } else {
      if (depth == 4) RPU_LAUNCH_REST(4, 2);
      else if (depth == 2) RPU_LAUNCH_REST(2, 2);
      else RPU_LAUNCH_REST(1, 2);
    }
#undef RPU_LAUNCH_REST
    return;
  }
#define RPU_LAUNCH_ROUND(PD, WMODE) hipLaunchKernelGGL((k_mvm_round<PD, WMODE>), grid, dim3(256), 0, s, a)
  if (mode == 0) {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 0);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 0);
    else RPU_LAUNCH_ROUND(1, 0);
  } else if (mode == 1) {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 1);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 1);
    else RPU_LAUNCH_ROUND(1, 1);
  } else {
    if (depth == 4) RPU_LAUNCH_ROUND(4, 2);
    else if (depth == 2) RPU_LAUNCH_ROUND(2, 2);
    else RPU_LAUNCH_ROUND(1, 2);
  }
#undef RPU_LAUNCH_ROUND
}

bool conv_forward_supported(const MvmArgs &a) {
  if (a.O > 32 || a.transposed) return false;
  if (a.io.perfect) return true;
  const int nm = a.io.noise_management, bm = a.io.bound_management;
  return (nm == RPU_NM_NONE || nm == RPU_NM_ABS_MAX || nm == RPU_NM_MAX || nm == RPU_NM_CONSTANT) &&
         (bm == RPU_BM_NONE || bm == RPU_BM_ITERATIVE);
}

void launch_conv_forward(const MvmArgs &a, const ConvArgs &c, hipStream_t s) {
  const long tiles = ((long)c.n_images * c.patches + 31) / 32;
  const dim3 grid((unsigned)((tiles + 3) / 4));
  const bool stoch = !a.io.perfect && (a.io.inp_sto_round || a.io.out_sto_round || a.io.inp_noise > 0.0f);
#define RPU_LAUNCH_CONV(STOCH, WOC)                                                                                  \
  {                                                                                                                   \
    if (a.K <= 32) hipLaunchKernelGGL((k_conv_forward<true, STOCH, WOC>), grid, dim3(256), 0, s, a, c);              \
    else if (a.K <= 64) hipLaunchKernelGGL((k_conv_forward<false, STOCH, WOC>), grid, dim3(256), 0, s, a, c);        \
    else hipLaunchKernelGGL((k_conv_forward_split<STOCH, WOC>), dim3((unsigned)tiles), dim3(256), 0, s, a, c);       \
  }
  if (stoch) {
    if (a.w_oc) RPU_LAUNCH_CONV(true, true) else RPU_LAUNCH_CONV(true, false)
  } else {
    if (a.w_oc) RPU_LAUNCH_CONV(false, true) else RPU_LAUNCH_CONV(false, false)
  }
#undef RPU_LAUNCH_CONV
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
