// Launch interface between the host tile class and the HIP kernels (gfx950).
#pragma once
#include "../../include/rpu_amd.h"
#include "philox.h"
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rpu_amd {

// IO non-idealities of one pass, absolute steps (see IOPar::initialize).
struct IoDev {
  float inp_res, inp_bound, inp_noise, inp_asym;
  float out_res, out_bound, out_noise, out_asym, out_scale;
  float nm_thres, nm_assumed_wmax, max_bm_res;
  int noise_management, bound_management, bm_test_negative_bound, max_bm_factor;
  int inp_sto_round, out_sto_round;
  int perfect;
};

// Per-sample bookkeeping of the noisy MVM, all arrays of length >= m_batch.
constexpr int MVM_COUNT_WORDS = 256; // MvmState::count: [0, 40) per round; [MVM_ARRIVE_BASE + 4 r, + 4): counter and flag of the
                                     // arrivals after round r, counter and flag of the wait before round r
constexpr int MVM_ARRIVE_BASE = 64;
constexpr int MVM_ABORT_WORD = 255;  // MvmState::count[MVM_ABORT_WORD]: raised by a workgroup whose wait for the others ran out

struct MvmState {
  float *nm;       // noise-management scale
  float *nm_np;    // AbsMaxNPSum scale (IterativeWorstCase only)
  float *red;      // bound-management reduction of the current round
  float *scale;    // input scale of the current round
  float *fin;      // factor applied to the ADC output (0 = sample short-cut to zero)
  int *rounds;     // rounds run so far
  int *hit_up;     // 1 + largest output index that hit the upper bound this round (0 = none)
  int *hit_lo;     // same for the lower bound
  int *list[2];    // ping-pong lists of samples that need another round
  int *row[2];     // row[i][pos]: row of xq[i] that holds the quantized input of the sample at list[i][pos]
  float *next_scale[2]; // next_scale[i][pos]: input scale that sample would use one round later (0: no such round)
  int *count;      // count[r] = number of samples in the list read by round r (r >= 1); MVM_COUNT_WORDS words, the
                   // upper half the arrival counters of the launches that run several rounds
  int *tile_done;  // tile_done[r * tiles_b + t] = workgroups of round r that have finished sample tile t
};

// Rounds 0 and 1 of a call in one launch (samples that need a second round are the rule on some workloads):
// the state of that launch and of the selection that the following launch starts with.
struct DualDev {
  float *buf[3]; // buf[r]: [m_batch][O] outputs of round r of the fused launch
  int *sel;      // [m_batch] which of them is the sample's output (0 .. rounds - 1); rounds: the sample is listed
                 // for the round after the fused launch
  int *hit1;     // [2][m_batch] saturation marks of round 1: upper, lower (as MvmState::hit_up / hit_lo)
  int *hit2;     // the same of round 2 (three fused rounds)
  float *xq2;    // quantized rows of round 2: written by the fused launch of two rounds while round 0's rows are still
                 // read, by the init kernel for a fused launch of three
  int rounds;    // rounds of the fused launch: 2 or 3 (0: the call has none)
  int *seen;     // host-visible: [0] samples of the last call that needed round 1, [1] its batch, [2] the last round
                 // that listed a sample (0: none after round 0), [3] 1 + the round at which a wait between the
                 // workgroups of a launch gave up (0: none); null: not kept
  int on;        // 1: the fused launch; 2: this launch starts with the selection of the fused launch's results
};

struct MvmArgs {
  // The weight matrix as it is stored: rows of w_ld elements.  w_oc = 0: a row holds the contraction index of one
  // output (out[o] = sum_k w[o * w_ld + k] in[k]); w_oc = 1: a row holds the outputs of one contraction index
  // (out[o] = sum_k w[k * w_ld + o] in[k]).  A tile that stores [d_size][x_size] runs forward with w_oc = 0 and
  // backward with w_oc = 1; one that stores [x_size][d_size] (the layout of the reference's CUDA tiles) the other way
  // round.  Set by mvm_set_weights.
  const float *w;
  int w_oc, w_ld;
  int x_size, d_size;
  const float *in;
  long in_sb, in_sk; // input element (b, k) at in[b * in_sb + k * in_sk]
  float *out;
  long out_sb, out_so; // output element (b, o) at out[b * out_sb + o * out_so]
  int m_batch;
  int K, O;       // contraction length and number of outputs
  int k_pad;      // K rounded up to the step of the contraction kernel (mvm_k_pad)
  float *xq[2];   // ping-pong scratch [rows][k_pad]: DAC-quantized inputs, zero padded (rows: see MvmState::row)
  int transposed; // 0: forward pass (out = W in), 1: backward pass (out = W^T in); decides the scales of a round, not
                  // how the weights are addressed (w_oc)
  int round;      // bound-management round, 0-based
  int max_rounds; // rounds launched for this call (mvm_max_rounds)
  int speculate;  // 1: each round also quantizes every row for the round after it (short path between rounds, for
                  // small batches); 0: only the rows of samples that saturated are quantized, once that is known
  int rows_ahead_in_init; // 1: the init kernel also writes the rows of round 1 (round 0 then prepares nothing)
  int big_from;   // > 0: rounds with at least this many samples are run by the large-tile kernel; < 0: round 0 is
  float alpha, beta; // only used when io.perfect: out = alpha * acc + beta * out
  IoDev io;
  MvmState st;
  PhiloxKey key;
  uint32_t call;
  // Analog non-idealities that add to the sums before the ADC stage (output-referred weight noise, IR drop):
  // pre_add[row * O + o] for the output o of the sample whose quantized input is row `row` of xq[round & 1];
  // null: none.  Only the 32 x 32 round kernels read it.
  const float *pre_add;
  int pre_is_total;         // 1: pre_add holds the whole analog value before quantization (the kernel's own sums are unused)
  // PosNegSeparateDigitalSum (rpu_forward_backward_pass.cpp:861-877): post_add[row * O + o] is the finished ADC value
  // of the negative pass, added after this pass's own quantization and clipping; post_hit_up / post_hit_lo[row] hold
  // that pass's saturation marks (1 + largest output index that hit the bound), read and cleared when the sample is
  // advanced.  All null otherwise.
  const float *post_add;
  int *post_hit_up, *post_hit_lo;
  int nm_phase;             // running-average noise management: 1 = the init kernel only stores every sample's
                            // largest absolute input in st.nm, 2 = it takes the scales from st.nm; 0 otherwise
  int small_tiles_only;     // 1: never the large-tile kernel (its row padding differs)
  const int *skip_if_zero;  // non-null: a round launch does nothing when this device value is zero
  DualDev dual;
  int rest_in_one;          // 1: this launch runs round `round` and every round after it (k_mvm_rounds_rest)
  int wait_spins;           // polls after which a wait between the workgroups of such a launch gives up (0: the default)
  int wait_extra;           // arrivals such a wait expects beyond the launch's workgroups (0; tests of the give-up path: 1)
  // Tiles of a group call that quantize the same input the same way (the column blocks of a layer split over several
  // tiles) share the rows of rounds 0 and 1: with xq_first[0] set, those rounds read xq_first[round] instead of
  // xq[round & 1] (every later round uses the tile's own xq as usual), and the init kernel writes the shared rows
  // for the one tile that has xq_first_writer = 1.  Requires rows_ahead_in_init (or a single round).
  float *xq_first[2];
  int xq_first_writer;
  // Input gathered through an index (the patches of a convolution, never materialized) when in_index is set:
  // sample b is patch b % in_group of image b / in_group, images are in_gs apart in `in`, and element k of the sample
  // is what in_index[(b % in_group) * K + k] names: 0, 1 (bias) or, from 2 on, element j - 2 of the image.
  // in_index_lines is the same index line-major, [K][in_group] (the init kernels read it with lanes along the
  // patches).  Only for calls that read their input row by row (the gathering init kernels, rows of a further round
  // written once it is known who goes on: speculate = 0, or a single round).
  const int *in_index;
  const int *in_index_lines;
  int in_group;
  long in_gs;
};

// weight operand of a call: the matrix at w with rows of `ld` elements, stored [d_size][x_size] (xd_storage = false) or
// [x_size][d_size]; a.transposed must be set
inline void mvm_set_weights(MvmArgs &a, const float *w, int ld, bool xd_storage) {
  a.w = w;
  a.w_ld = ld;
  a.w_oc = (a.transposed != 0) != xd_storage ? 1 : 0;
}
// noise management + per-sample state for round 0
void launch_mvm_init(const MvmArgs &a, hipStream_t s);
// one round of DAC -> MFMA contraction -> ADC
void launch_mvm_round(const MvmArgs &a, hipStream_t s);
// rounds 0 and 1 in one launch (a.dual filled in); the launches of rounds 2 .. follow with a.dual.on = 2 on the first
// of them and a.xq[0] = a.dual.xq2
bool mvm_can_fuse_rounds(const MvmArgs &a);
// the rounds from a.round on in one launch (a.rest_in_one = 1 for launch_mvm_round): for calls that expect them empty
// resident_limit: workgroups of that launch that the GPU holds at once (mvm_rest_resident_limit)
bool mvm_can_merge_rest(const MvmArgs &a, int resident_limit);
int mvm_rest_resident_limit(const MvmArgs &a);
void launch_mvm_dual(const MvmArgs &a, hipStream_t s);
// AverageAbsMax noise management (rpu_forward_backward_pass.cpp:138-149): nm[b] holds the largest absolute input of
// sample b and becomes the running average after that sample, in batch order; aux carries the value between calls
// (negative: not started)
void launch_nm_running_average(float *nm, int m_batch, float decay, float *aux, hipStream_t s);
// Several tiles in one launch: args[t] are the tiles' arguments in HBM, start[t] .. start[t + 1] the workgroups of
// tile t in a round launch (all tiles share m_batch).  The tiles of one round launch share a kernel variant.
struct MvmGroup {
  const MvmArgs *args;
  const int *start; // [n + 1]
  int n;
  int m_batch;
  // waits between the workgroups of k_mvm_rest_group (see MvmArgs::wait_spins / wait_extra); wait_failed: host-visible
  // word that takes 1 + the round at which a wait gave up
  int wait_spins = 0, wait_extra = 0;
  int *wait_failed = nullptr;
};
void launch_mvm_init_group(const MvmGroup &g, int max_k, hipStream_t s);
// seen: host-visible pair (any tile lists a sample for round 1, batch) written by the launch of round 1; may be null
void launch_mvm_round_group(const MvmGroup &g, int prefetch_depth, int weight_mode, int total_workgroups, int round,
                            hipStream_t s, int *seen = nullptr);
// the rounds from round_first on in one launch, for calls that expect them to list nothing (see k_mvm_rounds_rest)
bool mvm_group_can_merge_rest(const MvmGroup &g, int weight_mode);
int mvm_group_rest_resident_limit(int weight_mode); // workgroups of k_mvm_rest_group that the GPU holds at once
void launch_mvm_rest_group(const MvmGroup &g, int weight_mode, int round_first, int rounds, int workgroups, int *seen,
                           hipStream_t s);
int mvm_round_workgroups(const MvmArgs &a);            // workgroups of a round launch for this tile
// Large-tile (128 x 128) variant for round 0 of a group: args[t].big_from < 0 marks the tiles it runs, start[]
// counts its workgroups (mvm_big_workgroups; 0 for the other tiles).
int mvm_big_workgroups(const MvmArgs &a, int bb);
// bb: samples of a workgroup tile, 128 or 64 (mvm_big_sample_tile: by the workgroups the launch would have with 128)
int mvm_big_sample_tile(int workgroups_128, int n_cus);
// w_oc: how the tiles of the launch address their weights (MvmArgs::w_oc; the same for all of them)
void launch_mvm_big_group(const MvmGroup &g, int total_workgroups, int bb, bool w_oc, hipStream_t s);
void mvm_round_variant(const MvmArgs &a, int &prefetch_depth, int &weight_mode);

// Fused convolution forward (unfold + noisy MVM with its bound-management rounds) for tiles of at most 32 outputs:
// images [n_images][image_size], idx_t the transposed index matrix [patches][x_size], out [n_images][d_size][patches].
// MvmArgs carries the tile (w, sizes, io, key, call, max_rounds, st.rounds, alpha); in / out / xq are not used.
struct ConvArgs {
  const float *images;
  const int *idx_t;
  float *out;
  int patches, n_images;
  long image_size;
};
bool conv_forward_supported(const MvmArgs &a);
void launch_conv_forward(const MvmArgs &a, const ConvArgs &c, hipStream_t s);

// ---- analog non-idealities before the ADC (kernels_nonideal.hip), rpu_forward_backward_pass.cpp:325-433, 535-560
// transformed copy of the quantized input rows [rows][k_pad]: mode 0 x^2, 1 |x|, 2 x (1 - (1 - j / K)^2), 3 x
// part -1 / +1: only the negative / positive inputs (the others read as zero), before the transformation
void launch_side_rows(const float *xq, float *out, int rows, int k_pad, int K, int mode, int part, const int *skip_if_zero,
                      hipStream_t s);
void launch_abs_copy(const float *w, float *out, size_t n, hipStream_t s);
void launch_mul_copy(const float *w, const float *factors, float *out, size_t n, hipStream_t s); // out = w * factors
struct SideDev {
  int w_noise_type; // 0 none, 1 additive constant (row_sumsq), 2 PCM read (s_noise)
  float w_noise, ir_drop, a_scale; // a_scale = in_size / ir_drop_g_ratio
  // total mode (s_y non-null): the analog value itself is made here, with the per-line terms of the periphery
  // (applyVoltageOffsets and finalizeOutput up to the output noise, rpu_forward_backward_pass.cpp:436-506, 679-698)
  const float *s_y;        // W x_q per row and output
  const float *x_accum;    // sum of x_q per row (only read with v_offset_w_min != 0)
  const float *v_offset;   // per output, null: no voltage offsets / series resistance
  const float *out_nl;     // per output, null: no non-linearity
  const float *out_noise;  // per output, null: out_noise_all for every output
  float r_series, r_series_max_total, v_offset_w_min, nl_factor, out_noise_all, out_asym;
  // two passes (PosNegSeparate): the first stops after the weight noise (ni_only), the second adds that result
  // (add_ni) before the non-linearity
  int ni_only;
  const float *add_ni;
  // PosNegSeparateDigitalSum: the pass ends with its own ADC here (quantization, clipping, saturation marks per row)
  int adc_here, adc_sto_round;
  float adc_res, adc_bound;
  int *hit_up, *hit_lo; // [rows], null: no bound management
  // rounds after the first: row_sample[row] = the sample whose quantized input the row holds (made by
  // launch_side_row_samples); null: row r holds sample r.  The random draws are keyed by the sample, not by the row:
  // which row a sample gets in a later round depends on the order in which workgroups finished the round before.
  const int *row_sample;
};
// row_sample[row[pos]] = list[pos] for pos < *count (the list of a bound-management round and its rows)
void launch_side_row_samples(int *row_sample, const int *list, const int *row, const int *count, int rows, hipStream_t s);
// addend mode: pre[row][o] = w_noise term * N(0, 1) - IR-drop term; s_cur / s_ir are null without IR drop.
// total mode: pre[row][o] = asymmetry(nonlinearity(offsets(s_y - IR drop) + w_noise term)) + output noise
void launch_side_combine(float *pre, const float *s_noise, const float *row_sumsq, const float *s_cur, const float *s_ir,
                         const SideDev &p, int rows, int O, PhiloxKey key, uint32_t call, int round,
                         const int *skip_if_zero, hipStream_t s);

// number of rounds that can ever be needed with these IO settings
int mvm_max_rounds(const IoDev &io);
// row length of the quantized-input scratch for a contraction length K
int mvm_k_pad(int K, bool tight = false);
// whether a call of this shape has rounds run by the large-tile kernel (then the padding can be tight)
bool mvm_uses_large_tiles(int m_batch, int O);

// [B][X-1] (or [X-1][B]) -> [B][X] with a trailing column of ones (always batch-first output)
void launch_make_bias(const float *in, float *out, int m_batch, int x_size, int in_trans, hipStream_t s);
// [B][X] -> [B][X-1] (or [X-1][B]) dropping the last column
void launch_drop_bias(const float *in, float *out, int m_batch, int x_size, int out_trans, hipStream_t s);

// ----- pulsed update ---------------------------------------------------------------------------

struct UpdateDev {
  int pulse_type, desired_bl, fixed_bl, update_management, update_bl_management, sto_round;
  float um_grad_scale, res, x_res_implicit, d_res_implicit;
};

struct DeviceDev {
  int kind;
  int ls_mult_noise;
  float dw_min, dw_min_std;
  const float *w_max, *w_min, *scale_up, *scale_down, *slope_up, *slope_down; // [d_size][x_size]
};

struct UpdateArgs {
  float *w; // [d_size][x_size]
  // swapped = 1: the view of a tile that stores [x_size][d_size], for the kernels that work cross-point by cross-point:
  // everything named x here belongs to the tile's d lines and the other way round (sizes, words, planes, line values,
  // inputs), so that "rows" are again what is contiguous in memory.  The kernels that make the lines never see it.
  int swapped;
  int x_size, d_size, m_batch;
  // The stochastic pulse loop on a tile that stores [x_size][d_size]: it walks a row-major copy of the weights (w) with
  // the tile's row-major parameter copies and stores cross-point (i, j) to w_out[i * wo_si + j * wo_sj], the tile's own
  // matrix.  The copy is made from wt_src ([x_size][d_size]) by extra workgroups of the kernel that makes the pulse
  // trains, or by launch_transpose.  All null / zero on a row-major tile: the loop then stores to w in place.
  float *w_out;
  long wo_si, wo_sj;
  const float *wt_src;
  const float *x;
  long x_sb, x_sj; // x element (b, j) at x[b * x_sb + j * x_sj]
  const float *d;
  long d_sb, d_si;
  // Lines read in place from the image tensors of the indexed interface (all zero / null otherwise; only the kernels
  // that make the lines look at these).  x_index set: sample b is patch b % x_group of image b / x_group, the images
  // are x_gs apart in x, and element j of the sample is what x_index[(b % x_group) * x_size + j] names: 0, 1 (bias)
  // or, from 2 on, element idx - 2 of the image.  d_group > 0: element (b, i) of d is at
  // d[(b / d_group) * d_gs + (b % d_group) * d_sb + i * d_si] (the [image][output][patch] tensor of a convolution).
  const int *x_index;
  const int *x_index_lines; // the same index line-major, [x_size][x_group], for kernels with their lanes along the samples
  int x_group;
  long x_gs;
  int d_group;
  long d_gs;
  float lr;
  UpdateDev up;
  DeviceDev dev;
  // per-call scratch
  int *bl;       // [B] bit-line length per sample
  float *prob_a; // [B] probability scale of d
  float *prob_b; // [B] probability scale of x
  uint32_t *x_words; // [B][X] packed pulse words
  uint32_t *d_words; // [B][D]
  // bit lines beyond 31 pulses: a sample takes words_per_sample consecutive rows of words (and bit positions in the
  // planes); m_batch then counts those rows, bl / prob_a / prob_b / x / d stay per sample (row r belongs to sample
  // r / words_per_sample and holds its pulse slots 31 (r % words_per_sample) + 1 ..).  0 or 1: one row per sample.
  int words_per_sample;
  // sample-transposed pulse bits: plane (chunk c, slot k) of line element e is the 32-bit word whose bit q
  // is pulse slot k of sample 32 c + q; element (c, k, e) at planes[(c * plane_slots + k) * size + e];
  // slot plane_slots - 1 holds the sign bits (bit 0 of the packed words)
  uint32_t *x_planes;
  uint32_t *d_planes;
  int plane_slots; // slots per chunk the plane buffers are laid out for
  int n_chunks;    // ceil(m_batch / 32)
  int *row_cost;   // [d_size] work of the pulse loop on each d row of this call (zeroed by the prepare kernel, summed by
                   // the kernel that makes the d pulse trains); null: not kept
  int *kmax;       // kmax[0..1]: largest BL of a batch (ping-pong by call), kmax[2]: constant 31, kmax[3]: longest line
                   // among pulse words made elsewhere (launch_words_kmax)
  int kmax_slot;   // which entry this call uses
  float *x_val;  // [B][X] implicit line values
  float *d_val;  // [B][D]
  PhiloxKey key;
  uint32_t call;
};

// Several tiles in one launch of an update kernel: args[t] in HBM, start[t] .. start[t + 1] the workgroups (blockIdx.x)
// of tile t in the launch at hand (each kernel has its own table); all tiles share m_batch.
struct UpdateGroup {
  const UpdateArgs *args;
  const int *start; // [n + 1]; unused by the set-up kernel
  int n;
  int m_batch;
};
void launch_update_prepare_group(const UpdateGroup &g, hipStream_t s);
// wide: 16 line elements per workgroup (else 4); total_blocks: sum of the tiles' element blocks; rows of words = m_batch
void launch_update_lines_group(const UpdateGroup &g, bool wide, int total_blocks, hipStream_t s);
int update_lines_blocks(const UpdateArgs &a, bool wide);
// the tiles must agree in what update_pulsed_variant returns; total_workgroups: sum of update_pulsed_workgroups
int update_pulsed_variant(const UpdateArgs &a);
bool update_reads_row_cost(const UpdateArgs &a); // by its shape: whether the pulse loop of this call looks at row_cost
int update_pulsed_workgroups(const UpdateArgs &a);
void launch_update_pulsed_group(const UpdateGroup &g, int variant, int total_workgroups, hipStream_t s);

// tables of the update kernels on the current device (once per GPU; blocking copy, no allocation)
void ensure_update_tables();
void launch_update_prepare(const UpdateArgs &a, hipStream_t s);       // BL, A, B per sample
void launch_update_lines(const UpdateArgs &a, hipStream_t s);         // stochastic pulse words and their bit planes
void launch_update_implicit_lines(const UpdateArgs &a, hipStream_t s); // deterministic line values
void launch_update_planes(const UpdateArgs &a, hipStream_t s);        // bit planes of pulse words made elsewhere
void launch_words_kmax(const UpdateArgs &a, hipStream_t s);           // a.kmax[a.kmax_slot] = longest bit line among such words
void launch_update_pulsed(const UpdateArgs &a, hipStream_t s);        // coincidences + device steps
// opt-in variant for LinearStep devices with multiplicative noise: per group of samples_per_step samples the
// coincidences are counted and applied in closed form with one normal draw for their summed noise
void launch_update_aggregated(const UpdateArgs &a, int samples_per_step, hipStream_t s);
void launch_update_implicit(const UpdateArgs &a, hipStream_t s);
// the swapped view of a call's arguments (UpdateArgs::swapped)
UpdateArgs update_swapped_view(const UpdateArgs &a);
void launch_implicit_counts(const UpdateArgs &a, int32_t *counts, hipStream_t s);
// after an update of the persistent weights: w_apparent = w_persistent + noise_std * N(0, 1) at every cross-point that
// took a pulse (from the planes / line values of that update)
void launch_write_noise_touched(const UpdateArgs &a, float *w_apparent, const float *w_persistent, float noise_std,
                                bool implicit, hipStream_t s);
// the same at every cross-point (after weight maintenance and set_weights)
void launch_write_noise_all(float *w_apparent, const float *w_persistent, float noise_std, PhiloxKey key, uint32_t call,
                            size_t n, hipStream_t s);
// floating-point update with the device bounds applied after every sample (x, d, strides, lr, w, dev.w_min / w_max)
void launch_update_fp_clipped(const UpdateArgs &a, hipStream_t s);
// How the cross-point arrays of a tile are stored: element (row i of d, column j of x) at i * x_size + j (xd = 0) or at
// j * d_size + i (xd = 1, the layout of the reference's CUDA tiles).  Kernels that work element by element do not
// care; those with rows or columns in their meaning take this.
struct MatLayout {
  int x_size, d_size, xd;
  __host__ __device__ size_t size() const { return (size_t)x_size * (size_t)d_size; }
  __host__ __device__ size_t at(int i, int j) const {
    return xd ? (size_t)j * (size_t)d_size + (size_t)i : (size_t)i * (size_t)x_size + (size_t)j;
  }
  __host__ __device__ int col_of(size_t idx) const { return xd ? (int)(idx / (size_t)d_size) : (int)(idx % (size_t)x_size); }
  __host__ __device__ int row_of(size_t idx) const { return xd ? (int)(idx % (size_t)d_size) : (int)(idx / (size_t)x_size); }
};
// ----- weight maintenance between steps (kernels_state.hip); w_min / w_max may be null (no device bounds)
void launch_decay_device(float *w, const float *decay_scale, const float *reset_bias, const float *w_min,
                         const float *w_max, float alpha, int bias_no_decay, const MatLayout &lay, hipStream_t s);
void launch_decay_scalar(float *w, float scale, int bias_no_decay, const MatLayout &lay, hipStream_t s);
// rates == null: the same rate for every element
void launch_diffuse(float *w, const float *rates, float rate, const float *w_min, const float *w_max, PhiloxKey key,
                    uint32_t call, size_t n, hipStream_t s);
// clip to +- clip (clip < 0: bounds only); clip_dev != null: the value is read from device memory and a value
// that is not positive leaves the weights alone
void launch_clip_value(float *w, const float *w_min, const float *w_max, float clip, const float *clip_dev, size_t n,
                       hipStream_t s);
void launch_clip_value_gaussian(const float *w, size_t n, float sigma, float fixed_value, float *clip_out, hipStream_t s);
void launch_clip_value_channel(const float *w, const MatLayout &lay, float fixed_value, float *row_max, float *clip_out,
                               hipStream_t s);
void launch_reset_cols(float *w, const float *reset_bias, const float *w_min, const float *w_max, float reset_std,
                       int start_col, int n_cols, float reset_prob, const MatLayout &lay, PhiloxKey key, uint32_t call,
                       hipStream_t s);
// prev_w_and_delta holds the weights from before an update: it becomes scale * (w - previous), w gets them back
void launch_delta_finish(float *w, float *prev_w_and_delta, float scale, size_t n, hipStream_t s);
// out[c][r] = in[r][c] for a row-major [rows][cols] matrix
void launch_transpose(const float *in, float *out, int rows, int cols, hipStream_t s);

// power-law drift of every weight that has stayed within reset_tol of its value after the last call
// (WeightDrifter::apply, weight_drifter.cpp:108-150); nu == null: the same nu0 for every element
struct DriftDev {
  float nu0, nu_std, wg_ratio, g_offset, w_offset, nu_k, log_g0, reset_tol, w_read_std;
  float a; // g_offset * wg_ratio + w_offset, zero when within reset_tol of zero
};
void launch_device_drift(float *w, float *prev, float *w0, float *t, const float *nu, const float *w_min,
                         const float *w_max, const DriftDev &p, float current_t, PhiloxKey key, uint32_t call, size_t n,
                         hipStream_t s);

// per-row statistic of the first n_cols columns: largest absolute value, or sum of squares
void launch_row_stat(const float *w, const MatLayout &lay, int n_cols, int sum_squares, float *row_out, hipStream_t s);
// out[0] = largest of v[0..n-1] when positive, else 1
void launch_max_or_one(const float *v, int n, float *out, hipStream_t s);
// WeightRemapper::apply (weight_remapper.cpp:19-190): from the row statistic in row_stat the per-row factors
// mul / div and the new scales; then w[i][j] = w[i][j] * mul[i] / div[i]
struct RemapDev {
  int type, clip_if;
  float max_scale_range, max_scale_ref, row_norm, remapped_wmax;
};
void launch_remap(float *w, float *scales, float *row_stat, float *mul, float *div, const MatLayout &lay,
                  const RemapDev &p, hipStream_t s);

// WeightModifier::apply (weight_modifier.cpp:28-224): out = modified copy of w; amax_dev == null: assumed_wmax
struct ModifierDev {
  int type, sto_round, copy_last_column, n_coeffs;
  float std_dev, res, dorefa_clip, pdrop, g_max, assumed_wmax;
  float coeffs[8];
};
void launch_modify(float *out, const float *w, const ModifierDev &p, const float *amax_dev, PhiloxKey key, uint32_t call,
                   const MatLayout &lay, hipStream_t s);

// adds the coincidences of the batch to the per-cross-point counters: pos where the signs of x and d agree,
// neg where they differ (kernelPulseCounter, cuda/pwu_kernel.h:1523-1627); implicit: from the line values
void launch_count_pulses(const UpdateArgs &a, unsigned long long *pos, unsigned long long *neg, bool implicit,
                         hipStream_t s);

// clip weights into [w_min, w_max]
void launch_clip(float *w, const float *w_min, const float *w_max, size_t n, hipStream_t s);

// ---- inference weight pipeline (kernels_inference.hip) ------------------------------------------
struct PcmDev {
  float g_max, g_min, prog_noise_scale, read_noise_scale, drift_scale;
  float c0, c1, c2, sig_scale; // programming-noise polynomial and g_max / prog_coeff_g_max_reference
  float drift_base_log2;       // log2(t / t_0) when t > t_0, else 0 (no drift)
  float read_sigma;            // sqrt(ln((t + t_read) / (2 t_read))) when t > 0, else < 0 (no read noise)
};
// abs_max_bits[0] = bits of max |w| (non-negative floats order like their bit patterns)
void launch_abs_max(const float *w, size_t n, uint32_t *abs_max_bits, hipStream_t s);
void launch_pcm_program(const float *w_ref, float *w_prog, float *nu_plus, float *nu_minus, size_t n,
                        const uint32_t *abs_max_bits, const PcmDev &p, PhiloxKey key, uint32_t call, hipStream_t s);
void launch_pcm_drift(const float *w_prog, const float *nu_plus, const float *nu_minus, float *w_out, size_t n,
                      const uint32_t *abs_max_bits, const PcmDev &p, PhiloxKey key, uint32_t call, hipStream_t s);
// out[0] = mean |v| over n values, one workgroup, fixed summation order
void launch_mean_abs(const float *v, size_t n, float *out, hipStream_t s);

// ---- indexed (convolution) interface: RPUSimple::copyIndexedInput / copyIndexedOutput / permute132 with
// trans = true (rpu.cpp:1017-1115, math_util.cpp:319-346).  The caller's index is [x_size][patches]: 0 = padding
// zero, 1 = bias one, j >= 2 = element j - 2 of the image; images are `image_size` apart.
// x_mat[(n * patches + p) * x_ld + k] = value of patch p of image n (x_ld >= x_size: rows may be padded so that they
// start on cache lines)
void launch_gather_indexed(float *x_mat, const float *images, const int *indices, int x_size, int x_ld, int patches,
                           int n_images, long image_size, hipStream_t s);
// images[(j - 2) + n * image_size] = sum of the patch entries gathered from that element, without atomics and in the
// reference's order.  Here x_mat is line-major, [x_size][n_images * patches]; ptr [image_size + 1] and kp list, per
// image element, the pairs (k, p) of the entries gathered from it (every image element is written; no zeroing before)
void launch_fold_indexed(float *images, const float *x_mat, const int *ptr, const int *kp, int x_size, int patches,
                         int n_images, long image_size, hipStream_t s);
// [n][line][p] <-> [line][(n, p)]: what a contraction call reads or writes with its transposed layouts
void launch_images_to_lines(float *lines_major, const float *images, int n_images, int lines, int patches, hipStream_t s);
void launch_lines_to_images(float *images, const float *lines_major, int n_images, int lines, int patches, hipStream_t s);
// [n][d][p] -> [(n, p)][d]
void launch_ndp_to_bd(float *bd, const float *ndp, int n_images, int d_size, int patches, hipStream_t s);
void launch_fill(float *p, float value, size_t n, hipStream_t s);

// n_vec unit vectors of length `size`: row v is e_((start + v) % size)
void launch_unit_vectors(float *out, int n_vec, int size, int start, hipStream_t s);

// out = sum_k gamma[k] * w[k], k < n (VectorRPUDevice::reduceToWeights, rpu_vector_device.cpp:530-536)
struct ReduceArgs {
  const float *w[RPU_MAX_VECTOR_DEVICES];
  float gamma[RPU_MAX_VECTOR_DEVICES];
  int n;
};
void launch_reduce_weights(float *out, const ReduceArgs &r, size_t size, hipStream_t s);

} // namespace rpu_amd
