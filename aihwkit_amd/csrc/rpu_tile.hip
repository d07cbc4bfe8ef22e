// The analog tile object behind the C ABI: host-side state (parameters, sampled device arrays,
// weights) plus, once moved to a GPU, the HBM-resident weights / per-device parameters and the scratch
// buffers of the kernels.  It plays the role of the reference's RPUPulsed (src/rpucuda/rpu_pulsed.{h,cpp})
// and RPUCudaPulsed (src/rpucuda/cuda/rpucuda_pulsed.{h,cu}) pair.
#include "../../include/rpu_amd.h"
#include "kernels.h"
#include "rpu_host.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <memory>
#include <cstdlib>
#include <mutex>
#include <random>
#include <string>
#include <vector>

// Scratch of rpu_tile_update_noalloc, the entry point for callers that cannot allocate: one array per GPU the
// library runs on, held until the process ends.  Host code never uses the array's name as an address: the device
// address is looked up once per device (noalloc_scratch) and only that pointer is passed on.
static __device__ __align__(256) unsigned char scratch[RPU_NOALLOC_MAX_SCRATCH_BYTES];

namespace rpu_amd {

#define RPU_HIP_CHECK(expr)                                                                         \
  do {                                                                                              \
    hipError_t _e = (expr);                                                                         \
    if (_e != hipSuccess) {                                                                         \
      throw RpuError(std::string("HIP error: ") + hipGetErrorString(_e) + " in " #expr);            \
    }                                                                                               \
  } while (0)

namespace {

// device allocations made by the library's buffers so far (rpu_device_allocation_count)
std::atomic<long> g_device_allocations{0};

// Test switch: with RPU_AMD_POISON_NEW_BUFFERS set in the environment every new device buffer of the library is filled
// with 0xff bytes (NaN as a float, -1 as an integer), so that a kernel that reads scratch memory nothing has written
// shows up in the results instead of finding plausible values that an earlier call left there.
static bool poison_new_buffers() {
  static const bool on = std::getenv("RPU_AMD_POISON_NEW_BUFFERS") != nullptr;
  return on;
}

template <typename T> struct DevBuf {
  T *p = nullptr;
  size_t n = 0;
  bool owned = true;
  void ensure(size_t count) {
    if (count <= n) return;
    if (!owned) throw RpuError("A buffer that belongs to the caller cannot grow.");
    release();
    RPU_HIP_CHECK(hipMalloc((void **)&p, count * sizeof(T)));
    g_device_allocations.fetch_add(1, std::memory_order_relaxed);
    n = count;
    if (poison_new_buffers()) RPU_HIP_CHECK(hipMemset(p, 0xff, count * sizeof(T)));
  }
  // use memory of the caller from now on (never freed here)
  void adopt(T *external, size_t count) {
    release();
    p = external;
    n = count;
    owned = false;
  }
  void release() {
    if (p && owned) (void)hipFree(p);
    p = nullptr;
    n = 0;
    owned = true;
  }
};

class DeviceGuard {
public:
  explicit DeviceGuard(int device) {
    RPU_HIP_CHECK(hipGetDevice(&prev_));
    if (device != prev_) {
      RPU_HIP_CHECK(hipSetDevice(device));
      changed_ = true;
    }
  }
  ~DeviceGuard() {
    if (changed_) (void)hipSetDevice(prev_);
  }

private:
  int prev_ = 0;
  bool changed_ = false;
};

__global__ void k_philox_probe(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                               uint32_t *out) {
  const Philox4 r = philox4x32_10(c0, c1, c2, c3, k0, k1);
  out[0] = r.v[0];
  out[1] = r.v[1];
  out[2] = r.v[2];
  out[3] = r.v[3];
}

__global__ void k_init_kmax(int *kmax) {
  if (threadIdx.x < 4) kmax[threadIdx.x] = threadIdx.x == 2 ? 31 : 0;
}

// device address of the static scratch array on the current device, looked up at the first call per device
unsigned char *noalloc_scratch(int device) {
  static std::mutex m;
  static unsigned char *ptr[64] = {};
  if (device < 0 || device >= 64) throw RpuError("Device number out of range for the static scratch array.");
  // every GPU holds its own copy of the array at its own address, and the lookup answers for the current device
  int current = -1;
  RPU_HIP_CHECK(hipGetDevice(&current));
  if (current != device) throw RpuError("The static scratch array is looked up with its device current.");
  std::lock_guard<std::mutex> lock(m);
  if (!ptr[device]) {
    unsigned char *p = nullptr;
    RPU_HIP_CHECK(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
    if (!p) throw RpuError("The static scratch array has no device address.");
    ptr[device] = p;
  }
  return ptr[device];
}

const char *const kHiddenNames[10] = {"max_bound",       "min_bound",  "dwmin_up", "dwmin_down", "decay_scales",
                                      "diffusion_rates", "reset_bias", "drift_nu", "slope_up",   "slope_down"};

} // namespace

// One physical device matrix of a compound: its parameters, sampled arrays and weights.
struct DeviceSlot {
  DevicePar par;
  DeviceArrays arr;
  std::vector<float> w_host; // weights while the tile is not resident on a GPU
  DevBuf<float> d_w, d_wmax, d_wmin, d_sup, d_sdown, d_slup, d_sldown, d_rbias;
  void release() {
    d_w.release(); d_wmax.release(); d_wmin.release(); d_sup.release(); d_sdown.release();
    d_slup.release(); d_sldown.release(); d_rbias.release();
  }
  void clip_host() {
    for (size_t i = 0; i < w_host.size(); ++i) {
      w_host[i] = std::min(w_host[i], arr.w_max[i]);
      w_host[i] = std::max(w_host[i], arr.w_min[i]);
    }
  }
  void upload(size_t n, bool with_weights) {
    const size_t bytes = n * sizeof(float);
    d_rbias.release(); // uploaded again when a transfer resets columns of this device
    d_wmax.ensure(n); d_wmin.ensure(n); d_sup.ensure(n); d_sdown.ensure(n);
    RPU_HIP_CHECK(hipMemcpy(d_wmax.p, arr.w_max.data(), bytes, hipMemcpyHostToDevice));
    RPU_HIP_CHECK(hipMemcpy(d_wmin.p, arr.w_min.data(), bytes, hipMemcpyHostToDevice));
    RPU_HIP_CHECK(hipMemcpy(d_sup.p, arr.scale_up.data(), bytes, hipMemcpyHostToDevice));
    RPU_HIP_CHECK(hipMemcpy(d_sdown.p, arr.scale_down.data(), bytes, hipMemcpyHostToDevice));
    if (par.linear()) {
      d_slup.ensure(n); d_sldown.ensure(n);
      RPU_HIP_CHECK(hipMemcpy(d_slup.p, arr.slope_up.data(), bytes, hipMemcpyHostToDevice));
      RPU_HIP_CHECK(hipMemcpy(d_sldown.p, arr.slope_down.data(), bytes, hipMemcpyHostToDevice));
    }
    if (with_weights) {
      d_w.ensure(n);
      RPU_HIP_CHECK(hipMemcpy(d_w.p, w_host.data(), bytes, hipMemcpyHostToDevice));
    }
  }
};

// what the update kernels need to know about the device matrix they write
struct DeviceView {
  float *w;
  const float *w_max, *w_min, *scale_up, *scale_down, *slope_up, *slope_down;
  const DevicePar *par;
  float granularity; // dw_min used for BL and the pulse probabilities
};

struct Tile {
  int X = 0, D = 0;
  IOPar fio, bio;
  UpdatePar up;
  DevicePar dev;
  DeviceArrays arr;          // host copy of the per-device parameters (never changed by the kernels)
  std::vector<float> w_host; // weights while the tile is not resident on a GPU
  float lr = 0.0f;           // as RPUAbstract: zero until set_learning_rate
  uint64_t seed = 0;
  uint32_t call = 0;
  std::mutex mutex;

  // GPU residency
  int device_id = -1;
  hipStream_t last_stream = nullptr;
  DevBuf<float> d_w, d_wmax, d_wmin, d_sup, d_sdown, d_slup, d_sldown;
  // MVM scratch
  DevBuf<float> s_nsc0, s_nsc1, s_nm, s_nmnp, s_red, s_scale, s_fin, s_bias, s_xq0, s_xq1;
  // rounds 0 and 1 of a forward call in one launch: kept outputs of both, choice per sample, marks of round 1, rows of
  // round 2; the host-visible pair (samples of the last call that needed round 1, its batch) that the choice between
  // the fused and the separate launches is made from (fused_rounds: -1 by those values, 0 never, 1 .. 3 as forced)
  DevBuf<float> s_dual0, s_dual1, s_dual2, s_xq2;
  DevBuf<int> s_dsel, s_dhit1, s_dhit2;
  int *seen_host = nullptr, *seen_dev = nullptr;
  int rest_from = 0, rest_quiet = 0; // the last round that listed samples in the recent calls, and calls since it did
  int fused_rounds = -1;
  // A launch that runs several rounds makes its workgroups wait for each other; a wait that runs out is written to
  // seen_host[3] by the kernel.  The next compute call on the tile reports it (the results of that forward call are
  // invalid) and from then on the tile runs one launch per round.  The hook values shorten the wait and make it expect
  // one arrival too many, for the test of that path.
  bool merged_off = false;
  uint32_t merged_call = 0; // random-stream index of the last forward call that used such a launch
  int wait_spins_hook = 0, wait_extra_hook = 0;
  void check_round_waits() {
    if (!seen_host) return;
    const int failed = *(volatile int *)&seen_host[3];
    if (!failed) return;
    *(volatile int *)&seen_host[3] = 0;
    merged_off = true;
    throw RpuError("forward round barrier timed out in round " + std::to_string(failed - 1) + "; results of call " +
                   std::to_string(merged_call) + " are invalid (the tile now runs one launch per round).");
  }
  int cu_count = 0;
  int n_cus() {
    if (!cu_count) {
      hipDeviceProp_t prop;
      RPU_HIP_CHECK(hipGetDeviceProperties(&prop, device_id));
      cu_count = prop.multiProcessorCount;
    }
    return cu_count;
  }
  DevBuf<int> s_rounds, s_hitup, s_hitlo, s_list0, s_list1, s_row0, s_row1, s_count, s_tiledone;
  // update scratch
  DevBuf<int> u_bl, u_rowcost;
  DevBuf<float> u_a, u_b, u_xval, u_dval;
  DevBuf<uint32_t> u_xw, u_dw, u_xpl, u_dpl;
  DevBuf<int> u_kmax;
  uint32_t update_calls = 0;
  int update_variant = RPU_UPDATE_VARIANT_EXACT, update_variant_samples = 32;
  // where the last pulsed update left its per-sample values and packed words (own buffers or the static scratch)
  int *last_bl = nullptr;
  float *last_a = nullptr, *last_b = nullptr;
  uint32_t *last_xw = nullptr, *last_dw = nullptr;
  int last_words_per_sample = 1;
  // transfer compound (rpu_transfer_device.{h,cpp}): device 0 takes the gradient update, device j is read
  // column by column and written onto device j + 1; the tile's weights d_w are the weighted sum, or the
  // last device itself when that one alone is visible
  std::unique_ptr<TransferPar> tr;
  std::vector<std::unique_ptr<DeviceSlot>> slots;
  uint64_t update_idx = 0;
  std::vector<int> slice_idx;
  DevBuf<float> t_unit, t_read;
  // inference weight pipeline: reference and programmed weights, drift coefficients of both conductances
  DevBuf<float> i_ref, i_prog, i_nu_plus, i_nu_minus, i_scalar;
  DevBuf<uint32_t> i_absmax;
  bool has_reference = false, programmed = false;
  // indexed (convolution) interface: index matrix [X][patches] and the unfolded matrices
  std::vector<int32_t> idx_host;
  int idx_patches = 0;
  int32_t idx_max = 0; // largest entry of the index matrix
  DevBuf<int> x_idx, x_idx_t; // the index matrix as set, [X][patches], and patch-major, [patches][X] (fused forward)
  DevBuf<int> x_fold_ptr, x_fold_off; // per image element the patch entries gathered from it (backward_indexed)
  long fold_image_size = -1;
  DevBuf<float> x_mat, d_mat;
  int last_update_batch = 0;
  int last_update_pulse = -1;
  int last_forward_batch = 0;
  // weight maintenance: per-device decay scales, diffusion rates and reset biases (uploaded at first use),
  // clip value computed on the device, and the caller's buffer that takes the updates instead of the weights
  DevBuf<float> d_decay, d_diff, d_rbias, s_clip;
  bool state_params_valid = false;
  float *delta_w = nullptr;
  // the reference's CUDA tiles exchange shared and delta weights as [x_size][d_size] (column-major) tensors
  // (rpu_base_tiles_cuda.cpp:88-130).  The matrices of this library stay row-major [d_size][x_size]; a caller's
  // column-major tensor is kept in step by transposition: read into the tile before a call that uses the weights,
  // written back after a call that changes them.
  float *shared_xd = nullptr;
  float *delta_xd = nullptr;
  DevBuf<float> d_delta_own;
  // Zero-copy form of the same binding (RPUCudaSimple::setSharedWeights, cuda/rpucuda.cu:322-334): the caller's
  // [x_size][d_size] tensor IS the weight matrix, and every other cross-point array of the tile (device parameters,
  // drift clocks, modified weights, inference arrays) is kept in that layout too, transposed once when the tensor is
  // bound.  The kernels then read the weights with the roles of rows and columns exchanged: forward addresses them as
  // backward does on a row-major tile and the other way round (MvmArgs::w_oc), the update kernels see x and d swapped.
  // Plain tiles take this form; transfer compounds, write noise, pulse counters and the analog terms before the ADC
  // keep the mirror above.
  bool xd = false;
  // The stochastic pulse loop is the exception: it walks the d pulses of a row of W with its lanes along x, which on
  // the usual workloads (inputs denser than errors) takes half the passes of the walk the other way round.  For it
  // the tile keeps the device parameters row-major as well (r_*) and a row-major scratch copy of the weights (u_wrm),
  // filled by workgroups that the launch of the pulse trains carries along; the loop stores its results into the
  // bound tensor directly.
  DevBuf<float> r_wmax, r_wmin, r_sup, r_sdown, r_slup, r_sldown, u_wrm;
  int w_ld() const { return xd ? D : X; } // row length of the stored matrices
  MatLayout layout() const { return MatLayout{X, D, xd ? 1 : 0}; }
  // Host matrices are row-major [D][X] on every interface; the device copies follow the tile's storage.
  void upload_mat(float *dst_dev, const float *src_host) {
    const size_t bytes = size() * sizeof(float);
    if (!xd) {
      RPU_HIP_CHECK(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
      return;
    }
    std::vector<float> t(size());
    for (int i = 0; i < D; ++i)
      for (int j = 0; j < X; ++j) t[(size_t)j * D + i] = src_host[(size_t)i * X + j];
    RPU_HIP_CHECK(hipMemcpy(dst_dev, t.data(), bytes, hipMemcpyHostToDevice));
  }
  void download_mat(float *dst_host, const float *src_dev) const {
    const size_t bytes = size() * sizeof(float);
    if (!xd) {
      RPU_HIP_CHECK(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
      return;
    }
    std::vector<float> t(size());
    RPU_HIP_CHECK(hipMemcpy(t.data(), src_dev, bytes, hipMemcpyDeviceToHost));
    for (int i = 0; i < D; ++i)
      for (int j = 0; j < X; ++j) dst_host[(size_t)i * X + j] = t[(size_t)j * D + i];
  }
  // row-major [D][X] device matrix -> [X][D] in place (through a temporary), on the last stream, waited for
  void to_xd_in_place(DevBuf<float> &b) {
    if (!b.p || b.n < size()) return;
    DevBuf<float> tmp;
    tmp.ensure(size());
    launch_transpose(b.p, tmp.p, D, X, last_stream);
    RPU_HIP_CHECK(hipMemcpyAsync(b.p, tmp.p, size() * sizeof(float), hipMemcpyDeviceToDevice, last_stream));
    RPU_HIP_CHECK(hipStreamSynchronize(last_stream));
    tmp.release();
  }
  // hardware-aware training: the modified copy of the weights that forward / backward contract with, scratch of
  // the remapper ([3 D + 1]: row statistic, multiplier, divisor, one scalar), the drift clock per weight and the
  // pulse counters [2][size]
  DevBuf<float> d_fbw, s_rowstat;
  bool fb_during_test = false;
  // write noise: the persistent weights the pulses and the maintenance act on; d_w then holds the shown weights
  DevBuf<float> d_wp;
  // analog non-idealities before the ADC: the addend per output, up to three side contractions, the transformed
  // input rows, |W| and the squared row norms
  DevBuf<float> n_pre, n_s1, n_s2, n_s3, n_s4, n_rows, n_absw, n_sumsq, n_xsum, n_part, n_neg;
  DevBuf<int> n_neghit; // [2][B] saturation marks of the negative pass (PosNegSeparateDigitalSum)
  DevBuf<int> n_rowsample; // [B] sample of every row of a later round (SideDev::row_sample)
  // per direction: voltage offsets, non-linearity coefficients, output noise levels, read-asymmetry factors
  // per-line values on the device: of the forward IO, the backward IO and the IO of a transfer compound's read
  DevBuf<float> d_line[3][4];
  bool line_valid[3][4] = {{false, false, false, false}, {false, false, false, false}, {false, false, false, false}};
  int line_set = -1; // 2 while the read of a transfer runs (pre_adc_terms then takes that IO's lines), else by direction
  DevBuf<float> n_wneg, n_absneg; // weights of the negative pass with read asymmetry, and their absolute values
  // running AverageAbsMax noise-management scale, one value shared by forward and backward as in the reference
  // (rpu_forward_backward_pass.h:241); negative: not started
  DevBuf<float> nm_aux;
  float nm_aux_host = -1.0f; // its value while no device copy exists, and what extra state reads / writes
  DevBuf<float> dr_prev, dr_w0, dr_t, d_nu;
  float drift_t = 0.0f;
  bool nu_valid = false;
  DevBuf<unsigned long long> d_cnt;

  // optional per-kernel timing with HIP events on the launch stream
  bool profiling = false;
  std::vector<hipEvent_t> prof_events;
  std::vector<const char *> prof_names;
  size_t prof_used = 0;

  void prof_begin(hipStream_t s) {
    if (!profiling) return;
    prof_used = 0;
    prof_names.clear();
    prof_mark(s, nullptr);
    // an empty bracket first: what two consecutive event records cost on this stream, for callers that want
    // to take the bracket's own time out of the kernel figures
    prof_mark(s, "_bracket");
  }
  void prof_mark(hipStream_t s, const char *name) {
    if (!profiling) return;
    if (prof_used == prof_events.size()) {
      hipEvent_t e;
      RPU_HIP_CHECK(hipEventCreate(&e));
      prof_events.push_back(e);
    }
    RPU_HIP_CHECK(hipEventRecord(prof_events[prof_used++], s));
    if (name) prof_names.push_back(name);
  }

  bool resident() const { return device_id >= 0; }
  bool is_transfer() const { return tr != nullptr; }
  // the matrix forward / backward contract with
  float *wdev() { return (tr && tr->fully_hidden) ? slots.back()->d_w.p : d_w.p; }
  bool persistent() const { return !tr && dev.persistent_weights(); }
  // the matrix that pulses and weight maintenance change
  float *wp_dev() { return persistent() ? d_wp.p : d_w.p; }
  // PulsedRPUDevice::applyUpdateWriteNoise (rpu_pulsed_device.cpp:573-588): all shown weights are redrawn
  void refresh_shown_weights(hipStream_t s) {
    if (!persistent()) return;
    launch_write_noise_all(d_w.p, d_wp.p, dev.scaled_write_noise(), key(), call++, size(), s);
  }

  // RPUSimple::getFBWeights (rpu.cpp:1483-1487): once modified weights exist, forward and backward use them,
  // during evaluation only if the modifier asked for it
  const float *mvm_weights(bool is_test) {
    return (d_fbw.p && (!is_test || fb_during_test)) ? d_fbw.p : wdev();
  }
  size_t size() const { return (size_t)X * (size_t)D; }

  ~Tile() {
    if (resident()) {
      try {
        DeviceGuard g(device_id);
        (void)hipDeviceSynchronize();
        for (hipEvent_t e : prof_events) (void)hipEventDestroy(e);
        release_all();
      } catch (...) {
      }
    }
  }

  void release_all() {
    d_w.release(); d_wmax.release(); d_wmin.release(); d_sup.release(); d_sdown.release();
    d_slup.release(); d_sldown.release();
    s_dual0.release(); s_dual1.release(); s_dual2.release(); s_xq2.release(); s_dsel.release(); s_dhit1.release();
    s_dhit2.release();
    if (seen_host) {
      (void)hipHostFree(seen_host);
      seen_host = seen_dev = nullptr;
    }
    s_nsc0.release(); s_nsc1.release(); s_nm.release(); s_nmnp.release(); s_red.release(); s_scale.release(); s_fin.release(); s_bias.release(); s_xq0.release(); s_xq1.release();
    s_rounds.release(); s_hitup.release(); s_hitlo.release(); s_list0.release(); s_list1.release(); s_row0.release(); s_row1.release(); s_count.release(); s_tiledone.release();
    u_rowcost.release();
    u_bl.release(); u_a.release(); u_b.release(); u_xval.release(); u_dval.release(); u_xw.release(); u_dw.release();
    u_xpl.release(); u_dpl.release(); u_kmax.release();
    r_wmax.release(); r_wmin.release(); r_sup.release(); r_sdown.release(); r_slup.release(); r_sldown.release(); u_wrm.release();
    last_bl = nullptr; last_a = last_b = nullptr; last_xw = last_dw = nullptr;
    t_unit.release(); t_read.release();
    i_ref.release(); i_prog.release(); i_nu_plus.release(); i_nu_minus.release(); i_scalar.release(); i_absmax.release();
    has_reference = programmed = false;
    x_idx.release(); x_idx_t.release(); x_fold_ptr.release(); x_fold_off.release(); fold_image_size = -1;
    x_mat.release(); d_mat.release();
    d_decay.release(); d_diff.release(); d_rbias.release(); s_clip.release();
    state_params_valid = false;
    delta_w = nullptr;
    shared_xd = nullptr;
    delta_xd = nullptr;
    xd = false;
    d_delta_own.release();
    n_pre.release(); n_s1.release(); n_s2.release(); n_s3.release(); n_rows.release(); n_absw.release();
    n_sumsq.release();
    n_s4.release();
    n_xsum.release();
    n_part.release();
    n_neg.release();
    n_neghit.release();
    n_rowsample.release();
    n_wneg.release();
    n_absneg.release();
    for (auto &dir : d_line) for (auto &b : dir) b.release();
    for (auto &dir : line_valid) for (bool &v : dir) v = false;
    nm_aux.release();
    d_wp.release();
    d_fbw.release(); s_rowstat.release(); dr_prev.release(); dr_w0.release(); dr_t.release(); d_nu.release();
    d_cnt.release();
    fb_during_test = false;
    drift_t = 0.0f;
    nu_valid = false;
    for (auto &sl : slots) sl->release();
  }

  // brings nm_aux_host and the device copy in line (to_host: before the value is read on the host)
  void sync_nm_aux(bool to_host) {
    if (!resident() || !nm_aux.p) return;
    if (to_host) {
      sync_last();
      RPU_HIP_CHECK(hipMemcpy(&nm_aux_host, nm_aux.p, sizeof(float), hipMemcpyDeviceToHost));
    } else {
      sync_last();
      RPU_HIP_CHECK(hipMemcpy(nm_aux.p, &nm_aux_host, sizeof(float), hipMemcpyHostToDevice));
    }
  }

  PhiloxKey key() const {
    PhiloxKey k;
    k.k0 = (uint32_t)(seed & 0xffffffffu);
    k.k1 = (uint32_t)(seed >> 32);
    return k;
  }

  void clip_host(std::vector<float> &w) const {
    if (!dev.pulsed()) return;
    for (size_t i = 0; i < w.size(); ++i) {
      w[i] = std::min(w[i], arr.w_max[i]);
      w[i] = std::max(w[i], arr.w_min[i]);
    }
  }

  void upload_params() {
    state_params_valid = false;
    nu_valid = false;
    if (!dev.pulsed()) return;
    const size_t n = size(), bytes = n * sizeof(float);
    d_wmax.ensure(n); d_wmin.ensure(n); d_sup.ensure(n); d_sdown.ensure(n);
    upload_mat(d_wmax.p, arr.w_max.data());
    upload_mat(d_wmin.p, arr.w_min.data());
    upload_mat(d_sup.p, arr.scale_up.data());
    upload_mat(d_sdown.p, arr.scale_down.data());
    if (dev.linear()) {
      d_slup.ensure(n); d_sldown.ensure(n);
      upload_mat(d_slup.p, arr.slope_up.data());
      upload_mat(d_sldown.p, arr.slope_down.data());
    }
    if (xd) { // the row-major copies of the pulse loop
      r_wmax.ensure(n); r_wmin.ensure(n); r_sup.ensure(n); r_sdown.ensure(n);
      RPU_HIP_CHECK(hipMemcpy(r_wmax.p, arr.w_max.data(), bytes, hipMemcpyHostToDevice));
      RPU_HIP_CHECK(hipMemcpy(r_wmin.p, arr.w_min.data(), bytes, hipMemcpyHostToDevice));
      RPU_HIP_CHECK(hipMemcpy(r_sup.p, arr.scale_up.data(), bytes, hipMemcpyHostToDevice));
      RPU_HIP_CHECK(hipMemcpy(r_sdown.p, arr.scale_down.data(), bytes, hipMemcpyHostToDevice));
      if (dev.linear()) {
        r_slup.ensure(n); r_sldown.ensure(n);
        RPU_HIP_CHECK(hipMemcpy(r_slup.p, arr.slope_up.data(), bytes, hipMemcpyHostToDevice));
        RPU_HIP_CHECK(hipMemcpy(r_sldown.p, arr.slope_down.data(), bytes, hipMemcpyHostToDevice));
      }
    }
  }

  void to_device(int dev_id) {
    if (resident()) throw RpuError("Tile is already resident on a GPU.");
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
      throw RpuError("No HIP device available: this library has no CPU compute path.");
    }
    int target = dev_id;
    if (target < 0) RPU_HIP_CHECK(hipGetDevice(&target));
    if (target >= count) throw RpuError("Invalid HIP device id.");
    DeviceGuard g(target);
    device_id = target;
    cu_count = 0;
    try {
      if (is_transfer()) {
        for (auto &sl : slots) sl->upload(size(), true);
        if (!tr->fully_hidden) {
          d_w.ensure(size());
          RPU_HIP_CHECK(hipMemcpy(d_w.p, w_host.data(), size() * sizeof(float), hipMemcpyHostToDevice));
        }
      } else {
        d_w.ensure(size());
        RPU_HIP_CHECK(hipMemcpy(d_w.p, w_host.data(), size() * sizeof(float), hipMemcpyHostToDevice));
        if (persistent()) {
          if (arr.persistent.size() != size()) arr.persistent = w_host;
          d_wp.ensure(size());
          RPU_HIP_CHECK(hipMemcpy(d_wp.p, arr.persistent.data(), size() * sizeof(float), hipMemcpyHostToDevice));
        }
        upload_params();
      }
      s_count.ensure(MVM_COUNT_WORDS);
      ensure_update_tables();
    } catch (...) {
      release_all();
      device_id = -1;
      throw;
    }
  }

  void sync_last() {
    RPU_HIP_CHECK(hipStreamSynchronize(last_stream));
  }

  void ensure_mvm_scratch(int B) {
    const size_t n = (size_t)B;
    s_nsc0.ensure(n); s_nsc1.ensure(n); s_nm.ensure(n); s_nmnp.ensure(n); s_red.ensure(n); s_scale.ensure(n); s_fin.ensure(n);
    s_rounds.ensure(n); s_hitup.ensure(n); s_hitlo.ensure(n); s_list0.ensure(n); s_list1.ensure(n); s_row0.ensure(n); s_row1.ensure(n);
    s_count.ensure(MVM_COUNT_WORDS);
    s_tiledone.ensure((size_t)32 * ((n + 31) / 32));
  }

  IoDev io_dev(const IOPar &io) const {
    IoDev d;
    d.inp_res = io.p.inp_res; d.inp_bound = io.p.inp_bound; d.inp_noise = io.p.inp_noise; d.inp_asym = io.p.inp_asymmetry;
    d.out_res = io.p.out_res; d.out_bound = io.p.out_bound; d.out_noise = io.p.out_noise; d.out_asym = io.p.out_asymmetry;
    d.out_scale = io.p.out_scale; d.nm_thres = io.p.nm_thres; d.nm_assumed_wmax = io.p.nm_assumed_wmax;
    d.max_bm_res = io.p.max_bm_res; d.noise_management = io.p.noise_management;
    d.bound_management = io.p.bound_management; d.bm_test_negative_bound = io.p.bm_test_negative_bound;
    d.max_bm_factor = io.p.max_bm_factor; d.inp_sto_round = io.p.inp_sto_round; d.out_sto_round = io.p.out_sto_round;
    d.perfect = io.perfect ? 1 : 0;
    return d;
  }

  // false: an empty batch, nothing to do (the reference's loops over the samples run zero times; pointers of an empty
  // tensor may be null)
  bool check_compute(int m_batch, const void *p0, const void *p1) {
    if (!resident()) throw RpuError("Tile is not resident on a GPU: forward / backward / update need rpu_tile_to_device first.");
    check_round_waits();
    if (m_batch < 0) throw RpuError("m_batch must not be negative.");
    if (m_batch == 0) return false;
    if (!p0 || !p1) throw RpuError("Null device pointer.");
    return true;
  }

  // shared driver of forward (transposed = 0) and backward (transposed = 1)
  // arguments of the MVM kernels for one call, scratch sized for B samples; the caller sets in / out
  MvmArgs mvm_args(int B, bool transposed, const float *w_other, const IOPar &io, int large_tiles = -1) {
    const int K = transposed ? D : X;
    const int O = transposed ? X : D;
    ensure_mvm_scratch(B);
    MvmArgs a{};
    a.x_size = X; a.d_size = D; a.m_batch = B; a.K = K; a.O = O;
    a.transposed = transposed ? 1 : 0;
    mvm_set_weights(a, w_other ? w_other : wdev(), w_ld(), xd);
    a.io = io_dev(io);
    a.alpha = io.p.out_scale; a.beta = 0.0f;
    a.key = key(); a.call = call++;
    a.st.next_scale[0] = s_nsc0.p; a.st.next_scale[1] = s_nsc1.p;
    a.st.nm = s_nm.p; a.st.nm_np = s_nmnp.p; a.st.red = s_red.p; a.st.scale = s_scale.p; a.st.fin = s_fin.p;
    a.st.rounds = s_rounds.p; a.st.hit_up = s_hitup.p; a.st.hit_lo = s_hitlo.p;
    a.st.list[0] = s_list0.p; a.st.list[1] = s_list1.p; a.st.row[0] = s_row0.p; a.st.row[1] = s_row1.p;
    a.st.count = s_count.p;
    a.st.tile_done = s_tiledone.p;
    // large_tiles: whether rounds of this call run on the large-tile kernel (-1: what the shape alone decides)
    const bool tight = large_tiles < 0 ? mvm_uses_large_tiles(B, O) : large_tiles != 0;
    a.k_pad = mvm_k_pad(K, tight);
    s_xq0.ensure((size_t)B * a.k_pad);
    if (!io.perfect && io.p.bound_management != RPU_BM_NONE) s_xq1.ensure((size_t)B * a.k_pad);
    a.xq[0] = s_xq0.p; a.xq[1] = s_xq1.p;
    a.max_rounds = io.perfect ? 0 : mvm_max_rounds(a.io);
    // rows for the next bound-management round are quantized ahead when the batch is small (shortest path between
    // rounds) or when at least four workgroups per sample tile share that work; a large batch on a narrow tile
    // quantizes only the rows of the samples that saturated
    a.speculate = mvm_speculates(B, O) ? 1 : 0;
    a.rows_ahead_in_init = a.speculate;
    return a;
  }
  static bool mvm_speculates(int B, int O) { return B <= 1024 || O > 96; }

  // whether a pass with these IO parameters has non-idealities that add to the sums before the ADC
  static bool has_pre_adc_terms(const IOPar &io) {
    return !io.perfect && ((io.p.w_noise_type != 0 && io.p.w_noise > 0.0f) || io.p.ir_drop > 0.0f || io.has_line_terms());
  }

  // per-line values of both directions; a fixed construction seed fixes them too
  void populate_lines(unsigned int construction_seed) {
    fio.populate_lines(D, construction_seed ? construction_seed * 2654435761u + 1u : 0u, size());
    bio.populate_lines(X, construction_seed ? construction_seed * 2654435761u + 2u : 0u, size());
  }

  // device copies of the per-line values of a direction (0 forward, 1 backward, 2 the read of a transfer)
  const float *line_values(int dir, int which, const std::vector<float> &host) {
    if (host.empty()) return nullptr;
    DevBuf<float> &buf = d_line[dir][which];
    if (!line_valid[dir][which]) {
      buf.ensure(host.size());
      RPU_HIP_CHECK(hipMemcpy(buf.p, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
      line_valid[dir][which] = true;
    }
    return buf.p;
  }

  // The addend of every output of round a.round from the quantized inputs of that round: weight noise and IR drop
  // (ForwardBackwardPassIOManaged::applyNonIdealities, rpu_forward_backward_pass.cpp:535-560).  The extra
  // contractions run on the round kernel without its ADC stage; rounds that list no sample do nothing.
  void pre_adc_terms(MvmArgs &a, const IOPar &io, hipStream_t s) {
    const int B = a.m_batch, r = a.round;
    const size_t out_n = (size_t)B * a.O, row_n = (size_t)B * a.k_pad;
    const int *skip = r > 0 ? a.st.count + r : nullptr;
    const float *xq = a.xq[r & 1];
    const bool noisy = io.p.w_noise_type != 0 && io.p.w_noise > 0.0f;
    const bool ir = io.p.ir_drop > 0.0f;
    const bool need_abs = ir || (noisy && io.p.w_noise_type == 2);
    const bool total = io.has_line_terms();
    n_pre.ensure(out_n);
    n_rows.ensure(row_n);
    if (need_abs && r == 0) {
      n_absw.ensure(size());
      launch_abs_copy(a.w, n_absw.p, size(), s);
    }
    // PosNegSeparate: the negative and the positive inputs see the array one after the other, each pass with its
    // own IR drop, offsets and weight noise; the sums of both go through the ADC (rpu_forward_backward_pass.cpp:832-893)
    // a later round keeps its samples in rows handed out in the order in which the round before finished them
    const int *row_sample = nullptr;
    if (r > 0) {
      if (n_rowsample.n < (size_t)B) {
        n_rowsample.ensure((size_t)B);
        launch_fill(reinterpret_cast<float *>(n_rowsample.p), 0.0f, (size_t)B, s); // rows without a sample: any valid key
      }
      launch_side_row_samples(n_rowsample.p, a.st.list[r & 1], a.st.row[r & 1], a.st.count + r, B, s);
      row_sample = n_rowsample.p;
    }
    const bool separate = io.separate_passes();
    for (int pass = 0; pass < (separate ? 2 : 1); ++pass) {
      const int part = separate ? (pass == 0 ? -1 : 1) : 0;
      // the negative pass reads every weight through its own asymmetry factor (rpu_forward_backward_pass.cpp:845-856)
      const float *w_pass = a.w, *absw_pass = n_absw.p;
      if (part < 0 && io.p.w_read_asymmetry_dtod > 0.0f && !io.w_asymmetry.empty()) {
        if (r == 0) {
          n_wneg.ensure(size());
          launch_mul_copy(a.w, line_values(line_set >= 0 ? line_set : (a.transposed ? 1 : 0), 3, io.w_asymmetry), n_wneg.p, size(), s);
          if (need_abs) {
            n_absneg.ensure(size());
            launch_abs_copy(n_wneg.p, n_absneg.p, size(), s);
          }
        }
        w_pass = n_wneg.p;
        absw_pass = n_absneg.p;
      }
      const float *xin = xq;
      if (part) {
        n_part.ensure(row_n);
        launch_side_rows(xq, n_part.p, B, a.k_pad, a.K, 3, part, skip, s);
        xin = n_part.p;
      }
      const auto contract = [&](const float *w, int mode, float *dst) {
        if (mode != 3) launch_side_rows(xin, n_rows.p, B, a.k_pad, a.K, mode, 0, skip, s);
        MvmArgs g{};
        g.x_size = X; g.d_size = D; g.m_batch = B; g.K = a.K; g.O = a.O; g.k_pad = a.k_pad;
        g.transposed = a.transposed;
        mvm_set_weights(g, w, w_ld(), xd);
        g.xq[0] = mode != 3 ? n_rows.p : const_cast<float *>(xin); g.xq[1] = nullptr;
        g.out = dst; g.out_sb = a.O; g.out_so = 1;
        g.io = a.io; g.io.perfect = 1;
        g.alpha = 1.0f; g.beta = 0.0f; g.round = 0;
        g.key = a.key; g.call = a.call;
        g.small_tiles_only = 1;
        g.skip_if_zero = skip;
        launch_mvm_round(g, s);
      };
      if (noisy && io.p.w_noise_type == 1) {
        n_sumsq.ensure((size_t)B);
        launch_row_stat(xin, MatLayout{a.k_pad, B, 0}, a.K, 1, n_sumsq.p, s);
      } else if (noisy) {
        n_s1.ensure(out_n);
        contract(absw_pass, 0, n_s1.p);
      }
      if (ir) {
        n_s2.ensure(out_n); n_s3.ensure(out_n);
        contract(absw_pass, 1, n_s2.p);
        contract(w_pass, 2, n_s3.p);
      }
      SideDev p{};
      p.row_sample = row_sample;
      p.w_noise_type = noisy ? io.p.w_noise_type : 0;
      p.w_noise = io.p.w_noise; p.ir_drop = ir ? io.p.ir_drop : 0.0f;
      p.a_scale = (float)a.K / io.p.ir_drop_g_ratio;
      if (total) {
        // the value itself is made beside the round kernel, whose ADC stage then only quantizes and clips
        const int dir = line_set >= 0 ? line_set : (a.transposed ? 1 : 0);
        n_s4.ensure(out_n);
        contract(w_pass, 3, n_s4.p);
        p.s_y = n_s4.p;
        if (io.has_voltage_offsets()) {
          p.v_offset = line_values(dir, 0, io.v_offset);
          if (io.p.v_offset_w_min != 0.0f) {
            n_xsum.ensure((size_t)B);
            launch_row_stat(xin, MatLayout{a.k_pad, B, 0}, a.K, 2, n_xsum.p, s);
            p.x_accum = n_xsum.p;
          }
        }
        if (io.has_nl_calibration()) p.out_nl = line_values(dir, 1, io.out_nl);
        p.out_noise = line_values(dir, 2, io.out_noise_values);
        p.r_series = io.p.r_series; p.r_series_max_total = io.p.r_series_max_total;
        p.v_offset_w_min = io.p.v_offset_w_min; p.nl_factor = io.nl_factor;
        p.out_noise_all = io.p.out_noise; p.out_asym = io.p.out_asymmetry;
        a.pre_is_total = 1;
        a.io.out_noise = 0.0f;
        a.io.out_asym = 0.0f;
      }
      float *dst = n_pre.p;
      const bool digital = io.digital_sum();
      if (separate && pass == 0) {
        n_neg.ensure(out_n);
        dst = n_neg.p;
        if (digital) {
          // the pass goes through the ADC stage on its own (rpu_forward_backward_pass.cpp:861-863)
          p.adc_here = 1;
          p.adc_res = a.io.out_res; p.adc_bound = a.io.out_bound; p.adc_sto_round = a.io.out_sto_round;
          if (io.p.bound_management != RPU_BM_NONE) {
            n_neghit.ensure(2 * (size_t)B);
            // every round: the pass also converts rows that no sample of this round uses, whose marks nobody clears
            launch_fill(reinterpret_cast<float *>(n_neghit.p), 0.0f, 2 * (size_t)B, s); // all-zero bits
            p.hit_up = n_neghit.p;
            p.hit_lo = n_neghit.p + B;
          }
        } else {
          p.ni_only = 1;
        }
      } else if (separate && digital) {
        a.post_add = n_neg.p;
        if (io.p.bound_management != RPU_BM_NONE) {
          a.post_hit_up = n_neghit.p;
          a.post_hit_lo = n_neghit.p + B;
        }
      } else if (separate) {
        p.add_ni = n_neg.p;
      }
      // the second pass draws its own noise
      launch_side_combine(dst, n_s1.p, n_sumsq.p, n_s2.p, n_s3.p, p, B, a.O, a.key, a.call, r + 64 * pass, skip, s);
    }
    a.pre_add = n_pre.p;
    prof_mark(s, "pre_adc_terms");
  }

  // Input of a forward call whose samples are the patches of images, read through the index matrix (MvmArgs::in_index):
  // `in` then points to the images
  struct GatherSource {
    const int *index_patch_major; // [patches][X]
    const int *index_line_major;  // [X][patches]
    int patches;                  // per image
    long image_size;
  };

  const GatherSource *lines_in_place = nullptr; // set while update_indexed runs a pulsed update (pulsed_update_args)

  // in_ld: row stride of a plain row-major input with padded rows (0: the rows are dense)
  void mvm(const float *in, float *out, int B, bool bias, bool in_trans, bool out_trans, bool transposed, hipStream_t s,
           const float *w_other = nullptr, const IOPar *io_other = nullptr, bool is_test = false, long in_ld = 0,
           const GatherSource *gather = nullptr, long out_ld = 0) {
    const IOPar &io = io_other ? *io_other : (transposed ? bio : fio);
    const bool side = has_pre_adc_terms(io);
    MvmArgs a = mvm_args(B, transposed, w_other ? w_other : mvm_weights(is_test), io, side ? 0 : -1);
    a.small_tiles_only = side ? 1 : 0;

    // the x side carries the optional bias column: input of forward, output of backward
    float *final_out = out;
    if (!transposed) {
      if (bias) {
        s_bias.ensure((size_t)B * X);
        launch_make_bias(in, s_bias.p, B, X, in_trans ? 1 : 0, s);
        a.in = s_bias.p; a.in_sb = X; a.in_sk = 1;
      } else {
        a.in = in; a.in_sb = in_trans ? 1 : X; a.in_sk = in_trans ? B : 1;
      }
      a.out = out; a.out_sb = out_trans ? 1 : D; a.out_so = out_trans ? B : 1;
    } else {
      a.in = in; a.in_sb = in_trans ? 1 : D; a.in_sk = in_trans ? B : 1;
      if (bias) {
        s_bias.ensure((size_t)B * X);
        a.out = s_bias.p; a.out_sb = X; a.out_so = 1;
      } else {
        a.out = out; a.out_sb = out_trans ? 1 : X; a.out_so = out_trans ? B : 1;
      }
    }

    if (in_ld) { // padded rows of a plain row-major input
      if (in_trans || bias || gather) throw RpuError("A row stride goes with a plain row-major input only.");
      a.in_sb = in_ld;
    }
    if (out_ld) { // padded rows of a plain row-major output
      if (out_trans || bias) throw RpuError("A row stride goes with a plain row-major output only.");
      a.out_sb = out_ld;
    }
    if (gather) { // the samples are patches gathered from the images `in` (see MvmArgs::in_index)
      if (in_trans || bias || transposed || side || gather->patches <= 0) throw RpuError("Gathered input: plain forward calls only.");
      if (a.speculate && a.max_rounds > 1) throw RpuError("Gathered input: not with rows quantized ahead.");
      const int nm = io.p.noise_management;
      if (!io.perfect && ((nm != RPU_NM_NONE && nm != RPU_NM_CONSTANT && nm != RPU_NM_ABS_MAX && nm != RPU_NM_MAX) ||
                          io.p.bound_management == RPU_BM_ITERATIVE_WORST_CASE)) {
        throw RpuError("Gathered input: not with this noise or bound management.");
      }
      a.in_index = gather->index_patch_major; a.in_index_lines = gather->index_line_major; a.in_group = gather->patches;
      a.in_gs = gather->image_size;
      a.in_sb = 0; a.in_sk = 0;
    }

    prof_begin(s);
    if (io.perfect) {
      a.round = 0;
      launch_mvm_init(a, s);
      prof_mark(s, "mvm_init");
      launch_mvm_round(a, s);
      prof_mark(s, "mvm_round");
    } else {
      if (io.p.noise_management == RPU_NM_AVERAGE_ABS_MAX || io.p.noise_management == RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE) {
        // per-sample maxima, the recurrence over the batch in its order, then the usual set-up with those scales
        if (!nm_aux.p) {
          nm_aux.ensure(1);
          launch_fill(nm_aux.p, nm_aux_host, 1, s);
        }
        a.nm_phase = 1;
        launch_mvm_init(a, s);
        launch_nm_running_average(a.st.nm, B, io.p.nm_decay, nm_aux.p, s);
        a.nm_phase = 2;
      }
      // Where most samples need a second round (as the last call on this tile showed), rounds 0 and 1 run as one
      // launch: one chain of latencies instead of two.  Results are the same either way.
      bool fuse = false;
      int fused = 0;      // rounds of the fused launch: 2, or 3 where the recent calls listed samples for round 2
      int merge_from = 0; // > 0: the rounds from this one on run as one launch
      if (!transposed && !w_other && !side && io.p.bound_management != RPU_BM_NONE && fused_rounds != 0) {
        if (!seen_host) {
          RPU_HIP_CHECK(hipHostMalloc((void **)&seen_host, 4 * sizeof(int), hipHostMallocMapped));
          seen_host[0] = seen_host[1] = seen_host[2] = seen_host[3] = 0;
          RPU_HIP_CHECK(hipHostGetDevicePointer((void **)&seen_dev, seen_host, 0));
        }
        a.dual.seen = seen_dev;
        const int needed = *(volatile int *)&seen_host[0], of = *(volatile int *)&seen_host[1];
        const int last_listed = *(volatile int *)&seen_host[2];
        fuse = mvm_can_fuse_rounds(a) &&
               ((fused_rounds > 0 && (fused_rounds & 1)) || (fused_rounds < 0 && of > 0 && 2 * (long)needed > of));
        // The last round that listed samples in the recent calls is expected to be the last one of this call too: the
        // rounds after it share a launch, whose workgroups find the first of their lists empty and leave.  The
        // estimate rises at once and falls only after eight calls below it: a round that does run inside that launch
        // costs a wait of all its workgroups for each other (about 8 us, tens if yet another round follows), an extra
        // launch only a few microseconds.
        if (of > 0) {
          if (last_listed >= rest_from) {
            rest_from = last_listed;
            rest_quiet = 0;
          } else if (++rest_quiet >= 8) {
            rest_from = last_listed;
            rest_quiet = 0;
          }
        }
        // a third round in the fused launch costs half of what its own launch does, even for a few samples
        if (fuse) fused = (a.max_rounds >= 4 && ((fused_rounds > 0 && (fused_rounds & 4)) || (fused_rounds < 0 && rest_from >= 2))) ? 3 : 2;
        const int first_mergeable = fuse ? fused : 1;
        if (!merged_off && mvm_can_merge_rest(a, mvm_rest_resident_limit(a))) {
          if (fused_rounds > 0 && (fused_rounds & 2)) merge_from = first_mergeable;
          else if (fused_rounds < 0 && of > 0) merge_from = std::max(first_mergeable, rest_from + 1);
          if (merge_from + 1 >= a.max_rounds) merge_from = 0; // the last round alone: a plain launch
          if (merge_from > 0) {
            a.wait_spins = wait_spins_hook;
            a.wait_extra = wait_extra_hook;
            merged_call = a.call;
          }
        }
      }
      if (fuse) {
        s_dual0.ensure((size_t)B * a.O); s_dual1.ensure((size_t)B * a.O); s_xq2.ensure((size_t)B * a.k_pad);
        s_dsel.ensure((size_t)B);
        if (s_dhit1.n < 2 * (size_t)B) {
          s_dhit1.ensure(2 * (size_t)B);
          RPU_HIP_CHECK(hipMemset(s_dhit1.p, 0, s_dhit1.n * sizeof(int))); // cleared by every call after use
        }
        a.dual.buf[0] = s_dual0.p; a.dual.buf[1] = s_dual1.p; a.dual.sel = s_dsel.p; a.dual.hit1 = s_dhit1.p;
        a.dual.xq2 = s_xq2.p;
        a.dual.rounds = fused;
        if (fused == 3) {
          s_dual2.ensure((size_t)B * a.O);
          if (s_dhit2.n < 2 * (size_t)B) {
            s_dhit2.ensure(2 * (size_t)B);
            RPU_HIP_CHECK(hipMemset(s_dhit2.p, 0, s_dhit2.n * sizeof(int)));
          }
          a.dual.buf[2] = s_dual2.p; a.dual.hit2 = s_dhit2.p;
        }
      }
      launch_mvm_init(a, s);
      prof_mark(s, "mvm_init");
      // every round after the first works on the samples whose ADC saturated in the one before; the
      // last workgroup to finish a sample tile sets up the next round for that tile
      if (fuse) {
        launch_mvm_dual(a, s);
        prof_mark(s, "mvm_round");
        // two fused rounds: the launch wrote the rows of round 2 into the third buffer, at each sample's own row; three:
        // the row of a sample listed for round 3 replaced its row of round 1
        if (fused == 2) a.xq[0] = s_xq2.p;
        for (int r = fused; r < a.max_rounds; ++r) {
          a.round = r;
          a.dual.on = r == fused ? 2 : 0;
          a.rest_in_one = (merge_from > 0 && r == merge_from) ? 1 : 0;
          launch_mvm_round(a, s);
          prof_mark(s, "mvm_round");
          if (a.rest_in_one) break;
        }
      } else {
        for (int r = 0; r < a.max_rounds; ++r) {
          a.round = r;
          if (side) pre_adc_terms(a, io, s);
          a.rest_in_one = (merge_from > 0 && r == merge_from) ? 1 : 0;
          launch_mvm_round(a, s);
          prof_mark(s, "mvm_round");
          if (a.rest_in_one) break;
        }
      }
    }
    if (transposed && bias) launch_drop_bias(s_bias.p, final_out, B, X, out_trans ? 1 : 0, s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
    if (!transposed && !w_other) last_forward_batch = B;
  }

  // Carves the scratch of a stochastic pulsed update out of a caller-provided block (256-byte aligned parts) and
  // returns the bytes used; with base == nullptr only the size is computed.
  static size_t carve_update_scratch(unsigned char *base, int X, int D, int B, bool bias, UpdateArgs *a, float **bias_rows) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
      unsigned char *p = base ? base + off : nullptr;
      off += (bytes + 255) & ~(size_t)255;
      return p;
    };
    const size_t chunks = ((size_t)B + 31) / 32, slots = 32;
    int *kmax = (int *)take(4 * sizeof(int));
    int *row_cost = (int *)take((size_t)D * 4);
    int *bl = (int *)take((size_t)B * 4);
    float *pa = (float *)take((size_t)B * 4), *pb = (float *)take((size_t)B * 4);
    uint32_t *xw = (uint32_t *)take((size_t)B * X * 4), *dw = (uint32_t *)take((size_t)B * D * 4);
    uint32_t *xpl = (uint32_t *)take(chunks * slots * X * 4), *dpl = (uint32_t *)take(chunks * slots * D * 4);
    float *rows = bias ? (float *)take((size_t)B * X * 4) : nullptr;
    if (a) {
      a->kmax = kmax; a->row_cost = row_cost; a->bl = bl; a->prob_a = pa; a->prob_b = pb; a->x_words = xw; a->d_words = dw;
      a->x_planes = xpl; a->d_planes = dpl; a->plane_slots = (int)slots; a->n_chunks = (int)chunks;
    }
    if (bias_rows) *bias_rows = rows;
    return off;
  }

  void set_plane_args(UpdateArgs &a, int B) {
    const int slots = 32; // 31 pulse slots and the sign plane
    const int chunks = (B + 31) / 32;
    u_xpl.ensure((size_t)chunks * slots * X);
    u_dpl.ensure((size_t)chunks * slots * D);
    if (!u_kmax.p) {
      u_kmax.ensure(4);
      const int init[4] = {0, 0, 31, 0};
      RPU_HIP_CHECK(hipMemcpy(u_kmax.p, init, sizeof(init), hipMemcpyHostToDevice));
    }
    a.x_planes = u_xpl.p; a.d_planes = u_dpl.p; a.plane_slots = slots; a.n_chunks = chunks;
    a.kmax = u_kmax.p;
  }

  // device steps for pulse words made elsewhere (the reference's updateVectorWithCounts debug protocol)
  void update_with_words(const uint32_t *x_words, const uint32_t *d_words, int B, hipStream_t s) {
    if (lr == 0.0f) return;
    if (is_transfer()) throw RpuError("update_with_words is not provided for a transfer compound.");
    if (!dev.pulsed()) throw RpuError("update_with_words needs a pulsed device.");
    UpdateArgs a{};
    a.w = wp_dev(); a.x_size = X; a.d_size = D; a.m_batch = B; a.lr = lr;
    a.dev.kind = dev.p.kind; a.dev.ls_mult_noise = dev.p.ls_mult_noise; a.dev.dw_min = dev.p.dw_min;
    a.dev.dw_min_std = dev.p.dw_min_std;
    a.dev.w_max = d_wmax.p; a.dev.w_min = d_wmin.p; a.dev.scale_up = d_sup.p; a.dev.scale_down = d_sdown.p;
    a.dev.slope_up = d_slup.p; a.dev.slope_down = d_sldown.p;
    a.x_words = const_cast<uint32_t *>(x_words); a.d_words = const_cast<uint32_t *>(d_words);
    a.key = key(); a.call = call++;
    set_plane_args(a, B);
    if (xd) { // see r_wmax
      row_major_pulse_loop(a);
      launch_transpose(d_w.p, u_wrm.p, X, D, s);
    }
    // words from outside: the longest bit line among them picks the pulse loop, as the batch's largest BL does for the
    // tile's own words (short lines then take the same loop, and the same noise stream, as in rpu_tile_update)
    a.kmax_slot = 3;
    prof_begin(s);
    launch_words_kmax(a, s);
    launch_update_planes(a, s);
    prof_mark(s, "update_planes");
    if (dev.p.count_pulses) count_pulses(a, false, s);
    launch_update_pulsed(a, s);
    prof_mark(s, "update_pulsed");
    if (persistent()) launch_write_noise_touched(a, d_w.p, d_wp.p, dev.scaled_write_noise(), false, s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // With delta weights set the update lands in the caller's buffer as the gradient-like quantity dW with
  // W_new = W - lr * dW and the weights stay as they are (RPUPulsed::updateMatrix, rpu_pulsed.cpp:560-585;
  // RPUSimple::updateMatrix with getUpWeights / getUpBeta, rpu.cpp:624-634, 1489-1510).
  void update(const float *x, const float *d, int B, bool bias, bool x_trans, bool d_trans, hipStream_t s) {
    // NoneWithDevice: the floating-point update, then the device bounds (rpu_weight_updater.cpp:216-224)
    const bool with_device = up.p.pulse_type == RPU_PULSE_NONE_WITH_DEVICE;
    const bool fp_update = !dev.pulsed() || up.p.pulse_type == RPU_PULSE_NONE || with_device;
    if (delta_w && !fp_update) {
      if (lr == 0.0f) throw RpuError("Delta weights of a pulsed update need a learning rate.");
      RPU_HIP_CHECK(hipMemcpyAsync(delta_w, d_w.p, size() * sizeof(float), hipMemcpyDeviceToDevice, s));
      float *delta = delta_w;
      delta_w = nullptr;
      try {
        update(x, d, B, bias, x_trans, d_trans, s);
      } catch (...) {
        delta_w = delta;
        throw;
      }
      delta_w = delta;
      launch_delta_finish(d_w.p, delta_w, -1.0f / lr, size(), s);
      RPU_HIP_CHECK(hipGetLastError());
      return;
    }
    if (lr == 0.0f && !delta_w) return;
    const float *xin = x;
    long x_sb = x_trans ? 1 : X, x_sj = x_trans ? B : 1;
    if (bias) {
      s_bias.ensure((size_t)B * X);
      launch_make_bias(x, s_bias.p, B, X, x_trans ? 1 : 0, s);
      xin = s_bias.p; x_sb = X; x_sj = 1;
    }
    const long d_sb = d_trans ? 1 : D, d_si = d_trans ? B : 1;

    if (with_device && dev.pulsed() && !delta_w && !is_transfer()) {
      // the bounds after every sample make the batch a sequence per cross-point
      UpdateArgs a{};
      a.w = wp_dev(); a.x_size = X; a.d_size = D; a.m_batch = B; a.lr = lr;
      a.x = xin; a.x_sb = x_sb; a.x_sj = x_sj; a.d = d; a.d_sb = d_sb; a.d_si = d_si;
      a.dev.w_max = d_wmax.p; a.dev.w_min = d_wmin.p;
      prof_begin(s);
      launch_update_fp_clipped(cross_point_view(a), s);
      prof_mark(s, "update_fp_clipped");
      refresh_shown_weights(s); // clipWeights ends with applyUpdateWriteNoise (rpu_pulsed_device.cpp:448-467)
      RPU_HIP_CHECK(hipGetLastError());
      last_stream = s;
      last_update_batch = B;
      last_update_pulse = RPU_PULSE_NONE_WITH_DEVICE;
      return;
    }
    if (fp_update) {
      // W += -lr * d^T x as a contraction over the batch (rpu.cpp:624-634): "weights" = d, K = batch
      MvmArgs a{};
      a.transposed = d_trans ? 0 : 1; // element (o = i, k = b): d[b * D + i] or d[i * B + b]
      a.x_size = d_trans ? B : D; a.d_size = d_trans ? D : B;
      mvm_set_weights(a, d, a.x_size, false);
      a.K = B; a.O = D; a.m_batch = X;
      a.in = xin; a.in_sb = x_sj; a.in_sk = x_sb; // "sample" = column j of x, contraction over b
      a.out = delta_w ? delta_w : d_w.p; // W[i][j] of sample j, output i
      a.out_sb = xd ? D : 1; a.out_so = xd ? 1 : X;
      a.io = io_dev(fio); a.io.perfect = 1;
      a.alpha = delta_w ? 1.0f : -lr; a.beta = delta_w ? 0.0f : 1.0f; a.round = 0;
      a.key = key(); a.call = call++;
      a.k_pad = mvm_k_pad(B);
      s_xq0.ensure((size_t)X * a.k_pad);
      a.xq[0] = s_xq0.p; a.xq[1] = nullptr;
      prof_begin(s);
      launch_mvm_init(a, s);
      prof_mark(s, "fp_update_gather");
      launch_mvm_round(a, s);
      prof_mark(s, "fp_update");
      RPU_HIP_CHECK(hipGetLastError());
      last_stream = s;
      last_update_batch = B;
      last_update_pulse = RPU_PULSE_NONE;
      return;
    }

    if (is_transfer()) {
      transfer_update(xin, x_sb, x_sj, d, d_sb, d_si, B, s);
      return;
    }
    if (persistent() && delta_w) throw RpuError("Delta weights are not provided for a device with write noise.");
    DeviceView dv{wp_dev(), d_wmax.p, d_wmin.p, d_sup.p, d_sdown.p, d_slup.p, d_sldown.p, &dev, dev.p.dw_min};
    pulsed_update_on(dv, up, lr, xin, x_sb, x_sj, d, d_sb, d_si, B, s);
  }

  // ----- weight maintenance between steps (decay, diffusion, clipping, column reset) ------------------------------

  void ensure_state_params() {
    if (!dev.pulsed() || state_params_valid) return;
    const size_t n = size(), bytes = n * sizeof(float);
    (void)bytes;
    d_decay.ensure(n); d_diff.ensure(n); d_rbias.ensure(n);
    upload_mat(d_decay.p, arr.decay_scale.data());
    upload_mat(d_diff.p, arr.diffusion_rate.data());
    upload_mat(d_rbias.p, arr.reset_bias.data());
    state_params_valid = true;
  }

  void check_maintenance(const char *what) {
    if (!resident()) throw RpuError(std::string(what) + " needs the tile on a GPU (rpu_tile_to_device).");
    if (is_transfer()) throw RpuError(std::string(what) + " is not provided for a transfer compound.");
  }

  // RPUPulsed::decayWeights -> PulsedRPUDevice::decayWeights (rpu_pulsed_device.cpp:392-420) for a pulsed device,
  // SimpleRPUDevice::decayWeights (rpu_simple_device.cpp:96-115) otherwise
  void decay_weights(float alpha, bool bias_no_decay, hipStream_t s) {
    check_maintenance("decay_weights");
    if (dev.pulsed()) {
      ensure_state_params();
      launch_decay_device(wp_dev(), d_decay.p, d_rbias.p, d_wmin.p, d_wmax.p, alpha, bias_no_decay ? 1 : 0, layout(), s);
      refresh_shown_weights(s);
    } else {
      const float rate = dev.p.lifetime > 1.0f ? 1.0f / dev.p.lifetime : 0.0f;
      const float scale = 1.0f - alpha * rate;
      if (scale > 0.0f && scale < 1.0f) launch_decay_scalar(d_w.p, scale, bias_no_decay ? 1 : 0, layout(), s);
    }
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // rpu_pulsed_device.cpp:432-446, rpu_simple_device.cpp:124-134
  void diffuse_weights(hipStream_t s) {
    check_maintenance("diffuse_weights");
    if (dev.pulsed()) {
      ensure_state_params();
      launch_diffuse(wp_dev(), d_diff.p, 0.0f, d_wmin.p, d_wmax.p, key(), call++, size(), s);
      refresh_shown_weights(s);
    } else if (dev.p.diffusion > 0.0f) {
      launch_diffuse(d_w.p, nullptr, dev.p.diffusion, nullptr, nullptr, key(), call++, size(), s);
    }
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // RPUPulsed::clipWeights (rpu_pulsed.cpp:263-278), WeightClipper::apply (weight_clipper.cpp:30-106)
  void clip_weights(int type, float fixed_value, float sigma, hipStream_t s) {
    check_maintenance("clip_weights");
    if (type == RPU_CLIP_FIXED_VALUE) {
      if (dev.pulsed()) {
        launch_clip_value(wp_dev(), d_wmin.p, d_wmax.p, fixed_value, nullptr, size(), s);
        refresh_shown_weights(s);
      } else if (fixed_value >= 0.0f) launch_clip_value(d_w.p, nullptr, nullptr, fixed_value, nullptr, size(), s);
    } else if (type == RPU_CLIP_NONE) {
      if (dev.pulsed()) throw RpuError("Sophisticated clipping is NOT implemented for most training devices");
    } else if (type == RPU_CLIP_LAYER_GAUSSIAN || type == RPU_CLIP_AVERAGE_CHANNEL_MAX) {
      if (dev.pulsed()) throw RpuError("Sophisticated clipping is NOT implemented for most training devices");
      s_clip.ensure(1 + (size_t)D);
      if (type == RPU_CLIP_LAYER_GAUSSIAN) launch_clip_value_gaussian(d_w.p, size(), sigma, fixed_value, s_clip.p, s);
      else launch_clip_value_channel(d_w.p, layout(), fixed_value, s_clip.p + 1, s_clip.p, s);
      launch_clip_value(d_w.p, nullptr, nullptr, 0.0f, s_clip.p, size(), s);
    } else {
      throw RpuError("Clipping type not implemented.");
    }
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // RPUPulsed::resetCols -> rpu_pulsed_device.cpp:469-494 / rpu_simple_device.cpp:148-168
  void reset_columns(int start_col, int n_cols, float reset_prob, hipStream_t s) {
    check_maintenance("reset_columns");
    if (start_col < 0 || start_col >= X) throw RpuError("start_column_idx out of range.");
    int n = n_cols >= 0 ? n_cols : X;
    if (n > X) n = X; // the wrapped range covers every column once
    if (n == 0) return;
    if (dev.pulsed()) {
      ensure_state_params();
      launch_reset_cols(wp_dev(), d_rbias.p, d_wmin.p, d_wmax.p, dev.p.reset_std, start_col, n, reset_prob, layout(), key(),
                        call++, s);
      refresh_shown_weights(s);
    } else {
      launch_reset_cols(d_w.p, nullptr, nullptr, nullptr, dev.p.reset_std, start_col, n, reset_prob, layout(), key(), call++, s);
    }
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // RPUPulsed::driftWeights -> PulsedRPUDevice::driftWeights (rpu_pulsed_device.cpp:422-430) for a pulsed device,
  // which drifts only when its parameters ask for it; RPUSimple::driftWeights (rpu.cpp:1581-1587) otherwise, with
  // the one nu of the parameters.  WeightDrifter::apply (weight_drifter.cpp:108-150) starts the clocks at its
  // first call.
  void drift_device_weights(float time_since_last_call, hipStream_t s) {
    check_maintenance("drift_weights");
    const rpu_device_params &q = dev.p;
    if (dev.pulsed() && !(q.drift_nu > 0.0f)) return;
    const size_t n = size();
    const bool per_device = arr.drift_nu.size() == n;
    if (per_device && !nu_valid) {
      d_nu.ensure(n);
      upload_mat(d_nu.p, arr.drift_nu.data());
      nu_valid = true;
    }
    if (!dr_prev.p) {
      dr_prev.ensure(n); dr_w0.ensure(n); dr_t.ensure(n);
      RPU_HIP_CHECK(hipMemcpyAsync(dr_prev.p, wp_dev(), n * sizeof(float), hipMemcpyDeviceToDevice, s));
      RPU_HIP_CHECK(hipMemcpyAsync(dr_w0.p, wp_dev(), n * sizeof(float), hipMemcpyDeviceToDevice, s));
      launch_fill(dr_t.p, 0.0f, n, s);
      drift_t = 0.0f;
    }
    drift_t += time_since_last_call / q.drift_t0;
    DriftDev p{};
    p.nu0 = q.drift_nu; p.nu_std = q.drift_nu_std; p.wg_ratio = q.drift_wg_ratio; p.g_offset = q.drift_g_offset;
    p.w_offset = q.drift_w_offset; p.nu_k = q.drift_nu_k; p.log_g0 = q.drift_log_g0; p.reset_tol = q.drift_reset_tol;
    p.w_read_std = q.drift_w_read_std;
    p.a = q.drift_g_offset * q.drift_wg_ratio + q.drift_w_offset;
    if (std::fabs(p.a) < p.reset_tol) p.a = 0.0f;
    const bool random = p.nu_std > 0.0f || p.w_read_std > 0.0f;
    launch_device_drift(wp_dev(), dr_prev.p, dr_w0.p, dr_t.p, per_device ? d_nu.p : nullptr,
                        dev.pulsed() ? d_wmin.p : nullptr, dev.pulsed() ? d_wmax.p : nullptr, p, drift_t, key(),
                        random ? call++ : call, n, s);
    refresh_shown_weights(s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // RPUSimple::remapWeights (rpu.cpp:1740-1747), WeightRemapper::apply (weight_remapper.cpp:19-190)
  void remap_weights(const rpu_remap_params &q, float *scales_dev, hipStream_t s) {
    check_maintenance("remap_weights");
    switch (q.type) {
    case RPU_REMAP_NONE:
      return;
    case RPU_REMAP_LAYERWISE_SYMMETRIC:
    case RPU_REMAP_CHANNELWISE_SYMMETRIC:
    case RPU_REMAP_CHANNELWISE_NORM:
      break;
    case RPU_REMAP_CHANNELWISE_ASYMMETRIC:
      throw RpuError("Expect scales and biases given.");
    default:
      throw RpuError("Remapping type not implemented.");
    }
    if (!scales_dev) throw RpuError("Expect scales given.");
    if (q.type == RPU_REMAP_CHANNELWISE_NORM && !(q.row_norm > 0.0f)) throw RpuError("Expect row_norm >0.");
    if (q.type == RPU_REMAP_CHANNELWISE_SYMMETRIC && q.max_scale_range > 0.0f && q.remapped_wmax != 1.0f) {
      throw RpuError("For max_scales set, expect wrmpar.remapped_wmax to be 1.");
    }
    s_rowstat.ensure(3 * (size_t)D + 1);
    RemapDev p{};
    p.type = q.type; p.clip_if = q.clip_if; p.max_scale_range = q.max_scale_range; p.max_scale_ref = q.max_scale_ref;
    p.row_norm = q.row_norm; p.remapped_wmax = q.remapped_wmax;
    launch_remap(d_w.p, scales_dev, s_rowstat.p, s_rowstat.p + D, s_rowstat.p + 2 * (size_t)D, layout(), p, s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // RPUSimple::modifyFBWeights (rpu.cpp:1749-1758), WeightModifier::apply (weight_modifier.cpp:28-224)
  void modify_weights(const rpu_modifier_params &q, hipStream_t s) {
    check_maintenance("modify_weights");
    if (q.type < RPU_MODIFIER_COPY || q.type > RPU_MODIFIER_PROG_NOISE) {
      throw RpuError("Requested WeightModifierType not implemented.");
    }
    if (q.type == RPU_MODIFIER_PCM_NOISE) throw RpuError("Requested WeightModifierType not implemented in CPU version.");
    if (q.type != RPU_MODIFIER_COPY && q.per_batch_sample) throw RpuError("Per batch sample is not implemented in RPUCuda");
    if (q.n_coeffs < 0 || q.n_coeffs > RPU_MAX_MODIFIER_COEFFS) throw RpuError("Too many modifier coefficients.");
    const size_t n = size();
    d_fbw.ensure(n);
    fb_during_test = q.enable_during_test != 0;
    ModifierDev p{};
    p.type = q.type; p.sto_round = q.sto_round; p.copy_last_column = q.copy_last_column; p.n_coeffs = q.n_coeffs;
    p.std_dev = q.std_dev; p.res = q.res; p.dorefa_clip = q.dorefa_clip; p.pdrop = q.pdrop; p.g_max = q.g_max;
    p.assumed_wmax = q.assumed_wmax;
    for (int c = 0; c < q.n_coeffs; ++c) p.coeffs[c] = q.coeffs[c];
    const float *amax_dev = nullptr;
    if (q.rel_to_actual_wmax && q.type != RPU_MODIFIER_COPY) {
      s_rowstat.ensure(3 * (size_t)D + 1);
      launch_row_stat(d_w.p, layout(), q.copy_last_column ? X - 1 : X, 0, s_rowstat.p, s);
      launch_max_or_one(s_rowstat.p, D, s_rowstat.p + 3 * (size_t)D, s);
      amax_dev = s_rowstat.p + 3 * (size_t)D;
    }
    launch_modify(d_fbw.p, d_w.p, p, amax_dev, key(), call++, layout(), s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  // two 64-bit counters per cross-point, made at the first counted update
  void count_pulses(const UpdateArgs &a, bool implicit, hipStream_t s) {
    if (!d_cnt.p) {
      d_cnt.ensure(2 * size());
      launch_fill(reinterpret_cast<float *>(d_cnt.p), 0.0f, 4 * size(), s); // all-zero bits
    }
    launch_count_pulses(a, d_cnt.p, d_cnt.p + size(), implicit, s);
    prof_mark(s, "count_pulses");
  }

  // RPUSimple::setSharedWeights (rpu.cpp:1384-1398): the caller's memory becomes the weight matrix
  void set_shared_weights(float *w_dev) {
    check_maintenance("set_shared_weights");
    if (!w_dev) throw RpuError("Null device pointer.");
    if (xd || shared_xd) throw RpuError("The tile already uses an [x_size, d_size] shared weight tensor.");
    if (w_dev == d_w.p) return;
    sync_last();
    RPU_HIP_CHECK(hipMemcpy(w_dev, d_w.p, size() * sizeof(float), hipMemcpyDeviceToDevice));
    d_w.adopt(w_dev, size());
  }

  // RPUSimple::setDeltaWeights (rpu.cpp:1459-1481): null ends the mode
  void set_delta_weights(float *dw_dev) {
    if (dw_dev) check_maintenance("set_delta_weights");
    if (dw_dev && xd) throw RpuError("A tile with [x_size, d_size] weights takes its delta weights in that layout.");
    delta_w = dw_dev;
    delta_xd = nullptr;
  }

  // RPUCudaSimple::setSharedWeights (cuda/rpucuda.cu:322-334) with the CUDA tiles' [x_size][d_size] layout.  A plain
  // tile takes the tensor as its weight matrix (see `xd`); the kinds of tile named there keep their row-major matrix
  // and mirror it into the tensor around every call.
  bool takes_xd_storage() const {
    return !is_transfer() && !persistent() && !dev.p.count_pulses && !has_pre_adc_terms(fio) && !has_pre_adc_terms(bio) &&
           !d_cnt.p && !delta_w;
  }
  void set_shared_weights_xd(float *w_xd_dev) {
    check_maintenance("set_shared_weights");
    if (!w_xd_dev) throw RpuError("Null device pointer.");
    if (xd) { // bound already: the weights move to the new tensor
      if (w_xd_dev == d_w.p) return;
      sync_last();
      RPU_HIP_CHECK(hipMemcpy(w_xd_dev, d_w.p, size() * sizeof(float), hipMemcpyDeviceToDevice));
      d_w.adopt(w_xd_dev, size());
      return;
    }
    if (!d_w.owned) throw RpuError("The tile already uses a row-major shared weight buffer.");
    sync_last();
    launch_transpose(d_w.p, w_xd_dev, D, X, last_stream);
    RPU_HIP_CHECK(hipGetLastError());
    RPU_HIP_CHECK(hipStreamSynchronize(last_stream));
    if (shared_xd || !takes_xd_storage()) {
      shared_xd = w_xd_dev;
      return;
    }
    d_w.adopt(w_xd_dev, size());
    // the device parameters: the row-major arrays stay for the pulse loop, copies in the tensor's layout serve the rest
    {
      DevBuf<float> *own[6] = {&d_wmax, &d_wmin, &d_sup, &d_sdown, &d_slup, &d_sldown};
      DevBuf<float> *kept[6] = {&r_wmax, &r_wmin, &r_sup, &r_sdown, &r_slup, &r_sldown};
      for (int k = 0; k < 6; ++k) {
        if (!own[k]->p) continue;
        std::swap(*own[k], *kept[k]);
        own[k]->ensure(size());
        launch_transpose(kept[k]->p, own[k]->p, D, X, last_stream);
      }
      RPU_HIP_CHECK(hipStreamSynchronize(last_stream));
    }
    if (dev.pulsed()) u_wrm.ensure(size()); // here, so that no update call has to allocate it
    for (DevBuf<float> *b : {&d_nu, &dr_prev, &dr_w0, &dr_t, &d_fbw, &i_ref, &i_prog, &i_nu_plus, &i_nu_minus}) {
      to_xd_in_place(*b);
    }
    if (state_params_valid) {
      for (DevBuf<float> *b : {&d_decay, &d_diff, &d_rbias}) to_xd_in_place(*b);
    }
    xd = true;
  }
  void set_delta_weights_xd(float *dw_xd_dev) {
    if (!dw_xd_dev) {
      set_delta_weights(nullptr);
      return;
    }
    check_maintenance("set_delta_weights");
    if (xd) { // the tile's own layout: the buffer is written in place
      delta_w = dw_xd_dev;
      delta_xd = nullptr;
      return;
    }
    d_delta_own.ensure(size());
    delta_w = d_delta_own.p;
    delta_xd = dw_xd_dev;
  }
  // before a call that reads the weights / after a call that may have changed them (or the delta buffer)
  void shared_in(hipStream_t s) {
    if (shared_xd) launch_transpose(shared_xd, d_w.p, X, D, s);
  }
  void shared_out(hipStream_t s) {
    if (shared_xd) launch_transpose(d_w.p, shared_xd, D, X, s);
    if (delta_xd) launch_transpose(d_delta_own.p, delta_xd, D, X, s);
  }

  DeviceView view_of(DeviceSlot &sl, float granularity) {
    return DeviceView{sl.d_w.p, sl.d_wmax.p, sl.d_wmin.p, sl.d_sup.p, sl.d_sdown.p, sl.d_slup.p, sl.d_sldown.p,
                      &sl.par, granularity};
  }

  // pulsed update of one device matrix (rpu_weight_updater.cpp:197-294)
  // ws != nullptr: the per-call scratch is carved out of that block and nothing is allocated (stochastic pulses only)
  // Rows of pulse words per sample.  The longest bit line a call can choose (calculateBlAB,
  // rpu_pulsed_meta_parameter.cpp:152-181) is desired_BL, or ceil(lr / dw_min) when neither a fixed BL nor BL
  // management holds it there.  A packed word holds 31 pulses; longer lines take several rows of words per sample.
  static int words_per_sample_for(const UpdatePar &up, float lr, float granularity) {
    int bl_max = up.p.desired_bl;
    if (!up.p.fixed_bl && !up.p.update_bl_management && granularity * (float)up.p.desired_bl < fabsf(lr)) {
      const float need = ceilf(fabsf(lr) / granularity);
      if (up.p.pulse_type == RPU_PULSE_STOCHASTIC_COMPRESSED && !(need <= (float)RPU_MAX_BL)) {
        throw RpuError("This learning rate needs a bit line of " + std::to_string((long)need) +
                       " pulses (fixed_BL and update_bl_management are off); stochastic pulse trains hold at most " +
                       std::to_string(RPU_MAX_BL) + ".");
      }
      bl_max = std::max((int)need, 1);
    }
    return up.p.pulse_type == RPU_PULSE_STOCHASTIC_COMPRESSED ? std::max((bl_max + 30) / 31, 1) : 1;
  }

  // Arguments of the update kernels for one call (lr != 0): scratch sized for B samples (or carved out of ws), the
  // call's random-stream index taken; wps returns the rows of pulse words per sample.
  UpdateArgs pulsed_update_args(const DeviceView &dv, const UpdatePar &up, float lr, const float *xin, long x_sb, long x_sj,
                                const float *d, long d_sb, long d_si, int B, hipStream_t s, unsigned char *ws, int &wps_out) {
    const DevicePar &dev = *dv.par;
    const int wps = words_per_sample_for(up, lr, dv.granularity);
    if (wps > 1 && ws) throw RpuError("update_noalloc holds bit lines of at most 31 pulses.");
    if (wps > 1 && (long)B * wps > 0x7fffffffL) throw RpuError("Too many rows of pulse words for this batch.");
    const int rows = B * wps; // rows of pulse words
    UpdateArgs a{};
    a.w = dv.w; a.x_size = X; a.d_size = D; a.m_batch = B;
    a.x = xin; a.x_sb = x_sb; a.x_sj = x_sj; a.d = d; a.d_sb = d_sb; a.d_si = d_si;
    if (lines_in_place) { // update_indexed: xin and d are the caller's image tensors
      a.x_index = lines_in_place->index_patch_major; a.x_index_lines = lines_in_place->index_line_major; a.x_group = lines_in_place->patches; a.x_gs = lines_in_place->image_size;
      a.x_sb = 0; a.x_sj = 0;
      a.d_group = lines_in_place->patches; a.d_gs = (long)D * lines_in_place->patches; a.d_sb = 1; a.d_si = lines_in_place->patches;
    }
    a.lr = lr;
    a.up.pulse_type = up.p.pulse_type; a.up.desired_bl = up.p.desired_bl; a.up.fixed_bl = up.p.fixed_bl;
    a.up.update_management = up.p.update_management; a.up.update_bl_management = up.p.update_bl_management;
    a.up.sto_round = up.p.sto_round; a.up.um_grad_scale = up.p.um_grad_scale; a.up.res = up.p.res;
    a.up.x_res_implicit = up.p.x_res_implicit; a.up.d_res_implicit = up.p.d_res_implicit;
    a.dev.kind = dev.p.kind; a.dev.ls_mult_noise = dev.p.ls_mult_noise; a.dev.dw_min = dv.granularity;
    a.dev.dw_min_std = dev.p.dw_min_std;
    a.dev.w_max = const_cast<float *>(dv.w_max); a.dev.w_min = const_cast<float *>(dv.w_min);
    a.dev.scale_up = const_cast<float *>(dv.scale_up); a.dev.scale_down = const_cast<float *>(dv.scale_down);
    a.dev.slope_up = const_cast<float *>(dv.slope_up); a.dev.slope_down = const_cast<float *>(dv.slope_down);
    a.key = key(); a.call = call++;
    if (ws) {
      carve_update_scratch(ws, X, D, B, false, &a, nullptr);
      // the array keeps the last call's contents: the largest-BL slots start from zero again
      hipLaunchKernelGGL(k_init_kmax, dim3(1), dim3(64), 0, s, a.kmax);
      a.kmax_slot = 0;
    } else {
      u_bl.ensure(B); u_a.ensure(B); u_b.ensure(B);
      a.bl = u_bl.p; a.prob_a = u_a.p; a.prob_b = u_b.p;
      if (up.p.pulse_type == RPU_PULSE_STOCHASTIC_COMPRESSED) {
        u_xw.ensure((size_t)rows * X); u_dw.ensure((size_t)rows * D);
        a.x_words = u_xw.p; a.d_words = u_dw.p;
        set_plane_args(a, rows);
        a.kmax_slot = (int)(update_calls++ & 1u);
        if (update_reads_row_cost(a)) {
          u_rowcost.ensure((size_t)D);
          a.row_cost = u_rowcost.p;
        }
      } else {
        u_xval.ensure((size_t)B * X); u_dval.ensure((size_t)B * D);
        a.x_val = u_xval.p; a.d_val = u_dval.p;
      }
    }
    wps_out = wps;
    return a;
  }

  // the pulse loop of a tile that stores [x_size][d_size]: on the row-major copies, results into the tile's matrix
  void row_major_pulse_loop(UpdateArgs &a) {
    u_wrm.ensure(size());
    a.w = u_wrm.p;
    a.w_out = d_w.p; a.wo_si = 1; a.wo_sj = D;
    a.dev.w_max = r_wmax.p; a.dev.w_min = r_wmin.p; a.dev.scale_up = r_sup.p; a.dev.scale_down = r_sdown.p;
    a.dev.slope_up = r_slup.p; a.dev.slope_down = r_sldown.p;
  }

  // the arguments of a pulsed update as the kernels that work cross-point by cross-point take them: as they are on a
  // row-major tile, with x and d exchanged on one that stores [x_size][d_size] (UpdateArgs::swapped)
  UpdateArgs cross_point_view(const UpdateArgs &a) const { return xd ? update_swapped_view(a) : a; }

  // what the debug hooks read after a pulsed update
  void note_pulsed_update(const UpdateArgs &a, int B, int wps, int pulse_type, hipStream_t s) {
    last_stream = s;
    last_update_batch = B;
    last_words_per_sample = wps;
    last_update_pulse = pulse_type;
    last_bl = a.bl; last_a = a.prob_a; last_b = a.prob_b; last_xw = a.x_words; last_dw = a.d_words;
  }

  void pulsed_update_on(const DeviceView &dv, const UpdatePar &up, float lr, const float *xin, long x_sb, long x_sj,
                        const float *d, long d_sb, long d_si, int B, hipStream_t s, unsigned char *ws = nullptr) {
    if (lr == 0.0f) return;
    const DevicePar &dev = *dv.par;
    int wps = 1;
    UpdateArgs a = pulsed_update_args(dv, up, lr, xin, x_sb, x_sj, d, d_sb, d_si, B, s, ws, wps);
    const int rows = B * wps;
    prof_begin(s);
    launch_update_prepare(a, s);
    prof_mark(s, "update_prepare");
    const bool counting = dev.p.count_pulses && !is_transfer();
    if (up.p.pulse_type == RPU_PULSE_STOCHASTIC_COMPRESSED) {
      // from here on the kernels walk rows of words; a longer bit line is several rows of one sample in a row
      a.m_batch = rows;
      a.words_per_sample = wps;
      const bool aggregated = update_variant == RPU_UPDATE_VARIANT_AGGREGATED && dev.linear() && dev.p.ls_mult_noise && !is_transfer();
      if (xd && !aggregated && dv.w == d_w.p) {
        row_major_pulse_loop(a);
        a.wt_src = d_w.p; // the launch of the pulse trains makes the row-major copy
      }
      launch_update_lines(a, s);
      prof_mark(s, "update_lines");
      if (counting) count_pulses(a, false, s);
      if (aggregated) {
        launch_update_aggregated(cross_point_view(a), update_variant_samples, s);
        prof_mark(s, "update_aggregated");
      } else {
        launch_update_pulsed(a, s);
        prof_mark(s, "update_pulsed");
      }
    } else {
      launch_update_implicit_lines(a, s);
      prof_mark(s, "update_implicit_lines");
      if (counting) count_pulses(a, true, s);
      launch_update_implicit(cross_point_view(a), s);
      prof_mark(s, "update_implicit");
    }
    // write noise: cross-points that took a pulse show their new persistent weight with fresh noise
    if (dv.w == d_wp.p && persistent()) {
      launch_write_noise_touched(a, d_w.p, d_wp.p, dev.scaled_write_noise(),
                                 up.p.pulse_type != RPU_PULSE_STOCHASTIC_COMPRESSED, s);
      prof_mark(s, "write_noise");
    }
    RPU_HIP_CHECK(hipGetLastError());
    note_pulsed_update(a, B, wps, up.p.pulse_type, s);
  }

  // Whether this tile's update is the plain stochastic pulsed one that a group launch provides; else why not.
  const char *group_update_obstacle() const {
    if (!dev.pulsed() || up.p.pulse_type != RPU_PULSE_STOCHASTIC_COMPRESSED) return "only stochastic pulses on a pulsed device";
    if (is_transfer()) return "no transfer compounds";
    if (persistent()) return "no write noise";
    if (delta_w) return "no delta weights";
    if (dev.p.count_pulses) return "no pulse counters";
    if (update_variant == RPU_UPDATE_VARIANT_AGGREGATED) return "no update variants";
    if (shared_xd) return "no mirrored shared weights";
    if (lr != 0.0f && words_per_sample_for(up, lr, dev.p.dw_min) > 1) return "bit lines of at most 31 pulses";
    return nullptr;
  }

  // arguments of the plain pulsed update on this tile's own weights (see group_update_obstacle)
  UpdateArgs group_update_args(const float *x, long x_ld, const float *d, long d_ld, int B, hipStream_t s, int &wps) {
    DeviceView dv{wp_dev(), d_wmax.p, d_wmin.p, d_sup.p, d_sdown.p, d_slup.p, d_sldown.p, &dev, dev.p.dw_min};
    UpdateArgs a = pulsed_update_args(dv, up, lr, x, x_ld, 1, d, d_ld, 1, B, s, nullptr, wps);
    a.row_cost = nullptr; // the group launches deal the rows out in their order
    return a;
  }

  // The stochastic pulsed update without any allocation: every buffer beyond inputs and weights lives in the
  // static scratch array of this GPU.  Same kernels, same random streams and therefore the same weights as update().
  void update_noalloc(const float *x, const float *d, int B, bool bias, bool x_trans, bool d_trans, hipStream_t s) {
    if (!dev.pulsed() || up.p.pulse_type != RPU_PULSE_STOCHASTIC_COMPRESSED) {
      throw RpuError("update_noalloc is provided for stochastic pulses on a pulsed device only.");
    }
    if (is_transfer() || persistent() || delta_w || dev.p.count_pulses) {
      throw RpuError("update_noalloc is not provided for transfer compounds, write noise, delta weights or pulse counters.");
    }
    float *rows = nullptr;
    const size_t need = carve_update_scratch(nullptr, X, D, B, bias, nullptr, nullptr);
    if (need > (size_t)RPU_NOALLOC_MAX_SCRATCH_BYTES) {
      throw RpuError("update_noalloc: this call needs " + std::to_string(need) + " bytes of scratch, the static array holds " +
                     std::to_string((size_t)RPU_NOALLOC_MAX_SCRATCH_BYTES) + ".");
    }
    if (lr == 0.0f) return;
    // refused before anything is written to the shared array
    if (words_per_sample_for(up, lr, dev.p.dw_min) > 1) throw RpuError("update_noalloc holds bit lines of at most 31 pulses.");
    unsigned char *ws = noalloc_scratch(device_id);
    carve_update_scratch(ws, X, D, B, bias, nullptr, &rows);
    const float *xin = x;
    long x_sb = x_trans ? 1 : X, x_sj = x_trans ? B : 1;
    if (bias) {
      launch_make_bias(x, rows, B, X, x_trans ? 1 : 0, s);
      xin = rows; x_sb = X; x_sj = 1;
    }
    const long d_sb = d_trans ? 1 : D, d_si = d_trans ? B : 1;
    DeviceView dv{wp_dev(), d_wmax.p, d_wmin.p, d_sup.p, d_sdown.p, d_slup.p, d_sldown.p, &dev, dev.p.dw_min};
    const bool was_profiling = profiling;
    profiling = false; // event creation allocates
    try {
      pulsed_update_on(dv, up, lr, xin, x_sb, x_sj, d, d_sb, d_si, B, s, ws);
    } catch (...) {
      profiling = was_profiling;
      throw;
    }
    profiling = was_profiling;
  }

  // ---- indexed (convolution) interface ---------------------------------------------------------------

  // the index matrix as the fused forward kernels read it: [patches][X], the order of the rows of the patch matrix
  void ensure_patch_major_index() {
    if (x_idx_t.p) return;
    std::vector<int32_t> tr((size_t)X * idx_patches);
    for (int k = 0; k < X; ++k)
      for (int p = 0; p < idx_patches; ++p) tr[(size_t)p * X + k] = idx_host[(size_t)k * idx_patches + p];
    x_idx_t.ensure(tr.size());
    RPU_HIP_CHECK(hipMemcpy(x_idx_t.p, tr.data(), tr.size() * sizeof(int32_t), hipMemcpyHostToDevice));
  }

  // samples of an indexed call: the kernels count them in 32 bits
  int indexed_samples(int n_images) const {
    const long B = (long)n_images * idx_patches;
    if (B >= (1L << 31) || B * std::max(X, D) >= (1L << 40)) throw RpuError("Too many patches for one call: split the images.");
    return (int)B;
  }

  void ensure_line_major_index() {
    if (x_idx.p) return;
    x_idx.ensure(idx_host.size());
    RPU_HIP_CHECK(hipMemcpy(x_idx.p, idx_host.data(), idx_host.size() * sizeof(int32_t), hipMemcpyHostToDevice));
  }

  // rows of the patch matrix start on 128-byte lines: a workgroup's stores then fill whole lines
  int x_mat_ld() const { return (X + 31) & ~31; }

  void ensure_indexed(int n_images) {
    if (idx_patches <= 0) throw RpuError("The index matrix has not been set (set_matrix_indices).");
    if (n_images <= 0) throw RpuError("n_images must be positive.");
    (void)indexed_samples(n_images);
    ensure_line_major_index();
    const size_t B = (size_t)n_images * idx_patches;
    x_mat.ensure(B * (size_t)x_mat_ld());
    d_mat.ensure(B * D);
  }

  void forward_indexed(const float *x, float *d, int n_images, long image_size, bool is_test, hipStream_t s) {
    if (idx_patches <= 0) throw RpuError("The index matrix has not been set (set_matrix_indices).");
    if (n_images <= 0) throw RpuError("n_images must be positive.");
    if (D <= 32 && (long)n_images * idx_patches < (1L << 31) && !has_pre_adc_terms(fio)) {
      // narrow tile: unfold, contraction and bound management fused in one kernel, nothing materialized
      const int B = n_images * idx_patches;
      s_rounds.ensure((size_t)B); // the only per-patch state that leaves the kernel: rounds run (get_bm_rounds)
      MvmArgs a{};
      a.x_size = X; a.d_size = D; a.m_batch = B; a.K = X; a.O = D;
      mvm_set_weights(a, mvm_weights(is_test), w_ld(), xd);
      a.io = io_dev(fio);
      a.alpha = fio.p.out_scale;
      a.max_rounds = fio.perfect ? 0 : mvm_max_rounds(a.io);
      a.st.rounds = s_rounds.p;
      if (conv_forward_supported(a)) {
        ensure_patch_major_index();
        a.key = key(); a.call = call++;
        ConvArgs c{x, x_idx_t.p, d, idx_patches, n_images, image_size};
        prof_begin(s);
        launch_conv_forward(a, c, s);
        prof_mark(s, "conv_forward");
        RPU_HIP_CHECK(hipGetLastError());
        last_stream = s;
        last_forward_batch = B;
        return;
      }
    }
    const int B = indexed_samples(n_images);
    {
      // a call that reads its input row by row only (one round, or the rows of a further round written once it is
      // known who goes on) gathers the patches in the init kernel: the patch matrix is never written
      MvmArgs probe{};
      probe.io = io_dev(fio);
      const bool one_round = fio.perfect || mvm_max_rounds(probe.io) <= 1;
      const int nm = fio.p.noise_management;
      const bool nm_ok = fio.perfect || ((nm == RPU_NM_NONE || nm == RPU_NM_CONSTANT || nm == RPU_NM_ABS_MAX || nm == RPU_NM_MAX) &&
                                         fio.p.bound_management != RPU_BM_ITERATIVE_WORST_CASE);
      if ((one_round || !mvm_speculates(B, D)) && !has_pre_adc_terms(fio) && nm_ok) {
        ensure_patch_major_index();
        ensure_line_major_index();
        d_mat.ensure((size_t)B * D);
        const GatherSource patches_of{x_idx_t.p, x_idx.p, idx_patches, image_size};
        mvm(x, d_mat.p, B, false, false, true, false, s, nullptr, nullptr, is_test, 0, &patches_of);
        launch_lines_to_images(d, d_mat.p, n_images, D, idx_patches, s);
        RPU_HIP_CHECK(hipGetLastError());
        return;
      }
    }
    ensure_indexed(n_images);
    launch_gather_indexed(x_mat.p, x, x_idx.p, X, x_mat_ld(), idx_patches, n_images, image_size, s);
    // the outputs come out line-major, [D][N P] (stores of a wave, one sample per lane, are unit stride), and move to
    // the caller's [image][output][patch] tensor in runs of a patch row
    mvm(x_mat.p, d_mat.p, B, false, false, true, false, s, nullptr, nullptr, is_test, x_mat_ld());
    launch_lines_to_images(d, d_mat.p, n_images, D, idx_patches, s);
    RPU_HIP_CHECK(hipGetLastError());
  }

  void backward_indexed(const float *d, float *x, int n_images, long image_size, hipStream_t s) {
    ensure_indexed(n_images);
    const int B = indexed_samples(n_images);
    // the caller's [image][output][patch] tensor moves to line-major [D][N P] in runs of a patch row and is read
    // transposed; the patch matrix comes out line-major too, [X][N P]: stores of a wave (one sample per lane) and the
    // reads of the fold (neighbouring image elements meet neighbouring patches) are then unit stride
    launch_images_to_lines(d_mat.p, d, n_images, D, idx_patches, s);
    mvm(d_mat.p, x_mat.p, B, false, true, true, true, s);
    if (fold_image_size != image_size) {
      // per image element, the entries of the patch matrix that were gathered from it, in the order in which the
      // reference's loop adds them up (k, then p)
      if (image_size <= 0 || (long)idx_max - 2 >= image_size) throw RpuError("The index matrix points beyond the image.");
      std::vector<int> ptr((size_t)image_size + 1, 0);
      for (int32_t j : idx_host) {
        if (j > 1) ++ptr[(size_t)(j - 2) + 1];
      }
      for (long e = 0; e < image_size; ++e) ptr[(size_t)e + 1] += ptr[(size_t)e];
      std::vector<int> off(2 * (size_t)ptr[(size_t)image_size]), cursor(ptr.begin(), ptr.end() - 1);
      for (int k = 0; k < X; ++k) {
        for (int p = 0; p < idx_patches; ++p) {
          const int32_t j = idx_host[(size_t)k * idx_patches + p];
          if (j > 1) {
            const size_t at = 2 * (size_t)cursor[(size_t)(j - 2)]++;
            off[at] = k;
            off[at + 1] = p;
          }
        }
      }
      sync_last(); // the lists of another image size may still be read
      x_fold_ptr.ensure(ptr.size());
      x_fold_off.ensure(std::max<size_t>(off.size(), 1));
      RPU_HIP_CHECK(hipMemcpy(x_fold_ptr.p, ptr.data(), ptr.size() * sizeof(int), hipMemcpyHostToDevice));
      if (!off.empty()) RPU_HIP_CHECK(hipMemcpy(x_fold_off.p, off.data(), off.size() * sizeof(int), hipMemcpyHostToDevice));
      fold_image_size = image_size;
    }
    launch_fold_indexed(x, x_mat.p, x_fold_ptr.p, x_fold_off.p, X, idx_patches, n_images, image_size, s);
    RPU_HIP_CHECK(hipGetLastError());
  }

  void update_indexed(const float *x, const float *d, int n_images, long image_size, hipStream_t s) {
    if (idx_patches <= 0) throw RpuError("The index matrix has not been set (set_matrix_indices).");
    if (n_images <= 0) throw RpuError("n_images must be positive.");
    const int B = indexed_samples(n_images);
    const int pt = up.p.pulse_type;
    if (dev.pulsed() && !is_transfer() && pt != RPU_PULSE_NONE && pt != RPU_PULSE_NONE_WITH_DEVICE) {
      // pulsed update: the kernels that make the pulse trains read the patches through the index matrix and the
      // gradients where the caller keeps them; neither the patch matrix nor a patch-major copy of d is written
      // (the reference walks both tensors through iterators, cuda/io_iterator.h:160-696, cuda/rpucuda_pulsed.cu:575-604)
      ensure_patch_major_index();
      ensure_line_major_index();
      const GatherSource patches_of{x_idx_t.p, x_idx.p, idx_patches, image_size};
      lines_in_place = &patches_of;
      try {
        update(x, d, B, false, false, false, s);
      } catch (...) {
        lines_in_place = nullptr;
        throw;
      }
      lines_in_place = nullptr;
      RPU_HIP_CHECK(hipGetLastError());
      return;
    }
    ensure_indexed(n_images);
    launch_gather_indexed(x_mat.p, x, x_idx.p, X, X, idx_patches, n_images, image_size, s);
    launch_ndp_to_bd(d_mat.p, d, n_images, D, idx_patches, s);
    update(x_mat.p, d_mat.p, B, false, false, false, s);
    RPU_HIP_CHECK(hipGetLastError());
  }

  // ---- inference weight pipeline ------------------------------------------------------------------

  static PcmDev pcm_dev(const rpu_pcm_noise_params &q, float t_inference) {
    if (!(q.g_max > 0.0f) || q.g_min < 0.0f || q.g_min >= q.g_max) throw RpuError("g_min should be smaller than g_max");
    PcmDev p{};
    p.g_max = q.g_max; p.g_min = q.g_min;
    p.prog_noise_scale = q.prog_noise_scale; p.read_noise_scale = q.read_noise_scale; p.drift_scale = q.drift_scale;
    p.c0 = q.prog_coeff[0]; p.c1 = q.prog_coeff[1]; p.c2 = q.prog_coeff[2];
    p.sig_scale = q.g_max / q.prog_coeff_g_max_reference;
    const double t = (double)t_inference + (double)q.t_0; // pcm.py:138-152
    p.drift_base_log2 = t > (double)q.t_0 ? (float)std::log2(t / (double)q.t_0) : 0.0f;
    p.read_sigma = t > 0.0 ? (float)std::sqrt(std::log((t + (double)q.t_read) / (2.0 * (double)q.t_read))) : -1.0f;
    return p;
  }

  void check_inference_tile() {
    if (!resident()) throw RpuError("Tile is not resident on a GPU.");
    if (is_transfer() || dev.pulsed()) {
      throw RpuError("The inference weight pipeline needs a tile with an ideal device (as InferenceRPUConfig has).");
    }
  }

  void program_weights(const rpu_pcm_noise_params &q, bool from_reference, hipStream_t s) {
    check_inference_tile();
    const size_t n = size();
    i_ref.ensure(n); i_prog.ensure(n); i_nu_plus.ensure(n); i_nu_minus.ensure(n); i_absmax.ensure(1);
    if (!from_reference || !has_reference) {
      RPU_HIP_CHECK(hipMemcpyAsync(i_ref.p, d_w.p, n * sizeof(float), hipMemcpyDeviceToDevice, s));
      has_reference = true;
    }
    const PcmDev p = pcm_dev(q, 0.0f);
    launch_abs_max(i_ref.p, n, i_absmax.p, s);
    launch_pcm_program(i_ref.p, i_prog.p, i_nu_plus.p, i_nu_minus.p, n, i_absmax.p, p, key(), call++, s);
    RPU_HIP_CHECK(hipMemcpyAsync(d_w.p, i_prog.p, n * sizeof(float), hipMemcpyDeviceToDevice, s));
    RPU_HIP_CHECK(hipGetLastError());
    programmed = true;
    last_stream = s;
  }

  void drift_weights(const rpu_pcm_noise_params &q, float t_inference, hipStream_t s) {
    check_inference_tile();
    if (!programmed) program_weights(q, true, s);
    const size_t n = size();
    const PcmDev p = pcm_dev(q, t_inference);
    launch_abs_max(i_prog.p, n, i_absmax.p, s);
    launch_pcm_drift(i_prog.p, i_nu_plus.p, i_nu_minus.p, d_w.p, n, i_absmax.p, p, key(), call++, s);
    RPU_HIP_CHECK(hipGetLastError());
    last_stream = s;
  }

  float drift_readout(hipStream_t s) {
    check_inference_tile();
    t_unit.ensure((size_t)X * X);
    t_read.ensure((size_t)X * D);
    i_scalar.ensure(1);
    launch_unit_vectors(t_unit.p, X, X, 0, s);
    mvm(t_unit.p, t_read.p, X, false, false, false, false, s);
    launch_mean_abs(t_read.p, (size_t)X * D, i_scalar.p, s);
    float value = 0.0f;
    RPU_HIP_CHECK(hipMemcpyAsync(&value, i_scalar.p, sizeof(float), hipMemcpyDeviceToHost, s));
    RPU_HIP_CHECK(hipStreamSynchronize(s));
    last_stream = s;
    return std::max(value, 0.0001f);
  }

  // ---- transfer compound ----------------------------------------------------------------------

  // tile weights = sum_k gamma_k w_k, unless the last device alone is visible (rpu_transfer_device.cpp:596-602)
  void reduce_to_weights(hipStream_t s) {
    if (tr->fully_hidden) return;
    ReduceArgs r{};
    r.n = tr->n();
    for (int k = 0; k < r.n; ++k) {
      r.w[k] = slots[k]->d_w.p;
      r.gamma[k] = tr->gamma_vec[k];
    }
    launch_reduce_weights(d_w.p, r, size(), s);
  }

  // TransferRPUDevice::transfer / readAndUpdate (rpu_transfer_device.cpp:428-516): the next
  // n_reads_per_transfer columns (rows) of device `from` are read through transfer_io with unit vectors
  // (scaled by -1 so that the write adds) and written onto device `to` with a pulsed update under
  // transfer_up.  Reading all of them before writing is the same as one by one: `from` is not written.
  void do_transfer(int to, int from, float current_lr, hipStream_t s) {
    const TransferPar &tp = *tr;
    const int in_size = tp.in_size, out_size = tp.out_size;
    const bool cols = tp.p.transfer_columns != 0;
    // the two host draws of a transfer (the reference's rw_rng_): one Philox call keyed by (device, update counter)
    const PhiloxKey k = key();
    const Philox4 draw = philox4x32_10((uint32_t)from, (uint32_t)update_idx, (uint32_t)(update_idx >> 32), RNG_TRANSFER, k.k0, k.k1);
    int start = slice_idx[from];
    if (tp.p.random_selection) { // rpu_transfer_device.cpp:486-488
      start = std::max(std::min((int)floorf(u32_to_uniform(draw.v[0]) * (float)in_size), in_size - 1), 0);
    }
    const int n_vec = std::min(tp.p.n_reads_per_transfer, in_size);
    slice_idx[from] = (start + n_vec) % in_size;
    const float lr_t = tp.transfer_lr(from, current_lr);
    if (lr_t != 0.0f && to != from) {
      t_unit.ensure((size_t)n_vec * in_size);
      t_read.ensure((size_t)n_vec * out_size);
      launch_unit_vectors(t_unit.p, n_vec, in_size, start, s);
      IOPar io = tp.io;
      io.p.out_scale = -io.p.out_scale;
      line_set = 2; // the periphery of the read has its own per-line values (rpu_transfer_device.cpp:198-213)
      try {
        mvm(t_unit.p, t_read.p, n_vec, false, false, false, !cols, s, slots[from]->d_w.p, &io);
      } catch (...) {
        line_set = -1;
        throw;
      }
      line_set = -1;
      DeviceView dv = view_of(*slots[to], slots[to]->par.weight_granularity());
      if (cols) pulsed_update_on(dv, tp.up, lr_t, t_unit.p, X, 1, t_read.p, D, 1, n_vec, s);
      else pulsed_update_on(dv, tp.up, lr_t, t_read.p, X, 1, t_unit.p, D, 1, n_vec, s);
    }
    // the columns that were read start again from their reset values with probability with_reset_prob per transfer,
    // after all of them were read and written (cuda/rpucuda_transfer_device.cu:320-324)
    if (cols && tp.p.with_reset_prob > 0.0f && u32_to_uniform(draw.v[1]) < tp.p.with_reset_prob) {
      DeviceSlot &src = *slots[from];
      if (src.d_rbias.n < size()) {
        src.d_rbias.ensure(size());
        RPU_HIP_CHECK(hipMemcpy(src.d_rbias.p, src.arr.reset_bias.data(), size() * sizeof(float), hipMemcpyHostToDevice));
      }
      launch_reset_cols(src.d_w.p, src.d_rbias.p, src.d_wmin.p, src.d_wmax.p, src.par.p.reset_std, start, n_vec, 1.0f, layout(),
                        k, call++, s);
    }
  }

  // TransferRPUDevice::doSparseUpdate / finishUpdateCycle per update vector (rpu_transfer_device.cpp:520-557):
  // the gradient goes onto device 0; after every vector the update counter advances and each device whose
  // period divides it transfers.  The batch is cut at those points (C/rpucuda_transfer_device.cu:393-510).
  void transfer_update(const float *xin, long x_sb, long x_sj, const float *d, long d_sb, long d_si, int B, hipStream_t s) {
    const TransferPar &tp = *tr;
    const float lr_fast = tp.fast_lr(lr);
    const int n_dev = tp.n();
    std::vector<int> every(n_dev);
    for (int j = 0; j < n_dev; ++j) every[j] = tp.transfer_every(j, B);
    DeviceView dv0 = view_of(*slots[0], tp.granularity());
    int b0 = 0;
    while (b0 < B) {
      // vectors until the next transfer of any device
      uint64_t chunk = (uint64_t)(B - b0);
      for (int j = 0; j < n_dev; ++j) {
        if (every[j] > 0) chunk = std::min<uint64_t>(chunk, (uint64_t)every[j] - update_idx % (uint64_t)every[j]);
      }
      pulsed_update_on(dv0, up, lr_fast, xin + (long)b0 * x_sb, x_sb, x_sj, d + (long)b0 * d_sb, d_sb, d_si, (int)chunk, s);
      update_idx += chunk;
      b0 += (int)chunk;
      for (int j = 0; j < n_dev; ++j) {
        if (every[j] > 0 && update_idx % (uint64_t)every[j] == 0) do_transfer(std::min(j + 1, n_dev - 1), j, lr, s);
      }
    }
    reduce_to_weights(s);
    last_stream = s;
    last_update_batch = B;
  }

  // TransferRPUDevice::onSetWeights (rpu_transfer_device.cpp:559-594): every device to zero, the last one gets
  // the weights over its significance, each is clipped into its own bounds, counters restart
  void transfer_set_weights_host(const float *w) {
    const int last = tr->n() - 1;
    const size_t n = size();
    for (auto &sl : slots) sl->w_host.assign(n, 0.0f);
    const float g = tr->fully_hidden ? 1.0f : tr->gamma_vec[last];
    for (size_t i = 0; i < n; ++i) slots[last]->w_host[i] = tr->fully_hidden ? w[i] : w[i] / g;
    for (auto &sl : slots) sl->clip_host();
    update_idx = 0;
    std::fill(slice_idx.begin(), slice_idx.end(), 0);
    transfer_reduce_host();
  }

  void transfer_reduce_host() {
    const size_t n = size();
    w_host.assign(n, 0.0f);
    if (tr->fully_hidden) {
      w_host = slots.back()->w_host;
      return;
    }
    for (int k = 0; k < tr->n(); ++k) {
      for (size_t i = 0; i < n; ++i) w_host[i] += tr->gamma_vec[k] * slots[k]->w_host[i];
    }
  }

  // device -> host copies of all matrices of the compound
  void transfer_download() {
    const size_t bytes = size() * sizeof(float);
    for (auto &sl : slots) {
      sl->w_host.resize(size());
      RPU_HIP_CHECK(hipMemcpy(sl->w_host.data(), sl->d_w.p, bytes, hipMemcpyDeviceToHost));
    }
    w_host.resize(size());
    RPU_HIP_CHECK(hipMemcpy(w_host.data(), wdev(), bytes, hipMemcpyDeviceToHost));
  }

  void transfer_upload_weights() {
    const size_t bytes = size() * sizeof(float);
    for (auto &sl : slots) RPU_HIP_CHECK(hipMemcpy(sl->d_w.p, sl->w_host.data(), bytes, hipMemcpyHostToDevice));
    if (!tr->fully_hidden) RPU_HIP_CHECK(hipMemcpy(d_w.p, w_host.data(), bytes, hipMemcpyHostToDevice));
  }
};

} // namespace rpu_amd

// ---------------------------------------------------------------------------------------------------
// C ABI

using namespace rpu_amd;

struct rpu_tile {
  Tile t;
};

namespace {
thread_local std::string g_last_error;

template <typename F> int guarded(F &&f) {
  try {
    f();
    return 0;
  } catch (const std::exception &e) {
    g_last_error = e.what();
    return 1;
  } catch (...) {
    g_last_error = "unknown error";
    return 2;
  }
}
} // namespace

extern "C" {

const char *rpu_last_error(void) { return g_last_error.c_str(); }
int rpu_abi_version(void) { return RPU_AMD_ABI_VERSION; }

int rpu_tile_config_default(rpu_tile_config *cfg, int device_kind) {
  return guarded([&] {
    if (!cfg) throw RpuError("cfg is null");
    fill_default_config(cfg, device_kind);
  });
}

int rpu_tile_create(rpu_tile_t **out, int x_size, int d_size, const rpu_tile_config *cfg) {
  return guarded([&] {
    if (!out || !cfg) throw RpuError("null argument");
    if (x_size <= 0 || d_size <= 0) throw RpuError("x_size and d_size must be positive.");
    auto h = std::make_unique<rpu_tile>();
    Tile &t = h->t;
    t.X = x_size;
    t.D = d_size;
    t.fio.p = cfg->f_io;
    t.bio.p = cfg->b_io;
    t.up.p = cfg->up;
    t.dev.p = cfg->device;
    t.fio.initialize(false);
    t.bio.initialize(true);
    t.populate_lines(cfg->device.construction_seed);
    t.up.initialize();
    t.dev.initialize();
    t.dev.populate(x_size, d_size, t.arr);
    t.w_host.assign(t.size(), 0.0f);
    t.clip_host(t.w_host);
    *out = h.release();
  });
}

int rpu_transfer_params_default(rpu_transfer_params *tp, int device_kind) {
  return guarded([&] {
    if (!tp) throw RpuError("tp is null");
    fill_default_transfer(tp, device_kind);
  });
}

int rpu_tile_create_transfer(rpu_tile_t **out, int x_size, int d_size, const rpu_tile_config *cfg,
                             const rpu_transfer_params *tp) {
  return guarded([&] {
    if (!out || !cfg || !tp) throw RpuError("null argument");
    if (x_size <= 0 || d_size <= 0) throw RpuError("Tile sizes must be positive.");
    auto h = std::make_unique<rpu_tile>();
    Tile &t = h->t;
    t.X = x_size;
    t.D = d_size;
    t.fio.p = cfg->f_io;
    t.bio.p = cfg->b_io;
    t.up.p = cfg->up;
    t.fio.initialize(false);
    t.bio.initialize(true);
    t.populate_lines(tp->construction_seed);
    t.up.initialize();
    if (t.up.p.pulse_type == RPU_PULSE_NONE || t.up.p.pulse_type == RPU_PULSE_NONE_WITH_DEVICE) {
      throw RpuError("A transfer compound needs a pulsed update (pulse_type None is not provided).");
    }
    t.tr = std::make_unique<TransferPar>();
    t.tr->p = *tp;
    t.tr->initialize(x_size, d_size);
    t.tr->io.populate_lines(t.tr->out_size, tp->construction_seed ? tp->construction_seed * 2654435761u + 3u : 0u, 0);
    t.dev = t.tr->devs[0]; // the device the gradient update sees
    std::vector<DeviceArrays> arrays;
    populate_chain(t.tr->devs, tp->construction_seed, x_size, d_size, arrays);
    for (int k = 0; k < t.tr->n(); ++k) {
      auto sl = std::make_unique<DeviceSlot>();
      sl->par = t.tr->devs[k];
      sl->arr = std::move(arrays[k]);
      t.slots.push_back(std::move(sl));
    }
    t.slice_idx.assign(t.tr->n(), 0);
    std::vector<float> zeros(t.size(), 0.0f);
    t.transfer_set_weights_host(zeros.data());
    *out = h.release();
  });
}

int rpu_tile_set_matrix_indices(rpu_tile_t *tile, const int32_t *indices_host, int x_size, int patches) {
  return guarded([&] {
    if (!tile || !indices_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (x_size != t.X) throw RpuError("The index matrix must have x_size rows.");
    if (patches <= 0) throw RpuError("patches must be positive.");
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_last();
      t.x_idx.release();
      t.x_idx_t.release();
      t.x_fold_ptr.release();
      t.x_fold_off.release();
    }
    t.fold_image_size = -1;
    t.idx_host.assign(indices_host, indices_host + (size_t)x_size * patches);
    t.idx_max = 0;
    for (int32_t j : t.idx_host) {
      if (j < 0) throw RpuError("Negative entry in the index matrix.");
      t.idx_max = std::max(t.idx_max, j);
    }
    t.idx_patches = patches;
  });
}

int rpu_tile_has_matrix_indices(const rpu_tile_t *tile) { return tile ? tile->t.idx_patches : 0; }

#define RPU_INDEXED_ENTRY(NAME, CALL)                                                          \
  return guarded([&] {                                                                         \
    if (!tile) throw RpuError("null tile");                                                    \
    Tile &t = tile->t;                                                                         \
    std::lock_guard<std::mutex> lock(t.mutex);                                                 \
    if (!t.check_compute(n_images, x_dev, d_dev)) return;                                      \
    if (image_size <= 0) throw RpuError("image_size must be positive.");                       \
    if ((long)t.idx_max - 2 >= image_size) throw RpuError("Index matrix entry beyond the image size."); \
    DeviceGuard g(t.device_id);                                                                \
    t.shared_in((hipStream_t)stream);                                                          \
    CALL;                                                                                      \
    t.shared_out((hipStream_t)stream);                                                         \
  })

int rpu_tile_forward_indexed(rpu_tile_t *tile, const float *x_dev, float *d_dev, int n_images, long image_size,
                             int is_test, void *stream) {
  RPU_INDEXED_ENTRY(forward, t.forward_indexed(x_dev, d_dev, n_images, image_size, is_test != 0, (hipStream_t)stream));
}

int rpu_tile_backward_indexed(rpu_tile_t *tile, const float *d_dev, float *x_dev, int n_images, long image_size,
                              void *stream) {
  RPU_INDEXED_ENTRY(backward, t.backward_indexed(d_dev, x_dev, n_images, image_size, (hipStream_t)stream));
}

int rpu_tile_update_indexed(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int n_images, long image_size,
                            void *stream) {
  RPU_INDEXED_ENTRY(update, t.update_indexed(x_dev, d_dev, n_images, image_size, (hipStream_t)stream));
}
#undef RPU_INDEXED_ENTRY

// ---- weight maintenance between steps, shared and delta weights, extra state --------------------------

#define RPU_MAINTENANCE_ENTRY(CALL)                                \
  return guarded([&] {                                             \
    if (!tile) throw RpuError("null tile");                        \
    Tile &t = tile->t;                                             \
    std::lock_guard<std::mutex> lock(t.mutex);                     \
    if (!t.resident()) {                                           \
      CALL;                                                        \
      return;                                                      \
    }                                                              \
    DeviceGuard g(t.device_id);                                    \
    t.shared_in((hipStream_t)stream);                              \
    CALL;                                                          \
    t.shared_out((hipStream_t)stream);                             \
  })

#define RPU_MAINTENANCE_ENTRY_NOSYNC(CALL)                         \
  return guarded([&] {                                             \
    if (!tile) throw RpuError("null tile");                        \
    Tile &t = tile->t;                                             \
    std::lock_guard<std::mutex> lock(t.mutex);                     \
    if (!t.resident()) {                                           \
      CALL;                                                        \
      return;                                                      \
    }                                                              \
    DeviceGuard g(t.device_id);                                    \
    CALL;                                                          \
  })

int rpu_tile_decay_weights(rpu_tile_t *tile, float alpha, int bias_no_decay, void *stream) {
  RPU_MAINTENANCE_ENTRY(t.decay_weights(alpha, bias_no_decay != 0, (hipStream_t)stream));
}

int rpu_tile_diffuse_weights(rpu_tile_t *tile, void *stream) {
  RPU_MAINTENANCE_ENTRY(t.diffuse_weights((hipStream_t)stream));
}

int rpu_tile_clip_weights(rpu_tile_t *tile, int clip_type, float fixed_value, float sigma, void *stream) {
  RPU_MAINTENANCE_ENTRY(t.clip_weights(clip_type, fixed_value, sigma, (hipStream_t)stream));
}

int rpu_tile_reset_columns(rpu_tile_t *tile, int start_column_idx, int num_columns, float reset_prob, void *stream) {
  RPU_MAINTENANCE_ENTRY(t.reset_columns(start_column_idx, num_columns, reset_prob, (hipStream_t)stream));
}

int rpu_tile_drift_device_weights(rpu_tile_t *tile, float time_since_last_call, void *stream) {
  RPU_MAINTENANCE_ENTRY(t.drift_device_weights(time_since_last_call, (hipStream_t)stream));
}

int rpu_tile_remap_weights(rpu_tile_t *tile, const rpu_remap_params *p, float *scales_dev, void *stream) {
  if (!p) return guarded([] { throw RpuError("null parameters"); });
  RPU_MAINTENANCE_ENTRY(t.remap_weights(*p, scales_dev, (hipStream_t)stream));
}

int rpu_tile_modify_weights(rpu_tile_t *tile, const rpu_modifier_params *p, void *stream) {
  if (!p) return guarded([] { throw RpuError("null parameters"); });
  RPU_MAINTENANCE_ENTRY(t.modify_weights(*p, (hipStream_t)stream));
}

int rpu_tile_get_modified_weights(rpu_tile_t *tile, float *w_host) {
  return guarded([&] {
    if (!tile || !w_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || !t.d_fbw.p) throw RpuError("No modified weights: modify_weights has not been called.");
    DeviceGuard g(t.device_id);
    t.sync_last();
    t.download_mat(w_host, t.d_fbw.p);
  });
}

static std::vector<float> &read_asymmetry_of(Tile &t, int backward) {
  IOPar &io = backward ? t.bio : t.fio;
  if (io.w_asymmetry.empty()) throw RpuError("No read asymmetry factors: w_read_asymmetry_dtod of this direction is 0.");
  return io.w_asymmetry;
}

int rpu_tile_get_read_asymmetry(rpu_tile_t *tile, int backward, float *factors_host) {
  return guarded([&] {
    if (!tile || !factors_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    const std::vector<float> &v = read_asymmetry_of(t, backward);
    std::memcpy(factors_host, v.data(), v.size() * sizeof(float));
  });
}

int rpu_tile_set_read_asymmetry(rpu_tile_t *tile, int backward, const float *factors_host) {
  return guarded([&] {
    if (!tile || !factors_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    std::vector<float> &v = read_asymmetry_of(t, backward);
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_last(); // a call in flight may still read the device copy that the next call replaces
    }
    std::memcpy(v.data(), factors_host, v.size() * sizeof(float));
    t.line_valid[backward ? 1 : 0][3] = false;
  });
}

int rpu_tile_pulse_counter_count(const rpu_tile_t *tile) {
  return (tile && !tile->t.is_transfer() && tile->t.dev.pulsed() && tile->t.dev.p.count_pulses) ? 2 : 0;
}

int rpu_tile_get_pulse_counters(rpu_tile_t *tile, uint64_t *counters_host) {
  return guarded([&] {
    if (!tile || !counters_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!rpu_tile_pulse_counter_count(tile)) throw RpuError("The tile does not count pulses (count_pulses).");
    const size_t bytes = 2 * t.size() * sizeof(uint64_t);
    if (!t.resident() || !t.d_cnt.p) {
      std::memset(counters_host, 0, bytes); // nothing counted yet
      return;
    }
    DeviceGuard g(t.device_id);
    t.sync_last();
    RPU_HIP_CHECK(hipMemcpy(counters_host, t.d_cnt.p, bytes, hipMemcpyDeviceToHost));
  });
}

int rpu_tile_set_forward_out_scale(rpu_tile_t *tile, float out_scale) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.fio.p.out_scale = out_scale;
  });
}

int rpu_tile_set_shared_weights(rpu_tile_t *tile, float *weights_dev) {
  RPU_MAINTENANCE_ENTRY_NOSYNC(t.set_shared_weights(weights_dev));
}

int rpu_tile_get_shared_weights_if(const rpu_tile_t *tile) {
  return (tile && (!tile->t.d_w.owned || tile->t.shared_xd)) ? 1 : 0;
}

int rpu_tile_set_shared_weights_xd(rpu_tile_t *tile, float *weights_xd_dev) {
  RPU_MAINTENANCE_ENTRY_NOSYNC(t.set_shared_weights_xd(weights_xd_dev));
}

int rpu_tile_set_delta_weights_xd(rpu_tile_t *tile, float *delta_weights_xd_dev) {
  RPU_MAINTENANCE_ENTRY_NOSYNC(t.set_delta_weights_xd(delta_weights_xd_dev));
}

int rpu_tile_set_delta_weights(rpu_tile_t *tile, float *delta_weights_dev) {
  RPU_MAINTENANCE_ENTRY_NOSYNC(t.set_delta_weights(delta_weights_dev));
}
#undef RPU_MAINTENANCE_ENTRY

// The state beyond weights and device parameters that decides what the next calls compute: the seed and the
// call counter of the random streams, the update counters and, for a transfer compound, its transfer counters.
static int64_t float_bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, sizeof(u));
  return (int64_t)u;
}
static float bits_float(int64_t b) {
  const uint32_t u = (uint32_t)b;
  float v;
  std::memcpy(&v, &u, sizeof(v));
  return v;
}
constexpr int kFixedExtras = 6;

// floats travel as their bit patterns
static void extra_fields(const Tile &t, std::vector<std::string> &names, std::vector<int64_t> &values) {
  names = {"seed", "call", "update_calls", "transfer.update_idx", "nm_running_average.bits", "drift_time.bits"};
  values = {(int64_t)t.seed, (int64_t)t.call, (int64_t)t.update_calls, (int64_t)t.update_idx, float_bits(t.nm_aux_host),
            float_bits(t.drift_t)};
  for (size_t k = 0; k < t.slice_idx.size(); ++k) {
    names.push_back("transfer.slice_idx_" + std::to_string(k));
    values.push_back(t.slice_idx[k]);
  }
  // per-line values of the periphery (the reference's "fwd.v_offset", "fwd.out_nonlinearity", ... entries,
  // rpu_forward_backward_pass.cpp:62-80), one entry per line
  const auto lines = [&](const char *prefix, const char *what, const std::vector<float> &v) {
    for (size_t k = 0; k < v.size(); ++k) {
      names.push_back(std::string(prefix) + what + "_" + std::to_string(k) + ".bits");
      values.push_back(float_bits(v[k]));
    }
  };
  const IOPar *ios[3] = {&t.fio, &t.bio, t.tr ? &t.tr->io : nullptr};
  const char *prefixes[3] = {"fwd.", "bwd.", "transfer.io."};
  for (int dir = 0; dir < 3; ++dir) {
    if (!ios[dir]) continue;
    lines(prefixes[dir], "v_offset", ios[dir]->v_offset);
    lines(prefixes[dir], "out_nonlinearity", ios[dir]->out_nl);
    lines(prefixes[dir], "out_noise_values", ios[dir]->out_noise_values);
  }
}
static size_t line_entries(const Tile &t) {
  size_t n = t.fio.v_offset.size() + t.fio.out_nl.size() + t.fio.out_noise_values.size() + t.bio.v_offset.size() +
             t.bio.out_nl.size() + t.bio.out_noise_values.size();
  if (t.tr) n += t.tr->io.v_offset.size() + t.tr->io.out_nl.size() + t.tr->io.out_noise_values.size();
  return n;
}
static thread_local std::string g_extra_name;

int rpu_tile_extra_count(const rpu_tile_t *tile) {
  return tile ? kFixedExtras + (int)tile->t.slice_idx.size() + (int)line_entries(tile->t) : 0;
}

const char *rpu_tile_extra_name(const rpu_tile_t *tile, int idx) {
  if (!tile || idx < 0 || idx >= rpu_tile_extra_count(tile)) return nullptr;
  std::vector<std::string> names;
  std::vector<int64_t> values;
  extra_fields(tile->t, names, values);
  g_extra_name = names[idx];
  return g_extra_name.c_str();
}

int rpu_tile_get_extra(rpu_tile_t *tile, int64_t *values_host) {
  return guarded([&] {
    if (!tile || !values_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    std::vector<std::string> names;
    std::vector<int64_t> values;
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_nm_aux(true);
    }
    extra_fields(t, names, values);
    std::memcpy(values_host, values.data(), values.size() * sizeof(int64_t));
  });
}

int rpu_tile_set_extra(rpu_tile_t *tile, const int64_t *values_host, int count) {
  return guarded([&] {
    if (!tile || !values_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (count != rpu_tile_extra_count(tile)) throw RpuError("Extra state of a different tile layout.");
    t.seed = (uint64_t)values_host[0];
    t.call = (uint32_t)values_host[1];
    t.update_calls = (uint32_t)values_host[2];
    t.update_idx = (uint64_t)values_host[3];
    t.nm_aux_host = bits_float(values_host[4]);
    t.drift_t = bits_float(values_host[5]);
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_nm_aux(false);
    }
    for (size_t k = 0; k < t.slice_idx.size(); ++k) t.slice_idx[k] = (int)values_host[kFixedExtras + k];
    size_t at = kFixedExtras + t.slice_idx.size();
    IOPar *ios[3] = {&t.fio, &t.bio, t.tr ? &t.tr->io : nullptr};
    for (int dir = 0; dir < 3; ++dir) {
      if (!ios[dir]) continue;
      for (std::vector<float> *v : {&ios[dir]->v_offset, &ios[dir]->out_nl, &ios[dir]->out_noise_values}) {
        for (float &x : *v) x = bits_float(values_host[at++]);
      }
      ios[dir]->set_nl_factor();
      for (bool &valid : t.line_valid[dir]) valid = false;
    }
  });
}

// ---- grouped forward over several tiles ------------------------------------------------------------

struct rpu_group {
  std::vector<rpu_tile *> tiles;
  int device_id = -1;
  DevBuf<MvmArgs> d_args;
  DevBuf<int> d_start;
  MvmArgs *h_args = nullptr; // pinned staging
  int *h_start = nullptr;
  hipEvent_t copied = nullptr;
  // host-visible pairs (any tile listed a sample for round 1, batch), one per kernel variant of the group's last call:
  // the next call runs the rounds after round 0 in one launch where nothing was listed
  int *seen_host = nullptr, *seen_dev = nullptr;
  // the word after the pairs: 1 + the round at which a wait between the workgroups of a merged-round launch gave up;
  // reported by the next call, after which the group runs one launch per round
  bool merged_off = false;
  int wait_spins_hook = 0, wait_extra_hook = 0;
  int cu_count = 0;
  // quantized rows of rounds 0 and 1 shared by tiles that read the same input with the same DAC (two buffers per set)
  std::vector<DevBuf<float>> first_rows;
  int shared_sets = 0, shared_tiles = 0; // of the last call
  // grouped update: the tiles' argument blocks and the workgroup tables of its launches
  DevBuf<UpdateArgs> d_uargs;
  DevBuf<int> d_ustart;
  UpdateArgs *h_uargs = nullptr; // pinned staging
  int *h_ustart = nullptr;
  std::mutex mutex;
  ~rpu_group() {
    if (device_id >= 0) {
      try {
        DeviceGuard g(device_id);
        if (copied) {
          (void)hipEventSynchronize(copied);
          (void)hipEventDestroy(copied);
        }
        if (h_args) (void)hipHostFree(h_args);
        if (h_start) (void)hipHostFree(h_start);
        if (seen_host) (void)hipHostFree(seen_host);
        if (h_uargs) (void)hipHostFree(h_uargs);
        if (h_ustart) (void)hipHostFree(h_ustart);
        d_uargs.release();
        d_ustart.release();
        d_args.release();
        d_start.release();
        for (auto &b : first_rows) b.release();
      } catch (...) {
      }
    }
  }
};

int rpu_group_create(rpu_group_t **out, rpu_tile_t *const *tiles, int n_tiles) {
  return guarded([&] {
    if (!out || !tiles || n_tiles <= 0) throw RpuError("null or empty tile list");
    auto g = std::make_unique<rpu_group>();
    for (int i = 0; i < n_tiles; ++i) {
      if (!tiles[i]) throw RpuError("null tile in the list");
      for (int j = 0; j < i; ++j) {
        if (tiles[j] == tiles[i]) throw RpuError("A tile may be in a group only once.");
      }
      Tile &t = tiles[i]->t;
      if (!t.resident()) throw RpuError("All tiles of a group must be resident on a GPU.");
      if (t.shared_xd) throw RpuError("A tile that mirrors its weights into a shared tensor cannot be in a group.");
      if (g->device_id < 0) g->device_id = t.device_id;
      if (t.device_id != g->device_id) throw RpuError("All tiles of a group must be on the same GPU.");
      g->tiles.push_back(tiles[i]);
    }
    DeviceGuard dg(g->device_id);
    const size_t n = (size_t)n_tiles;
    g->d_args.ensure(n);
    g->d_start.ensure(3 * n + 4);
    RPU_HIP_CHECK(hipHostMalloc((void **)&g->h_args, n * sizeof(MvmArgs), hipHostMallocDefault));
    RPU_HIP_CHECK(hipHostMalloc((void **)&g->h_start, (3 * n + 4) * sizeof(int), hipHostMallocDefault));
    RPU_HIP_CHECK(hipEventCreateWithFlags(&g->copied, hipEventDisableTiming));
    *out = g.release();
  });
}

// Stochastic pulsed update of all tiles of a group: one set-up launch, one launch for the pulse trains and one update
// launch per kernel variant among the tiles (device step, noise, columns per lane), instead of three launches per tile
int rpu_group_update_strided(rpu_group_t *group, const float *const *x_dev, const long *x_ld, const float *const *d_dev,
                             const long *d_ld, int m_batch, void *stream) {
  return guarded([&] {
    if (!group || !x_dev || !d_dev) throw RpuError("null argument");
    if (m_batch < 0) throw RpuError("m_batch must not be negative.");
    if (m_batch == 0) return;
    std::lock_guard<std::mutex> glock(group->mutex);
    DeviceGuard dg(group->device_id);
    hipStream_t s = (hipStream_t)stream;
    const int n = (int)group->tiles.size();
    if (!group->h_uargs) {
      // per tile the arguments of the kernels that make the lines and, after those of all tiles, the view that the
      // cross-point kernels take (the same, or with x and d exchanged for a tile that stores [x_size][d_size])
      group->d_uargs.ensure(2 * (size_t)n);
      group->d_ustart.ensure(2 * (size_t)n + 16);
      RPU_HIP_CHECK(hipHostMalloc((void **)&group->h_uargs, 2 * (size_t)n * sizeof(UpdateArgs), hipHostMallocDefault));
      RPU_HIP_CHECK(hipHostMalloc((void **)&group->h_ustart, (2 * (size_t)n + 16) * sizeof(int), hipHostMallocDefault));
    }
    // the staging buffers may still feed the copy of the previous call
    RPU_HIP_CHECK(hipEventSynchronize(group->copied));
    ensure_update_tables();

    // every tile is checked before any tile's call counter moves
    for (int i = 0; i < n; ++i) {
      Tile &t = group->tiles[i]->t;
      std::lock_guard<std::mutex> lock(t.mutex);
      (void)t.check_compute(m_batch, x_dev[i], d_dev[i]);
      if (const char *why = t.group_update_obstacle()) {
        throw RpuError(std::string("The grouped update runs the plain stochastic pulsed update (") + why +
                       "): call this tile's own update.");
      }
      if ((x_ld && x_ld[i] < t.X) || (d_ld && d_ld[i] < t.D)) throw RpuError("A row stride is shorter than the row.");
    }
    std::vector<UpdateArgs> args, views;
    std::vector<int> variant;
    for (int i = 0; i < n; ++i) {
      Tile &t = group->tiles[i]->t;
      std::lock_guard<std::mutex> lock(t.mutex);
      const long xl = x_ld ? x_ld[i] : t.X, dl = d_ld ? d_ld[i] : t.D;
      if (t.lr == 0.0f) continue; // as the tile's own update: nothing happens, no random-stream index is used
      int wps = 1;
      UpdateArgs a = t.group_update_args(x_dev[i], xl, d_dev[i], dl, m_batch, s, wps);
      a.words_per_sample = 1;
      t.note_pulsed_update(a, m_batch, 1, RPU_PULSE_STOCHASTIC_COMPRESSED, s);
      args.push_back(a);
      UpdateArgs v = a;
      if (t.xd) { // the pulse loop runs on row-major copies (Tile::r_wmax); here the copy of the weights is a launch of its own
        t.row_major_pulse_loop(v);
        launch_transpose(t.d_w.p, t.u_wrm.p, t.X, t.D, s);
      }
      views.push_back(v);
      variant.push_back(update_pulsed_variant(views.back()));
    }
    const int m = (int)args.size();
    if (m == 0) return;
    // tiles that share a kernel variant sit next to each other
    std::vector<int> order(m);
    for (int i = 0; i < m; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return variant[a] < variant[b]; });
    long lines_blocks_16 = 0;
    for (int i = 0; i < m; ++i) lines_blocks_16 += update_lines_blocks(args[i], true);
    const bool wide_lines = lines_blocks_16 * ((m_batch + 63) / 64) >= 256;
    int cursor = 0, blocks = 0;
    const int lines_offset = cursor;
    for (int i = 0; i < m; ++i) {
      group->h_ustart[cursor++] = blocks;
      blocks += update_lines_blocks(args[order[i]], wide_lines);
    }
    group->h_ustart[cursor++] = blocks;
    struct Segment { int first, count, variant, start_offset, workgroups; };
    std::vector<Segment> segments;
    for (int i = 0; i < m;) {
      Segment seg{i, 0, variant[order[i]], cursor, 0};
      int wg = 0, j = i;
      for (; j < m && variant[order[j]] == seg.variant; ++j) {
        group->h_ustart[cursor++] = wg;
        wg += update_pulsed_workgroups(views[order[j]]);
      }
      group->h_ustart[cursor++] = wg;
      seg.count = j - i;
      seg.workgroups = wg;
      segments.push_back(seg);
      i = j;
    }
    for (int i = 0; i < m; ++i) {
      group->h_uargs[i] = args[order[i]];
      group->h_uargs[m + i] = views[order[i]];
    }
    RPU_HIP_CHECK(hipMemcpyAsync(group->d_uargs.p, group->h_uargs, 2 * (size_t)m * sizeof(UpdateArgs), hipMemcpyHostToDevice, s));
    RPU_HIP_CHECK(hipMemcpyAsync(group->d_ustart.p, group->h_ustart, (size_t)cursor * sizeof(int), hipMemcpyHostToDevice, s));
    RPU_HIP_CHECK(hipEventRecord(group->copied, s));

    UpdateGroup all{group->d_uargs.p, group->d_ustart.p + lines_offset, m, m_batch};
    launch_update_prepare_group(all, s);
    launch_update_lines_group(all, wide_lines, blocks, s);
    for (const Segment &seg : segments) {
      UpdateGroup g{group->d_uargs.p + m + seg.first, group->d_ustart.p + seg.start_offset, seg.count, m_batch};
      launch_update_pulsed_group(g, seg.variant, seg.workgroups, s);
    }
    RPU_HIP_CHECK(hipGetLastError());
  });
}

int rpu_group_get_shared_input_sets(rpu_group_t *group, int *n_sets, int *n_tiles) {
  return guarded([&] {
    if (!group) throw RpuError("null argument");
    std::lock_guard<std::mutex> glock(group->mutex);
    if (n_sets) *n_sets = group->shared_sets;
    if (n_tiles) *n_tiles = group->shared_tiles;
  });
}

int rpu_group_destroy(rpu_group_t *group) {
  return guarded([&] { delete group; });
}

static int group_mvm(rpu_group_t *group, const float *const *x_dev, const long *x_ld, float *const *y_dev,
                     const long *y_ld, int m_batch, bool transposed, bool is_test, void *stream);

int rpu_group_forward(rpu_group_t *group, const float *const *x_dev, float *const *y_dev, int m_batch, int is_test,
                      void *stream) {
  return rpu_group_forward_strided(group, x_dev, nullptr, y_dev, nullptr, m_batch, is_test, stream);
}

int rpu_group_forward_strided(rpu_group_t *group, const float *const *x_dev, const long *x_ld, float *const *y_dev,
                              const long *y_ld, int m_batch, int is_test, void *stream) {
  return group_mvm(group, x_dev, x_ld, y_dev, y_ld, m_batch, false, is_test != 0, stream);
}

int rpu_group_backward_strided(rpu_group_t *group, const float *const *d_dev, const long *d_ld, float *const *x_dev,
                               const long *x_ld, int m_batch, void *stream) {
  return group_mvm(group, d_dev, d_ld, x_dev, x_ld, m_batch, true, false, stream);
}

// forward (inputs x, outputs y) or backward (inputs d, outputs x) of all tiles of a group
static int group_mvm(rpu_group_t *group, const float *const *x_dev, const long *x_ld, float *const *y_dev,
                     const long *y_ld, int m_batch, bool transposed, bool is_test, void *stream) {
  return guarded([&] {
    if (!group || !x_dev || !y_dev) throw RpuError("null argument");
    if (m_batch < 0) throw RpuError("m_batch must not be negative.");
    if (m_batch == 0) return;
    std::lock_guard<std::mutex> glock(group->mutex);
    DeviceGuard dg(group->device_id);
    hipStream_t s = (hipStream_t)stream;
    const int n = (int)group->tiles.size();
    constexpr int kSeenPairs = 16;
    if (group->seen_host && *(volatile int *)&group->seen_host[2 * kSeenPairs]) {
      const int failed = *(volatile int *)&group->seen_host[2 * kSeenPairs];
      *(volatile int *)&group->seen_host[2 * kSeenPairs] = 0;
      group->merged_off = true;
      throw RpuError("forward round barrier timed out in round " + std::to_string(failed - 1) +
                     "; results of the group's last forward call are invalid (the group now runs one launch per round).");
    }
    // Tiles whose pass has terms that the group launches do not carry (the periphery terms before the ADC: weight noise
    // referred to the output, IR drop, per-line offsets and non-linearities, separate passes for the two input signs;
    // running-average noise management, a recurrence over the batch): the call runs the tiles one after the other on
    // the stream, each with its own launches -- same results as rpu_tile_forward / rpu_tile_backward on each tile.
    {
      bool one_by_one = false;
      for (int i = 0; i < n && !one_by_one; ++i) {
        const Tile &t = group->tiles[i]->t;
        const IOPar &gio = transposed ? t.bio : t.fio;
        one_by_one = Tile::has_pre_adc_terms(gio) ||
                     (!gio.perfect && (gio.p.noise_management == RPU_NM_AVERAGE_ABS_MAX ||
                                       gio.p.noise_management == RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE));
      }
      if (one_by_one) {
        for (int i = 0; i < n; ++i) {
          Tile &t = group->tiles[i]->t;
          std::lock_guard<std::mutex> lock(t.mutex);
          (void)t.check_compute(m_batch, x_dev[i], y_dev[i]);
          if (t.shared_xd) throw RpuError("A tile that mirrors its weights into a shared tensor cannot be in a group.");
          const int in_size = transposed ? t.D : t.X, out_size = transposed ? t.X : t.D;
          const long in_ld = x_ld ? x_ld[i] : in_size, out_ld = y_ld ? y_ld[i] : out_size;
          if (in_ld < in_size || out_ld < out_size) throw RpuError("A row stride is shorter than the row.");
          t.mvm(x_dev[i], y_dev[i], m_batch, false, false, false, transposed, s, nullptr, nullptr, is_test,
                in_ld == in_size ? 0 : in_ld, nullptr, out_ld == out_size ? 0 : out_ld);
          t.last_stream = s;
          if (!transposed) t.last_forward_batch = m_batch;
        }
        group->shared_sets = group->shared_tiles = 0;
        return;
      }
    }
    // the staging buffers may still feed the copy of the previous call
    RPU_HIP_CHECK(hipEventSynchronize(group->copied));

    // a batch of 1024 or more on tiles at least 128 outputs wide: the large-tile kernel runs round 0 of those tiles,
    // if the group has enough of its workgroups to fill the chip
    int big_total = 0, big_bb = 128;
    if (m_batch >= 1024) {
      if (group->cu_count == 0) {
        hipDeviceProp_t prop;
        RPU_HIP_CHECK(hipGetDeviceProperties(&prop, group->device_id));
        group->cu_count = prop.multiProcessorCount;
      }
      int total_128 = 0, total_64 = 0;
      for (int i = 0; i < n; ++i) {
        MvmArgs shape{};
        shape.O = transposed ? group->tiles[i]->t.X : group->tiles[i]->t.D;
        shape.m_batch = m_batch;
        total_128 += mvm_big_workgroups(shape, 128);
        total_64 += mvm_big_workgroups(shape, 64);
      }
      big_bb = mvm_big_sample_tile(total_128, group->cu_count);
      big_total = big_bb == 128 ? total_128 : total_64;
    }
    // with the half tiles, one workgroup on every second CU already beats the 32 x 32 kernel
    const bool use_big = big_total >= (big_bb == 128 ? 256 : 128);
    bool all_big = use_big;
    // per tile: arguments of a plain forward call (row-major x [m_batch][x_size], y [m_batch][d_size])
    std::vector<MvmArgs> args(n);
    std::vector<int> depth(n), mode(n);
    int rounds = 1;
    bool storage_xd = false;
    for (int i = 0; i < n; ++i) {
      Tile &t = group->tiles[i]->t;
      std::lock_guard<std::mutex> lock(t.mutex);
      (void)t.check_compute(m_batch, x_dev[i], y_dev[i]);
      if (t.shared_xd) throw RpuError("A tile that mirrors its weights into a shared tensor cannot be in a group.");
      if (i == 0) storage_xd = t.xd;
      if (t.xd != storage_xd) throw RpuError("The tiles of a group must store their weights the same way (all bound to [x_size, d_size] tensors, or none).");
      const int in_size = transposed ? t.D : t.X, out_size = transposed ? t.X : t.D;
      const bool big = use_big && out_size >= 128;
      MvmArgs a = t.mvm_args(m_batch, transposed, t.mvm_weights(is_test), transposed ? t.bio : t.fio, big ? 1 : 0);
      a.in = x_dev[i]; a.in_sb = x_ld ? x_ld[i] : in_size; a.in_sk = 1;
      a.out = y_dev[i]; a.out_sb = y_ld ? y_ld[i] : out_size; a.out_so = 1;
      if (a.in_sb < in_size || a.out_sb < out_size) throw RpuError("A row stride is shorter than the row.");
      a.big_from = big ? -1 : 0;
      if (!big) all_big = false;
      mvm_round_variant(a, depth[i], mode[i]);
      rounds = std::max(rounds, a.max_rounds);
      args[i] = a;
      t.last_stream = s;
      if (!transposed) t.last_forward_batch = m_batch;
    }
    // Tiles that quantize the same input the same way (the column blocks of a layer that was split over several
    // tiles) share the rows of rounds 0 and 1: one of them writes the rows, all of them read them.  Rows of later
    // rounds sit at list positions that differ from tile to tile and stay in each tile's own scratch.
    {
      auto shares = [](const MvmArgs &a) {
        if (a.io.perfect) return true;
        if (a.io.inp_noise > 0.0f || a.io.inp_sto_round) return false; // random streams are the tile's own
        return a.max_rounds <= 1 || (a.rows_ahead_in_init && (a.speculate || a.big_from < 0));
      };
      auto same_rows = [](const MvmArgs &a, const MvmArgs &b) {
        const IoDev &p = a.io, &q = b.io;
        return a.in == b.in && a.in_sb == b.in_sb && a.in_sk == b.in_sk && a.K == b.K && a.k_pad == b.k_pad &&
               a.max_rounds == b.max_rounds && a.rows_ahead_in_init == b.rows_ahead_in_init && p.perfect == q.perfect &&
               (p.perfect || (p.inp_res == q.inp_res && p.inp_bound == q.inp_bound && p.inp_asym == q.inp_asym &&
                              p.nm_thres == q.nm_thres && p.max_bm_res == q.max_bm_res &&
                              p.max_bm_factor == q.max_bm_factor && p.noise_management == q.noise_management &&
                              p.bound_management == q.bound_management &&
                              (p.out_scale != 0.0f) == (q.out_scale != 0.0f) &&
                              // the output range enters the input scale only through the worst-case estimate
                              (!(p.noise_management == RPU_NM_ABS_MAX_NP_SUM ||
                                 p.bound_management == RPU_BM_ITERATIVE_WORST_CASE) ||
                               (p.nm_assumed_wmax == q.nm_assumed_wmax &&
                                ((std::isinf(p.out_bound) && std::isinf(q.out_bound)) || p.out_bound == q.out_bound)))));
      };
      std::vector<int> first_of; // first tile of each set
      std::vector<int> set_of(n, -1), members;
      for (int i = 0; i < n; ++i) {
        if (!shares(args[i])) continue;
        for (size_t c = 0; c < first_of.size() && set_of[i] < 0; ++c) {
          if (same_rows(args[i], args[first_of[c]])) set_of[i] = (int)c;
        }
        if (set_of[i] < 0) {
          set_of[i] = (int)first_of.size();
          first_of.push_back(i);
          members.push_back(0);
        }
        ++members[set_of[i]];
      }
      if (group->first_rows.size() < 2 * first_of.size()) group->first_rows.resize(2 * first_of.size());
      group->shared_sets = group->shared_tiles = 0;
      for (size_t c = 0; c < members.size(); ++c) {
        if (members[c] >= 2) {
          ++group->shared_sets;
          group->shared_tiles += members[c];
        }
      }
      for (int i = 0; i < n; ++i) {
        const int c = set_of[i];
        if (c < 0 || members[c] < 2) continue;
        MvmArgs &a = args[i];
        DevBuf<float> &r0 = group->first_rows[2 * c], &r1 = group->first_rows[2 * c + 1];
        r0.ensure((size_t)m_batch * a.k_pad);
        if (a.max_rounds > 1) r1.ensure((size_t)m_batch * a.k_pad);
        a.xq_first[0] = r0.p;
        a.xq_first[1] = a.max_rounds > 1 ? r1.p : nullptr;
        a.xq_first_writer = first_of[c] == i ? 1 : 0;
      }
    }
    // tiles that share a kernel variant sit next to each other
    std::vector<int> order(n);
    for (int i = 0; i < n; ++i) order[i] = i;
    std::stable_sort(order.begin(), order.end(),
                     [&](int a, int b) { return depth[a] * 4 + mode[a] < depth[b] * 4 + mode[b]; });
    struct Segment { int first, count, depth, mode, start_offset, workgroups; };
    std::vector<Segment> segments;
    int cursor = 0; // position in h_start
    for (int i = 0; i < n;) {
      Segment seg{i, 0, depth[order[i]], mode[order[i]], cursor, 0};
      int wg = 0;
      int j = i;
      for (; j < n && depth[order[j]] == seg.depth && mode[order[j]] == seg.mode; ++j) {
        group->h_start[cursor++] = wg;
        wg += mvm_round_workgroups(args[order[j]]);
      }
      group->h_start[cursor++] = wg;
      seg.count = j - i;
      seg.workgroups = wg;
      segments.push_back(seg);
      i = j;
    }
    const int big_offset = cursor; // table of the large-tile launch over all tiles, in the order of d_args
    if (use_big) {
      int wg = 0;
      for (int i = 0; i < n; ++i) {
        group->h_start[cursor++] = wg;
        if (args[order[i]].big_from != 0) wg += mvm_big_workgroups(args[order[i]], big_bb);
      }
      group->h_start[cursor++] = wg;
    }
    for (int i = 0; i < n; ++i) group->h_args[i] = args[order[i]];
    RPU_HIP_CHECK(hipMemcpyAsync(group->d_args.p, group->h_args, (size_t)n * sizeof(MvmArgs), hipMemcpyHostToDevice, s));
    RPU_HIP_CHECK(hipMemcpyAsync(group->d_start.p, group->h_start, (size_t)cursor * sizeof(int), hipMemcpyHostToDevice, s));
    RPU_HIP_CHECK(hipEventRecord(group->copied, s));

    MvmGroup all{group->d_args.p, nullptr, n, m_batch};
    int max_k = 0;
    for (int i = 0; i < n; ++i) max_k = std::max(max_k, args[i].K);
    launch_mvm_init_group(all, max_k, s);
    if (!group->seen_host) {
      RPU_HIP_CHECK(hipHostMalloc((void **)&group->seen_host, (2 * kSeenPairs + 1) * sizeof(int), hipHostMallocMapped));
      for (int i = 0; i < 2 * kSeenPairs + 1; ++i) group->seen_host[i] = 0;
      RPU_HIP_CHECK(hipHostGetDevicePointer((void **)&group->seen_dev, group->seen_host, 0));
      hipDeviceProp_t prop;
      RPU_HIP_CHECK(hipGetDeviceProperties(&prop, group->device_id));
      group->cu_count = prop.multiProcessorCount;
    }
    std::vector<bool> merged(segments.size(), false);
    for (int r = 0; r < rounds; ++r) {
      if (use_big && r == 0) {
        MvmGroup g{group->d_args.p, group->d_start.p + big_offset, n, m_batch};
        launch_mvm_big_group(g, big_total, big_bb, transposed != storage_xd, s);
        if (all_big) continue;
      }
      for (size_t k = 0; k < segments.size(); ++k) {
        const Segment &seg = segments[k];
        if (merged[k]) continue;
        MvmGroup g{group->d_args.p + seg.first, group->d_start.p + seg.start_offset, seg.count, m_batch};
        int *seen = k < (size_t)kSeenPairs ? group->seen_dev + 2 * k : nullptr;
        // the last call of this group listed nothing for round 1: one launch for all rounds after round 0
        const int rest_wgs = (r == 1 && rounds >= 3) ? std::min(256, mvm_group_rest_resident_limit(seg.mode)) : 0;
        if (rest_wgs > 0 && seen && !transposed && !group->merged_off && mvm_group_can_merge_rest(g, seg.mode) &&
            *(volatile int *)&group->seen_host[2 * k + 1] == m_batch && *(volatile int *)&group->seen_host[2 * k] == 0) {
          g.wait_spins = group->wait_spins_hook;
          g.wait_extra = group->wait_extra_hook;
          g.wait_failed = group->seen_dev + 2 * kSeenPairs;
          launch_mvm_rest_group(g, seg.mode, 1, rounds, rest_wgs, seen, s);
          merged[k] = true;
          continue;
        }
        launch_mvm_round_group(g, seg.depth, seg.mode, seg.workgroups, r, s, seen);
      }
    }
    RPU_HIP_CHECK(hipGetLastError());
  });
}

int rpu_pcm_noise_params_default(rpu_pcm_noise_params *p) {
  return guarded([&] {
    if (!p) throw RpuError("null argument");
    rpu_pcm_noise_params q{};
    q.g_max = 25.0f; q.g_min = 0.0f; q.t_read = 250.0e-9f; q.t_0 = 20.0f;
    q.prog_noise_scale = 1.0f; q.read_noise_scale = 1.0f; q.drift_scale = 1.0f;
    q.prog_coeff[0] = 0.26348f; q.prog_coeff[1] = 1.9650f; q.prog_coeff[2] = -1.1731f;
    q.prog_coeff_g_max_reference = 25.0f;
    *p = q;
  });
}

int rpu_tile_program_weights(rpu_tile_t *tile, const rpu_pcm_noise_params *p, int from_reference, void *stream) {
  return guarded([&] {
    if (!tile || !p) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident()) throw RpuError("Tile is not resident on a GPU.");
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.program_weights(*p, from_reference != 0, (hipStream_t)stream);
    t.shared_out((hipStream_t)stream);
  });
}

int rpu_tile_drift_weights(rpu_tile_t *tile, const rpu_pcm_noise_params *p, float t_inference, void *stream) {
  return guarded([&] {
    if (!tile || !p) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident()) throw RpuError("Tile is not resident on a GPU.");
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.drift_weights(*p, t_inference, (hipStream_t)stream);
    t.shared_out((hipStream_t)stream);
  });
}

int rpu_tile_get_drift_state(rpu_tile_t *tile, float *programmed_host, float *nu_plus_host, float *nu_minus_host) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || !t.programmed) throw RpuError("The weights have not been programmed.");
    DeviceGuard g(t.device_id);
    t.sync_last();
    const size_t bytes = t.size() * sizeof(float);
    (void)bytes;
    if (programmed_host) t.download_mat(programmed_host, t.i_prog.p);
    if (nu_plus_host) t.download_mat(nu_plus_host, t.i_nu_plus.p);
    if (nu_minus_host) t.download_mat(nu_minus_host, t.i_nu_minus.p);
  });
}

int rpu_tile_drift_readout(rpu_tile_t *tile, float *mean_abs_host, void *stream) {
  return guarded([&] {
    if (!tile || !mean_abs_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident()) throw RpuError("Tile is not resident on a GPU.");
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    *mean_abs_host = t.drift_readout((hipStream_t)stream);
  });
}

int rpu_tile_get_transfer_state(rpu_tile_t *tile, uint64_t *update_idx, int32_t *slice_indices_host) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.is_transfer()) throw RpuError("Not a transfer compound.");
    if (update_idx) *update_idx = t.update_idx;
    if (slice_indices_host) {
      for (int k = 0; k < t.tr->n(); ++k) slice_indices_host[k] = t.slice_idx[k];
    }
  });
}

int rpu_tile_clone(rpu_tile_t **out, const rpu_tile_t *src_c) {
  return guarded([&] {
    if (!out || !src_c) throw RpuError("null argument");
    rpu_tile *src = const_cast<rpu_tile *>(src_c);
    std::lock_guard<std::mutex> lock(src->t.mutex);
    auto h = std::make_unique<rpu_tile>();
    Tile &t = h->t;
    const Tile &s = src->t;
    t.X = s.X; t.D = s.D; t.fio = s.fio; t.bio = s.bio; t.up = s.up; t.dev = s.dev; t.arr = s.arr;
    t.lr = s.lr; t.seed = s.seed; t.call = s.call;
    if (s.resident()) {
      DeviceGuard g(s.device_id);
      const_cast<Tile &>(s).sync_nm_aux(true);
    }
    t.nm_aux_host = s.nm_aux_host;
    t.w_host = s.w_host;
    t.idx_host = s.idx_host;
    t.idx_patches = s.idx_patches;
    t.idx_max = s.idx_max;
    t.update_calls = s.update_calls;
    t.update_variant = s.update_variant;
    t.update_variant_samples = s.update_variant_samples;
    t.fused_rounds = s.fused_rounds;
    if (s.is_transfer()) {
      t.tr = std::make_unique<TransferPar>(*s.tr);
      t.update_idx = s.update_idx;
      t.slice_idx = s.slice_idx;
      if (s.resident()) {
        DeviceGuard g(s.device_id);
        RPU_HIP_CHECK(hipStreamSynchronize(s.last_stream));
        const_cast<Tile &>(s).transfer_download();
        t.w_host = s.w_host;
      }
      for (const auto &sl : s.slots) {
        auto c = std::make_unique<DeviceSlot>();
        c->par = sl->par;
        c->arr = sl->arr;
        c->w_host = sl->w_host;
        t.slots.push_back(std::move(c));
      }
      if (s.resident()) t.to_device(s.device_id);
    } else if (s.resident()) {
      DeviceGuard g(s.device_id);
      RPU_HIP_CHECK(hipStreamSynchronize(s.last_stream));
      t.w_host.resize(s.size());
      s.download_mat(t.w_host.data(), s.d_w.p);
      t.to_device(s.device_id);
      // modified weights, drift clocks and pulse counters travel with the copy
      const size_t n = s.size();
      // the copy owns its weights and stores them row-major, whatever the source is bound to
      const auto dup = [&](DevBuf<float> &dst, const DevBuf<float> &from) {
        if (!from.p) return;
        dst.ensure(n);
        if (s.xd) {
          launch_transpose(from.p, dst.p, s.X, s.D, s.last_stream);
          RPU_HIP_CHECK(hipStreamSynchronize(s.last_stream));
        } else {
          RPU_HIP_CHECK(hipMemcpy(dst.p, from.p, n * sizeof(float), hipMemcpyDeviceToDevice));
        }
      };
      dup(t.d_fbw, s.d_fbw);
      dup(t.d_wp, s.d_wp);
      t.fb_during_test = s.fb_during_test;
      dup(t.dr_prev, s.dr_prev);
      dup(t.dr_w0, s.dr_w0);
      dup(t.dr_t, s.dr_t);
      t.drift_t = s.drift_t;
      if (s.d_cnt.p) {
        t.d_cnt.ensure(2 * n);
        RPU_HIP_CHECK(hipMemcpy(t.d_cnt.p, s.d_cnt.p, 2 * n * sizeof(unsigned long long), hipMemcpyDeviceToDevice));
      }
    }
    *out = h.release();
  });
}

int rpu_tile_to_device(rpu_tile_t *tile, int device_id) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.to_device(device_id);
  });
}

int rpu_tile_destroy(rpu_tile_t *tile) {
  return guarded([&] { delete tile; });
}

int rpu_tile_forward(rpu_tile_t *tile, const float *x_dev, float *y_dev, int m_batch, int bias, int x_trans,
                     int d_trans, int is_test, void *stream) {
  // the analog forward pass is the same in training and evaluation (rpu_forward_backward_pass.cpp:816-818); is_test
  // only decides whether modified weights are used
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.check_compute(m_batch, x_dev, y_dev)) return;
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.mvm(x_dev, y_dev, m_batch, bias != 0, x_trans != 0, d_trans != 0, false, (hipStream_t)stream, nullptr, nullptr,
          is_test != 0);
  });
}

int rpu_tile_backward(rpu_tile_t *tile, const float *d_dev, float *x_dev, int m_batch, int bias, int d_trans,
                      int x_trans, void *stream) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.check_compute(m_batch, d_dev, x_dev)) return;
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.mvm(d_dev, x_dev, m_batch, bias != 0, d_trans != 0, x_trans != 0, true, (hipStream_t)stream);
  });
}

int rpu_tile_update(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int m_batch, int bias, int x_trans,
                    int d_trans, void *stream) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.check_compute(m_batch, x_dev, d_dev)) return;
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.update(x_dev, d_dev, m_batch, bias != 0, x_trans != 0, d_trans != 0, (hipStream_t)stream);
    t.shared_out((hipStream_t)stream);
  });
}

int rpu_tile_update_noalloc(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int m_batch, int bias, int x_trans,
                            int d_trans, void *stream) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.check_compute(m_batch, x_dev, d_dev)) return;
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.update_noalloc(x_dev, d_dev, m_batch, bias != 0, x_trans != 0, d_trans != 0, (hipStream_t)stream);
    t.shared_out((hipStream_t)stream);
  });
}

int rpu_tile_update_with_words(rpu_tile_t *tile, const uint32_t *x_words_dev, const uint32_t *d_words_dev, int m_batch,
                               void *stream) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.check_compute(m_batch, x_words_dev, d_words_dev)) return;
    DeviceGuard g(t.device_id);
    t.shared_in((hipStream_t)stream);
    t.update_with_words(x_words_dev, d_words_dev, m_batch, (hipStream_t)stream);
    t.shared_out((hipStream_t)stream);
  });
}

int rpu_tile_get_x_size(const rpu_tile_t *tile) { return tile ? tile->t.X : -1; }
int rpu_tile_get_d_size(const rpu_tile_t *tile) { return tile ? tile->t.D : -1; }
int rpu_tile_is_on_device(const rpu_tile_t *tile) { return (tile && tile->t.resident()) ? 1 : 0; }

int rpu_tile_set_learning_rate(rpu_tile_t *tile, float lr) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.lr = lr;
  });
}
float rpu_tile_get_learning_rate(const rpu_tile_t *tile) { return tile ? tile->t.lr : 0.0f; }

int rpu_tile_set_weights(rpu_tile_t *tile, const float *w_host) {
  return guarded([&] {
    if (!tile || !w_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (t.is_transfer()) {
      if (t.resident()) {
        DeviceGuard g(t.device_id);
        t.sync_last();
        t.transfer_set_weights_host(w_host);
        t.transfer_upload_weights();
      } else {
        t.transfer_set_weights_host(w_host);
      }
      return;
    }
    std::vector<float> w(w_host, w_host + t.size());
    t.clip_host(w);
    // onSetWeights (rpu_pulsed_device.cpp:545-571): with write noise the given weights become the persistent ones and
    // the shown ones are those, with fresh noise if apply_write_noise_on_set
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_last();
      t.upload_mat(t.d_w.p, w.data());
      if (t.persistent()) {
        RPU_HIP_CHECK(hipMemcpy(t.d_wp.p, w.data(), t.size() * sizeof(float), hipMemcpyHostToDevice));
        if (t.dev.p.apply_write_noise_on_set) {
          t.refresh_shown_weights(t.last_stream);
          RPU_HIP_CHECK(hipStreamSynchronize(t.last_stream));
        }
      }
      if (t.shared_xd) {
        t.shared_out(t.last_stream);
        RPU_HIP_CHECK(hipStreamSynchronize(t.last_stream));
      }
    } else {
      if (t.persistent()) {
        t.arr.persistent = w;
        if (t.dev.p.apply_write_noise_on_set) {
          // a host tile draws its noise on the CPU, from the tile's seed and call counter
          std::mt19937 engine((uint32_t)(t.seed ^ (t.seed >> 32)) + 0x9e3779b9u * (++t.call));
          std::normal_distribution<float> normal(0.0f, 1.0f);
          const float std_ = t.dev.scaled_write_noise();
          for (float &v : w) v += std_ * normal(engine);
        }
      }
      t.w_host.swap(w);
    }
  });
}

int rpu_tile_get_weights(rpu_tile_t *tile, float *w_host) {
  return guarded([&] {
    if (!tile || !w_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.shared_in(t.last_stream);
      t.sync_last();
      t.download_mat(w_host, t.wdev());
    } else {
      std::memcpy(w_host, t.w_host.data(), t.size() * sizeof(float));
    }
  });
}

int rpu_tile_weights_device_ptr(rpu_tile_t *tile, float **w_dev) {
  return guarded([&] {
    if (!tile || !w_dev) throw RpuError("null argument");
    *w_dev = tile->t.resident() ? tile->t.wdev() : nullptr;
  });
}

// entry idx of a transfer compound's hidden parameters: (device, index within the device); the index one
// past the device's own arrays is its weight matrix "hidden_weights_k" (rpu_vector_device.cpp:188-203)
static void compound_entry(const Tile &t, int idx, int &device, int &local, int &n_local) {
  device = 0;
  for (const auto &sl : t.slots) {
    n_local = sl->par.linear() ? 10 : 8;
    if (idx <= n_local) {
      local = idx;
      return;
    }
    idx -= n_local + 1;
    ++device;
  }
  device = -1;
}

int rpu_tile_hidden_parameter_count(const rpu_tile_t *tile) {
  if (!tile) return 0;
  if (tile->t.is_transfer()) {
    int n = 0;
    for (const auto &sl : tile->t.slots) n += (sl->par.linear() ? 10 : 8) + 1;
    return n;
  }
  if (!tile->t.dev.pulsed()) return 0;
  return (tile->t.dev.linear() ? 10 : 8) + (tile->t.persistent() ? 1 : 0);
}

// index into kHiddenNames of entry idx of a single tile, or -1 for the persistent weights, which sit between the
// base entries and the slopes (PulsedRPUDevice::getDPNames then LinearStepRPUDevice's, rpu_pulsed_device.cpp:235-253)
static int single_hidden_code(const Tile &t, int idx) {
  if (!t.persistent() || idx < 8) return idx;
  return idx == 8 ? -1 : idx - 1;
}

const char *rpu_tile_hidden_parameter_name(const rpu_tile_t *tile, int idx) {
  if (idx < 0 || idx >= rpu_tile_hidden_parameter_count(tile)) return nullptr;
  if (tile->t.is_transfer()) {
    static thread_local std::string name;
    int device, local, n_local;
    compound_entry(tile->t, idx, device, local, n_local);
    name = std::string(local < n_local ? kHiddenNames[local] : "hidden_weights") + "_" + std::to_string(device);
    return name.c_str();
  }
  const int code = single_hidden_code(tile->t, idx);
  return code < 0 ? "persistent_weights" : kHiddenNames[code];
}

static std::vector<float> *hidden_array(DeviceArrays &arr, int idx) {
  switch (idx) {
  case 0: return &arr.w_max;
  case 1: return &arr.w_min;
  case 2: return &arr.scale_up;
  case 3: return &arr.scale_down;
  case 4: return &arr.decay_scale;
  case 5: return &arr.diffusion_rate;
  case 6: return &arr.reset_bias;
  case 7: return arr.drift_nu.empty() ? nullptr : &arr.drift_nu; // without a drifter reported as zeros
  case 8: return &arr.slope_up;
  case 9: return &arr.slope_down;
  default: return nullptr;
  }
}

static std::vector<float> *hidden_slot(Tile &t, int idx) {
  const int code = single_hidden_code(t, idx);
  return code < 0 ? &t.arr.persistent : hidden_array(t.arr, code);
}

int rpu_tile_get_hidden_parameters(rpu_tile_t *tile, float *data_host) {
  return guarded([&] {
    if (!tile || !data_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    const size_t n = t.size();
    const int count = rpu_tile_hidden_parameter_count(tile);
    if (t.is_transfer()) {
      if (t.resident()) {
        DeviceGuard g(t.device_id);
        t.sync_last();
        t.transfer_download();
      }
      for (int k = 0; k < count; ++k) {
        int device, local, n_local;
        compound_entry(t, k, device, local, n_local);
        DeviceSlot &sl = *t.slots[device];
        std::vector<float> *a = local < n_local ? hidden_array(sl.arr, local) : &sl.w_host;
        if (a) std::memcpy(data_host + (size_t)k * n, a->data(), n * sizeof(float));
        else std::memset(data_host + (size_t)k * n, 0, n * sizeof(float));
      }
      return;
    }
    if (t.persistent()) {
      // the persistent weights live on the GPU while the tile is resident
      t.arr.persistent.resize(n);
      if (t.resident()) {
        DeviceGuard g(t.device_id);
        t.sync_last();
        RPU_HIP_CHECK(hipMemcpy(t.arr.persistent.data(), t.d_wp.p, n * sizeof(float), hipMemcpyDeviceToHost));
      } else if (t.arr.persistent.empty()) {
        t.arr.persistent = t.w_host;
      }
    }
    for (int k = 0; k < count; ++k) {
      std::vector<float> *a = hidden_slot(t, k);
      if (a && a->size() == n) std::memcpy(data_host + (size_t)k * n, a->data(), n * sizeof(float));
      else std::memset(data_host + (size_t)k * n, 0, n * sizeof(float));
    }
  });
}

int rpu_tile_set_hidden_parameters(rpu_tile_t *tile, const float *data_host) {
  return guarded([&] {
    if (!tile || !data_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    const size_t n = t.size();
    const int count = rpu_tile_hidden_parameter_count(tile);
    if (t.is_transfer()) {
      // VectorRPUDevice::setDeviceParameter (rpu_vector_device.cpp:286-325): per device its weights, then its
      // arrays (which clip those weights), then the tile weights are reduced again
      if (t.resident()) {
        DeviceGuard g(t.device_id);
        t.sync_last();
      }
      for (int k = 0; k < count; ++k) {
        int device, local, n_local;
        compound_entry(t, k, device, local, n_local);
        DeviceSlot &sl = *t.slots[device];
        std::vector<float> *a = local < n_local ? hidden_array(sl.arr, local) : &sl.w_host;
        if (a) {
          a->resize(n);
          std::memcpy(a->data(), data_host + (size_t)k * n, n * sizeof(float));
        }
      }
      for (auto &sl : t.slots) sl->clip_host();
      t.transfer_reduce_host();
      if (t.resident()) {
        DeviceGuard g(t.device_id);
        for (auto &sl : t.slots) sl->upload(n, true);
        t.transfer_upload_weights();
      }
      return;
    }
    for (int k = 0; k < count; ++k) {
      std::vector<float> *a = hidden_slot(t, k);
      if (a) {
        a->resize(n);
        std::memcpy(a->data(), data_host + (size_t)k * n, n * sizeof(float));
      }
    }
    // new bounds apply to the current weights at once (rpu_pulsed_device.cpp setDeviceParameter -> onSetWeights);
    // with write noise onSetWeights then takes the clipped shown weights as the persistent ones, whatever was given
    if (t.resident()) {
      DeviceGuard g(t.device_id);
      t.sync_last();
      t.upload_params();
      t.shared_in(t.last_stream);
      launch_clip(t.d_w.p, t.d_wmin.p, t.d_wmax.p, n, t.last_stream);
      if (t.persistent()) {
        RPU_HIP_CHECK(hipMemcpyAsync(t.d_wp.p, t.d_w.p, n * sizeof(float), hipMemcpyDeviceToDevice, t.last_stream));
        if (t.dev.p.apply_write_noise_on_set) t.refresh_shown_weights(t.last_stream);
      }
      t.shared_out(t.last_stream);
      RPU_HIP_CHECK(hipStreamSynchronize(t.last_stream));
    } else {
      t.clip_host(t.w_host);
      if (t.persistent()) t.arr.persistent = t.w_host;
    }
  });
}

int rpu_tile_set_update_variant(rpu_tile_t *tile, int variant, int samples_per_step) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (variant != RPU_UPDATE_VARIANT_EXACT && variant != RPU_UPDATE_VARIANT_AGGREGATED) throw RpuError("Unknown update variant.");
    if (variant == RPU_UPDATE_VARIANT_AGGREGATED) {
      if (t.is_transfer() || !t.dev.linear() || !t.dev.p.ls_mult_noise || t.persistent()) {
        throw RpuError("The aggregated update variant is provided for LinearStep / SoftBounds devices with multiplicative "
                       "noise only (no transfer compound, no write noise).");
      }
      if (samples_per_step < 32 || samples_per_step % 32 != 0) throw RpuError("samples_per_step must be a positive multiple of 32.");
    }
    t.update_variant = variant;
    t.update_variant_samples = samples_per_step;
  });
}

int rpu_tile_set_seed(rpu_tile_t *tile, uint64_t seed) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.seed = seed;
    tile->t.call = 0;
  });
}

int rpu_tile_get_update_words(rpu_tile_t *tile, uint32_t *x_words_host, uint32_t *d_words_host, int32_t *bl_host,
                              int m_batch) {
  return guarded([&] {
    if (!tile || !x_words_host || !d_words_host || !bl_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || t.last_update_pulse != RPU_PULSE_STOCHASTIC_COMPRESSED || m_batch != t.last_update_batch) {
      throw RpuError("No stochastic update of this batch size has run on this tile.");
    }
    DeviceGuard g(t.device_id);
    t.sync_last();
    const size_t rows = (size_t)m_batch * t.last_words_per_sample;
    RPU_HIP_CHECK(hipMemcpy(x_words_host, t.last_xw, rows * t.X * 4, hipMemcpyDeviceToHost));
    RPU_HIP_CHECK(hipMemcpy(d_words_host, t.last_dw, rows * t.D * 4, hipMemcpyDeviceToHost));
    RPU_HIP_CHECK(hipMemcpy(bl_host, t.last_bl, (size_t)m_batch * 4, hipMemcpyDeviceToHost));
  });
}

int rpu_tile_set_fused_rounds(rpu_tile_t *tile, int mode) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    if (mode < -1 || mode > 7 || mode == 4 || mode == 6) {
      throw RpuError("fused rounds: mode must be -1 (by the last calls), 0 (never), 1 (rounds 0 and 1 in one launch whenever "
                     "possible), 2 (the rounds after round 0 in one launch whenever possible), 3 (rounds 0 and 1 in one "
                     "launch and the rounds after them in another), or 5 / 7 (as 1 / 3 with round 2 in the first launch too).");
    }
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.fused_rounds = mode;
    tile->t.merged_off = false; // an explicit choice re-arms the merged launches after a reported time-out
  });
}

long rpu_device_allocation_count(void) { return g_device_allocations.load(std::memory_order_relaxed); }

int rpu_tile_set_round_wait_test_hook(rpu_tile_t *tile, int spin_limit, int extra_arrivals) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    if (spin_limit < 0 || extra_arrivals < 0 || extra_arrivals > 1) throw RpuError("round wait hook: spin_limit >= 0, extra_arrivals 0 or 1");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.wait_spins_hook = spin_limit;
    tile->t.wait_extra_hook = extra_arrivals;
  });
}

int rpu_group_set_round_wait_test_hook(rpu_group_t *group, int spin_limit, int extra_arrivals) {
  return guarded([&] {
    if (!group) throw RpuError("null group");
    if (spin_limit < 0 || extra_arrivals < 0 || extra_arrivals > 1) throw RpuError("round wait hook: spin_limit >= 0, extra_arrivals 0 or 1");
    std::lock_guard<std::mutex> lock(group->mutex);
    group->wait_spins_hook = spin_limit;
    group->wait_extra_hook = extra_arrivals;
  });
}

int rpu_tile_get_update_words_per_sample(rpu_tile_t *tile, int32_t *words_per_sample) {
  return guarded([&] {
    if (!tile || !words_per_sample) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || t.last_update_pulse != RPU_PULSE_STOCHASTIC_COMPRESSED) {
      throw RpuError("No stochastic update has run on this tile.");
    }
    *words_per_sample = t.last_words_per_sample;
  });
}

int rpu_tile_get_update_ab(rpu_tile_t *tile, float *a_host, float *b_host, int m_batch) {
  return guarded([&] {
    if (!tile || !a_host || !b_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || !t.last_a || m_batch != t.last_update_batch || t.last_update_pulse == RPU_PULSE_NONE ||
        t.last_update_pulse == RPU_PULSE_NONE_WITH_DEVICE) {
      throw RpuError("No pulsed update of this batch size has run on this tile.");
    }
    DeviceGuard g(t.device_id);
    t.sync_last();
    RPU_HIP_CHECK(hipMemcpy(a_host, t.last_a, (size_t)m_batch * 4, hipMemcpyDeviceToHost));
    RPU_HIP_CHECK(hipMemcpy(b_host, t.last_b, (size_t)m_batch * 4, hipMemcpyDeviceToHost));
  });
}

int rpu_tile_get_implicit_counts(rpu_tile_t *tile, int32_t *counts_host, int m_batch) {
  return guarded([&] {
    if (!tile || !counts_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || m_batch != t.last_update_batch ||
        (t.last_update_pulse != RPU_PULSE_DETERMINISTIC_IMPLICIT && t.last_update_pulse != RPU_PULSE_MEAN_COUNT)) {
      throw RpuError("No deterministic implicit update of this batch size has run on this tile.");
    }
    DeviceGuard g(t.device_id);
    t.sync_last();
    const size_t total = (size_t)m_batch * t.size();
    DevBuf<int32_t> tmp;
    tmp.ensure(total);
    UpdateArgs a{};
    a.x_size = t.X; a.d_size = t.D; a.m_batch = m_batch;
    a.bl = t.u_bl.p; a.x_val = t.u_xval.p; a.d_val = t.u_dval.p;
    a.up.pulse_type = t.last_update_pulse;
    try {
      launch_implicit_counts(a, tmp.p, t.last_stream);
      RPU_HIP_CHECK(hipStreamSynchronize(t.last_stream));
      RPU_HIP_CHECK(hipMemcpy(counts_host, tmp.p, total * 4, hipMemcpyDeviceToHost));
    } catch (...) {
      tmp.release();
      throw;
    }
    tmp.release();
  });
}

int rpu_tile_get_bm_rounds(rpu_tile_t *tile, int32_t *rounds_host, int m_batch) {
  return guarded([&] {
    if (!tile || !rounds_host) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    if (!t.resident() || m_batch != t.last_forward_batch || t.fio.perfect) {
      throw RpuError("No analog forward pass of this batch size has run on this tile.");
    }
    DeviceGuard g(t.device_id);
    t.sync_last();
    RPU_HIP_CHECK(hipMemcpy(rounds_host, t.s_rounds.p, (size_t)m_batch * 4, hipMemcpyDeviceToHost));
  });
}

int rpu_tile_set_profiling(rpu_tile_t *tile, int enable) {
  return guarded([&] {
    if (!tile) throw RpuError("null tile");
    std::lock_guard<std::mutex> lock(tile->t.mutex);
    tile->t.profiling = enable != 0;
    tile->t.prof_used = 0;
    tile->t.prof_names.clear();
  });
}

int rpu_tile_get_profile(rpu_tile_t *tile, float *ms_host, int capacity, int *count) {
  return guarded([&] {
    if (!tile || !count) throw RpuError("null argument");
    Tile &t = tile->t;
    std::lock_guard<std::mutex> lock(t.mutex);
    const int n = (int)t.prof_names.size();
    *count = n;
    if (n == 0 || !ms_host) return;
    if (capacity < n) throw RpuError("profile buffer too small");
    DeviceGuard g(t.device_id);
    t.sync_last();
    for (int i = 0; i < n; ++i) {
      RPU_HIP_CHECK(hipEventElapsedTime(&ms_host[i], t.prof_events[i], t.prof_events[i + 1]));
    }
  });
}

const char *rpu_tile_profile_name(const rpu_tile_t *tile, int idx) {
  if (!tile || idx < 0 || idx >= (int)tile->t.prof_names.size()) return nullptr;
  return tile->t.prof_names[idx];
}

int rpu_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
  return guarded([&] {
    if (!counter || !key || !out) throw RpuError("null argument");
    const Philox4 r = philox4x32_10(counter[0], counter[1], counter[2], counter[3], key[0], key[1]);
    for (int i = 0; i < 4; ++i) out[i] = r.v[i];
  });
}

int rpu_philox4x32_10_device(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4], int device_id) {
  return guarded([&] {
    if (!counter || !key || !out) throw RpuError("null argument");
    int target = device_id;
    if (target < 0) RPU_HIP_CHECK(hipGetDevice(&target));
    DeviceGuard g(target);
    DevBuf<uint32_t> buf;
    buf.ensure(4);
    hipLaunchKernelGGL(k_philox_probe, dim3(1), dim3(1), 0, nullptr, counter[0], counter[1], counter[2], counter[3],
                       key[0], key[1], buf.p);
    hipError_t e = hipMemcpy(out, buf.p, 16, hipMemcpyDeviceToHost);
    buf.release();
    if (e != hipSuccess) throw RpuError(std::string("HIP error: ") + hipGetErrorString(e));
  });
}

} // extern "C"
