// TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
//
// CPU restatement of the analog-tile semantics of IBM/aihwkit's rpucuda CPU path (forward /
// backward noisy MVM and pulsed update for the Ideal, ConstantStep and LinearStep / SoftBounds
// devices).  It exists so that tests, the smoke check and the cpu_baseline leg of the benchmark have
// something independent of the GPU code to compare against and to time.  Nothing in the shipped
// library links, loads or calls this file.
//
// Every function cites the reference file:line it restates (R/ = src/rpucuda/ of the reference).
// The reference itself cannot be compiled in the build container: all of its translation units include
// R/math_util.h, which needs a cblas.h or mkl.h header that the image does not have, so this file is
// pinned by closed forms, brute force on small cases and invariants (see tests/test_oracle_*.py).
//
// The draw order of the device-to-device parameters in populate_pulsed() / populate_linear_step()
// (R/rpu_pulsed_device.cpp:593-733, R/rpu_linearstep_device.cpp:20-74) is pinned against the raw libstdc++
// stream (tests/rawstream.cpp, tests/test_draw_order_pins.py), cross-point by cross-point.
//
// Layout: weights and all per-device arrays are row-major [d_size][x_size] (R/rpu.h:674).
// Built with -O2 -ffp-contract=off so that every expression is evaluated with the reference's
// operation order in plain fp32.

#include "../include/rpu_amd.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <memory>
#include <random>
#include <string>
#include <vector>

namespace {

thread_local std::string g_err;

// ---------------------------------------------------------------------------------------------
// RNG used for everything but construction.  R/rng.h:64-118, R/rng.cpp:83-121: uniform = rand() /
// RAND_MAX; Gaussian = a random entry of a 32768-entry table that is re-drawn from
// std::normal_distribution<float> over std::default_random_engine(seed) whenever the seed is set.
// The integer source here is xoshiro256++ instead of libc rand() (rand() is process global); the
// distribution of what is returned is the same.
struct OrcRng {
  uint64_t s[4];
  std::vector<float> table;
  bool use_table = true;
  bool have_spare = false;
  float spare = 0.f;

  static uint64_t splitmix(uint64_t &z) {
    z += 0x9E3779B97F4A7C15ull;
    uint64_t r = z;
    r = (r ^ (r >> 30)) * 0xBF58476D1CE4E5B9ull;
    r = (r ^ (r >> 27)) * 0x94D049BB133111EBull;
    return r ^ (r >> 31);
  }
  static inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
  inline uint64_t next() {
    const uint64_t result = rotl(s[0] + s[3], 23) + s[0];
    const uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl(s[3], 45);
    return result;
  }
  void seed(unsigned int seed_in) {
    unsigned int sd = seed_in;
    if (sd == 0) { // R/rng.cpp:73-81 randomizeSeed
      sd = (unsigned int)std::chrono::high_resolution_clock::now().time_since_epoch().count();
    }
    uint64_t z = sd;
    for (int i = 0; i < 4; ++i) s[i] = splitmix(z);
    have_spare = false;
    // R/rng.cpp:94-121 generateNewList
    std::default_random_engine generator{sd};
    std::normal_distribution<float> dist{};
    table.resize(32768);
    for (auto &v : table) v = dist(generator);
  }
  // R/rng.h:88 sampleUniform: (float)rand() / (float)RAND_MAX, a value in [0, 1]
  inline float uniform() { return (float)(next() >> 33) / (float)2147483647; }
  // R/rng.h:98-112 sampleGauss
  inline float gauss() {
    if (use_table) {
      return table[(next() >> 33) % 32768u];
    }
    if (have_spare) {
      have_spare = false;
      return spare;
    }
    double u1, u2;
    do {
      u1 = (double)(next() >> 11) * (1.0 / 9007199254740992.0);
    } while (u1 <= 0.0);
    u2 = (double)(next() >> 11) * (1.0 / 9007199254740992.0);
    double r = std::sqrt(-2.0 * std::log(u1));
    spare = (float)(r * std::sin(6.283185307179586 * u2));
    have_spare = true;
    return (float)(r * std::cos(6.283185307179586 * u2));
  }
};

// R/rng.h:45-61 RealWorldRNG: construction-time generator.  One engine, one persistent
// normal_distribution<float> object (it caches its second value) and one uniform distribution.
struct OrcRealWorldRng {
  std::default_random_engine gen;
  std::uniform_real_distribution<float> udist{0.0f, 1.0f};
  std::normal_distribution<float> ndist{0.0f, 1.0f};
  explicit OrcRealWorldRng(unsigned int seed) {
    unsigned int sd = seed;
    if (!sd) { // R/rng.cpp:23-27
      sd = (unsigned int)std::chrono::high_resolution_clock::now().time_since_epoch().count();
    }
    gen = std::default_random_engine(sd);
  }
  float gauss() { return ndist(gen); }
  float uniform() { return udist(gen); }
};

// R/utility_functions.h:186-210 getDiscretizedValue / getDiscretizedValueSR
inline float discretize(float value, float res, bool sto_round, OrcRng &rng) {
  if (res <= 0.0f) return value;
  if (sto_round) return rintf(value / res + (rng.uniform() - 0.5f)) * res;
  return rintf(value / res) * res;
}

// R/rpu_pulsed_meta_parameter.cpp:26-37 checkRes / checkAndSetRes
inline float check_res(float res) {
  float r = res < 0.0f ? 0.0f : res;
  return r > 1.0f ? 1.0f / r : r;
}

struct OrcIO {
  rpu_io_params p;
  bool perfect = false;
};

// R/rpu_pulsed_meta_parameter.cpp:39-128 initializeForForward / initializeForBackward
bool init_io(OrcIO &io, bool backward) {
  rpu_io_params &p = io.p;
  if (p.mv_type == RPU_MV_IDEAL) p.is_perfect = 1;
  if (p.is_perfect) {
    p.mv_type = RPU_MV_IDEAL;
    io.perfect = true;
    return true;
  }
  if (p.mv_type != RPU_MV_ONE_PASS && p.mv_type != RPU_MV_POS_NEG_SEPARATE &&
      p.mv_type != RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM) {
    g_err = "oracle: only mv_type Ideal / OnePass / PosNegSeparate / PosNegSeparateDigitalSum restated";
    return false;
  }
  p.out_res = check_res(p.out_res) * (2.0f * p.out_bound);
  p.inp_res = check_res(p.inp_res) * (2.0f * p.inp_bound);
  if (p.noise_management != RPU_NM_NONE) {
    if (p.inp_bound != 1.0f) {
      g_err = backward ? "Backward noise managment expects input bound==1"
                       : "Forward noise managment expects bound==1";
      return false;
    }
  } else {
    p.nm_thres = 0.0f;
  }
  if (p.out_bound <= 0.0f) p.out_bound = std::numeric_limits<float>::infinity();
  if (p.inp_bound <= 0.0f) p.inp_bound = std::numeric_limits<float>::infinity();
  if (backward) p.bound_management = RPU_BM_NONE;
  if (p.w_noise_type < 0 || p.w_noise_type > 2) {
    g_err = "Output noise type not implemented";
    return false;
  }
  return true;
}

// R/rpu_pulsed_meta_parameter.h:112-119
bool io_perfect(const rpu_io_params &p) { return p.is_perfect || p.mv_type == RPU_MV_IDEAL; }
bool has_voltage_offsets(const rpu_io_params &p) { return p.v_offset_std > 0.0f || p.r_series > 0.0f; }
bool has_out_nonlinearity(const rpu_io_params &p) { return p.out_nonlinearity > 0.0f && !io_perfect(p); }
bool has_nl_calibration(const rpu_io_params &p) { return has_out_nonlinearity(p) || p.r_series > 0.0f; }

struct OrcTile {
  int X = 0, D = 0;
  OrcIO fio, bio;
  rpu_update_params up;
  rpu_device_params dev;
  float lr = 0.01f; // R/rpu.h:186 default learning rate is set by the caller; 0.01 here
  float granularity = 0.0f; // 0: the device's dw_min
  OrcRng rng;
  std::vector<float> w;
  // R/rpu_pulsed_device.h:296-312 per-device arrays
  std::vector<float> w_max, w_min, scale_up, scale_down, decay_scale, diffusion_rate, reset_bias;
  // R/rpu_linearstep_device.h:199-200
  std::vector<float> slope_up, slope_down;
  std::vector<int32_t> last_rounds;
  // write noise (R/rpu_pulsed_device.h:89-104): the weights the pulses act on; w then holds the shown weights
  std::vector<float> w_persistent;
  // R/rpu_forward_backward_pass.h:17-26 MVParameter of the forward [0] and backward [1] pass
  struct Lines {
    std::vector<float> v_offset, out_nl, out_noise;
    std::vector<float> w_asymmetry; // [D][X] factors of the negative pass of PosNegSeparate
    float nl_factor = 1.0f;
  } lines[2];
  float aux_nm = -1.0f; // running AverageAbsMax scale (R/rpu_forward_backward_pass.h:241), negative: not started
  // scratch
  std::vector<float> in_buf, bias_buf;
  std::vector<std::vector<int>> x_idx, d_idx;
  std::vector<int> x_cnt, d_cnt;
  std::vector<float> xv, dv;
  std::vector<int> coinc;
};

bool is_pulsed_device(const OrcTile &t) { return t.dev.kind != RPU_DEVICE_IDEAL; }
bool uses_persistent(const OrcTile &t) {
  return (t.dev.kind == RPU_DEVICE_LINEAR_STEP || t.dev.kind == RPU_DEVICE_SOFT_BOUNDS) && t.dev.write_noise_std > 0.0f;
}
bool is_linear_device(const OrcTile &t) {
  return t.dev.kind == RPU_DEVICE_LINEAR_STEP || t.dev.kind == RPU_DEVICE_SOFT_BOUNDS;
}

// R/rpu_pulsed_device.cpp:593-733 PulsedRPUDevice::populate
bool populate_pulsed(OrcTile &t, OrcRealWorldRng &rng) {
  const rpu_device_params &par = t.dev;
  const int X = t.X, D = t.D;
  const size_t n = (size_t)X * D;
  t.w_max.assign(n, 0.f);
  t.w_min.assign(n, 0.f);
  t.scale_up.assign(n, 0.f);
  t.scale_down.assign(n, 0.f);
  t.decay_scale.assign(n, 1.f);
  t.diffusion_rate.assign(n, 0.f);
  t.reset_bias.assign(n, 0.f);

  float up_down = par.up_down;
  float up_down_std = par.up_down_dtod;
  float up_bias = up_down > 0.0f ? 0.0f : up_down;
  float down_bias = up_down > 0.0f ? -up_down : 0.0f;
  float gain_std = par.dw_min_dtod;

  if ((par.w_min > 0.0f) || (par.w_max < 0.0f)) {
    g_err = "The closed interval [w_min,w_max] needs to contain 0.";
    return false;
  }
  for (int j = 0; j < X; ++j) {
    for (int i = 0; i < D; ++i) {
      const size_t k = (size_t)i * X + j;
      float &mx = t.w_max[k], &mn = t.w_min[k], &su = t.scale_up[k], &sd = t.scale_down[k];
      mx = par.w_max * (1.0f + par.w_max_dtod * rng.gauss());
      mn = par.w_min * (1.0f + par.w_min_dtod * rng.gauss());
      float gain;
      if (par.dw_min_dtod_log_normal) {
        gain = expf(gain_std * rng.gauss());
      } else {
        gain = (1.0f + gain_std * rng.gauss());
      }
      float r = up_down_std * rng.gauss();
      su = (up_bias + gain + r) * par.dw_min;
      sd = (down_bias + gain - r) * par.dw_min;

      if (par.enforce_consistency) {
        su = fabsf(su);
        sd = fabsf(sd);
        if (mn > mx) std::swap(mn, mx);
        mx = fabsf(mx);
        mn = -fabsf(mn);
      } else {
        if (mn > mx) {
          float m = mx + (mn - mx) / 2.0f;
          mx = m;
          mn = m;
        }
      }
      if (par.adjust_bounds_with_up_down) {
        if (mn > mx) std::swap(mn, mx);
        float up_down_alpha = su / (su + sd);
        float mm = mx - mn;
        float new_min_bound = 0.0f;
        float dev = par.adjust_bounds_with_up_down_dev;
        if (dev > 0.0f) {
          new_min_bound = -(((float)tanh((float)((up_down_alpha - 0.5f) / dev)) + 1.0f) / 2.0f) * mm;
        } else {
          if (up_down_alpha < 0.5f)
            new_min_bound = 0;
          else if (up_down_alpha == 0.5f)
            new_min_bound = -mm / 2.0f;
          else
            new_min_bound = -mm;
        }
        mn = new_min_bound;
        mx = new_min_bound + mm;
      }
      // one uniform is always drawn here (R/rpu_pulsed_device.cpp:684)
      if (par.corrupt_devices_prob > rng.uniform()) {
        float lo = std::max(std::min(mx, mn), -fabsf(par.corrupt_devices_range));
        float hi = std::min(std::max(mx, mn), fabsf(par.corrupt_devices_range));
        float value = lo + (hi - lo) * rng.uniform();
        mx = value;
        mn = value;
        su = 0.0f;
        sd = 0.0f;
      }
      if (par.perfect_bias && (j == X - 1)) {
        su = par.dw_min;
        sd = par.dw_min;
        mn = 100.f * par.w_min;
        mx = 100.f * par.w_max;
      }
      t.diffusion_rate[k] = fabsf(par.diffusion * (1.0f + par.diffusion_dtod * rng.gauss()));
      t.reset_bias[k] = par.reset + par.reset_dtod * rng.gauss();
      if (par.lifetime > 0.0f) {
        float lt = par.lifetime * (1.0f + par.lifetime_dtod * rng.gauss());
        t.decay_scale[k] = (lt > 1.0f) ? (1.0f - (1.0f / lt)) : 0.0f;
      } else {
        t.decay_scale[k] = 1.0f;
      }
    }
  }
  return true;
}

// R/rpu_linearstep_device.cpp:20-74 LinearStepRPUDevice::populate
bool populate_linear_step(OrcTile &t, OrcRealWorldRng &rng) {
  const rpu_device_params &par = t.dev;
  const int X = t.X, D = t.D;
  t.slope_up.assign((size_t)X * D, 0.f);
  t.slope_down.assign((size_t)X * D, 0.f);
  if ((par.ls_reverse_up || par.ls_reverse_down) && !par.ls_mult_noise) {
    g_err = "Only mulitplicative noise supported with reverse up/down!";
    return false;
  }
  for (int i = 0; i < D; ++i) {
    for (int j = 0; j < X; ++j) {
      const size_t k = (size_t)i * X + j;
      float up = par.ls_decrease_up + par.ls_decrease_up_dtod * rng.gauss();
      float down = par.ls_decrease_down + par.ls_decrease_down_dtod * rng.gauss();
      if (!par.ls_allow_increasing_slope) {
        up = fabsf(up);
        down = fabsf(down);
      }
      float w_ref_up, w_ref_down;
      if (par.ls_mean_bound_reference) {
        w_ref_up = par.ls_reverse_up ? par.w_min - par.ls_reverse_offset : par.w_max;
        w_ref_down = par.ls_reverse_down ? par.w_max + par.ls_reverse_offset : par.w_min;
      } else {
        w_ref_up = par.ls_reverse_up ? t.w_min[k] - par.ls_reverse_offset : t.w_max[k];
        w_ref_down = par.ls_reverse_down ? t.w_max[k] + par.ls_reverse_offset : t.w_min[k];
      }
      t.slope_up[k] = (w_ref_up != 0.0f) ? -up * t.scale_up[k] / w_ref_up : 0.0f;
      t.slope_down[k] = (w_ref_down != 0.0f) ? -down * t.scale_down[k] / w_ref_down : 0.0f;
    }
  }
  return true;
}

// R/rpu_pulsed_device.cpp:545-571 onSetWeights (hard bounds; no persistent weights here)
void clip_to_bounds(OrcTile &t) {
  if (!is_pulsed_device(t)) return;
  const size_t n = t.w.size();
  for (size_t i = 0; i < n; ++i) {
    t.w[i] = std::min(t.w[i], t.w_max[i]);
    t.w[i] = std::max(t.w[i], t.w_min[i]);
  }
}

// ---------------------------------------------------------------------------------------------
// forward / backward

// R/rpu_forward_backward_pass.cpp:112-178 computeNoiseManagement
float noise_management(const float *in, int size, int inc, int nm_type, const rpu_io_params &io, float &aux) {
  switch (nm_type) {
  case RPU_NM_AVERAGE_ABS_MAX:
  case RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE: { // :138-149, one running value shared by forward and backward
    float amax = 0.f;
    for (int j = 0; j < size; ++j) amax = std::max(amax, fabsf(in[(size_t)j * inc]));
    if (aux < 0.0f) {
      aux = amax;
    } else {
      aux = aux * (1.0f - io.nm_decay) + io.nm_decay * amax;
    }
    return aux;
  }
  case RPU_NM_NONE:
    return 1.0f;
  case RPU_NM_ABS_MAX: {
    float amax = 0.f; // isamax + fabsf of that entry
    for (int j = 0; j < size; ++j) amax = std::max(amax, fabsf(in[(size_t)j * inc]));
    return io.nm_thres > 0.0f ? std::min(amax, io.nm_thres) : amax;
  }
  case RPU_NM_CONSTANT:
    return io.nm_thres > 0.0f ? io.nm_thres : 1.0f;
  case RPU_NM_MAX: {
    float mx = in[0];
    for (int j = 1; j < size; ++j) mx = std::max(mx, in[(size_t)j * inc]);
    return io.nm_thres > 0.0f ? std::min(mx, io.nm_thres) : mx;
  }
  case RPU_NM_ABS_MAX_NP_SUM: {
    float amax = 0.f;
    for (int j = 0; j < size; ++j) amax = std::max(amax, fabsf(in[(size_t)j * inc]));
    float bound = std::isinf(io.out_bound) ? 1.0f : io.out_bound;
    float psum = 0, nsum = 0;
    for (int j = 0; j < size; ++j) {
      float x = in[(size_t)j * inc];
      psum += x > 0.0f ? x : 0.0f;
      nsum += x < 0.0f ? x : 0.0f;
    }
    float sum = std::max(psum, -nsum);
    amax = io.nm_thres > 0.0f ? std::min(amax, io.nm_thres) : amax;
    float npsum_scale = sum * io.nm_assumed_wmax / bound;
    if (io.inp_res > 0.0f) {
      npsum_scale = std::min(amax / io.inp_res * io.max_bm_res, npsum_scale);
    }
    return std::max(amax, npsum_scale);
  }
  default:
    return -1.0f; // rejected at creation
  }
}

// R/rpu_forward_backward_pass.cpp:571-604 prepareInputImplStage4 (the DAC)
void prepare_input(OrcTile &t, float *out, const float *in, int in_size, int in_inc, float scale,
                   bool scaling, const rpu_io_params &io) {
  const float bound = io.inp_bound > 0.0f ? io.inp_bound : std::numeric_limits<float>::infinity();
  const float noise = io.inp_noise;
  const float asymmetry_scale = (1.0f - io.inp_asymmetry);
  const float res = io.inp_res;
  const bool sr = io.inp_sto_round != 0;
  for (int j = 0; j < in_size; ++j) {
    float value = in[(size_t)j * in_inc];
    if (scaling) value *= scale;
    value = discretize(value, res, sr, t.rng);
    value = (value > bound) ? bound : value;
    value = (value < -bound) ? -bound : value;
    if (noise > 0.0f) value += noise * t.rng.gauss();
    if (io.inp_asymmetry != 0.0f) value = value < 0.0f ? value * asymmetry_scale : value;
    out[j] = value;
  }
}

// R/rpu_forward_backward_pass.cpp:38-61 gemv (row-major W [D][X]); the accumulation order of a
// BLAS is unspecified, so a blocked sum is as good a stand-in as a sequential one.
void gemv(const OrcTile &t, const float *in, float *out, int out_inc, bool transposed) {
  const int X = t.X, D = t.D;
  const float *w = t.w.data();
  if (!transposed) {
    for (int i = 0; i < D; ++i) {
      const float *row = w + (size_t)i * X;
      float acc = 0.f;
#pragma omp simd reduction(+ : acc)
      for (int j = 0; j < X; ++j) acc += row[j] * in[j];
      out[(size_t)i * out_inc] = acc;
    }
  } else {
    std::vector<float> acc((size_t)X, 0.f);
    for (int i = 0; i < D; ++i) {
      const float *row = w + (size_t)i * X;
      const float di = in[i];
#pragma omp simd
      for (int j = 0; j < X; ++j) acc[j] += row[j] * di;
    }
    for (int j = 0; j < X; ++j) out[(size_t)j * out_inc] = acc[j];
  }
}

// R/rpu_forward_backward_pass.cpp:666-719 finalizeOutputImplStage5 (the ADC).  A Gaussian is drawn
// for every output even when out_noise == 0 (:750-756 instantiate with_noise = true in both branches).
bool finalize_output(OrcTile &t, float *out, int out_size, int out_inc, const rpu_io_params &io,
                     const OrcTile::Lines &mv) {
  bool bound_test_passed = true;
  const bool with_nl = has_nl_calibration(io); // :738-745
  const float nlf = mv.nl_factor;
  const float bound = io.out_bound > 0.0f ? io.out_bound : std::numeric_limits<float>::infinity();
  const float asymmetry_scale = (1.0f - io.out_asymmetry);
  const float res = io.out_res;
  const bool with_bm = io.bound_management != RPU_BM_NONE;
  const bool sr = io.out_sto_round != 0;
  for (int i = 0; i < out_size; ++i) {
    float value = out[(size_t)i * out_inc];
    if (with_nl) value = nlf * value / (1.0f + std::fabs(mv.out_nl[i] * value)); // :686-688
    if (io.out_asymmetry > 0.0f) value = value < 0.0f ? value * asymmetry_scale : value;
    const float noise_std = io.out_noise_std > 0.0f ? mv.out_noise[i] : io.out_noise; // :696
    value += noise_std * t.rng.gauss();
    value = discretize(value, res, sr, t.rng);
    if (with_bm) {
      if (value > bound) {
        value = bound;
        bound_test_passed = false;
      } else if (value < -bound) {
        value = -bound;
        bound_test_passed = !io.bm_test_negative_bound;
      }
    } else {
      value = value > bound ? bound : value;
      value = value < -bound ? -bound : value;
    }
    out[(size_t)i * out_inc] = value;
  }
  return bound_test_passed;
}

// R/rpu_forward_backward_pass.cpp:283-295: the slope calibration factor of the non-linearity
void set_nl_factor(const rpu_io_params &io, OrcTile::Lines &mv, int out_size) {
  mv.nl_factor = 1.0f;
  const float out_bound = io.out_bound > 0.0f && io.out_bound < std::numeric_limits<float>::infinity() ? io.out_bound : 1.0f;
  if (io.slope_calibration > 0.0f) {
    float sum_nonlinearity = 0.0f;
    if (has_out_nonlinearity(io)) {
      for (int i = 0; i < out_size; ++i) sum_nonlinearity += std::fabs(mv.out_nl[i]);
    }
    const float r_correction = io.r_series;
    const float f = 1.0f + (sum_nonlinearity / (float)out_size + r_correction) * io.slope_calibration * out_bound;
    mv.nl_factor = f * f;
  }
}

// R/rpu_forward_backward_pass.cpp:254-318 the populate lambda of populateFBParameter (values drawn from the tile's
// run-time generator)
void populate_lines(OrcTile &t, const rpu_io_params &io, OrcTile::Lines &mv, int out_size) {
  mv = OrcTile::Lines();
  if (io_perfect(io)) return;
  if (has_voltage_offsets(io)) {
    mv.v_offset.resize(out_size);
    for (int i = 0; i < out_size; ++i) mv.v_offset[i] = std::max(io.v_offset_std * t.rng.gauss(), 0.0f);
  }
  const float out_bound = io.out_bound > 0.0f && io.out_bound < std::numeric_limits<float>::infinity() ? io.out_bound : 1.0f;
  if (has_nl_calibration(io)) {
    mv.out_nl.resize(out_size);
    for (int i = 0; i < out_size; ++i) {
      mv.out_nl[i] =
          std::fabs(io.out_nonlinearity / out_bound * (1.0f + std::max(io.out_nonlinearity_std, 0.0f) * t.rng.gauss()));
    }
  }
  set_nl_factor(io, mv, out_size);
  if (io.w_read_asymmetry_dtod != 0.0f) { // :297-304
    mv.w_asymmetry.resize((size_t)t.X * t.D);
    for (float &v : mv.w_asymmetry) v = 1.0f + io.w_read_asymmetry_dtod * t.rng.gauss();
  }
  if (io.out_noise_std > 0.0f) {
    mv.out_noise.resize(out_size);
    for (int i = 0; i < out_size; ++i) mv.out_noise[i] = std::fabs(io.out_noise * (1.0f + io.out_noise_std * t.rng.gauss()));
  }
}

// R/rpu_forward_backward_pass.cpp:436-506 applyVoltageOffsets
void apply_voltage_offsets(float *out, int out_size, int out_inc, const float *in, int in_size,
                           const rpu_io_params &io, const OrcTile::Lines &mv) {
  if (!has_voltage_offsets(io)) return;
  const float rs = std::max(io.r_series, 0.0f);
  const float rs_max_total = io.r_series_max_total;
  if (io.v_offset_w_min == 0.0f) {
    for (int i = 0; i < out_size; ++i) {
      float &y = out[(size_t)i * out_inc];
      const float v_offs = mv.v_offset[i];
      if (rs <= 0.0f) {
        y = y * (1.0f - v_offs);
      } else {
        const float nom = 1.0f + std::min(rs * std::fabs(y), rs_max_total);
        y = (1.0f - v_offs) * y / nom;
      }
    }
    return;
  }
  float x_accum = 0.0f;
  for (int j = 0; j < in_size; ++j) x_accum += in[j];
  if (rs <= 0.0f) {
    const float y_ref2 = (-io.v_offset_w_min) * x_accum * 2.0f;
    for (int i = 0; i < out_size; ++i) {
      float &y = out[(size_t)i * out_inc];
      const float v_offs = mv.v_offset[i];
      y = y * (1.0f - v_offs) - v_offs * y_ref2;
    }
  } else {
    const float y_ref = (-io.v_offset_w_min) * x_accum;
    for (int i = 0; i < out_size; ++i) {
      float &y = out[(size_t)i * out_inc];
      const float v_offs = mv.v_offset[i];
      const float y_pos = y + y_ref;
      const float p_nom = 1.0f + std::min(rs * std::fabs(y_pos), rs_max_total);
      const float n_nom = 1.0f + std::min(rs * std::fabs(y_ref), rs_max_total);
      y = (1.0f - v_offs) * y_pos / p_nom - (1.0f + v_offs) * y_ref / n_nom;
    }
  }
}

// R/rpu_forward_backward_pass.cpp:508-530 computeTotalCurrent and :387-433 applyIrDrop
void apply_ir_drop(OrcTile &t, float *out, int out_size, int out_inc, const float *in, int in_size,
                   const rpu_io_params &io, bool transposed) {
  if (io.ir_drop <= 0.0f) return;
  const int X = t.X;
  const float *w = t.w.data();
  std::vector<float> current((size_t)out_size), c_values((size_t)out_size), pos_in((size_t)in_size);
  for (int i = 0; i < out_size; ++i) {
    float accum = 0.0f;
    for (int j = 0; j < in_size; ++j) {
      const float wij = transposed ? w[(size_t)j * X + i] : w[(size_t)i * X + j];
      accum += std::fabs(wij) * std::fabs(in[j]);
    }
    current[i] = accum;
  }
  const float a_scale = (float)in_size / io.ir_drop_g_ratio;
  for (int i = 0; i < out_size; ++i) {
    const float a = a_scale * current[i];
    c_values[i] = a * (a * (0.05f * a - 0.2f) + 0.5f);
  }
  for (int j = 0; j < in_size; ++j) {
    const float p = (1.0f - (float)j / (float)in_size);
    pos_in[j] = in[j] * (1.0f - p * p);
  }
  for (int i = 0; i < out_size; ++i) {
    float accum = 0.0f;
    for (int j = 0; j < in_size; ++j) {
      const float wij = transposed ? w[(size_t)j * X + i] : w[(size_t)i * X + j];
      accum += wij * pos_in[j];
    }
    out[(size_t)i * out_inc] -= c_values[i] * (io.ir_drop * accum);
  }
}

// R/rpu_forward_backward_pass.cpp:325-385 applyOutputWeightNoise
void apply_output_weight_noise(OrcTile &t, float *out, int out_size, int out_inc, const float *in, int in_size,
                               const rpu_io_params &io, bool transposed) {
  if (io.w_noise_type == 0 || !(io.w_noise > 0.0f)) return;
  const int X = t.X;
  const float *w = t.w.data();
  if (io.w_noise_type == 1) { // AdditiveConstant
    float sq = 0.0f;
    for (int j = 0; j < in_size; ++j) sq += in[j] * in[j];
    const float w_std = io.w_noise * std::sqrt(sq);
    for (int i = 0; i < out_size; ++i) out[(size_t)i * out_inc] += w_std * t.rng.gauss();
    return;
  }
  for (int i = 0; i < out_size; ++i) { // PCMRead
    float accum = 0.0f;
    for (int j = 0; j < in_size; ++j) {
      const float wij = transposed ? w[(size_t)j * X + i] : w[(size_t)i * X + j];
      accum += std::fabs(wij) * (in[j] * in[j]);
    }
    out[(size_t)i * out_inc] += io.w_noise * std::sqrt(accum) * t.rng.gauss();
  }
}

// R/rpu_forward_backward_pass.cpp:779-797 computeAnalogMVSinglePass: the contraction, then applyNonIdealities
// (:535-560): IR drop, voltage offsets, then the weight-dependent noise
void analog_mv_single_pass(OrcTile &t, const float *in, int in_size, float *out, int out_size, int out_inc,
                           const rpu_io_params &io, bool transposed) {
  const OrcTile::Lines &mv = t.lines[transposed ? 1 : 0];
  gemv(t, in, out, out_inc, transposed);
  apply_ir_drop(t, out, out_size, out_inc, in, in_size, io, transposed);
  apply_voltage_offsets(out, out_size, out_inc, in, in_size, io, mv);
  apply_output_weight_noise(t, out, out_size, out_inc, in, in_size, io, transposed);
}

// R/rpu_forward_backward_pass.cpp:800-897 computeAnalogMV: OnePass, PosNegSeparate and PosNegSeparateDigitalSum
bool analog_mv(OrcTile &t, const float *in, int in_size, int in_inc, float *out, int out_size,
               int out_inc, float scale, bool scaling, const rpu_io_params &io, bool transposed) {
  t.in_buf.resize(in_size);
  prepare_input(t, t.in_buf.data(), in, in_size, in_inc, scale, scaling, io);
  const OrcTile::Lines &mv = t.lines[transposed ? 1 : 0];
  if (io.mv_type == RPU_MV_POS_NEG_SEPARATE || io.mv_type == RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM) {
    // first the negative inputs, then the positive ones; the sums of both passes go through the ADC (:832-893),
    // or, with the digital sum, each pass through the ADC stage on its own (:861-877) and the codes are added
    const bool digital = io.mv_type == RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM;
    bool passed = false;
    std::vector<float> part((size_t)in_size), neg_out((size_t)out_size);
    for (int i = 0; i < in_size; ++i) part[i] = t.in_buf[i] < 0.0f ? t.in_buf[i] : 0.0f;
    if (io.w_read_asymmetry_dtod > 0.0f) {
      // the negative pass reads w_ij * asymmetry_ij, contraction and non-idealities alike (:845-860)
      std::vector<float> neg_w(t.w.size());
      for (size_t i = 0; i < neg_w.size(); ++i) neg_w[i] = t.w[i] * mv.w_asymmetry[i];
      t.w.swap(neg_w);
      analog_mv_single_pass(t, part.data(), in_size, neg_out.data(), out_size, 1, io, transposed);
      t.w.swap(neg_w);
    } else {
      analog_mv_single_pass(t, part.data(), in_size, neg_out.data(), out_size, 1, io, transposed);
    }
    if (digital) passed = finalize_output(t, neg_out.data(), out_size, 1, io, mv);
    for (int i = 0; i < in_size; ++i) part[i] = t.in_buf[i] > 0.0f ? t.in_buf[i] : 0.0f;
    analog_mv_single_pass(t, part.data(), in_size, out, out_size, out_inc, io, transposed);
    if (digital) passed = finalize_output(t, out, out_size, out_inc, io, mv) && passed;
    for (int j = 0; j < out_size; ++j) out[(size_t)j * out_inc] += neg_out[j];
    if (digital) return passed;
    return finalize_output(t, out, out_size, out_inc, io, mv);
  }
  analog_mv_single_pass(t, t.in_buf.data(), in_size, out, out_size, out_inc, io, transposed);
  return finalize_output(t, out, out_size, out_inc, io, mv);
}

// R/rpu_forward_backward_pass.cpp:900-988 ForwardBackwardPassIOManaged::forwardVector
int forward_vector(OrcTile &t, const float *x, int x_inc, float *y, int d_inc) {
  const rpu_io_params &io = t.fio.p;
  const int X = t.X, D = t.D;
  float nm_scale = noise_management(x, X, x_inc, io.noise_management, io, t.aux_nm);
  const bool nm = io.noise_management != RPU_NM_NONE;
  const bool bm = io.bound_management != RPU_BM_NONE;
  if (nm && (nm_scale <= 0.0f) && (io.inp_noise <= 0.0f)) {
    for (int i = 0; i < D; ++i) y[(size_t)i * d_inc] = 0.0f;
    return 0;
  }
  const float out_scale = io.out_scale * 1.0f; // alpha = 1
  bool passed = false;
  float reduction = 0.5f;
  float scale = 1.f;
  bool scaling = false;
  int bm_round = 0;
  while (!passed) {
    passed = true;
    reduction *= 2.0f;
    if (bm_round == 1 && io.bound_management == RPU_BM_ITERATIVE_WORST_CASE &&
        io.noise_management != RPU_NM_ABS_MAX_NP_SUM) {
      nm_scale = noise_management(x, X, x_inc, RPU_NM_ABS_MAX_NP_SUM, io, t.aux_nm);
      reduction = 1.0f;
    }
    bm_round++;
    scaling = false;
    scale = 1.0f;
    if (nm && nm_scale > 0.0f) {
      scale /= nm_scale;
      scaling = true;
    }
    if (bm) {
      scale /= reduction;
      scaling = true;
    }
    passed = analog_mv(t, x, X, x_inc, y, D, d_inc, scale, scaling, io, false);
    if (bm) {
      passed = passed || (((int)reduction > io.max_bm_factor) ||
                          ((io.inp_res > 0.0f) && (reduction > io.max_bm_res / io.inp_res)));
    } else {
      passed = true;
    }
  }
  if (scaling || out_scale != 1.0f) {
    const float f = out_scale / scale;
    for (int i = 0; i < D; ++i) y[(size_t)i * d_inc] *= f;
  }
  return bm_round;
}

// R/rpu_forward_backward_pass.cpp:990-1027 backwardVector
void backward_vector(OrcTile &t, const float *d, int d_inc, float *x, int x_inc) {
  const rpu_io_params &io = t.bio.p;
  const int X = t.X, D = t.D;
  float nm_scale = noise_management(d, D, d_inc, io.noise_management, io, t.aux_nm);
  const bool nm = io.noise_management != RPU_NM_NONE;
  const float out_scale = io.out_scale * 1.0f;
  const bool scaling = nm && nm_scale > 0.0f;
  if (nm && (nm_scale <= 0.0f)) {
    for (int j = 0; j < X; ++j) x[(size_t)j * x_inc] = 0.0f;
    return;
  }
  analog_mv(t, d, D, d_inc, x, X, x_inc, 1.0f / nm_scale, scaling, io, true);
  if (scaling || out_scale != 1.0f) {
    const float f = out_scale * nm_scale;
    for (int j = 0; j < X; ++j) x[(size_t)j * x_inc] *= f;
  }
}

// plain W x / W^T d with a strided in/out (is_perfect short cut, :14-36)
void fp_forward(const OrcTile &t, const float *x, int x_inc, float *y, int d_inc, float alpha) {
  for (int i = 0; i < t.D; ++i) {
    const float *row = t.w.data() + (size_t)i * t.X;
    float acc = 0.f;
    for (int j = 0; j < t.X; ++j) acc += row[j] * x[(size_t)j * x_inc];
    y[(size_t)i * d_inc] = alpha * acc;
  }
}
void fp_backward(const OrcTile &t, const float *d, int d_inc, float *x, int x_inc, float alpha) {
  for (int j = 0; j < t.X; ++j) {
    float acc = 0.f;
    for (int i = 0; i < t.D; ++i) acc += t.w[(size_t)i * t.X + j] * d[(size_t)i * d_inc];
    x[(size_t)j * x_inc] = alpha * acc;
  }
}

// ---------------------------------------------------------------------------------------------
// update

// R/rpu_pulsed_meta_parameter.cpp:152-181 calculateBlAB
bool calculate_bl_ab(const rpu_update_params &up, int &BL, float &A, float &B, float lr, float dw_min) {
  if (lr < 0.0f) {
    g_err = "lr should be positive !";
    return false;
  } else if (lr == 0.0f) {
    A = 0.0f;
    B = 0.0f;
    BL = 0;
    return true;
  }
  if (up.fixed_bl || up.update_bl_management) {
    BL = up.desired_bl;
    A = sqrtf(lr / (dw_min * (float)BL));
    B = A;
  } else {
    if ((dw_min * (float)up.desired_bl) < lr) {
      A = 1.0f;
      B = 1.0f;
      BL = std::max((int)ceilf(lr / dw_min), 1);
    } else {
      BL = up.desired_bl;
      A = sqrtf(lr / (dw_min * (float)BL));
      B = A;
    }
  }
  return true;
}

// R/rpu_pulsed_meta_parameter.cpp:183-236 performUpdateManagement
bool update_management(const rpu_update_params &up, int &BL, float &A, float &B, int max_BL,
                       float x_abs_max, float d_abs_max, float lr, float dw_min) {
  if (!calculate_bl_ab(up, BL, A, B, lr, dw_min)) return false;
  if (lr > 0.0f) {
    if (d_abs_max == 0.0f || x_abs_max == 0.0f) {
      A = 1;
      B = 1;
      BL = 0;
      return true;
    }
    if (up.update_bl_management || up.update_management) {
      float x_val = x_abs_max;
      float d_val = up.um_grad_scale * d_abs_max;
      float k_val = lr * x_val * d_val / dw_min;
      if (up.update_bl_management) {
        BL = (int)ceilf(k_val);
        if (BL > max_BL) BL = max_BL;
        A = sqrtf(lr / (dw_min * (float)BL));
        B = A;
      }
      if (up.update_management) {
        if (k_val > (float)max_BL) d_val *= (float)max_BL / k_val;
        A *= sqrtf(x_val / d_val);
        B *= sqrtf(d_val / x_val);
      }
    }
  }
  return true;
}

// R/utility_functions.h:277-286 Find_Absolute_Max
float find_abs_max(const float *v, int n, int inc) {
  float m = 0;
  for (int i = 0; i < n; ++i) {
    float a = v[(size_t)i * inc];
    a = (a >= 0.0f) ? a : -a;
    if (a > m) m = a;
  }
  return m;
}

// BL / A / B of one sample as R/sparse_bit_line_maker.cpp:299-314 and R/dense_bit_line_maker.cpp:285-300
bool sample_bl_ab(OrcTile &t, const float *x, int x_inc, const float *d, int d_inc, float lr_abs,
                  int &BL, float &A, float &B) {
  // weight granularity (R/rpu_constantstep_device.h:27, R/rpu_linearstep_device.h:58); a compound device gives
  // its own (R/rpu_vector_device.cpp:411-421), set through orc_set_weight_granularity
  const float dw_min = t.granularity > 0.0f ? t.granularity : t.dev.dw_min;
  A = 0;
  B = 0;
  BL = 0;
  if (t.up.update_bl_management || t.up.update_management) {
    float xm = find_abs_max(x, t.X, x_inc);
    float dm = find_abs_max(d, t.D, d_inc);
    return update_management(t.up, BL, A, B, t.up.desired_bl, xm, dm, lr_abs, dw_min);
  }
  return calculate_bl_ab(t.up, BL, A, B, lr_abs, dw_min);
}

// R/sparse_bit_line_maker.cpp:199-238 generateCounts (StochasticCompressed)
void generate_counts(OrcTile &t, std::vector<int> &counts, std::vector<std::vector<int>> &indices,
                     const float *v, int v_inc, int v_size, float P, int BL) {
  for (int k = 0; k < BL; ++k) counts[k] = 0;
  for (int j = 0; j < v_size; ++j) {
    float value = v[(size_t)j * v_inc];
    float PP = discretize(fabsf(value) * P, t.up.res, t.up.sto_round != 0, t.rng);
    if (PP == 0.0f) continue;
    int jp1 = (value > 0.0f) ? j + 1 : -(j + 1);
    for (int k = 0; k < BL; ++k) {
      if (PP > t.rng.uniform()) indices[k][counts[k]++] = jp1;
    }
  }
}

// One device pulse.  sign > 0 means "down".
// ConstantStep: R/rpu_constantstep_device.cpp:27-55 ; LinearStep: R/rpu_linearstep_device.cpp:112-164
inline void device_step(OrcTile &t, size_t k, int sign, bool dense_form) {
  const rpu_device_params &par = t.dev;
  const bool persist = uses_persistent(t);
  float &w = persist ? t.w_persistent[k] : t.w[k];
  const float std_ = par.dw_min_std;
  if (par.kind == RPU_DEVICE_CONSTANT_STEP) {
    if (std_ > 0.0f || dense_form) {
      // sparse form with noise: (1 + std * g) * scale ; dense form (:57-78): dw = std>0 ? std*g : 0
      float dwn = std_ > 0.0f ? std_ * t.rng.gauss() : 0.0f;
      if (sign > 0) {
        w -= (1.0f + dwn) * t.scale_down[k];
      } else {
        w += (1.0f + dwn) * t.scale_up[k];
      }
    } else {
      if (sign > 0) {
        w -= t.scale_down[k];
      } else {
        w += t.scale_up[k];
      }
    }
    w = std::min(w, t.w_max[k]);
    w = std::max(w, t.w_min[k]);
  } else {
    if (par.ls_mult_noise) {
      if (sign > 0) {
        w -= (t.slope_down[k] * w + t.scale_down[k]) * (1.0f + std_ * t.rng.gauss());
      } else {
        w += (t.slope_up[k] * w + t.scale_up[k]) * (1.0f + std_ * t.rng.gauss());
      }
    } else {
      if (sign > 0) {
        w -= t.slope_down[k] * w + t.scale_down[k] * (1.0f + std_ * t.rng.gauss());
      } else {
        w += t.slope_up[k] * w + t.scale_up[k] * (1.0f + std_ * t.rng.gauss());
      }
    }
    w = std::max(w, t.w_min[k]);
    w = std::min(w, t.w_max[k]);
    // update_once_mult / update_once_add (R/rpu_linearstep_device.cpp:112-164): the shown weight is redrawn
    if (persist) t.w[k] = w + par.write_noise_std * par.dw_min * t.rng.gauss();
  }
}

// R/rpu_weight_updater.cpp:263-283 : slot-major sparse loop + PULSED_UPDATE_W_LOOP (R/rpu_pulsed_device.h:450-459)
void sparse_update(OrcTile &t, int BL, int lr_sign) {
  for (int k = 0; k < BL; ++k) {
    for (int ii = 0; ii < t.d_cnt[k]; ++ii) {
      int i_signed = t.d_idx[k][ii];
      int d_sign = i_signed < 0 ? -lr_sign : lr_sign;
      int i = i_signed < 0 ? -i_signed - 1 : i_signed - 1;
      for (int jj = 0; jj < t.x_cnt[k]; ++jj) {
        int j_signed = t.x_idx[k][jj];
        int sign = (j_signed < 0) ? -d_sign : d_sign;
        int j = (j_signed < 0) ? -j_signed - 1 : j_signed - 1;
        device_step(t, (size_t)i * t.X + j, sign, false);
      }
    }
  }
}

void ensure_sparse_containers(OrcTile &t, int bl = 0) {
  const int K = std::max(std::max(t.up.desired_bl, bl), 1);
  if ((int)t.x_idx.size() < K) {
    t.x_idx.assign(K, std::vector<int>(t.X));
    t.d_idx.assign(K, std::vector<int>(t.D));
    t.x_cnt.assign(K, 0);
    t.d_cnt.assign(K, 0);
  }
}

// R/dense_bit_line_maker.cpp:209-235 generateDetImplicit
void generate_det_implicit(OrcTile &t, float *pcounts, const float *v, int v_inc, int v_size, float p,
                           float res, float lr) {
  for (int j = 0; j < v_size; ++j) {
    float value = lr < 0.0f ? -v[(size_t)j * v_inc] : v[(size_t)j * v_inc];
    float pp = discretize(fabsf(value) * p, res, t.up.sto_round != 0, t.rng);
    pp = std::max(std::min(pp, 1.0f), 0.0f);
    pcounts[j] = (value >= 0.0f) ? pp : -pp;
  }
}

// R/dense_bit_line_maker.cpp:237-264 generateCoincidencesDetI
void generate_coincidences_det(int *coinc, const float *xv, int X, const float *dv, int D, int BL) {
  size_t idx = 0;
  for (int i = 0; i < D; ++i) {
    float dc = dv[i];
    if (dc != 0.0f) {
      dc *= BL;
      for (int j = 0; j < X; ++j) coinc[idx++] = (int)rintf(dc * xv[j]);
    } else {
      for (int j = 0; j < X; ++j) coinc[idx++] = 0;
    }
  }
}

// R/dense_bit_line_maker.cpp:140-170 generateCountsMean: the expected number of pulses of a line, signed
void generate_counts_mean(OrcTile &t, int *counts, const float *v, int v_inc, int v_size, float p, int BL, float lr) {
  for (int j = 0; j < v_size; ++j) {
    const float value = lr < 0.0f ? -v[(size_t)j * v_inc] : v[(size_t)j * v_inc];
    const float pp = discretize(fabsf(value) * p, t.up.res, t.up.sto_round != 0, t.rng);
    if (pp == 0.0f) {
      counts[j] = 0;
      continue;
    }
    const int ntimes = std::max(std::min((int)rintf((float)BL * pp), BL), 0);
    counts[j] = (value >= 0.0f) ? ntimes : -ntimes;
  }
}

// R/dense_bit_line_maker.cpp:176-201 generateCoincidences
void generate_coincidences_mean(int *coinc, const int *xc, int X, const int *dcnt, int D, int BL) {
  const float bl = (float)BL;
  size_t idx = 0;
  for (int i = 0; i < D; ++i) {
    float dc = (float)dcnt[i];
    if (dc != 0.0f) {
      dc /= bl;
      for (int j = 0; j < X; ++j) coinc[idx++] = (int)rintf(dc * (float)xc[j]);
    } else {
      for (int j = 0; j < X; ++j) coinc[idx++] = 0;
    }
  }
}

// the coincidences of one sample for either dense scheme (makeCoincidences, R/dense_bit_line_maker.cpp:267-331)
bool dense_coincidences(OrcTile &t, const float *x, int x_inc, const float *d, int d_inc, float lr, int *coinc) {
  const int X = t.X, D = t.D;
  int BL;
  float A, B;
  if (!sample_bl_ab(t, x, x_inc, d, d_inc, fabsf(lr), BL, A, B)) return false;
  if (t.up.pulse_type == RPU_PULSE_MEAN_COUNT) {
    std::vector<int> xc((size_t)X), dcnt((size_t)D);
    generate_counts_mean(t, xc.data(), x, x_inc, X, B, BL, lr);
    generate_counts_mean(t, dcnt.data(), d, d_inc, D, A, BL, lr);
    generate_coincidences_mean(coinc, xc.data(), X, dcnt.data(), D, BL);
    return true;
  }
  t.xv.resize(X);
  t.dv.resize(D);
  generate_det_implicit(t, t.xv.data(), x, x_inc, X, B, t.up.x_res_implicit, lr);
  generate_det_implicit(t, t.dv.data(), d, d_inc, D, A, t.up.d_res_implicit, lr);
  generate_coincidences_det(coinc, t.xv.data(), X, t.dv.data(), D, BL);
  return true;
}

// R/rpu_pulsed_device.h:461-474 PULSED_UPDATE_W_LOOP_DENSE
void dense_update(OrcTile &t, const int *coinc) {
  const size_t total = (size_t)t.X * t.D;
  for (size_t k = 0; k < total; ++k) {
    int c = coinc[k];
    if (c == 0) continue;
    int ac = abs(c);
    int sign = c > 0 ? 1 : -1;
    for (int n = 0; n < ac; ++n) device_step(t, k, sign, true);
  }
}

// R/rpu_weight_updater.cpp:197-294 updateVectorWithDevice
bool update_vector(OrcTile &t, const float *x, int x_inc, const float *d, int d_inc) {
  const float lr = t.lr; // R/rpu.cpp:1400-1403 getAlphaLearningRate with bwd_alpha = 1
  if (!lr) return true;
  const int X = t.X, D = t.D;
  if (!is_pulsed_device(t) || t.up.pulse_type == RPU_PULSE_NONE || t.up.pulse_type == RPU_PULSE_NONE_WITH_DEVICE) {
    // R/rpu.cpp:706-714 RPUSimple::updateVector: W += -lr * d x^T
    for (int i = 0; i < D; ++i) {
      const float di = -lr * d[(size_t)i * d_inc];
      float *row = t.w.data() + (size_t)i * X;
      for (int j = 0; j < X; ++j) row[j] += di * x[(size_t)j * x_inc];
    }
    if (is_pulsed_device(t) && t.up.pulse_type == RPU_PULSE_NONE_WITH_DEVICE) {
      // R/rpu_weight_updater.cpp:220-222 clipWeights(weights, -1): the device bounds only
      for (size_t k = 0; k < t.w.size(); ++k) {
        t.w[k] = std::min(t.w[k], t.w_max[k]);
        t.w[k] = std::max(t.w[k], t.w_min[k]);
      }
    }
    return true;
  }
  int BL;
  float A, B;
  // Stochastic differs from StochasticCompressed only in keeping positive and negative x in separate lists
  // (R/sparse_bit_line_maker.cpp:145-196): per cross-point the same pulses in the same order
  if (t.up.pulse_type == RPU_PULSE_STOCHASTIC_COMPRESSED || t.up.pulse_type == RPU_PULSE_STOCHASTIC) {
    if (!sample_bl_ab(t, x, x_inc, d, d_inc, lr < 0.0f ? -lr : lr, BL, A, B)) return false;
    if (BL == 0) return true;
    ensure_sparse_containers(t, BL); // without update management a large learning rate lengthens the bit line
    generate_counts(t, t.x_cnt, t.x_idx, x, x_inc, X, B, BL);
    generate_counts(t, t.d_cnt, t.d_idx, d, d_inc, D, A, BL);
    sparse_update(t, BL, lr < 0.0f ? -1 : 1);
    return true;
  }
  if (t.up.pulse_type == RPU_PULSE_DETERMINISTIC_IMPLICIT || t.up.pulse_type == RPU_PULSE_MEAN_COUNT) {
    t.coinc.resize((size_t)X * D);
    if (!dense_coincidences(t, x, x_inc, d, d_inc, lr, t.coinc.data())) return false;
    dense_update(t, t.coinc.data());
    return true;
  }
  g_err = "oracle: pulse type not restated";
  return false;
}

// R/rpu_weight_updater.cpp:297-324 getSparseCountsFromCounts (one 32-bit word per element, BL <= 31)
void words_to_sparse(std::vector<std::vector<int>> &indices, std::vector<int> &counts,
                     const uint32_t *words, int K, int size) {
  for (int k = 0; k < K; ++k) counts[k] = 0;
  for (int i = 0; i < size; ++i) {
    const uint32_t c = words[i];
    const uint32_t negative = c & 1u;
    for (int s = 0; s < K; ++s) {
      if ((c & (1u << (s + 1))) != 0) {
        indices[s][counts[s]++] = negative > 0 ? -(i + 1) : (i + 1);
      }
    }
  }
}

const float *with_bias(OrcTile &t, const float *x, int m_batch, bool x_trans) {
  // R/rpu.cpp:672-678 copyToMatrixBiasBuffer / math::makeBias: append a row / column of ones
  const int X = t.X;
  t.bias_buf.resize((size_t)m_batch * X);
  if (x_trans) { // [X-1][B] -> [X][B]
    memcpy(t.bias_buf.data(), x, sizeof(float) * (size_t)(X - 1) * m_batch);
    for (int b = 0; b < m_batch; ++b) t.bias_buf[(size_t)(X - 1) * m_batch + b] = 1.0f;
  } else {
    for (int b = 0; b < m_batch; ++b) {
      memcpy(&t.bias_buf[(size_t)b * X], x + (size_t)b * (X - 1), sizeof(float) * (X - 1));
      t.bias_buf[(size_t)b * X + X - 1] = 1.0f;
    }
  }
  return t.bias_buf.data();
}

} // namespace

extern "C" {

const char *orc_last_error(void) { return g_err.c_str(); }

// R/rpu_pulsed.cpp:460-495 populateParameter
void *orc_create(int x_size, int d_size, const rpu_tile_config *cfg) {
  auto t = std::make_unique<OrcTile>();
  t->X = x_size;
  t->D = d_size;
  t->fio.p = cfg->f_io;
  t->bio.p = cfg->b_io;
  t->up = cfg->up;
  t->dev = cfg->device;
  if (!init_io(t->fio, false) || !init_io(t->bio, true)) return nullptr;
  // R/rpu_pulsed_meta_parameter.cpp:134-150 initialize: UBLM implies UM
  t->up.update_management = t->up.update_management || t->up.update_bl_management;
  if (t->up.desired_bl < 1) {
    g_err = "oracle: desired_bl must be positive";
    return nullptr;
  }
  if (t->dev.kind == RPU_DEVICE_SOFT_BOUNDS) { // R/rpu_linearstep_device.h:68-80
    t->dev.ls_decrease_up = 1.0f;
    t->dev.ls_decrease_down = 1.0f;
    t->dev.ls_decrease_up_dtod = 0.0f;
    t->dev.ls_decrease_down_dtod = 0.0f;
    t->dev.ls_allow_increasing_slope = 0;
    t->dev.ls_mean_bound_reference = 0;
  }
  t->w.assign((size_t)x_size * d_size, 0.f);
  t->w_persistent.assign((size_t)x_size * d_size, 0.f);
  t->rng.seed(0);
  populate_lines(*t, t->fio.p, t->lines[0], d_size);
  populate_lines(*t, t->bio.p, t->lines[1], x_size);
  if (is_pulsed_device(*t)) {
    if (t->dev.write_noise_std > 0.f && !is_linear_device(*t)) { // R/rpu_pulsed_device.h:106-111
      g_err = "oracle: Device does not support write noise";
      return nullptr;
    }
    OrcRealWorldRng rw(t->dev.construction_seed);
    if (!populate_pulsed(*t, rw)) return nullptr;
    if (is_linear_device(*t) && !populate_linear_step(*t, rw)) return nullptr;
    clip_to_bounds(*t);
  }
  return t.release();
}

void orc_destroy(void *h) { delete static_cast<OrcTile *>(h); }

void orc_set_seed(void *h, unsigned int seed) { static_cast<OrcTile *>(h)->rng.seed(seed); }
void orc_use_gauss_table(void *h, int on) { static_cast<OrcTile *>(h)->rng.use_table = on != 0; }
void orc_set_learning_rate(void *h, float lr) { static_cast<OrcTile *>(h)->lr = lr; }
void orc_set_weight_granularity(void *h, float g) { static_cast<OrcTile *>(h)->granularity = g; }

// onSetWeights (R/rpu_pulsed_device.cpp:545-571) after the bounds: the given weights are the persistent ones, the shown
// ones get fresh noise if asked for
static void on_set_weights(OrcTile &t) {
  if (!uses_persistent(t)) return;
  t.w_persistent = t.w;
  if (t.dev.apply_write_noise_on_set) {
    const float std_ = t.dev.write_noise_std * t.dev.dw_min;
    for (size_t k = 0; k < t.w.size(); ++k) t.w[k] = t.w_persistent[k] + std_ * t.rng.gauss();
  }
}
void orc_set_weights(void *h, const float *w) { // R/rpu_pulsed.cpp:288-292
  auto *t = static_cast<OrcTile *>(h);
  memcpy(t->w.data(), w, sizeof(float) * t->w.size());
  clip_to_bounds(*t);
  on_set_weights(*t);
}
// per-line values of the periphery: dir 0 forward / 1 backward; which 0 v_offset, 1 out_nonlinearity, 2 out_noise_values,
// 3 w_asymmetry ([D][X])
// (the entries of the reference's state, R/rpu_forward_backward_pass.cpp:62-100).  Returns the length.
static std::vector<float> &line_vector(OrcTile &t, int dir, int which) {
  OrcTile::Lines &mv = t.lines[dir ? 1 : 0];
  return which == 0 ? mv.v_offset : (which == 1 ? mv.out_nl : (which == 2 ? mv.out_noise : mv.w_asymmetry));
}
int orc_get_lines(void *h, int dir, int which, float *out) {
  auto *t = static_cast<OrcTile *>(h);
  const std::vector<float> &v = line_vector(*t, dir, which);
  if (out) memcpy(out, v.data(), sizeof(float) * v.size());
  return (int)v.size();
}
int orc_set_lines(void *h, int dir, int which, const float *in, int n) {
  auto *t = static_cast<OrcTile *>(h);
  std::vector<float> &v = line_vector(*t, dir, which);
  if ((int)v.size() != n) return 1;
  memcpy(v.data(), in, sizeof(float) * v.size());
  set_nl_factor(dir ? t->bio.p : t->fio.p, t->lines[dir ? 1 : 0], dir ? t->X : t->D);
  return 0;
}
void orc_repopulate_lines(void *h) { // with the generator as it is now seeded
  auto *t = static_cast<OrcTile *>(h);
  populate_lines(*t, t->fio.p, t->lines[0], t->D);
  populate_lines(*t, t->bio.p, t->lines[1], t->X);
}
float orc_get_nl_factor(void *h, int dir) { return static_cast<OrcTile *>(h)->lines[dir ? 1 : 0].nl_factor; }

void orc_get_persistent(void *h, float *w) {
  auto *t = static_cast<OrcTile *>(h);
  const std::vector<float> &src = uses_persistent(*t) ? t->w_persistent : t->w;
  memcpy(w, src.data(), sizeof(float) * src.size());
}
void orc_get_weights(void *h, float *w) {
  auto *t = static_cast<OrcTile *>(h);
  memcpy(w, t->w.data(), sizeof(float) * t->w.size());
}

// order as R/rpu_pulsed_device.cpp:235-253 getDPNames (+ slope_up, slope_down for LinearStep)
int orc_hidden_count(void *h) {
  auto *t = static_cast<OrcTile *>(h);
  if (!is_pulsed_device(*t)) return 0;
  return is_linear_device(*t) ? 10 : 8;
}
static std::vector<float> *hidden_array(OrcTile *t, int idx) {
  switch (idx) {
  case 0: return &t->w_max;
  case 1: return &t->w_min;
  case 2: return &t->scale_up;
  case 3: return &t->scale_down;
  case 4: return &t->decay_scale;
  case 5: return &t->diffusion_rate;
  case 6: return &t->reset_bias;
  case 8: return &t->slope_up;
  case 9: return &t->slope_down;
  default: return nullptr; // 7 = drift_nu: zeros without a drifter
  }
}
void orc_get_hidden(void *h, float *data) {
  auto *t = static_cast<OrcTile *>(h);
  const size_t n = t->w.size();
  for (int k = 0; k < orc_hidden_count(h); ++k) {
    auto *a = hidden_array(t, k);
    if (a) memcpy(data + k * n, a->data(), sizeof(float) * n);
    else memset(data + k * n, 0, sizeof(float) * n);
  }
}
void orc_set_hidden(void *h, const float *data) { // R/rpu_pulsed_device.cpp:290-330 + onSetWeights
  auto *t = static_cast<OrcTile *>(h);
  const size_t n = t->w.size();
  for (int k = 0; k < orc_hidden_count(h); ++k) {
    auto *a = hidden_array(t, k);
    if (a) memcpy(a->data(), data + k * n, sizeof(float) * n);
  }
  clip_to_bounds(*t);
  on_set_weights(*t);
}

// R/rpu.cpp:508-533 forward + R/rpu.cpp:42-57 forwardMatrix loop
int orc_forward(void *h, const float *x_in, float *y, int m_batch, int bias, int x_trans, int d_trans) {
  auto *t = static_cast<OrcTile *>(h);
  const float *x = bias ? with_bias(*t, x_in, m_batch, x_trans) : x_in;
  const int x_offset = x_trans ? 1 : t->X, d_offset = d_trans ? 1 : t->D;
  const int x_inc = x_trans ? m_batch : 1, d_inc = d_trans ? m_batch : 1;
  t->last_rounds.assign(m_batch, 0);
  for (int b = 0; b < m_batch; ++b) {
    if (t->fio.perfect) {
      fp_forward(*t, x + (size_t)b * x_offset, x_inc, y + (size_t)b * d_offset, d_inc, t->fio.p.out_scale);
    } else {
      t->last_rounds[b] = forward_vector(*t, x + (size_t)b * x_offset, x_inc, y + (size_t)b * d_offset, d_inc);
    }
  }
  return 0;
}

void orc_get_bm_rounds(void *h, int32_t *rounds, int m_batch) {
  auto *t = static_cast<OrcTile *>(h);
  for (int b = 0; b < m_batch && b < (int)t->last_rounds.size(); ++b) rounds[b] = t->last_rounds[b];
}

// R/rpu.cpp:535-554 backward + :59-73 backwardMatrix loop (+ copyWithoutBias)
int orc_backward(void *h, const float *d, float *x_out, int m_batch, int bias, int d_trans, int x_trans) {
  auto *t = static_cast<OrcTile *>(h);
  const int X = t->X;
  std::vector<float> tmp;
  float *x = x_out;
  if (bias) {
    tmp.resize((size_t)m_batch * X);
    x = tmp.data();
  }
  const int x_offset = x_trans ? 1 : X, d_offset = d_trans ? 1 : t->D;
  const int x_inc = x_trans ? m_batch : 1, d_inc = d_trans ? m_batch : 1;
  for (int b = 0; b < m_batch; ++b) {
    if (t->bio.perfect) {
      fp_backward(*t, d + (size_t)b * d_offset, d_inc, x + (size_t)b * x_offset, x_inc, t->bio.p.out_scale);
    } else {
      backward_vector(*t, d + (size_t)b * d_offset, d_inc, x + (size_t)b * x_offset, x_inc);
    }
  }
  if (bias) {
    if (x_trans) {
      memcpy(x_out, x, sizeof(float) * (size_t)(X - 1) * m_batch);
    } else {
      for (int b = 0; b < m_batch; ++b)
        memcpy(x_out + (size_t)b * (X - 1), x + (size_t)b * X, sizeof(float) * (X - 1));
    }
  }
  return 0;
}

// R/rpu.cpp:556-575 update + :75-89 updateMatrix loop (R/rpu_pulsed.cpp:558-585)
int orc_update(void *h, const float *x_in, const float *d, int m_batch, int bias, int x_trans, int d_trans) {
  auto *t = static_cast<OrcTile *>(h);
  const float *x = bias ? with_bias(*t, x_in, m_batch, x_trans) : x_in;
  const int x_offset = x_trans ? 1 : t->X, d_offset = d_trans ? 1 : t->D;
  const int x_inc = x_trans ? m_batch : 1, d_inc = d_trans ? m_batch : 1;
  for (int b = 0; b < m_batch; ++b) {
    if (!update_vector(*t, x + (size_t)b * x_offset, x_inc, d + (size_t)b * d_offset, d_inc)) return 1;
  }
  return 0;
}

// R/rpu_weight_updater.cpp:327-393 updateVectorWithDeviceAndCounts, looped over the batch: drives the CPU
// device with packed pulse words made elsewhere.  x_words [m_batch][X], d_words [m_batch][D], bl [m_batch].
int orc_update_with_words(void *h, const uint32_t *x_words, const uint32_t *d_words, const int32_t *bl,
                          int m_batch) {
  auto *t = static_cast<OrcTile *>(h);
  if (!t->lr) return 0;
  ensure_sparse_containers(*t);
  const int lr_sign = t->lr < 0.0f ? -1 : 1;
  for (int b = 0; b < m_batch; ++b) {
    const int BL = bl[b];
    if (BL <= 0) continue;
    if (BL > 31) {
      g_err = "oracle: a packed word holds 31 pulses (longer bit lines come as several rows of words)";
      return 1;
    }
    words_to_sparse(t->x_idx, t->x_cnt, x_words + (size_t)b * t->X, BL, t->X);
    words_to_sparse(t->d_idx, t->d_cnt, d_words + (size_t)b * t->D, BL, t->D);
    sparse_update(*t, BL, lr_sign);
  }
  return 0;
}

// BL, A, B of every sample (R/rpu_pulsed_meta_parameter.cpp:152-236 through the bit line makers)
int orc_update_bl_ab(void *h, const float *x, const float *d, int m_batch, int32_t *bl, float *a, float *b_out) {
  auto *t = static_cast<OrcTile *>(h);
  for (int b = 0; b < m_batch; ++b) {
    int BL;
    float A, B;
    if (!sample_bl_ab(*t, x + (size_t)b * t->X, 1, d + (size_t)b * t->D, 1, fabsf(t->lr), BL, A, B)) return 1;
    bl[b] = BL;
    a[b] = A;
    b_out[b] = B;
  }
  return 0;
}

// signed coincidence counts of the deterministic implicit scheme for every sample: counts [m_batch][D][X]
int orc_implicit_counts(void *h, const float *x, const float *d, int m_batch, int32_t *counts) {
  auto *t = static_cast<OrcTile *>(h);
  const int X = t->X, D = t->D;
  for (int b = 0; b < m_batch; ++b) {
    if (!dense_coincidences(*t, x + (size_t)b * X, 1, d + (size_t)b * D, 1, t->lr, counts + (size_t)b * X * D)) return 1;
  }
  return 0;
}

} // extern "C"
