#include "rpu_host.h"

#include <algorithm>
#include <cfloat>
#include <chrono>
#include <cmath>
#include <limits>
#include <random>

namespace rpu_amd {

namespace {

// "1/steps" or "steps" -> fraction of the full range (rpu_pulsed_meta_parameter.cpp:26-30)
float normalized_resolution(float res) {
  const float r = res < 0.0f ? 0.0f : res;
  return r > 1.0f ? 1.0f / r : r;
}

// Construction-time generator: same engine and distributions as the reference's RealWorldRNG
// (rng.h:45-61) so that one construction_seed gives the same device arrays.
class ConstructionRng {
public:
  explicit ConstructionRng(unsigned int seed) {
    unsigned int s = seed;
    if (s == 0) {
      s = (unsigned int)std::chrono::high_resolution_clock::now().time_since_epoch().count();
    }
    engine_.seed(s);
  }
  float normal() { return normal_(engine_); }
  float uniform() { return uniform_(engine_); }

private:
  std::default_random_engine engine_;
  std::uniform_real_distribution<float> uniform_{0.0f, 1.0f};
  std::normal_distribution<float> normal_{0.0f, 1.0f};
};

} // namespace

void IOPar::initialize(bool backward) {
  if (p.mv_type == RPU_MV_IDEAL) {
    p.is_perfect = 1;
  }
  if (p.is_perfect) {
    p.mv_type = RPU_MV_IDEAL;
    perfect = true;
    return;
  }
  perfect = false;
  if (p.mv_type != RPU_MV_ONE_PASS && p.mv_type != RPU_MV_POS_NEG_SEPARATE &&
      p.mv_type != RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM) {
    throw RpuError("AnalogMVType not implemented on this path (only Ideal, OnePass, PosNegSeparate and "
                   "PosNegSeparateDigitalSum).");
  }
  if (p.w_noise_type < 0 || p.w_noise_type > 2) {
    throw RpuError("Output noise type not implemented");
  }
  switch (p.noise_management) {
  case RPU_NM_NONE:
  case RPU_NM_ABS_MAX:
  case RPU_NM_ABS_MAX_NP_SUM:
  case RPU_NM_MAX:
  case RPU_NM_CONSTANT:
  case RPU_NM_AVERAGE_ABS_MAX:
  case RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE:
    break;
  default:
    throw RpuError("Noise Management type not implemented!");
  }
  if (p.bound_management < RPU_BM_NONE || p.bound_management > RPU_BM_ITERATIVE_WORST_CASE) {
    throw RpuError("Bound management type not implemented!");
  }

  // absolute steps are taken with the bounds as given, before non-positive bounds turn into "no bound"
  p.out_res = normalized_resolution(p.out_res) * (2.0f * p.out_bound);
  p.inp_res = normalized_resolution(p.inp_res) * (2.0f * p.inp_bound);

  if (p.noise_management != RPU_NM_NONE) {
    if (p.inp_bound != 1.0f) {
      throw RpuError(
          backward ? "Backward noise managment expects input bound==1"
                   : "Forward noise managment expects bound==1");
    }
  } else {
    p.nm_thres = 0.0f;
  }
  if (p.out_bound <= 0.0f) {
    p.out_bound = std::numeric_limits<float>::infinity();
  }
  if (p.inp_bound <= 0.0f) {
    p.inp_bound = std::numeric_limits<float>::infinity();
  }
  if (backward) {
    p.bound_management = RPU_BM_NONE; // the backward pass never iterates (rpu_forward_backward_pass.cpp:1002)
  }
}

// Per-line values of the periphery (ForwardBackwardPassIOManaged::populateFBParameter,
// rpu_forward_backward_pass.cpp:254-318): voltage offsets, non-linearity coefficients with the slope calibration
// factor, and output noise levels.  The reference draws them from the tile's run-time generator; any stream will do.
void IOPar::populate_lines(int out_size, unsigned int seed, size_t n_weights) {
  v_offset.clear();
  out_nl.clear();
  out_noise_values.clear();
  w_asymmetry.clear();
  nl_factor = 1.0f;
  if (perfect) return;
  ConstructionRng rng(seed); // 0: from the clock
  if (has_voltage_offsets()) {
    v_offset.resize(out_size);
    for (float &v : v_offset) v = std::max(p.v_offset_std * rng.normal(), 0.0f);
  }
  const float out_bound = (p.out_bound > 0.0f && p.out_bound < std::numeric_limits<float>::infinity()) ? p.out_bound : 1.0f;
  if (has_nl_calibration()) {
    out_nl.resize(out_size);
    for (float &v : out_nl) {
      v = fabsf(p.out_nonlinearity / out_bound * (1.0f + std::max(p.out_nonlinearity_std, 0.0f) * rng.normal()));
    }
  }
  set_nl_factor();
  if (p.w_read_asymmetry_dtod != 0.0f) {
    w_asymmetry.resize(n_weights);
    for (float &v : w_asymmetry) v = 1.0f + p.w_read_asymmetry_dtod * rng.normal();
  }
  if (p.out_noise_std > 0.0f) {
    out_noise_values.resize(out_size);
    for (float &v : out_noise_values) v = fabsf(p.out_noise * (1.0f + p.out_noise_std * rng.normal()));
  }
}

void IOPar::set_nl_factor() {
  nl_factor = 1.0f;
  if (perfect || p.slope_calibration <= 0.0f) return;
  const float out_bound = (p.out_bound > 0.0f && p.out_bound < std::numeric_limits<float>::infinity()) ? p.out_bound : 1.0f;
  float sum_nl = 0.0f;
  if (p.out_nonlinearity > 0.0f) {
    for (float v : out_nl) sum_nl += fabsf(v);
  }
  const float n = out_nl.empty() ? 1.0f : (float)out_nl.size();
  const float f = 1.0f + (sum_nl / n + p.r_series) * p.slope_calibration * out_bound;
  nl_factor = f * f;
}

void UpdatePar::initialize() {
  p.update_management = (p.update_management || p.update_bl_management) ? 1 : 0;
  // Stochastic keeps the pulse trains of positive and negative inputs in separate lists
  // (sparse_bit_line_maker.cpp:145-196, 323-333); every cross-point sees the same pulses in the same order as with the
  // compressed lists, so the two types are one on this path
  if (p.pulse_type == RPU_PULSE_STOCHASTIC) p.pulse_type = RPU_PULSE_STOCHASTIC_COMPRESSED;
  switch (p.pulse_type) {
  case RPU_PULSE_NONE:
  case RPU_PULSE_NONE_WITH_DEVICE:
  case RPU_PULSE_STOCHASTIC_COMPRESSED:
  case RPU_PULSE_MEAN_COUNT:
  case RPU_PULSE_DETERMINISTIC_IMPLICIT:
    break;
  default:
    throw RpuError("PulseType not supported");
  }
  if (p.pulse_type != RPU_PULSE_NONE && p.pulse_type != RPU_PULSE_NONE_WITH_DEVICE && (p.desired_bl < 1 || p.desired_bl > RPU_MAX_BL)) {
    throw RpuError("desired_bl must be within 1.." + std::to_string(RPU_MAX_BL) + ".");
  }
}

void DevicePar::initialize() {
  if (p.kind < RPU_DEVICE_IDEAL || p.kind > RPU_DEVICE_SOFT_BOUNDS) {
    throw RpuError("Unknown device kind (a transfer compound is created with rpu_tile_create_transfer).");
  }
  if (p.kind == RPU_DEVICE_SOFT_BOUNDS) {
    // SoftBounds is LinearStep with zero step at the (actual) bounds (rpu_linearstep_device.h:68-80)
    p.ls_decrease_up = 1.0f;
    p.ls_decrease_down = 1.0f;
    p.ls_decrease_up_dtod = 0.0f;
    p.ls_decrease_down_dtod = 0.0f;
    p.ls_allow_increasing_slope = 0;
    p.ls_mean_bound_reference = 0;
  }
  if (pulsed()) {
    if (p.write_noise_std > 0.0f && !linear()) {
      throw RpuError("Device does not support write noise"); // rpu_pulsed_device.h:107-111
    }
    if (p.w_min > 0.0f || p.w_max < 0.0f) {
      throw RpuError("The closed interval [w_min,w_max] needs to contain 0.");
    }
    if (linear() && (p.ls_reverse_up || p.ls_reverse_down) && !p.ls_mult_noise) {
      throw RpuError("Only mulitplicative noise supported with reverse up/down!");
    }
    p.reset_dtod = std::max(p.reset_dtod, 0.0f);
    p.reset_std = std::max(p.reset_std, 0.0f);
    p.diffusion = std::max(p.diffusion, 0.0f);
    p.lifetime = std::max(p.lifetime, 0.0f);
  }
}

namespace {
void populate_from(const DevicePar &dev, ConstructionRng &rng, int x_size, int d_size, DeviceArrays &a);
}

void DevicePar::populate(int x_size, int d_size, DeviceArrays &a) const {
  ConstructionRng rng(p.construction_seed);
  populate_from(*this, rng, x_size, d_size, a);
}

void populate_chain(const std::vector<DevicePar> &pars, unsigned int seed, int x_size, int d_size,
                    std::vector<DeviceArrays> &out) {
  ConstructionRng rng(seed);
  out.assign(pars.size(), DeviceArrays());
  for (size_t k = 0; k < pars.size(); ++k) populate_from(pars[k], rng, x_size, d_size, out[k]);
}

namespace {
void populate_from(const DevicePar &dev, ConstructionRng &rng, int x_size, int d_size, DeviceArrays &a) {
  const rpu_device_params &p = dev.p;
  const auto pulsed = [&] { return dev.pulsed(); };
  const auto linear = [&] { return dev.linear(); };
  const size_t n = (size_t)x_size * (size_t)d_size;
  a = DeviceArrays();
  // the drift coefficients are drawn first, in memory order (SimpleRPUDevice::populate,
  // rpu_simple_device.cpp:171-182; WeightDrifter::populate, weight_drifter.cpp:57-65)
  if (p.drift_nu > 0.0f) {
    a.drift_nu.resize(n);
    for (size_t k = 0; k < n; ++k) a.drift_nu[k] = p.drift_nu + p.drift_nu_dtod * p.drift_nu * rng.normal();
  }
  if (!pulsed()) {
    return;
  }
  a.w_max.resize(n);
  a.w_min.resize(n);
  a.scale_up.resize(n);
  a.scale_down.resize(n);
  a.decay_scale.resize(n);
  a.diffusion_rate.resize(n);
  a.reset_bias.resize(n);

  const float bias_up = p.up_down > 0.0f ? 0.0f : p.up_down;
  const float bias_down = p.up_down > 0.0f ? -p.up_down : 0.0f;

  // Pass 1 walks the array column by column (x outer, d inner) with a fixed number of draws per
  // cross-point: bounds (2 normals), step gain, up/down asymmetry, one uniform for the corrupt-device
  // test, diffusion, reset and (only with a lifetime) decay.
  for (int col = 0; col < x_size; ++col) {
    for (int row = 0; row < d_size; ++row) {
      const size_t k = (size_t)row * x_size + col;
      float hi = p.w_max * (1.0f + p.w_max_dtod * rng.normal());
      float lo = p.w_min * (1.0f + p.w_min_dtod * rng.normal());
      const float g = rng.normal();
      const float gain = p.dw_min_dtod_log_normal ? expf(p.dw_min_dtod * g) : (1.0f + p.dw_min_dtod * g);
      const float asym = p.up_down_dtod * rng.normal();
      float up = (bias_up + gain + asym) * p.dw_min;
      float down = (bias_down + gain - asym) * p.dw_min;

      if (p.enforce_consistency) {
        up = fabsf(up);
        down = fabsf(down);
        if (lo > hi) {
          std::swap(lo, hi);
        }
        hi = fabsf(hi);
        lo = -fabsf(lo);
      } else if (lo > hi) {
        // inconsistent draw: collapse the window onto its centre
        const float centre = hi + (lo - hi) / 2.0f;
        hi = centre;
        lo = centre;
      }

      if (p.adjust_bounds_with_up_down) {
        if (lo > hi) {
          std::swap(lo, hi);
        }
        const float alpha = up / (up + down);
        const float width = hi - lo;
        float new_lo = 0.0f;
        if (p.adjust_bounds_with_up_down_dev > 0.0f) {
          new_lo = -(((float)tanh((float)((alpha - 0.5f) / p.adjust_bounds_with_up_down_dev)) + 1.0f) / 2.0f) * width;
        } else if (alpha < 0.5f) {
          new_lo = 0.0f;
        } else if (alpha == 0.5f) {
          new_lo = -width / 2.0f;
        } else {
          new_lo = -width;
        }
        lo = new_lo;
        hi = new_lo + width;
      }

      if (p.corrupt_devices_prob > rng.uniform()) {
        const float range = fabsf(p.corrupt_devices_range);
        const float from = std::max(std::min(hi, lo), -range);
        const float to = std::min(std::max(hi, lo), range);
        const float stuck = from + (to - from) * rng.uniform();
        hi = stuck;
        lo = stuck;
        up = 0.0f;
        down = 0.0f;
      }

      if (p.perfect_bias && col == x_size - 1) {
        up = p.dw_min;
        down = p.dw_min;
        lo = 100.0f * p.w_min;
        hi = 100.0f * p.w_max;
      }

      a.w_max[k] = hi;
      a.w_min[k] = lo;
      a.scale_up[k] = up;
      a.scale_down[k] = down;
      a.diffusion_rate[k] = fabsf(p.diffusion * (1.0f + p.diffusion_dtod * rng.normal()));
      a.reset_bias[k] = p.reset + p.reset_dtod * rng.normal();
      if (p.lifetime > 0.0f) {
        const float life = p.lifetime * (1.0f + p.lifetime_dtod * rng.normal());
        a.decay_scale[k] = (life > 1.0f) ? (1.0f - (1.0f / life)) : 0.0f;
      } else {
        a.decay_scale[k] = 1.0f;
      }
    }
  }

  if (!linear()) {
    return;
  }
  // Pass 2 (row by row): the two slopes of the linear step, two normals per cross-point.
  a.slope_up.resize(n);
  a.slope_down.resize(n);
  for (int row = 0; row < d_size; ++row) {
    for (int col = 0; col < x_size; ++col) {
      const size_t k = (size_t)row * x_size + col;
      float dec_up = p.ls_decrease_up + p.ls_decrease_up_dtod * rng.normal();
      float dec_down = p.ls_decrease_down + p.ls_decrease_down_dtod * rng.normal();
      if (!p.ls_allow_increasing_slope) {
        dec_up = fabsf(dec_up);
        dec_down = fabsf(dec_down);
      }
      float ref_up, ref_down;
      if (p.ls_mean_bound_reference) {
        ref_up = p.ls_reverse_up ? p.w_min - p.ls_reverse_offset : p.w_max;
        ref_down = p.ls_reverse_down ? p.w_max + p.ls_reverse_offset : p.w_min;
      } else {
        ref_up = p.ls_reverse_up ? a.w_min[k] - p.ls_reverse_offset : a.w_max[k];
        ref_down = p.ls_reverse_down ? a.w_max[k] + p.ls_reverse_offset : a.w_min[k];
      }
      a.slope_up[k] = ref_up != 0.0f ? -dec_up * a.scale_up[k] / ref_up : 0.0f;
      a.slope_down[k] = ref_down != 0.0f ? -dec_down * a.scale_down[k] / ref_down : 0.0f;
    }
  }
}
} // namespace

void TransferPar::initialize(int x_size, int d_size) {
  const int n_dev = p.n_devices;
  if (n_dev < 2) throw RpuError("Need at least 2 devices");
  if (n_dev > RPU_MAX_VECTOR_DEVICES) throw RpuError("At most 16 devices in a transfer chain.");
  if (p.with_reset_prob > 0.0f && !p.transfer_columns) {
    throw RpuError("Reset prob is only implemented for column-transfer so far."); // rpu_transfer_device.cpp:198-200
  }
  devs.clear();
  for (int k = 0; k < n_dev; ++k) {
    DevicePar d;
    d.p = k == 0 ? p.fast_device : p.rest_device;
    d.initialize();
    if (!d.pulsed()) throw RpuError("The devices of a transfer chain must be pulsed devices.");
    if (d.persistent_weights()) throw RpuError("write_noise_std > 0 is not provided for the devices of a transfer chain.");
    devs.push_back(d);
  }
  in_size = p.transfer_columns ? x_size : d_size;
  out_size = p.transfer_columns ? d_size : x_size;

  // weightening of the devices (rpu_transfer_device.cpp:146-168)
  gamma_vec.clear();
  if (p.n_gamma_vec > 0) {
    if (p.n_gamma_vec != n_dev) throw RpuError("If gamma_vec is set manually expect the same size as number of devices.");
    float g = 0.0f;
    for (int i = 0; i < n_dev; ++i) gamma_vec.push_back(p.gamma_vec[i]);
    for (int i = 0; i < n_dev - 1; ++i) g += gamma_vec[i];
    if (gamma_vec[n_dev - 1] == 0.0f) {
      throw RpuError("Expect that last device has some constribution to the network weights. [otherwise why transfer?]");
    }
    p.gamma = g;
  } else {
    gamma_vec.resize(n_dev);
    for (int i = 0; i < n_dev; ++i) gamma_vec[n_dev - i - 1] = powf(p.gamma, (float)i);
  }
  lr_vec.clear();
  if (p.n_transfer_lr_vec > 0) {
    if (p.n_transfer_lr_vec != n_dev) throw RpuError("Expect transfer_lr_vec of size n_devices.");
    for (int i = 0; i < n_dev; ++i) lr_vec.push_back(p.transfer_lr_vec[i]);
  } else {
    lr_vec.assign(n_dev, p.transfer_lr);
  }
  if (p.n_reads_per_transfer > in_size) p.n_reads_per_transfer = in_size;
  if (p.n_reads_per_transfer < 1) throw RpuError("n_reads_per_transfer must be positive.");
  every_vec.clear();
  if (p.n_transfer_every_vec > 0) {
    if (p.n_transfer_every_vec != n_dev) throw RpuError("Expect transfer_every_vec to be of length n_devices");
    for (int i = 0; i < n_dev; ++i) every_vec.push_back(p.transfer_every_vec[i]);
  } else {
    float every = p.transfer_every;
    for (int i = 0; i < n_dev; ++i) {
      every_vec.push_back(every);
      every *= (float)out_size / (float)p.n_reads_per_transfer;
    }
    if (p.no_self_transfer) every_vec[n_dev - 1] = 0.0f;
  }
  // IO of the read: management off (rpu_transfer_device.cpp:198-213)
  io.p = p.transfer_io;
  io.p.bound_management = RPU_BM_NONE;
  io.p.noise_management = RPU_NM_NONE;
  io.initialize(!p.transfer_columns);
  if (io.p.w_read_asymmetry_dtod != 0.0f) {
    throw RpuError("Read asymmetry of the negative pass (w_read_asymmetry_dtod) is not provided for the read of a transfer.");
  }
  up.p = p.transfer_up;
  up.initialize();
  fully_hidden = (p.gamma == 0.0f) && (gamma_vec.back() == 1.0f);
}

int TransferPar::transfer_every(int from_idx, int m_batch) const {
  if (p.units_in_mbatch) return std::max((int)ceilf(every_vec[from_idx] * (float)m_batch), 0);
  return std::max((int)roundf(every_vec[from_idx]), 0);
}

float TransferPar::granularity() const {
  float g = 0.0f;
  for (const DevicePar &d : devs) g += d.weight_granularity();
  return g / (float)devs.size();
}

void fill_default_config(rpu_tile_config *cfg, int device_kind) {
  rpu_io_params io{};
  io.is_perfect = 0;
  io.mv_type = RPU_MV_ONE_PASS;
  io.noise_management = RPU_NM_ABS_MAX;
  io.bound_management = RPU_BM_NONE;
  io.bm_test_negative_bound = 1;
  io.max_bm_factor = 1000;
  io.inp_sto_round = 0;
  io.out_sto_round = 0;
  io.inp_bound = 1.0f;
  io.inp_res = 1.0f / (powf(2.0f, 7.0f) - 2.0f);
  io.inp_noise = 0.0f;
  io.inp_asymmetry = 0.0f;
  io.out_bound = 12.0f;
  io.out_res = 1.0f / (powf(2.0f, 9.0f) - 2.0f);
  io.out_noise = 0.06f;
  io.out_asymmetry = 0.0f;
  io.out_scale = 1.0f;
  io.nm_thres = 0.0f;
  io.nm_assumed_wmax = 0.6f;
  io.max_bm_res = 0.25f;
  io.ir_drop_g_ratio = 5.7143e5f;
  io.nm_decay = 1e-3f;
  io.slope_calibration = 0.5f;
  io.v_offset_w_min = 0.0f;
  io.r_series_max_total = std::numeric_limits<float>::max();
  cfg->f_io = io;
  cfg->b_io = io;

  rpu_update_params up{};
  up.pulse_type = RPU_PULSE_STOCHASTIC_COMPRESSED;
  up.desired_bl = 31;
  up.fixed_bl = 1;
  up.update_management = 1;
  up.update_bl_management = 1;
  up.sto_round = 0;
  up.um_grad_scale = 1.0f;
  up.res = 0.0f;
  up.x_res_implicit = 0.0f;
  up.d_res_implicit = 0.0f;
  cfg->up = up;

  rpu_device_params d{};
  d.kind = device_kind;
  d.construction_seed = 0;
  d.enforce_consistency = 0;
  d.perfect_bias = 0;
  d.dw_min_dtod_log_normal = 0;
  d.adjust_bounds_with_up_down = 0;
  d.dw_min = 0.001f;
  d.dw_min_dtod = 0.3f;
  d.dw_min_std = 0.3f;
  d.w_min = -0.6f;
  d.w_min_dtod = 0.3f;
  d.w_max = 0.6f;
  d.w_max_dtod = 0.3f;
  d.up_down = 0.0f;
  d.up_down_dtod = 0.01f;
  d.adjust_bounds_with_up_down_dev = 0.0f;
  d.corrupt_devices_prob = 0.0f;
  d.corrupt_devices_range = FLT_MAX;
  d.lifetime = 0.0f;
  d.lifetime_dtod = 0.0f;
  d.diffusion = 0.0f;
  d.diffusion_dtod = 0.0f;
  d.reset = 0.0f;
  d.reset_dtod = 0.0f;
  d.reset_std = 0.01f;
  d.write_noise_std = 0.0f;
  d.apply_write_noise_on_set = 1;
  d.ls_allow_increasing_slope = 0;
  d.ls_mean_bound_reference = 1;
  d.ls_mult_noise = 1;
  d.ls_reverse_up = 0;
  d.ls_reverse_down = 0;
  d.ls_decrease_up = 0.0f;
  d.ls_decrease_down = 0.0f;
  d.ls_decrease_up_dtod = 0.05f;
  d.ls_decrease_down_dtod = 0.05f;
  d.ls_reverse_offset = 0.01f;
  // DriftParameter (weight_drifter.h:14-60)
  d.drift_nu = 0.0f;
  d.drift_nu_dtod = 0.0f;
  d.drift_nu_std = 0.0f;
  d.drift_wg_ratio = 1.0f;
  d.drift_g_offset = 0.0f;
  d.drift_w_offset = 0.0f;
  d.drift_nu_k = 0.0f;
  d.drift_log_g0 = 0.0f;
  d.drift_t0 = 1.0f;
  d.drift_reset_tol = 1e-7f;
  d.drift_w_read_std = 0.0f;
  d.count_pulses = 0;
  if (device_kind == RPU_DEVICE_SOFT_BOUNDS) {
    d.ls_decrease_up = 1.0f;
    d.ls_decrease_down = 1.0f;
    d.ls_decrease_up_dtod = 0.0f;
    d.ls_decrease_down_dtod = 0.0f;
    d.ls_mean_bound_reference = 0;
  }
  cfg->device = d;
}

void fill_default_transfer(rpu_transfer_params *tp, int device_kind) {
  rpu_tile_config cfg;
  fill_default_config(&cfg, device_kind);
  rpu_transfer_params t{};
  t.n_devices = 2;
  t.construction_seed = 0;
  t.units_in_mbatch = 0;
  t.n_reads_per_transfer = 1;
  t.no_self_transfer = 1;
  t.random_selection = 0;
  t.scale_transfer_lr = 1;
  t.scale_fast_lr = 1;
  t.transfer_columns = 1;
  t.gamma = 0.0f;
  t.transfer_every = 1.0f;
  t.with_reset_prob = 0.0f;
  t.fast_lr = 0.0f;
  t.transfer_lr = 1.0f;
  t.transfer_io = cfg.f_io;
  t.transfer_up = cfg.up;
  t.fast_device = cfg.device;
  t.rest_device = cfg.device;
  *tp = t;
}

} // namespace rpu_amd
