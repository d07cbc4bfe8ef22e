// Host-side C++ classes of the analog tile: meta-parameters and the per-crosspoint device model.
// They keep the roles of the reference's IOMetaParameter / PulsedUpdateMetaParameter
// (src/rpucuda/rpu_pulsed_meta_parameter.{h,cpp}) and PulsedRPUDevice / LinearStepRPUDevice
// (src/rpucuda/rpu_pulsed_device.cpp, rpu_linearstep_device.cpp): parameters are validated and the
// device-to-device variation is sampled on the CPU, then uploaded once.
#pragma once
#include "../../include/rpu_amd.h"

#include <stdexcept>
#include <string>
#include <vector>

namespace rpu_amd {

struct RpuError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Validated IO parameters with absolute DAC / ADC steps.
struct IOPar {
  rpu_io_params p{};
  bool perfect = false;
  void initialize(bool backward); // rpu_pulsed_meta_parameter.cpp:39-128
  // per-output-line values of the periphery (MVParameter, rpu_forward_backward_pass.h:17-26); empty when off
  std::vector<float> v_offset, out_nl, out_noise_values;
  std::vector<float> w_asymmetry; // [d_size][x_size] factors of the negative pass (PosNegSeparate), empty when off
  float nl_factor = 1.0f;
  bool has_voltage_offsets() const { return !perfect && (p.v_offset_std > 0.0f || p.r_series > 0.0f); }
  bool has_nl_calibration() const { return !perfect && (p.out_nonlinearity > 0.0f || p.r_series > 0.0f); }
  bool separate_passes() const {
    return !perfect && (p.mv_type == RPU_MV_POS_NEG_SEPARATE || p.mv_type == RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM);
  }
  bool digital_sum() const { return !perfect && p.mv_type == RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM; }
  // whether the analog value has to be built outside the contraction kernel
  bool has_line_terms() const {
    return has_voltage_offsets() || has_nl_calibration() || (!perfect && p.out_noise_std > 0.0f) || separate_passes();
  }
  void populate_lines(int out_size, unsigned int seed, size_t n_weights = 0);
  void set_nl_factor(); // from out_nl: after sampling and after the values were set from outside
};

struct UpdatePar {
  rpu_update_params p{};
  void initialize(); // rpu_pulsed_meta_parameter.cpp:134-150
};

// Per-crosspoint parameters, row-major [d_size][x_size].
struct DeviceArrays {
  std::vector<float> w_max, w_min, scale_up, scale_down, decay_scale, diffusion_rate, reset_bias;
  std::vector<float> slope_up, slope_down; // LinearStep / SoftBounds only
  std::vector<float> drift_nu;             // only with drift_nu > 0 in the parameters
  std::vector<float> persistent;           // persistent weights, only with write_noise_std > 0
};

struct DevicePar {
  rpu_device_params p{};
  void initialize();
  bool pulsed() const { return p.kind != RPU_DEVICE_IDEAL; }
  bool linear() const { return p.kind == RPU_DEVICE_LINEAR_STEP || p.kind == RPU_DEVICE_SOFT_BOUNDS; }
  bool persistent_weights() const { return linear() && p.write_noise_std > 0.0f; } // usesPersistentWeight
  float scaled_write_noise() const { return p.write_noise_std * p.dw_min; }        // getScaledWriteNoise
  float weight_granularity() const { return p.dw_min; }
  // rpu_pulsed_device.cpp:593-733 and rpu_linearstep_device.cpp:20-74
  void populate(int x_size, int d_size, DeviceArrays &out) const;
};

// Samples several devices one after the other from one stream seeded once, as VectorRPUDevice::populate
// hands the same RealWorldRNG to every sub-device (rpu_vector_device.cpp:397-431).
void populate_chain(const std::vector<DevicePar> &pars, unsigned int seed, int x_size, int d_size,
                    std::vector<DeviceArrays> &out);

// Validated parameters of the transfer compound (TransferRPUDeviceMetaParameter::initializeWithSize,
// rpu_transfer_device.cpp:119-217).
struct TransferPar {
  rpu_transfer_params p{};
  IOPar io;      // transfer_io, noise and bound management forced off
  UpdatePar up;  // transfer_up
  std::vector<DevicePar> devs;
  std::vector<float> gamma_vec, lr_vec, every_vec;
  bool fully_hidden = false; // gamma == 0 and the last gamma_vec entry is 1: the last device IS the tile's weights
  int in_size = 0, out_size = 0;
  void initialize(int x_size, int d_size);
  int n() const { return (int)devs.size(); }
  // rpu_transfer_device.cpp:219-230
  float transfer_lr(int from_idx, float current_lr) const {
    return p.scale_transfer_lr ? lr_vec[from_idx] * current_lr : lr_vec[from_idx];
  }
  // rpu_transfer_device.cpp:394-403
  int transfer_every(int from_idx, int m_batch) const;
  // rpu_transfer_device.cpp:366-383
  float fast_lr(float learning_rate) const {
    if (p.fast_lr > 0.0f) return p.scale_fast_lr ? p.fast_lr * learning_rate : p.fast_lr;
    return learning_rate;
  }
  // average over the devices (rpu_vector_device.cpp:411-421)
  float granularity() const;
};

void fill_default_config(rpu_tile_config *cfg, int device_kind);
void fill_default_transfer(rpu_transfer_params *tp, int device_kind);

} // namespace rpu_amd
