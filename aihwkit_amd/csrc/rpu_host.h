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
};

struct UpdatePar {
  rpu_update_params p{};
  void initialize(); // rpu_pulsed_meta_parameter.cpp:134-150
};

// Per-crosspoint parameters, row-major [d_size][x_size].
struct DeviceArrays {
  std::vector<float> w_max, w_min, scale_up, scale_down, decay_scale, diffusion_rate, reset_bias;
  std::vector<float> slope_up, slope_down; // LinearStep / SoftBounds only
};

struct DevicePar {
  rpu_device_params p{};
  void initialize();
  bool pulsed() const { return p.kind != RPU_DEVICE_IDEAL; }
  bool linear() const { return p.kind == RPU_DEVICE_LINEAR_STEP || p.kind == RPU_DEVICE_SOFT_BOUNDS; }
  float weight_granularity() const { return p.dw_min; }
  // rpu_pulsed_device.cpp:593-733 and rpu_linearstep_device.cpp:20-74
  void populate(int x_size, int d_size, DeviceArrays &out) const;
};

void fill_default_config(rpu_tile_config *cfg, int device_kind);

} // namespace rpu_amd
