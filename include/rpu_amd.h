/*
 * rpu_amd.h -- C ABI of the MI355X (gfx950) analog-tile library (librpu_amd.so).
 *
 * The entry points below are what the `rpu_base` binding layer of IBM/aihwkit
 * would bind for the analog-tile hot path (noisy forward / backward MVM and the
 * pulsed update).  Every declaration cites the reference interface it replaces
 * (paths relative to the reference checkout; R/ = src/rpucuda/,
 * C/ = src/rpucuda/cuda/, B/ = src/aihwkit/simulator/rpu_base_src/).
 *
 * Conventions
 *  - plain C: opaque handles, plain-old-data parameter structs, raw pointers.
 *  - every function returns 0 on success and a non-zero code on failure;
 *    rpu_last_error() returns the message of the last failure on the calling
 *    thread (the reference throws std::runtime_error, R/utility_functions.h:63-69;
 *    a binding layer turns the message into its RuntimeError).
 *  - `*_dev` pointers are device (HBM) pointers of the GPU the tile lives on,
 *    `*_host` pointers are host pointers.  `stream` is a hipStream_t passed as
 *    void* (NULL = the default stream).
 *  - weights are exchanged row-major [d_size][x_size] exactly like the reference
 *    (R/rpu.h:674, B/rpu_base_tiles.cpp:161-214).
 *  - compute entry points (forward / backward / update) exist for GPU-resident
 *    tiles only.  There is no CPU compute path in this library.
 *  - a tile owns its scratch memory (per-sample state, quantized inputs, pulse words): calls on one tile
 *    must be ordered on the device, i.e. issued on one stream or on streams the caller orders with events.
 *    Calls on different tiles are independent.  The library allocates device memory when a tile first meets
 *    a larger batch; after that, calls with the same or smaller shapes allocate nothing.
 */
#ifndef RPU_AMD_H
#define RPU_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RPU_AMD_ABI_VERSION 1

/* ---- enums: integer values equal the reference enum class order ------------ */

/* R/rpu_pulsed_meta_parameter.h:17-27 NoiseManagementType */
enum rpu_noise_management {
  RPU_NM_NONE = 0,
  RPU_NM_ABS_MAX = 1,
  RPU_NM_ABS_MAX_NP_SUM = 2,
  RPU_NM_MAX = 3,
  RPU_NM_CONSTANT = 4,
  RPU_NM_AVERAGE_ABS_MAX = 5,              /* running average over the samples seen so far (nm_decay) */
  RPU_NM_AVERAGE_ABS_MAX_SINGLE_VALUE = 6, /* the same on this path, as in the reference's CPU code */
  RPU_NM_ABS_MAX_SINGLE_VALUE = 7          /* not provided */
};

/* R/rpu_pulsed_meta_parameter.h:29 BoundManagementType */
enum rpu_bound_management {
  RPU_BM_NONE = 0,
  RPU_BM_ITERATIVE = 1,
  RPU_BM_ITERATIVE_WORST_CASE = 2
};

/* R/rpu_pulsed_meta_parameter.h:33-40 PulseType */
enum rpu_pulse_type {
  RPU_PULSE_NONE = 0,                  /* floating point rank-B update */
  RPU_PULSE_STOCHASTIC_COMPRESSED = 1,
  RPU_PULSE_STOCHASTIC = 2,            /* treated as STOCHASTIC_COMPRESSED: the same pulses per cross-point */
  RPU_PULSE_NONE_WITH_DEVICE = 3,      /* floating point update, device bounds after every sample */
  RPU_PULSE_MEAN_COUNT = 4,            /* deterministic counts round(BL p) per line (R/dense_bit_line_maker.cpp:140-208) */
  RPU_PULSE_DETERMINISTIC_IMPLICIT = 5
};

/* R/rpu_pulsed_meta_parameter.h:42-49 AnalogMVType */
enum rpu_mv_type {
  RPU_MV_IDEAL = 0,
  RPU_MV_ONE_PASS = 1,
  RPU_MV_POS_NEG_SEPARATE = 2, /* negative and positive inputs in two passes, summed before the ADC
                                  (R/rpu_forward_backward_pass.cpp:832-893) */
  RPU_MV_POS_NEG_SEPARATE_DIGITAL_SUM = 3 /* the two passes each through the ADC stage, the results added
                                             (R/rpu_forward_backward_pass.cpp:861-877) */
  /* SplitMode(4), BitWise(5): not provided */
};

/* device kinds; B/rpu_base_devices.cpp:545-656 */
enum rpu_device_kind {
  RPU_DEVICE_IDEAL = 0,         /* IdealResistiveDeviceParameter / FloatingPoint: no device physics */
  RPU_DEVICE_CONSTANT_STEP = 1, /* ConstantStepResistiveDeviceParameter */
  RPU_DEVICE_LINEAR_STEP = 2,   /* LinearStepResistiveDeviceParameter */
  RPU_DEVICE_SOFT_BOUNDS = 3,   /* SoftBoundsResistiveDeviceParameter (LinearStep with fixed ls_* values) */
  RPU_DEVICE_TRANSFER = 4       /* TransferResistiveDeviceParameter: a chain of the kinds above (rpu_transfer_params) */
};

/* ---- parameter structs ------------------------------------------------------ */

/* Replaces IOMetaParameter<float> (R/rpu_pulsed_meta_parameter.h:50-106) as bound by
 * AnalogTileInputOutputParameter (B/rpu_base_devices.cpp:485-519).  Field names and defaults are
 * the C++ ones; `inp_res` / `out_res` accept "1/steps" or "steps" and are converted to an absolute
 * step res * 2 * bound at creation (R/rpu_pulsed_meta_parameter.cpp:26-37,56-57).
 * A field marked "not provided" must be left at its inactive value or creation fails. */
typedef struct rpu_io_params {
  int32_t is_perfect;             /* 0 */
  int32_t mv_type;                /* RPU_MV_ONE_PASS */
  int32_t noise_management;       /* RPU_NM_ABS_MAX */
  int32_t bound_management;       /* RPU_BM_NONE (python default ITERATIVE) */
  int32_t bm_test_negative_bound; /* 1 */
  int32_t max_bm_factor;          /* 1000 */
  int32_t inp_sto_round;          /* 0 */
  int32_t out_sto_round;          /* 0 */
  float inp_bound;                /* 1 */
  float inp_res;                  /* 1/126 */
  float inp_noise;                /* 0 */
  float inp_asymmetry;            /* 0 */
  float out_bound;                /* 12 */
  float out_res;                  /* 1/510 */
  float out_noise;                /* 0.06 */
  float out_asymmetry;            /* 0 */
  float out_scale;                /* 1 */
  float nm_thres;                 /* 0 */
  float nm_assumed_wmax;          /* 0.6 */
  float max_bm_res;               /* 0.25 */
  /* output-referred weight noise (R/rpu_forward_backward_pass.cpp:325-385) and IR drop (:387-433) */
  int32_t w_noise_type;           /* 0 = None, 1 = AdditiveConstant, 2 = PCMRead */
  float w_noise;                  /* ignored while w_noise_type == 0 */
  float ir_drop;                  /* 0 */
  /* per-line variations of the periphery, sampled once per tile and direction (R/rpu_forward_backward_pass.cpp:244-318):
   * they are part of the extra state (rpu_tile_get_extra), "fwd.*" / "bwd.*" */
  float out_noise_std;            /* 0: relative spread of out_noise from output line to output line */
  float out_nonlinearity;         /* 0: y -> f y / (1 + nl_i |y|), nl_i = |out_nonlinearity / out_bound (1 + std xi)| */
  float out_nonlinearity_std;     /* 0 */
  float v_offset_std;             /* 0: voltage offset per output line, max(v_offset_std xi, 0) (:436-506) */
  float r_series;                 /* 0: series resistance, y -> y / (1 + min(r_series |y|, r_series_max_total)) */
  float w_read_asymmetry_dtod;    /* 0: the negative pass of PosNegSeparate reads w_ij (1 + dtod xi_ij) (:845-856) */
  float ir_drop_g_ratio;          /* 5.7143e5: wire conductance over g_max (ir_drop_Gw_div_gmax) */
  float nm_decay;                 /* 1e-3: weight of a new sample in the AverageAbsMax running average */
  float slope_calibration;        /* 0.5: y / out_bound at which the non-linearity has slope 1 on average (:283-295) */
  float v_offset_w_min;           /* 0: reference conductance of the offset, typically -1 */
  float r_series_max_total;       /* FLT_MAX */
} rpu_io_params;

/* Replaces PulsedUpdateMetaParameter<float> (R/rpu_pulsed_meta_parameter.h:248-323) as bound by
 * AnalogTileUpdateParameter (B/rpu_base_devices.cpp:469-483). */
typedef struct rpu_update_params {
  int32_t pulse_type;           /* RPU_PULSE_STOCHASTIC_COMPRESSED */
  int32_t desired_bl;           /* 31; up to RPU_MAX_BL (beyond 31 a sample takes several rows of pulse words) */
  int32_t fixed_bl;             /* 1 */
  int32_t update_management;    /* 1 */
  int32_t update_bl_management; /* 1 */
  int32_t sto_round;            /* 0 */
  float um_grad_scale;          /* 1 */
  float res;                    /* 0 : resolution of the pulse probability (0..1) */
  float x_res_implicit;         /* 0 */
  float d_res_implicit;         /* 0 */
} rpu_update_params;

/* Replaces PulsedRPUDeviceMetaParameter<float> (R/rpu_pulsed_device.h:52-114) plus the LinearStep
 * tail (R/rpu_linearstep_device.h:16-31) and the SimpleRPUDeviceMetaParameter fields that feed
 * device construction (R/rpu_simple_device.h:54,89).  For RPU_DEVICE_SOFT_BOUNDS the ls_* fields
 * are overwritten with the SoftBounds constants (R/rpu_linearstep_device.h:68-80). */
typedef struct rpu_device_params {
  int32_t kind;                    /* enum rpu_device_kind */
  uint32_t construction_seed;      /* 0 = time based (as the reference) */
  int32_t enforce_consistency;     /* 0 in C++, 1 in the python configs */
  int32_t perfect_bias;            /* 0 */
  int32_t dw_min_dtod_log_normal;  /* 0 */
  int32_t adjust_bounds_with_up_down; /* 0 */
  float dw_min;                    /* 0.001 */
  float dw_min_dtod;               /* 0.3 */
  float dw_min_std;                /* 0.3 (cycle-to-cycle) */
  float w_min;                     /* -0.6 */
  float w_min_dtod;                /* 0.3 */
  float w_max;                     /* 0.6 */
  float w_max_dtod;                /* 0.3 */
  float up_down;                   /* 0 */
  float up_down_dtod;              /* 0.01 */
  float adjust_bounds_with_up_down_dev; /* 0 */
  float corrupt_devices_prob;      /* 0 */
  float corrupt_devices_range;     /* FLT_MAX */
  float lifetime;                  /* 0 */
  float lifetime_dtod;             /* 0 */
  float diffusion;                 /* 0 */
  float diffusion_dtod;            /* 0 */
  float reset;                     /* 0 */
  float reset_dtod;                /* 0 */
  float reset_std;                 /* 0.01 */
  float write_noise_std;           /* 0 ; > 0 (LinearStep / SoftBounds): persistent weights, see apply_write_noise_on_set */
  /* LinearStep tail */
  int32_t ls_allow_increasing_slope; /* 0 */
  int32_t ls_mean_bound_reference;   /* 1 */
  int32_t ls_mult_noise;             /* 1 */
  int32_t ls_reverse_up;             /* 0 */
  int32_t ls_reverse_down;           /* 0 */
  float ls_decrease_up;              /* 0 */
  float ls_decrease_down;            /* 0 */
  float ls_decrease_up_dtod;         /* 0.05 */
  float ls_decrease_down_dtod;       /* 0.05 */
  float ls_reverse_offset;           /* 0.01 */
  /* Power-law drift of the device (DriftParameter, R/weight_drifter.h:14-60); active when drift_nu > 0. */
  float drift_nu;                    /* 0 */
  float drift_nu_dtod;               /* 0 */
  float drift_nu_std;                /* 0 (redrawn at every call) */
  float drift_wg_ratio;              /* 1 */
  float drift_g_offset;              /* 0 */
  float drift_w_offset;              /* 0 */
  float drift_nu_k;                  /* 0 */
  float drift_log_g0;                /* 0 */
  float drift_t0;                    /* 1 */
  float drift_reset_tol;             /* 1e-7 */
  float drift_w_read_std;            /* 0 */
  int32_t count_pulses;              /* 0 ; 1: every update also counts the pulses of each cross-point */
  /* Write noise (R/rpu_linearstep_device.cpp:112-164, R/rpu_pulsed_device.cpp:545-588): with write_noise_std > 0 the
   * pulses act on hidden persistent weights and the weights that forward / backward and get_weights see are those
   * plus write_noise_std * dw_min * N(0, 1), redrawn for a cross-point whenever it takes a pulse and for all after
   * weight maintenance; set_weights redraws it when this flag is set. */
  int32_t apply_write_noise_on_set;  /* 1 */
} rpu_device_params;

/* Replaces PulsedMetaParameter<float> (R/rpu_pulsed.h:127-151): forward IO, backward IO, update. */
typedef struct rpu_tile_config {
  rpu_io_params f_io;
  rpu_io_params b_io;
  rpu_update_params up;
  rpu_device_params device;
} rpu_tile_config;

/* Replaces TransferRPUDeviceMetaParameter<float> (R/rpu_transfer_device.h:52-127, with the gamma_vec of
 * VectorRPUDeviceMetaParameter, R/rpu_vector_device.h) as bound by TransferResistiveDeviceParameter
 * (B/rpu_base_devices.cpp:742-777; transfer_forward = transfer_io, transfer_update = transfer_up).  The
 * compound holds n_devices weight matrices: device 0 takes the gradient update, every transfer_every
 * updates n_reads_per_transfer columns (rows) of device j are read through transfer_io and written
 * onto device j + 1 with a pulsed update under transfer_up; the tile's weights are
 * sum_k gamma_vec[k] * w_k.  Device 0 is fast_device, all others rest_device (the reference allows only
 * the first to differ, R/rpu_transfer_device.cpp:136-144).  Empty vectors (n_* = 0) are filled as the
 * reference does (R/rpu_transfer_device.cpp:146-196). */
#define RPU_MAX_VECTOR_DEVICES 16
typedef struct rpu_transfer_params {
  int32_t n_devices;            /* 2 */
  uint32_t construction_seed;   /* 0 = time based; one stream samples all devices in order */
  int32_t units_in_mbatch;      /* 0 */
  int32_t n_reads_per_transfer; /* 1 */
  int32_t no_self_transfer;     /* 1 */
  int32_t random_selection;     /* 1: a transfer starts at column floor(u in_size), u uniform (R/rpu_transfer_device.cpp:486-488) */
  int32_t scale_transfer_lr;    /* 1 */
  int32_t scale_fast_lr;        /* 1 */
  int32_t transfer_columns;     /* 1 ; 0 = rows (read with the backward pass) */
  float gamma;                  /* 0 */
  float transfer_every;         /* 1 */
  float with_reset_prob;        /* probability per transfer that the columns just read are reset on the source device,
                                   after the write (C/rpucuda_transfer_device.cu:320-324); columns only */
  float fast_lr;                /* 0 */
  float transfer_lr;            /* 1 */
  int32_t n_gamma_vec;          /* 0 or n_devices */
  int32_t n_transfer_lr_vec;    /* 0 or n_devices */
  int32_t n_transfer_every_vec; /* 0 or n_devices */
  float gamma_vec[RPU_MAX_VECTOR_DEVICES];
  float transfer_lr_vec[RPU_MAX_VECTOR_DEVICES];
  float transfer_every_vec[RPU_MAX_VECTOR_DEVICES];
  rpu_io_params transfer_io;
  rpu_update_params transfer_up;
  rpu_device_params fast_device;
  rpu_device_params rest_device;
} rpu_transfer_params;

/* Replaces PCMLikeNoiseModel (src/aihwkit/inference/noise/pcm.py:27-158) over the
 * SinglePairConductanceConverter (src/aihwkit/inference/converter/conductance.py:24-82): statistical
 * programming noise, conductance drift and accumulated 1/f read noise of PCM devices, applied to the
 * weight matrix of an inference tile.  Defaults are the Python defaults. */
typedef struct rpu_pcm_noise_params {
  float g_max;                      /* 25 (uS) */
  float g_min;                      /* 0 */
  float t_read;                     /* 250e-9 (s) */
  float t_0;                        /* 20 (s) */
  float prog_noise_scale;           /* 1 */
  float read_noise_scale;           /* 1 */
  float drift_scale;                /* 1 */
  float prog_coeff[3];              /* 0.26348, 1.9650, -1.1731 */
  float prog_coeff_g_max_reference; /* 25 */
} rpu_pcm_noise_params;

typedef struct rpu_tile rpu_tile_t; /* opaque */

/* ---- defaults ---------------------------------------------------------------- */

/* Fill `cfg` with the C++ defaults of the reference structs cited above for the given device kind. */
int rpu_tile_config_default(rpu_tile_config *cfg, int device_kind);

/* ---- construction / residency --------------------------------------------------- */

/* Replaces PulsedMetaParameter::createRPUArray (R/rpu_pulsed.cpp:48-56) reached through
 * AnalogTileParameter.create_array (B/rpu_base_devices.cpp:453-467): builds the host-side tile,
 * samples the device-to-device parameters on the CPU with RealWorldRNG(construction_seed)
 * (R/rpu_pulsed.cpp:460-495, R/rpu_pulsed_device.cpp:593-733).  Touches no GPU. */
int rpu_tile_create(rpu_tile_t **out, int x_size, int d_size, const rpu_tile_config *cfg);

/* C++ defaults of TransferRPUDeviceMetaParameter with two devices of `device_kind`. */
int rpu_transfer_params_default(rpu_transfer_params *tp, int device_kind);

/* As rpu_tile_create with a transfer compound as the tile's device (cfg->device is ignored):
 * TransferRPUDeviceMetaParameter::createDevice -> TransferRPUDevice::populate
 * (R/rpu_transfer_device.cpp:333-358, R/rpu_vector_device.cpp:397-431).  Forward / backward act on the
 * reduced weights; rpu_tile_update follows TransferRPUDevice::doSparseUpdate / finishUpdateCycle
 * (R/rpu_transfer_device.cpp:520-557): the batch is cut where a transfer is due, as the reference's GPU
 * path does (C/rpucuda_transfer_device.cu:393-510).  Hidden parameters: per device k its arrays with
 * the suffix _k, then hidden_weights_k (R/rpu_vector_device.cpp:188-203). */
int rpu_tile_create_transfer(rpu_tile_t **out, int x_size, int d_size, const rpu_tile_config *cfg,
                             const rpu_transfer_params *tp);

/* Counters of a transfer tile: number of update vectors seen since the weights were set and the next
 * column (row) each device transfers (TransferRPUDevice::current_update_idx_, current_slice_indices_;
 * the reference exposes them through dumpExtra, R/rpu_transfer_device.cpp:672-688).
 * slice_indices_host is [n_devices]. */
int rpu_tile_get_transfer_state(rpu_tile_t *tile, uint64_t *update_idx, int32_t *slice_indices_host);

/* Deep copy (host state and, if resident, device state); B/rpu_base_tiles.cpp __copy__/__deepcopy__. */
int rpu_tile_clone(rpu_tile_t **out, const rpu_tile_t *src);

/* Replaces the CudaAnalogTile(cpu_tile) constructor (B/rpu_base_tiles_cuda.cpp:45-58,524-543;
 * C/rpucuda_pulsed.cu:69-88): allocates HBM on HIP device `device_id` (-1 = current) and uploads
 * weights and per-device parameters. */
int rpu_tile_to_device(rpu_tile_t *tile, int device_id);

int rpu_tile_destroy(rpu_tile_t *tile);

/* ---- hot path -------------------------------------------------------------------- */

/* Replaces RPUSimple::forward (R/rpu.cpp:508-533; GPU: C/rpucuda_pulsed.cu:646-659) as bound at
 * B/rpu_base_tiles_cuda.cpp:159-236.  x_dev is [m_batch][x_size - bias] (x_trans: [x_size - bias][m_batch]),
 * y_dev is [m_batch][d_size] (d_trans: [d_size][m_batch]).  Asynchronous on `stream`.  m_batch == 0 does nothing
 * and succeeds (here and in backward, update and the indexed and grouped calls); a negative value is an error. */
int rpu_tile_forward(rpu_tile_t *tile, const float *x_dev, float *y_dev, int m_batch, int bias,
                     int x_trans, int d_trans, int is_test, void *stream);

/* Replaces RPUSimple::backward (R/rpu.cpp:535-554) as bound at B/rpu_base_tiles.cpp:475-539. */
int rpu_tile_backward(rpu_tile_t *tile, const float *d_dev, float *x_dev, int m_batch, int bias,
                      int d_trans, int x_trans, void *stream);

/* Replaces RPUSimple::update -> RPUPulsed::updateMatrix (R/rpu.cpp:556-575, R/rpu_pulsed.cpp:558-585;
 * GPU: C/rpucuda_pulsed.cu:897-930, C/pulsed_weight_updater.cu:332-434) as bound at
 * B/rpu_base_tiles.cpp:541-620.  A zero learning rate makes this a no-op, as in the binding. */
int rpu_tile_update(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int m_batch, int bias,
                    int x_trans, int d_trans, void *stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory while they run -- code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc: the same update as rpu_tile_update for
 * RPU_PULSE_STOCHASTIC_COMPRESSED on a ConstantStep / LinearStep / SoftBounds tile (same kernels, same random
 * streams, bit-identical weights), but every buffer beyond the inputs and the tile's own matrices (per-sample BL and
 * probability scales, packed pulse words, bit planes, the rows with the bias column) lives in one static device
 * array of RPU_NOALLOC_MAX_SCRATCH_BYTES per GPU, which the library holds until the process ends.  The call makes
 * no hipMalloc / hipFree and records no events; a call whose scratch would not fit
 * (about 8 * m_batch * (x_size + d_size) bytes, + 4 * m_batch * x_size with bias) fails with a message that names both
 * sizes and changes nothing.  All tiles on a GPU share that GPU's array: calls that overlap in time on one GPU (other
 * streams, other threads) race, calls on one stream do not.  Not provided for transfer compounds, write noise, delta
 * weights, pulse counters and bit lines beyond 31 pulses (error).  rpu_tile_get_update_words / get_update_ab read this
 * call's words until the next no-allocation call on the same GPU overwrites them. */
#define RPU_NOALLOC_MAX_SCRATCH_BYTES (6u << 20)
int rpu_tile_update_noalloc(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int m_batch, int bias,
                            int x_trans, int d_trans, void *stream);

/* ---- state ------------------------------------------------------------------------ */

int rpu_tile_get_x_size(const rpu_tile_t *tile); /* R/rpu.h:76 getXSize */
int rpu_tile_get_d_size(const rpu_tile_t *tile); /* R/rpu.h:77 getDSize */
int rpu_tile_is_on_device(const rpu_tile_t *tile);

/* RPUAbstract::setLearningRate / getLearningRate (R/rpu.h:85-86, B/rpu_base_tiles.cpp get/set_learning_rate) */
int rpu_tile_set_learning_rate(rpu_tile_t *tile, float lr);
float rpu_tile_get_learning_rate(const rpu_tile_t *tile);

/* RPUPulsed::setWeights (clips into the per-device bounds, R/rpu_pulsed.cpp:288-292,
 * R/rpu_pulsed_device.cpp:545-571) and RPUSimple::getWeights; row-major [d_size][x_size] host buffers.
 * On a GPU tile these synchronise with the stream of the last compute call. */
int rpu_tile_set_weights(rpu_tile_t *tile, const float *w_host);
int rpu_tile_get_weights(rpu_tile_t *tile, float *w_host);

/* Device pointer of the weight matrix in HBM (NULL if not resident): row-major [d_size][x_size], or the bound
 * [x_size][d_size] tensor of a tile with the zero-copy binding of rpu_tile_set_shared_weights_xd. */
int rpu_tile_weights_device_ptr(rpu_tile_t *tile, float **w_dev);

/* Hidden per-device parameters: RPUPulsed::getDeviceParameterNames / getDeviceParameter /
 * setDeviceParameter (R/rpu_pulsed.cpp:392-410, R/rpu_pulsed_device.cpp:235-330) as bound at
 * B/rpu_base_tiles.cpp:763-825.  Names in order: max_bound, min_bound, dwmin_up, dwmin_down,
 * decay_scales, diffusion_rates, reset_bias, drift_nu [, slope_up, slope_down].
 * `data_host` is [n][d_size][x_size]. */
int rpu_tile_hidden_parameter_count(const rpu_tile_t *tile);
const char *rpu_tile_hidden_parameter_name(const rpu_tile_t *tile, int idx);
int rpu_tile_get_hidden_parameters(rpu_tile_t *tile, float *data_host);
int rpu_tile_set_hidden_parameters(rpu_tile_t *tile, const float *data_host);

/* Seed of the counter-based Philox4x32-10 generator that drives every random draw on the GPU
 * (output noise, stochastic rounding, pulse trains, cycle-to-cycle noise).  A draw is a pure
 * function of (seed, call index, purpose, element index); the call index restarts at 0 here.
 * Stands in for the per-context cuRAND state of the reference (C/cuda_util.cu:163-176,779-800). */
int rpu_tile_set_seed(rpu_tile_t *tile, uint64_t seed);

/* No counterpart in the reference.  Chooses how the stochastic pulsed update applies the coincidences of a batch:
 * RPU_UPDATE_VARIANT_EXACT (default): pulse by pulse in batch order with a normal draw per pulse, as
 * PulsedRPUWeightUpdater::updateVectorWithDevice (R/rpu_weight_updater.cpp:197-294) does.
 * RPU_UPDATE_VARIANT_AGGREGATED (opt-in; LinearStep / SoftBounds with multiplicative noise only): per group of
 * samples_per_step samples (a multiple of 32) a cross-point counts its coincidences by direction and takes them in
 * closed form (geometric approach to the soft bound) with one normal draw carrying the summed cycle-to-cycle
 * variance; same pulse trains, same counts, mean and variance of the weight change equal to first order in
 * n * slope.  A statistical equivalent, not the reference's arithmetic: labelled wherever it is measured. */
#define RPU_UPDATE_VARIANT_EXACT 0
#define RPU_UPDATE_VARIANT_AGGREGATED 1
int rpu_tile_set_update_variant(rpu_tile_t *tile, int variant, int samples_per_step);

/* ---- indexed (convolution) interface ----------------------------------------------------------- */

/* Replaces RPUSimple::setMatrixIndices (R/rpu.h:397-402) as bound at B/rpu_base_tiles.cpp:721-737: the index
 * matrix of an unfolded convolution, [x_size][patches] int32 on the host: 0 = zero padding, 1 = bias one,
 * j >= 2 = element j - 2 of one input image (src/aihwkit/nn/modules/conv.py:534-575). */
int rpu_tile_set_matrix_indices(rpu_tile_t *tile, const int32_t *indices_host, int x_size, int patches);
int rpu_tile_has_matrix_indices(const rpu_tile_t *tile); /* patches per image of the index matrix, 0 if none is set */

/* Replace RPUSimple::forwardIndexed / backwardIndexed / updateIndexed (R/rpu.cpp:1117-1239) as bound at
 * B/rpu_base_tiles.cpp:621-720 (always with trans = true, dim3 = images, m_batch = patches per image):
 * x_dev holds n_images input images of image_size floats (N, C, H, W), d_dev is [n_images][d_size][patches]
 * (N, C_out, H_out * W_out).  Forward gathers the patches through the index matrix and runs the tile's forward
 * pass over n_images * patches samples; backward runs the tile's backward pass and adds the patch gradients up
 * per image element (every element of x_dev is written, in a fixed order: nothing to zero, same bits on every
 * call); update runs the tile's update over the same samples: a pulsed update reads the patches through the index
 * matrix and the gradients from d_dev where they are (as the reference's iterators do, C/io_iterator.h:160-696; no
 * patch matrix is written, same weights as the update on the unfolded matrices bit for bit), the floating-point
 * update and a transfer compound unfold them first. */
int rpu_tile_forward_indexed(rpu_tile_t *tile, const float *x_dev, float *d_dev, int n_images, long image_size,
                             int is_test, void *stream);
int rpu_tile_backward_indexed(rpu_tile_t *tile, const float *d_dev, float *x_dev, int n_images, long image_size,
                              void *stream);
int rpu_tile_update_indexed(rpu_tile_t *tile, const float *x_dev, const float *d_dev, int n_images, long image_size,
                            void *stream);

/* ---- several tiles in one launch ------------------------------------------------------------ */

/* A layer larger than one tile is an array of tiles whose forward passes the reference runs one after the other
 * from Python (TileModuleArray.forward, src/aihwkit/simulator/tiles/array.py:155-182).  A group runs the forward
 * pass of all its tiles in a few launches (one per kernel variant and bound-management round) instead of
 * several per tile.  The tiles must be resident on the same GPU; each keeps its own state, seed and call
 * counter, and a grouped call gives every tile exactly what rpu_tile_forward with the same arguments would.
 * x_dev[i] is [m_batch][x_size_i], y_dev[i] is [m_batch][d_size_i] (no bias column, no transposed layouts).
 * A group that holds a tile whose pass has periphery terms before the ADC (output-referred weight noise, IR drop,
 * per-line offsets and non-linearities, separate passes per input sign) or running-average noise management runs
 * its tiles one after the other on the stream, each with the launches of rpu_tile_forward / rpu_tile_backward:
 * same results, no shared launches.  The tiles must outlive the group. */
typedef struct rpu_group rpu_group_t; /* opaque */
int rpu_group_create(rpu_group_t **out, rpu_tile_t *const *tiles, int n_tiles);
int rpu_group_forward(rpu_group_t *group, const float *const *x_dev, float *const *y_dev, int m_batch,
                      int is_test, void *stream);
/* The same with a row stride (in floats) per input and output, so that the tiles of a layer read column slices of
 * the layer's input [m_batch][in_total] and write column slices of one output [m_batch][out_total] in place
 * (what array.py:155-182 does with torch.split / torch.cat); null strides mean dense rows. */
int rpu_group_forward_strided(rpu_group_t *group, const float *const *x_dev, const long *x_ld, float *const *y_dev,
                              const long *y_ld, int m_batch, int is_test, void *stream);
/* Backward pass of all tiles of the group: d_dev[i] is [m_batch][d_size_i] with row stride d_ld[i], x_dev[i] receives
 * [m_batch][x_size_i] with row stride x_ld[i] (null strides: dense rows); every tile gets what rpu_tile_backward
 * gives it. */
int rpu_group_backward_strided(rpu_group_t *group, const float *const *d_dev, const long *d_ld, float *const *x_dev,
                               const long *x_ld, int m_batch, void *stream);
/* Stochastic pulsed update of all tiles of the group (the reference updates the tiles of an array one after the other
 * through autograd, tiles/array.py; three launches per tile): x_dev[i] is [m_batch][x_size_i] with row stride x_ld[i],
 * d_dev[i] is [m_batch][d_size_i] with row stride d_ld[i] (null strides: dense rows; no bias column, no transposed
 * layouts).  Every tile gets exactly what rpu_tile_update with the same arguments gives it (same seed and call
 * counter: same pulse trains, same weights).  Provided for the plain case -- stochastic compressed pulses on a pulsed
 * device, bit lines of at most 31 pulses, no transfer compound, write noise, delta weights, pulse counters or update
 * variant: any other tile in the group makes the call fail with a message that says so, before anything is launched. */
int rpu_group_update_strided(rpu_group_t *group, const float *const *x_dev, const long *x_ld, const float *const *d_dev,
                             const long *d_ld, int m_batch, void *stream);
/* Tiles of a group that are handed the same input (pointer, stride, length) and convert it with the same DAC, noise
 * and bound management and without random numbers (the column blocks of a split layer, array.py:155-182, which the
 * reference quantizes once per tile) share the quantized rows of rounds 0 and 1: one of them writes the rows, all read
 * them; results are unchanged.  This reports what the last call of the group did: the number of such sets of at
 * least two tiles, and the number of tiles in them. */
int rpu_group_get_shared_input_sets(rpu_group_t *group, int *n_sets, int *n_tiles);
int rpu_group_destroy(rpu_group_t *group);

/* ---- inference weight pipeline ------------------------------------------------------------- */

int rpu_pcm_noise_params_default(rpu_pcm_noise_params *p);

/* Replaces InferenceTileWithPeriphery.program_weights (src/aihwkit/simulator/tiles/inference.py:161-213) with
 * BaseNoiseModel.apply_programming_noise (src/aihwkit/inference/noise/base.py:82-103): the reference weights
 * (the current weights, taken anew unless from_reference != 0 and a reference exists) are mapped to a pair of
 * conductances per cross-point, programming noise is added and the drift coefficients of both conductances
 * are drawn (pcm.py:100-131); the tile's weights become the programmed weights.  All on the GPU: the
 * reference moves the matrix to the host and back.  GPU tiles with an ideal device only. */
int rpu_tile_program_weights(rpu_tile_t *tile, const rpu_pcm_noise_params *p, int from_reference, void *stream);

/* Replaces InferenceTileWithPeriphery.drift_weights (inference.py:215-262) with BaseNoiseModel.apply_drift_noise
 * (base.py:105-131, pcm.py:133-158): the tile's weights become the programmed weights drifted to t_inference
 * seconds after programming with accumulated read noise.  Programs first if that has not happened. */
int rpu_tile_drift_weights(rpu_tile_t *tile, const rpu_pcm_noise_params *p, float t_inference, void *stream);

/* Host copies [d_size][x_size] of the programmed weights and of the drift coefficients of the positive and
 * the negative conductance (InferenceTile.programmed_weights, drift_noise_parameters); NULL pointers are skipped. */
int rpu_tile_get_drift_state(rpu_tile_t *tile, float *programmed_host, float *nu_plus_host, float *nu_minus_host);

/* Read-out of GlobalDriftCompensation (src/aihwkit/inference/compensation/drift.py:21-41, base.py:25-62):
 * the unit vectors are forwarded through the tile and max(mean |output|, 1e-4) is returned; the ratio of the
 * value after programming to the value after drift is the output scale alpha. */
int rpu_tile_drift_readout(rpu_tile_t *tile, float *mean_abs_host, void *stream);

/* ---- weight maintenance between training steps ------------------------------------------- */
/* All of these work on the matrix in HBM of a resident tile, on `stream`; a transfer compound refuses them. */

/* decay_weights (src/aihwkit/simulator/rpu_base_src/rpu_base_tiles.cpp:276-291): a pulsed device decays each
 * weight towards its reset bias with its own decay scale and clips to its bounds,
 * w = (w - b) * (1 + alpha * (scale - 1)) + b   (src/rpucuda/rpu_pulsed_device.cpp:392-420);
 * other tiles scale by 1 - alpha / lifetime (src/rpucuda/rpu_simple_device.cpp:96-115).  bias_no_decay
 * leaves the last column alone. */
int rpu_tile_decay_weights(rpu_tile_t *tile, float alpha, int bias_no_decay, void *stream);

/* diffuse_weights (rpu_base_tiles.cpp:372-386): w += diffusion_rate * N(0, 1), then the bounds
 * (rpu_pulsed_device.cpp:432-446, rpu_simple_device.cpp:124-134). */
int rpu_tile_diffuse_weights(rpu_tile_t *tile, void *stream);

/* clip_weights (rpu_base_tiles.cpp:315-329) with the fields of WeightClipParameter
 * (src/rpucuda/weight_clipper.h:14-27).  Fixed value: +- fixed_value and, on a pulsed device, its bounds
 * (rpu_pulsed_device.cpp:448-467).  Layer Gaussian and average channel max (weight_clipper.cpp:38-93) are for
 * floating-point / ideal devices only, as in the reference (src/rpucuda/rpu_pulsed.cpp:269-278). */
enum rpu_clip_type {
  RPU_CLIP_NONE = 0,
  RPU_CLIP_FIXED_VALUE = 1,
  RPU_CLIP_LAYER_GAUSSIAN = 2,
  RPU_CLIP_AVERAGE_CHANNEL_MAX = 3
};
int rpu_tile_clip_weights(rpu_tile_t *tile, int clip_type, float fixed_value, float sigma, void *stream);

/* reset_columns (rpu_base_tiles.cpp:387-404): columns start .. start + num - 1 (wrapping; num < 0: all) are set
 * to reset_bias + reset_std * N(0, 1) and clipped, each element with probability reset_prob
 * (rpu_pulsed_device.cpp:469-494; without bias and bounds on other tiles, rpu_simple_device.cpp:148-168). */
int rpu_tile_reset_columns(rpu_tile_t *tile, int start_column_idx, int num_columns, float reset_prob, void *stream);

/* drift_weights of a training tile (rpu_base_tiles.cpp:293-313): power-law conductance drift
 * w = w0 * (delta_t / t0)^(-nu) of every weight that has not changed by more than reset_tol since the last call;
 * a changed weight restarts its drift clock (src/rpucuda/weight_drifter.cpp:108-150).  A pulsed device has its own
 * nu per cross-point (hidden parameter drift_nu) and saturates at its bounds (rpu_pulsed_device.cpp:422-430); other
 * tiles drift with the one nu of their parameters (src/rpucuda/rpu.cpp:1581-1587).  The drift fields of
 * rpu_device_params configure it; with drift_nu <= 0 on a pulsed device the call does nothing, as in the reference.
 * Not to be confused with rpu_tile_drift_weights, the PCM inference drift above. */
int rpu_tile_drift_device_weights(rpu_tile_t *tile, float time_since_last_call, void *stream);

/* remap_weights (rpu_base_tiles.cpp:330-356) with the fields of WeightRemapParameter
 * (src/rpucuda/weight_remapper.h:25-38): the rows of the weight matrix are divided by a factor that the per-row
 * output scales scales_dev[d_size] (device memory, updated in place) take up, so that scales[i] * W[i][:] stays
 * what it was (src/rpucuda/weight_remapper.cpp:19-190).  Layerwise symmetric: the largest absolute weight maps to
 * remapped_wmax; channelwise symmetric: that of each row does, optionally with the spread of the scales bounded
 * by max_scale_range; channelwise norm: rows whose norm exceeds row_norm are scaled down to it (the scales take the
 * factor unless clip_if).  The asymmetric types need biases, which the reference's binding does not pass, and
 * ChannelwiseExceeded needs the signal-channel bound management: both are refused. */
enum rpu_remap_type {
  RPU_REMAP_NONE = 0,
  RPU_REMAP_LAYERWISE_SYMMETRIC = 1,
  RPU_REMAP_CHANNELWISE_SYMMETRIC = 2,
  RPU_REMAP_CHANNELWISE_NORM = 3,
  RPU_REMAP_CHANNELWISE_EXCEEDED = 4,
  RPU_REMAP_LAYERWISE_ASYMMETRIC = 5,
  RPU_REMAP_CHANNELWISE_ASYMMETRIC = 6
};
typedef struct rpu_remap_params {
  int32_t type;          /* enum rpu_remap_type, NONE */
  int32_t clip_if;       /* 1 */
  float max_scale_range; /* 0 */
  float max_scale_ref;   /* 0 */
  float row_norm;        /* 1 */
  float remapped_wmax;   /* 1 */
} rpu_remap_params;
int rpu_tile_remap_weights(rpu_tile_t *tile, const rpu_remap_params *p, float *scales_dev, void *stream);

/* modify_weights (rpu_base_tiles.cpp:357-371) with the fields of WeightModifierParameter
 * (src/rpucuda/weight_modifier.h:27-50): makes a modified copy of the weights that forward and backward (not the
 * update) contract with from then on; during evaluation (is_test) only if enable_during_test
 * (src/rpucuda/rpu.cpp:1483-1487, 1749-1758; src/rpucuda/weight_modifier.cpp:28-224).  The reference value amax is
 * the largest absolute weight (rel_to_actual_wmax; without the last column under copy_last_column) or
 * assumed_wmax.  PCMNoise exists only in the reference's CUDA code and is refused; per_batch_sample is refused as
 * in the reference. */
enum rpu_modifier_type {
  RPU_MODIFIER_COPY = 0,
  RPU_MODIFIER_DISCRETIZE = 1,
  RPU_MODIFIER_MULT_NORMAL = 2,
  RPU_MODIFIER_ADD_NORMAL = 3,
  RPU_MODIFIER_DISCRETIZE_ADD_NORMAL = 4,
  RPU_MODIFIER_DOREFA = 5,
  RPU_MODIFIER_POLY = 6,
  RPU_MODIFIER_PCM_NOISE = 7,
  RPU_MODIFIER_DROP_CONNECT = 8,
  RPU_MODIFIER_PROG_NOISE = 9
};
#define RPU_MAX_MODIFIER_COEFFS 8
typedef struct rpu_modifier_params {
  int32_t type;               /* enum rpu_modifier_type, COPY */
  int32_t per_batch_sample;   /* 0 */
  int32_t sto_round;          /* 0 */
  int32_t enable_during_test; /* 0 */
  int32_t copy_last_column;   /* 0 */
  int32_t rel_to_actual_wmax; /* 1 */
  int32_t n_coeffs;           /* 3 */
  float std_dev;              /* 0 */
  float res;                  /* 0.1 */
  float dorefa_clip;          /* 0.6 */
  float pdrop;                /* 0 */
  float assumed_wmax;         /* 1 */
  float g_max;                /* 25 */
  float coeffs[RPU_MAX_MODIFIER_COEFFS]; /* 0.26348 / 25, 0.0768, -0.001877 * 25 */
} rpu_modifier_params;
int rpu_tile_modify_weights(rpu_tile_t *tile, const rpu_modifier_params *p, void *stream);
/* Host copy [d_size][x_size] of the modified weights; returns an error if none have been made. */
int rpu_tile_get_modified_weights(rpu_tile_t *tile, float *w_host);

/* The per-cross-point factors (1 + w_read_asymmetry_dtod xi) of the negative pass of PosNegSeparate, drawn at creation:
 * the "fwd.w_asymmetry" / "bwd.w_asymmetry" entries of the reference's state (R/rpu_forward_backward_pass.cpp:62-100,
 * :297-304).  backward = 0 / 1 selects the direction; [d_size][x_size] host floats, the layout of the weights.
 * Fails when w_read_asymmetry_dtod of that direction is 0 (there are no factors). */
int rpu_tile_get_read_asymmetry(rpu_tile_t *tile, int backward, float *factors_host);
int rpu_tile_set_read_asymmetry(rpu_tile_t *tile, int backward, const float *factors_host);

/* get_pulse_counters (rpu_base_tiles.cpp:845-868, src/rpucuda/cuda/rpucuda_pulsed_device.cu:316-343): with
 * count_pulses set in the device parameters every pulsed update adds, per cross-point, the number of up and of
 * down pulses it applies to two 64-bit counters.  counters_host is [2][d_size][x_size], positive first; the
 * return value of rpu_tile_pulse_counter_count is 2 when the tile counts and 0 otherwise. */
int rpu_tile_pulse_counter_count(const rpu_tile_t *tile);
int rpu_tile_get_pulse_counters(rpu_tile_t *tile, uint64_t *counters_host);

/* Replaces the out_scale of the forward IO parameters (rpu_io_params.out_scale) from now on.  No counterpart in the
 * reference, which applies run-time output factors such as the drift-compensation alpha to the output tensor in
 * Python (src/aihwkit/simulator/tiles/inference.py:264-282); here the factor rides on the ADC stage. */
int rpu_tile_set_forward_out_scale(rpu_tile_t *tile, float out_scale);

/* set_shared_weights (rpu_base_tiles.cpp:215-229, src/rpucuda/rpu.cpp:1384-1398): the tile's weights are copied
 * into the caller's device buffer [d_size][x_size], which is the weight matrix from then on (never freed by
 * the library; it must outlive the tile or its move off the GPU). */
int rpu_tile_set_shared_weights(rpu_tile_t *tile, float *weights_dev);
int rpu_tile_get_shared_weights_if(const rpu_tile_t *tile);

/* set_shared_weights / set_delta_weights as the reference's CUDA tiles bind them (rpu_base_tiles_cuda.cpp:88-130,
 * RPUCudaSimple::setSharedWeights, cuda/rpucuda.cu:322-334): a device tensor [x_size][d_size].  That is what the
 * reference's Python allocates for every tile whose class name contains "Cuda" and reads back through .t()
 * (src/aihwkit/simulator/tiles/base.py:392-446, tiles/rpucuda.py:166-183).
 * A plain tile (no transfer compound, no write noise, no pulse counters, no analog terms before the ADC beyond output
 * noise) takes the tensor as its weight matrix itself, zero copy: its weights are transposed into the tensor once,
 * every per-cross-point array of the tile (device parameters, drift clocks, modified weights, inference arrays) is
 * transposed once as well, and from then on the kernels address that layout in place: forward reads the weights
 * the way backward does on a row-major tile and the other way round, maintenance kernels know both layouts, the
 * deterministic and floating-point updates walk the cross-points with x and d exchanged.  The stochastic pulse loop
 * alone keeps its row-major form (lanes along x, walking the d pulses of a row: half the passes of the walk the other
 * way round where inputs are denser than errors): the tile keeps row-major copies of the device parameters for it, the
 * launch that makes the pulse trains also makes a row-major scratch copy of the weights, and the loop stores its
 * results straight into the tensor.  Results are bit for bit those of the row-major tile (same pulse trains, same noise
 * draws per cross-point, same ADC draws) for forward, backward, the stochastic pulse loop and the deterministic-implicit
 * update; the opt-in aggregated update deals its noise streams to lanes, which hold other cross-points in the other
 * layout, so its weights agree statistically.  Host-side interfaces (get / set weights, hidden parameters, ...) stay
 * [d_size][x_size]; rpu_tile_weights_device_ptr returns the tensor.  Such tiles can be members of a group when all
 * members are bound that way.
 * The other kinds of tile keep their row-major matrix and mirror it: the tensor takes the tile's weights when it is
 * set, is read into the tile before every call that uses the weights and written back after every call that may
 * change them (one or two transposition passes per call); they cannot be members of a group.
 * Delta weights: with the zero-copy binding the caller's [x_size][d_size] tensor is written in place, otherwise the
 * update lands in a buffer of the tile and is transposed into the tensor after the call; null ends the mode.  Not
 * provided for transfer compounds. */
int rpu_tile_set_shared_weights_xd(rpu_tile_t *tile, float *weights_xd_dev);
int rpu_tile_set_delta_weights_xd(rpu_tile_t *tile, float *delta_weights_xd_dev);

/* set_delta_weights / reset_delta_weights (rpu_base_tiles.cpp:230-251): while a device buffer [d_size][x_size]
 * is set, an update leaves the weights as they are and writes dW with W_new = W - lr * dW into the buffer
 * (rpu.cpp:1459-1510, rpu_pulsed.cpp:560-585); null ends the mode. */
int rpu_tile_set_delta_weights(rpu_tile_t *tile, float *delta_weights_dev);

/* dump_extra / load_extra (rpu_base_tiles.cpp:89-113): the state beyond weights and hidden parameters that
 * decides what the next calls compute, as named 64-bit integers: seed and call counter of the random streams,
 * update counter, transfer counters of a compound. */
int rpu_tile_extra_count(const rpu_tile_t *tile);
const char *rpu_tile_extra_name(const rpu_tile_t *tile, int idx);
int rpu_tile_get_extra(rpu_tile_t *tile, int64_t *values_host);
int rpu_tile_set_extra(rpu_tile_t *tile, const int64_t *values_host, int count);

/* No counterpart in the reference.  With iterative bound management the forward pass of a batch runs round after
 * round, one launch each, and a launch costs a few microseconds even when its round lists no sample.  Two shortcuts,
 * both with the same outputs, bit for bit, and the same round counts as the separate launches:
 *   1  rounds 0 and 1 as ONE launch that computes both from the same weights and keeps, per sample, the one the
 *      reference's loop would have ended with (pays where most samples need a second round: the outputs of the tile are
 *      large against out_bound);
 *   2  every round after round 0 as ONE launch: after a round its workgroups wait for each other's arrival (a few
 *      microseconds) and leave when the next round lists no sample; a round that does follow inside that launch waits for
 *      all workgroups once more, with the rows and lists of the round before made visible device-wide, which costs more
 *      than a launch;
 *   3  both: rounds 0 and 1 as one launch, the rounds after them as another;
 *   5, 7  as 1 and 3 with round 2 in the first launch as well (a third result from the same weights; needs at least
 *      four rounds to be possible): pays as soon as a call lists any sample for round 2, whose own launch costs more
 *      than the extra matrix work.
 * Mode -1 (default): the tile chooses by what its recent forward calls needed -- more than half of the samples in a
 * second round: rounds 0 and 1 in one launch, and round 2 with them when those calls listed samples for it; and the
 * rounds after the last one that listed any sample in those calls
 * (the estimate rises at once and falls after eight calls below it), which are expected to be empty, share one
 * launch.  0: always the separate launches.  1 / 2 / 3 / 5 / 7: that shortcut whenever the shape allows it
 * (single tile, rounds on the 32 x 32 kernel, for 2 and 3 no more workgroups than the GPU holds of that kernel at once
 * -- what the occupancy query reports per CU times the CUs --, no per-line periphery terms).
 * The waits of shortcut 2 are bounded (some tens of milliseconds).  They assume that the launch has the GPU's CUs to
 * itself; work on another stream that holds CUs at that moment can make a wait run out.  That is never passed over: the
 * launch stops, and the next forward / backward / update call on the tile fails with "forward round barrier timed out
 * ...; results of call N are invalid", after which the tile runs one launch per round (setting a mode again re-arms
 * the shortcut).  Tile groups report the same way at their next call. */
int rpu_tile_set_fused_rounds(rpu_tile_t *tile, int mode);

/* No counterpart in the reference; for the test of the time-out path above only.  spin_limit > 0 shortens the bounded
 * waits of the tile's (or group's) merged-round launches to that many polls, extra_arrivals = 1 makes every wait expect
 * one workgroup more than the launch has, so that it runs out while every workgroup still leaves its kernel normally.
 * 0, 0 restores the defaults. */
int rpu_tile_set_round_wait_test_hook(rpu_tile_t *tile, int spin_limit, int extra_arrivals);
int rpu_group_set_round_wait_test_hook(rpu_group_t *group, int spin_limit, int extra_arrivals);

/* ---- inspection hooks (mirror the reference's debug hooks) ------------------------------ */

/* After rpu_tile_update with a stochastic pulse type: copies the packed pulse words of that call
 * to the host.  Word format (R/rpu_weight_updater.cpp:297-324, C/bit_line_maker.cu:886-927):
 * bit 0 = sign (1 = negative input), bits 1..BL = pulses.  x_words_host is [m_batch][x_size],
 * d_words_host is [m_batch][d_size], bl_host is [m_batch] (the per-sample BL chosen by update
 * management).  Mirrors BitLineMaker::getCountsDebug (C/bit_line_maker.cu:1884). */
int rpu_tile_get_update_words(rpu_tile_t *tile, uint32_t *x_words_host, uint32_t *d_words_host,
                              int32_t *bl_host, int m_batch);

/* Bit lines longer than 31 pulses (the reference packs them into nK32 = BL / 32 + 1 words per line element,
 * R/rpu_pulsed_meta_parameter.h:278, word layout R/rpu_weight_updater.cpp:297-324): a sample whose call can need
 * up to BL_max pulses takes n = ceil(BL_max / 31) consecutive rows of words, each in the one-word format above (its own
 * copy of the sign bit, 31 pulse slots); row r of sample b holds slots 31 r + 1 .. min(BL_b, 31 r + 31) and is zero
 * beyond BL_b.  The device loop walks them as n samples in a row, which is the reference's slot order.
 * rpu_tile_get_update_words then returns [m_batch * n][x_size] and [m_batch * n][d_size] (bl_host stays [m_batch]);
 * *words_per_sample receives n of the last stochastic update (1 unless BL_max > 31). */
#define RPU_MAX_BL 992 /* 32 rows of 31 pulses */
int rpu_tile_get_update_words_per_sample(rpu_tile_t *tile, int32_t *words_per_sample);

/* After a pulsed rpu_tile_update: the per-sample probability scales of that call, A for the d line and B for the x
 * line (PulsedUpdateMetaParameter::calculateBlAB / performUpdateManagement, R/rpu_pulsed_meta_parameter.cpp:152-236),
 * each [m_batch]. */
int rpu_tile_get_update_ab(rpu_tile_t *tile, float *a_host, float *b_host, int m_batch);

/* After rpu_tile_update with RPU_PULSE_DETERMINISTIC_IMPLICIT: signed coincidence counts
 * n[b][i][j] = (int) rintf((dv_i * BL) * xv_j) (R/dense_bit_line_maker.cpp:237-264) recomputed on the
 * GPU from the stored line values of that call; counts_host is [m_batch][d_size][x_size]. */
int rpu_tile_get_implicit_counts(rpu_tile_t *tile, int32_t *counts_host, int m_batch);

/* Applies the device steps for packed pulse words made elsewhere (same word format, device pointers
 * x_words_dev [m_batch][x_size], d_words_dev [m_batch][d_size]); the words are taken as they are, bits
 * beyond a sample's BL must be clear.  Mirrors the reference's debug protocol
 * RPUPulsed::updateVectorWithCounts (R/rpu_pulsed.cpp:528-552, R/rpu_weight_updater.cpp:327-393). */
int rpu_tile_update_with_words(rpu_tile_t *tile, const uint32_t *x_words_dev, const uint32_t *d_words_dev,
                               int m_batch, void *stream);

/* After rpu_tile_forward with bound management: the number of rounds each sample took;
 * rounds_host is [m_batch]. */
int rpu_tile_get_bm_rounds(rpu_tile_t *tile, int32_t *rounds_host, int m_batch);

/* Per-kernel timing: while enabled, every compute call records HIP events on its launch stream
 * around each kernel; rpu_tile_get_profile waits for the last call and returns the kernel durations
 * in milliseconds in launch order (names through rpu_tile_profile_name).  Takes the place of the
 * reference's CUDA_TIMING_* event macros (C/cuda_util.h:144-163). */
int rpu_tile_set_profiling(rpu_tile_t *tile, int enable);
int rpu_tile_get_profile(rpu_tile_t *tile, float *ms_host, int capacity, int *count);
const char *rpu_tile_profile_name(const rpu_tile_t *tile, int idx);

/* Philox4x32-10 block function (Salmon, Moraes, Dror, Shaw, SC'11) as the kernels evaluate it, on the
 * host and, through a one-thread kernel, on GPU `device_id` (-1 = current).  For known-answer tests of
 * the generator; no counterpart in the reference, which uses cuRAND XORWOW (C/cuda_util.cu:163-176). */
int rpu_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
int rpu_philox4x32_10_device(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4],
                             int device_id);

/* ---- errors / info ------------------------------------------------------------------------ */

/* No counterpart in the reference.  Number of device allocations (hipMalloc) that the buffers of this library's tiles
 * and groups have made in this process so far; a caller, or a test, can hold it against the claim that a call allocates
 * nothing. */
long rpu_device_allocation_count(void);

const char *rpu_last_error(void);
int rpu_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* RPU_AMD_H */
