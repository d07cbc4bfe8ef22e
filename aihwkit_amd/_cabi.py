"""ctypes view of the C ABI declared in ``include/rpu_amd.h``.

The shared library is built in-tree (``aihwkit_amd/lib/librpu_amd.so``) by
``aihwkit_amd/csrc/Makefile``; it is loaded lazily and loading fails loudly when it is missing --
there is no Python or CPU fallback for the tile computations.
"""
import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librpu_amd.so")

i32, u32, f32 = C.c_int32, C.c_uint32, C.c_float


class IOParams(C.Structure):
    """``rpu_io_params``."""

    _fields_ = [
        ("is_perfect", i32), ("mv_type", i32), ("noise_management", i32), ("bound_management", i32),
        ("bm_test_negative_bound", i32), ("max_bm_factor", i32), ("inp_sto_round", i32),
        ("out_sto_round", i32),
        ("inp_bound", f32), ("inp_res", f32), ("inp_noise", f32), ("inp_asymmetry", f32),
        ("out_bound", f32), ("out_res", f32), ("out_noise", f32), ("out_asymmetry", f32),
        ("out_scale", f32), ("nm_thres", f32), ("nm_assumed_wmax", f32), ("max_bm_res", f32),
        ("w_noise_type", i32), ("w_noise", f32), ("ir_drop", f32), ("out_noise_std", f32),
        ("out_nonlinearity", f32), ("out_nonlinearity_std", f32), ("v_offset_std", f32),
        ("r_series", f32), ("w_read_asymmetry_dtod", f32), ("ir_drop_g_ratio", f32),
        ("nm_decay", f32), ("slope_calibration", f32), ("v_offset_w_min", f32), ("r_series_max_total", f32),
    ]


class UpdateParams(C.Structure):
    """``rpu_update_params``."""

    _fields_ = [
        ("pulse_type", i32), ("desired_bl", i32), ("fixed_bl", i32), ("update_management", i32),
        ("update_bl_management", i32), ("sto_round", i32),
        ("um_grad_scale", f32), ("res", f32), ("x_res_implicit", f32), ("d_res_implicit", f32),
    ]


class DeviceParams(C.Structure):
    """``rpu_device_params``."""

    _fields_ = [
        ("kind", i32), ("construction_seed", u32), ("enforce_consistency", i32),
        ("perfect_bias", i32), ("dw_min_dtod_log_normal", i32), ("adjust_bounds_with_up_down", i32),
        ("dw_min", f32), ("dw_min_dtod", f32), ("dw_min_std", f32),
        ("w_min", f32), ("w_min_dtod", f32), ("w_max", f32), ("w_max_dtod", f32),
        ("up_down", f32), ("up_down_dtod", f32), ("adjust_bounds_with_up_down_dev", f32),
        ("corrupt_devices_prob", f32), ("corrupt_devices_range", f32),
        ("lifetime", f32), ("lifetime_dtod", f32), ("diffusion", f32), ("diffusion_dtod", f32),
        ("reset", f32), ("reset_dtod", f32), ("reset_std", f32), ("write_noise_std", f32),
        ("ls_allow_increasing_slope", i32), ("ls_mean_bound_reference", i32), ("ls_mult_noise", i32),
        ("ls_reverse_up", i32), ("ls_reverse_down", i32),
        ("ls_decrease_up", f32), ("ls_decrease_down", f32), ("ls_decrease_up_dtod", f32),
        ("ls_decrease_down_dtod", f32), ("ls_reverse_offset", f32),
        ("drift_nu", f32), ("drift_nu_dtod", f32), ("drift_nu_std", f32), ("drift_wg_ratio", f32),
        ("drift_g_offset", f32), ("drift_w_offset", f32), ("drift_nu_k", f32), ("drift_log_g0", f32),
        ("drift_t0", f32), ("drift_reset_tol", f32), ("drift_w_read_std", f32), ("count_pulses", i32),
        ("apply_write_noise_on_set", i32),
    ]


class RemapParams(C.Structure):
    """``rpu_remap_params``."""

    _fields_ = [
        ("type", i32), ("clip_if", i32), ("max_scale_range", f32), ("max_scale_ref", f32),
        ("row_norm", f32), ("remapped_wmax", f32),
    ]


MAX_MODIFIER_COEFFS = 8


class ModifierParams(C.Structure):
    """``rpu_modifier_params``."""

    _fields_ = [
        ("type", i32), ("per_batch_sample", i32), ("sto_round", i32), ("enable_during_test", i32),
        ("copy_last_column", i32), ("rel_to_actual_wmax", i32), ("n_coeffs", i32),
        ("std_dev", f32), ("res", f32), ("dorefa_clip", f32), ("pdrop", f32), ("assumed_wmax", f32),
        ("g_max", f32), ("coeffs", f32 * MAX_MODIFIER_COEFFS),
    ]


class TileConfig(C.Structure):
    """``rpu_tile_config``."""

    _fields_ = [("f_io", IOParams), ("b_io", IOParams), ("up", UpdateParams), ("device", DeviceParams)]


MAX_VECTOR_DEVICES = 16


class TransferParams(C.Structure):
    """``rpu_transfer_params``."""

    _fields_ = [
        ("n_devices", i32), ("construction_seed", u32), ("units_in_mbatch", i32), ("n_reads_per_transfer", i32),
        ("no_self_transfer", i32), ("random_selection", i32), ("scale_transfer_lr", i32), ("scale_fast_lr", i32),
        ("transfer_columns", i32),
        ("gamma", f32), ("transfer_every", f32), ("with_reset_prob", f32), ("fast_lr", f32), ("transfer_lr", f32),
        ("n_gamma_vec", i32), ("n_transfer_lr_vec", i32), ("n_transfer_every_vec", i32),
        ("gamma_vec", f32 * MAX_VECTOR_DEVICES), ("transfer_lr_vec", f32 * MAX_VECTOR_DEVICES),
        ("transfer_every_vec", f32 * MAX_VECTOR_DEVICES),
        ("transfer_io", IOParams), ("transfer_up", UpdateParams),
        ("fast_device", DeviceParams), ("rest_device", DeviceParams),
    ]


class PcmNoiseParams(C.Structure):
    """``rpu_pcm_noise_params``."""

    _fields_ = [
        ("g_max", f32), ("g_min", f32), ("t_read", f32), ("t_0", f32), ("prog_noise_scale", f32),
        ("read_noise_scale", f32), ("drift_scale", f32), ("prog_coeff", f32 * 3),
        ("prog_coeff_g_max_reference", f32),
    ]


# every symbol include/rpu_amd.h declares: name -> (restype, argtypes)
_P = C.c_void_p
_FP = C.POINTER(C.c_float)
SYMBOLS = {
    "rpu_tile_config_default": (C.c_int, [C.POINTER(TileConfig), C.c_int]),
    "rpu_tile_create": (C.c_int, [C.POINTER(_P), C.c_int, C.c_int, C.POINTER(TileConfig)]),
    "rpu_transfer_params_default": (C.c_int, [C.POINTER(TransferParams), C.c_int]),
    "rpu_tile_create_transfer": (C.c_int, [C.POINTER(_P), C.c_int, C.c_int, C.POINTER(TileConfig),
                                           C.POINTER(TransferParams)]),
    "rpu_tile_get_transfer_state": (C.c_int, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_int32)]),
    "rpu_tile_set_matrix_indices": (C.c_int, [_P, _P, C.c_int, C.c_int]),
    "rpu_tile_has_matrix_indices": (C.c_int, [_P]),
    "rpu_tile_forward_indexed": (C.c_int, [_P, _P, _P, C.c_int, C.c_long, C.c_int, _P]),
    "rpu_tile_backward_indexed": (C.c_int, [_P, _P, _P, C.c_int, C.c_long, _P]),
    "rpu_tile_update_indexed": (C.c_int, [_P, _P, _P, C.c_int, C.c_long, _P]),
    "rpu_tile_decay_weights": (C.c_int, [_P, C.c_float, C.c_int, _P]),
    "rpu_tile_diffuse_weights": (C.c_int, [_P, _P]),
    "rpu_tile_clip_weights": (C.c_int, [_P, C.c_int, C.c_float, C.c_float, _P]),
    "rpu_tile_reset_columns": (C.c_int, [_P, C.c_int, C.c_int, C.c_float, _P]),
    "rpu_tile_drift_device_weights": (C.c_int, [_P, C.c_float, _P]),
    "rpu_tile_remap_weights": (C.c_int, [_P, C.POINTER(RemapParams), _P, _P]),
    "rpu_tile_modify_weights": (C.c_int, [_P, C.POINTER(ModifierParams), _P]),
    "rpu_tile_get_modified_weights": (C.c_int, [_P, _P]),
    "rpu_tile_get_read_asymmetry": (C.c_int, [_P, C.c_int, _P]),
    "rpu_tile_set_read_asymmetry": (C.c_int, [_P, C.c_int, _P]),
    "rpu_tile_pulse_counter_count": (C.c_int, [_P]),
    "rpu_tile_get_pulse_counters": (C.c_int, [_P, _P]),
    "rpu_tile_set_shared_weights": (C.c_int, [_P, _P]),
    "rpu_tile_set_shared_weights_xd": (C.c_int, [_P, _P]),
    "rpu_tile_set_delta_weights_xd": (C.c_int, [_P, _P]),
    "rpu_tile_get_shared_weights_if": (C.c_int, [_P]),
    "rpu_tile_set_delta_weights": (C.c_int, [_P, _P]),
    "rpu_tile_extra_count": (C.c_int, [_P]),
    "rpu_tile_extra_name": (C.c_char_p, [_P, C.c_int]),
    "rpu_tile_get_extra": (C.c_int, [_P, C.POINTER(C.c_int64)]),
    "rpu_tile_set_extra": (C.c_int, [_P, C.POINTER(C.c_int64), C.c_int]),
    "rpu_group_create": (C.c_int, [C.POINTER(_P), C.POINTER(_P), C.c_int]),
    "rpu_group_forward": (C.c_int, [_P, C.POINTER(_P), C.POINTER(_P), C.c_int, C.c_int, _P]),
    "rpu_group_forward_strided": (C.c_int, [_P, C.POINTER(_P), C.POINTER(C.c_long), C.POINTER(_P), C.POINTER(C.c_long),
                                            C.c_int, C.c_int, _P]),
    "rpu_group_backward_strided": (C.c_int, [_P, C.POINTER(_P), C.POINTER(C.c_long), C.POINTER(_P), C.POINTER(C.c_long),
                                             C.c_int, _P]),
    "rpu_group_update_strided": (C.c_int, [_P, C.POINTER(_P), C.POINTER(C.c_long), C.POINTER(_P), C.POINTER(C.c_long),
                                           C.c_int, _P]),
    "rpu_group_get_shared_input_sets": (C.c_int, [_P, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "rpu_group_destroy": (C.c_int, [_P]),
    "rpu_tile_set_forward_out_scale": (C.c_int, [_P, C.c_float]),
    "rpu_pcm_noise_params_default": (C.c_int, [C.POINTER(PcmNoiseParams)]),
    "rpu_tile_program_weights": (C.c_int, [_P, C.POINTER(PcmNoiseParams), C.c_int, _P]),
    "rpu_tile_drift_weights": (C.c_int, [_P, C.POINTER(PcmNoiseParams), C.c_float, _P]),
    "rpu_tile_get_drift_state": (C.c_int, [_P, _P, _P, _P]),
    "rpu_tile_drift_readout": (C.c_int, [_P, C.POINTER(C.c_float), _P]),
    "rpu_tile_clone": (C.c_int, [C.POINTER(_P), _P]),
    "rpu_tile_to_device": (C.c_int, [_P, C.c_int]),
    "rpu_tile_destroy": (C.c_int, [_P]),
    "rpu_tile_forward": (C.c_int, [_P, _P, _P, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _P]),
    "rpu_tile_backward": (C.c_int, [_P, _P, _P, C.c_int, C.c_int, C.c_int, C.c_int, _P]),
    "rpu_tile_update": (C.c_int, [_P, _P, _P, C.c_int, C.c_int, C.c_int, C.c_int, _P]),
    "rpu_tile_get_x_size": (C.c_int, [_P]),
    "rpu_tile_get_d_size": (C.c_int, [_P]),
    "rpu_tile_is_on_device": (C.c_int, [_P]),
    "rpu_tile_set_learning_rate": (C.c_int, [_P, C.c_float]),
    "rpu_tile_get_learning_rate": (C.c_float, [_P]),
    "rpu_tile_set_weights": (C.c_int, [_P, _P]),
    "rpu_tile_get_weights": (C.c_int, [_P, _P]),
    "rpu_tile_weights_device_ptr": (C.c_int, [_P, C.POINTER(_P)]),
    "rpu_tile_hidden_parameter_count": (C.c_int, [_P]),
    "rpu_tile_hidden_parameter_name": (C.c_char_p, [_P, C.c_int]),
    "rpu_tile_get_hidden_parameters": (C.c_int, [_P, _P]),
    "rpu_tile_set_hidden_parameters": (C.c_int, [_P, _P]),
    "rpu_tile_set_seed": (C.c_int, [_P, C.c_uint64]),
    "rpu_tile_set_update_variant": (C.c_int, [_P, C.c_int, C.c_int]),
    "rpu_tile_update_noalloc": (C.c_int, [_P, _P, _P, C.c_int, C.c_int, C.c_int, C.c_int, _P]),
    "rpu_tile_get_update_words": (C.c_int, [_P, _P, _P, _P, C.c_int]),
    "rpu_tile_get_update_words_per_sample": (C.c_int, [_P, _P]),
    "rpu_tile_set_fused_rounds": (C.c_int, [_P, C.c_int]),
    "rpu_tile_set_round_wait_test_hook": (C.c_int, [_P, C.c_int, C.c_int]),
    "rpu_group_set_round_wait_test_hook": (C.c_int, [_P, C.c_int, C.c_int]),
    "rpu_tile_get_update_ab": (C.c_int, [_P, _P, _P, C.c_int]),
    "rpu_tile_update_with_words": (C.c_int, [_P, _P, _P, C.c_int, _P]),
    "rpu_tile_get_implicit_counts": (C.c_int, [_P, _P, C.c_int]),
    "rpu_tile_get_bm_rounds": (C.c_int, [_P, _P, C.c_int]),
    "rpu_tile_set_profiling": (C.c_int, [_P, C.c_int]),
    "rpu_tile_get_profile": (C.c_int, [_P, _P, C.c_int, C.POINTER(C.c_int)]),
    "rpu_tile_profile_name": (C.c_char_p, [_P, C.c_int]),
    "rpu_philox4x32_10": (C.c_int, [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "rpu_philox4x32_10_device": (C.c_int, [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_int]),
    "rpu_device_allocation_count": (C.c_long, []),
    "rpu_last_error": (C.c_char_p, []),
    "rpu_abi_version": (C.c_int, []),
}

_lib = None
_lock = threading.Lock()


def lib():
    """Load ``librpu_amd.so`` (once).  Raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `make -C aihwkit_amd/csrc` "
                    "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
                    "There is no fallback implementation."
                )
            handle = C.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SYMBOLS.items():
                fn = getattr(handle, name)  # AttributeError if the symbol is not exported
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = handle
    return _lib


def check(code):
    """Turn a non-zero return code into the RuntimeError the reference's bindings raise."""
    if code != 0:
        raise RuntimeError(lib().rpu_last_error().decode("utf-8", "replace"))
