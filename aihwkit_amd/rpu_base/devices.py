"""Mirror of ``rpu_base.devices``: parameter structs and enums of the analog tile.

Class and field names are those of the reference bindings
(src/aihwkit/simulator/rpu_base_src/rpu_base_devices.cpp:436-656, rpu_base_utils.cpp:55-91) so that
``parameters_to_bindings`` style code (src/aihwkit/simulator/parameters/helpers.py:64-123), which copies
dataclass fields onto these objects by name, works unchanged.  Defaults are the C++ defaults of the
reference structs (src/rpucuda/rpu_pulsed_meta_parameter.h:50-106,248-323, rpu_pulsed_device.h:52-114,
rpu_linearstep_device.h:16-80).
"""
import enum
import sys

from .._cabi import MAX_VECTOR_DEVICES, DeviceParams, IOParams, TileConfig, TransferParams, UpdateParams

FLT_MAX = 3.4028234663852886e38


class BoundManagementType(enum.IntEnum):
    """rpu_base_utils.cpp:55-58."""

    # pylint: disable=invalid-name
    NONE = 0
    Iterative = 1
    IterativeWorstCase = 2


class NoiseManagementType(enum.IntEnum):
    """rpu_base_utils.cpp:66-72."""

    NONE = 0
    AbsMax = 1
    AbsMaxNPSum = 2
    Max = 3
    Constant = 4
    AverageAbsMax = 5


class WeightNoiseType(enum.IntEnum):
    """rpu_base_utils.cpp:74-77."""

    NONE = 0
    AdditiveConstant = 1
    PCMRead = 2


class PulseType(enum.IntEnum):
    """rpu_base_utils.cpp:79-85."""

    NONE = 0
    StochasticCompressed = 1
    Stochastic = 2
    NoneWithDevice = 3
    MeanCount = 4
    DeterministicImplicit = 5


class WeightClipType(enum.IntEnum):
    """src/rpucuda/weight_clipper.h:14-19."""

    NONE = 0
    FIXED_VALUE = 1
    LAYER_GAUSSIAN = 2
    AVERAGE_CHANNEL_MAX = 3


class WeightClipParameter:
    """src/rpucuda/weight_clipper.h:22-27 (``rpu_base.tiles.WeightClipParameter`` in the reference bindings)."""

    def __init__(self, type=WeightClipType.NONE, fixed_value: float = -1.0, sigma: float = 2.5):  # pylint: disable=redefined-builtin
        self.type = WeightClipType(type)
        self.fixed_value = float(fixed_value)
        self.sigma = float(sigma)


class WeightRemapType(enum.IntEnum):
    """src/rpucuda/weight_remapper.h:14-22 (the bindings expose the first three, rpu_base_utils.cpp:44-47)."""

    NONE = 0
    LayerwiseSymmetric = 1
    ChannelwiseSymmetric = 2
    ChannelwiseNorm = 3
    ChannelwiseExceeded = 4
    LayerwiseAsymmetric = 5
    ChannelwiseAsymmetric = 6


class WeightRemapParameter:
    """src/rpucuda/weight_remapper.h:25-38 (``rpu_base.tiles.WeightRemapParameter``, rpu_base_utils.cpp:24-29)."""

    def __init__(self):
        self.type = WeightRemapType.NONE
        self.max_scale_range = 0.0
        self.max_scale_ref = 0.0
        self.row_norm = 1.0
        self.remapped_wmax = 1.0
        self.clip_if = True


class WeightModifierType(enum.IntEnum):
    """src/rpucuda/weight_modifier.h:14-25 (rpu_base_utils.cpp:31-42)."""

    Copy = 0
    Discretize = 1
    MultNormal = 2
    AddNormal = 3
    DiscretizeAddNormal = 4
    DoReFa = 5
    Poly = 6
    PCMNoise = 7
    DropConnect = 8
    ProgNoise = 9


class WeightModifierParameter:
    """src/rpucuda/weight_modifier.h:27-50 (``rpu_base.tiles.WeightModifierParameter``, rpu_base_tiles.cpp:30-51).
    The pcm_* fields belong to the PCMNoise type, which only the reference's CUDA code has."""

    def __init__(self):
        self.type = WeightModifierType.Copy
        self.std_dev = 0.0
        self.per_batch_sample = False
        self.res = 0.1
        self.sto_round = False
        self.dorefa_clip = 0.6
        self.pdrop = 0.0
        self.enable_during_test = False
        self.copy_last_column = False
        self.rel_to_actual_wmax = True
        self.assumed_wmax = 1.0
        self.g_max = 25.0
        self.coeffs = [0.26348 / 25.0, 0.0768, -0.001877 * 25.0]
        self.pcm_zero_thres = 0.0
        self.pcm_t_inference = 0.0
        self.pcm_prob_at_reset = 0.0
        self.pcm_prob_at_gmax = 0.0
        self.pcm_prob_at_random = 0.0
        self.pcm_t0 = 20.0


class AnalogMVType(enum.IntEnum):
    """rpu_base_utils.cpp:87-91."""

    Ideal = 0
    OnePass = 1
    PosNegSeparate = 2
    PosNegSeparateDigitalSum = 3


# pybind exposes the member called "None" of each enum; Python's enum cannot define it in the class body.
for _e in (BoundManagementType, NoiseManagementType, WeightNoiseType, PulseType, WeightClipType, WeightRemapType):
    setattr(_e, "None", _e.NONE)  # reachable through getattr(Enum, "None") like the reference
setattr(WeightModifierType, "None", WeightModifierType.Copy)  # rpu_base_utils.cpp:42


class _Struct:
    """Attribute bag with fixed fields: unknown names raise, as on a pybind struct."""

    _defaults = {}

    def __init__(self):
        import copy

        for name, value in self._all_defaults().items():
            # a nested struct is this object's own
            object.__setattr__(self, name, copy.deepcopy(value) if isinstance(value, _Struct) else value)

    @classmethod
    def _all_defaults(cls):
        out = {}
        for klass in reversed(cls.__mro__):
            out.update(getattr(klass, "_defaults", {}))
        return out

    def __setattr__(self, name, value):
        if name not in self._all_defaults():
            raise AttributeError(f"{type(self).__name__} has no field {name!r}")
        object.__setattr__(self, name, value)

    def _all_values(self):
        return {k: getattr(self, k) for k in self._all_defaults()}

    def __eq__(self, other):
        return type(other) is type(self) and other._all_values() == self._all_values()

    __hash__ = None

    def __str__(self):
        fields = ", ".join(f"{k}={getattr(self, k)!r}" for k in self._all_defaults())
        return f"{type(self).__name__}({fields})"


class AnalogTileInputOutputParameter(_Struct):
    """rpu_base_devices.cpp:485-519 over IOMetaParameter (rpu_pulsed_meta_parameter.h:50-106)."""

    _defaults = dict(
        bm_test_negative_bound=True, bound_management=BoundManagementType.NONE, inp_bound=1.0,
        inp_noise=0.0, inp_res=1.0 / (2.0**7 - 2.0), inp_sto_round=False, is_perfect=False,
        max_bm_factor=1000, max_bm_res=0.25, nm_assumed_wmax=0.6, nm_decay=1e-3, nm_thres=0.0,
        noise_management=NoiseManagementType.AbsMax, out_bound=12.0, out_noise=0.06,
        out_noise_std=0.0, out_res=1.0 / (2.0**9 - 2.0), out_scale=1.0, out_sto_round=False,
        w_noise=0.0, w_noise_type=WeightNoiseType.NONE, ir_drop=0.0, ir_drop_g_ratio=5.7143e5,
        out_nonlinearity=0.0, out_nonlinearity_std=0.0, mv_type=AnalogMVType.OnePass,
        inp_asymmetry=0.0, out_asymmetry=0.0, slope_calibration=0.5, r_series=0.0, v_offset_std=0.0,
        v_offset_w_min=0.0, w_read_asymmetry_dtod=0.0,
        r_series_max_total=3.4028234663852886e38,   # IOMetaParameter field that the reference's binding leaves out
    )

    def _to_c(self) -> IOParams:
        p = IOParams()
        p.is_perfect = int(bool(self.is_perfect))
        p.mv_type = int(self.mv_type)
        p.noise_management = int(self.noise_management)
        p.bound_management = int(self.bound_management)
        p.bm_test_negative_bound = int(bool(self.bm_test_negative_bound))
        p.max_bm_factor = int(self.max_bm_factor)
        p.inp_sto_round = int(bool(self.inp_sto_round))
        p.out_sto_round = int(bool(self.out_sto_round))
        for name in ("inp_bound", "inp_res", "inp_noise", "inp_asymmetry", "out_bound", "out_res",
                     "out_noise", "out_asymmetry", "out_scale", "nm_thres", "nm_assumed_wmax",
                     "max_bm_res", "w_noise", "ir_drop", "out_noise_std", "out_nonlinearity",
                     "out_nonlinearity_std", "v_offset_std", "r_series", "w_read_asymmetry_dtod",
                     "ir_drop_g_ratio", "nm_decay", "slope_calibration", "v_offset_w_min", "r_series_max_total"):
            setattr(p, name, float(getattr(self, name)))
        p.w_noise_type = int(self.w_noise_type)
        return p


class AnalogTileUpdateParameter(_Struct):
    """rpu_base_devices.cpp:469-483 over PulsedUpdateMetaParameter (rpu_pulsed_meta_parameter.h:248-323)."""

    _defaults = dict(
        fixed_bl=True, desired_bl=31, d_res_implicit=0.0, pulse_type=PulseType.StochasticCompressed,
        res=0.0, sto_round=False, um_reg_scale=1.0, um_grad_scale=1.0, d_sparsity=False,
        update_management=True, update_bl_management=True, x_res_implicit=0.0,
    )

    def _to_c(self) -> UpdateParams:
        p = UpdateParams()
        p.pulse_type = int(self.pulse_type)
        p.desired_bl = int(self.desired_bl)
        p.fixed_bl = int(bool(self.fixed_bl))
        p.update_management = int(bool(self.update_management))
        p.update_bl_management = int(bool(self.update_bl_management))
        p.sto_round = int(bool(self.sto_round))
        p.um_grad_scale = float(self.um_grad_scale)
        p.res = float(self.res)
        p.x_res_implicit = float(self.x_res_implicit)
        p.d_res_implicit = float(self.d_res_implicit)
        return p


class DriftParameter(_Struct):
    """rpu_base_devices.cpp:521-533 over DriftParameter (src/rpucuda/weight_drifter.h:14-60): power-law drift
    w = w0 (delta_t / t_0)^(-nu) of a training tile; active on a pulsed device when nu > 0."""

    _defaults = dict(nu=0.0, nu_dtod=0.0, nu_std=0.0, wg_ratio=1.0, g_offset=0.0, w_offset=0.0, nu_k=0.0,
                     log_g0=0.0, t_0=1.0, reset_tol=1e-7, w_noise_std=0.0)

    _C_NAMES = dict(nu="drift_nu", nu_dtod="drift_nu_dtod", nu_std="drift_nu_std", wg_ratio="drift_wg_ratio",
                    g_offset="drift_g_offset", w_offset="drift_w_offset", nu_k="drift_nu_k",
                    log_g0="drift_log_g0", t_0="drift_t0", reset_tol="drift_reset_tol",
                    w_noise_std="drift_w_read_std")

    def _fill_c(self, p: DeviceParams, simple: bool = False) -> None:
        for name, c_name in self._C_NAMES.items():
            setattr(p, c_name, float(getattr(self, name)))
        if simple:
            p.drift_nu_dtod = 0.0  # DriftParameter::setSimpleDrift (weight_drifter.h:46-49)


class AbstractResistiveDeviceParameter(_Struct):
    """rpu_base_devices.cpp:536-539 (+ the SimpleMetaParameter fields diffusion / lifetime / drift)."""

    _defaults = dict(construction_seed=0, diffusion=0.0, lifetime=0.0, drift=DriftParameter())
    _kind = None

    def _fill_c(self, p: DeviceParams) -> None:
        p.construction_seed = int(self.construction_seed)
        p.diffusion = float(self.diffusion)
        p.lifetime = float(self.lifetime)
        if self.drift is not None:
            self.drift._fill_c(p)

    def _to_c(self) -> DeviceParams:
        from .._cabi import check, lib

        cfg = TileConfig()
        check(lib().rpu_tile_config_default(cfg, int(self._kind)))
        p = cfg.device
        self._fill_c(p)
        return p


class IdealResistiveDeviceParameter(AbstractResistiveDeviceParameter):
    """rpu_base_devices.cpp:545-552: no device physics; the update is a plain rank-B outer product."""

    _defaults = dict(reset_std=0.01)
    _kind = 0

    def _fill_c(self, p):
        super()._fill_c(p)
        p.reset_std = float(self.reset_std)


class PulsedResistiveDeviceParameter(AbstractResistiveDeviceParameter):
    """rpu_base_devices.cpp:554-581 over PulsedRPUDeviceMetaParameter (rpu_pulsed_device.h:52-114)."""

    _defaults = dict(
        corrupt_devices_prob=0.0, corrupt_devices_range=FLT_MAX, diffusion_dtod=0.0, dw_min=0.001,
        dw_min_dtod=0.3, dw_min_dtod_log_normal=False, dw_min_std=0.3, enforce_consistency=False,
        lifetime_dtod=0.0, perfect_bias=False, reset=0.0, reset_std=0.01, reset_dtod=0.0, up_down=0.0,
        up_down_dtod=0.01, w_max=0.6, w_max_dtod=0.3, w_min=-0.6, w_min_dtod=0.3, count_pulses=False,
    )

    def _fill_c(self, p):
        super()._fill_c(p)
        for name in ("corrupt_devices_prob", "corrupt_devices_range", "diffusion_dtod", "dw_min",
                     "dw_min_dtod", "dw_min_std", "lifetime_dtod", "reset", "reset_std", "reset_dtod",
                     "up_down", "up_down_dtod", "w_max", "w_max_dtod", "w_min", "w_min_dtod"):
            setattr(p, name, float(getattr(self, name)))
        p.dw_min_dtod_log_normal = int(bool(self.dw_min_dtod_log_normal))
        p.enforce_consistency = int(bool(self.enforce_consistency))
        p.perfect_bias = int(bool(self.perfect_bias))
        p.count_pulses = int(bool(self.count_pulses))

    def calc_weight_granularity(self) -> float:
        """rpu_constantstep_device.h:27, rpu_linearstep_device.h:58: the granularity is dw_min."""
        return float(self.dw_min)


class ConstantStepResistiveDeviceParameter(PulsedResistiveDeviceParameter):
    """rpu_base_devices.cpp:583-600."""

    _kind = 1


class LinearStepResistiveDeviceParameter(PulsedResistiveDeviceParameter):
    """rpu_base_devices.cpp:602-631 over the LinearStep tail (rpu_linearstep_device.h:16-31)."""

    _defaults = dict(
        gamma_up=0.0, gamma_down=0.0, gamma_up_dtod=0.05, gamma_down_dtod=0.05, allow_increasing=False,
        mean_bound_reference=True, write_noise_std=0.0, apply_write_noise_on_set=True, mult_noise=True,
        reverse_up=False, reverse_down=False, reverse_offset=0.01,
    )
    _kind = 2

    def _fill_c(self, p):
        super()._fill_c(p)
        p.ls_decrease_up = float(self.gamma_up)
        p.ls_decrease_down = float(self.gamma_down)
        p.ls_decrease_up_dtod = float(self.gamma_up_dtod)
        p.ls_decrease_down_dtod = float(self.gamma_down_dtod)
        p.ls_allow_increasing_slope = int(bool(self.allow_increasing))
        p.ls_mean_bound_reference = int(bool(self.mean_bound_reference))
        p.write_noise_std = float(self.write_noise_std)
        p.apply_write_noise_on_set = int(bool(self.apply_write_noise_on_set))
        p.ls_mult_noise = int(bool(self.mult_noise))
        p.ls_reverse_up = int(bool(self.reverse_up))
        p.ls_reverse_down = int(bool(self.reverse_down))
        p.ls_reverse_offset = float(self.reverse_offset)


class SoftBoundsResistiveDeviceParameter(LinearStepResistiveDeviceParameter):
    """rpu_base_devices.cpp:633-656 over SoftBoundsRPUDeviceMetaParameter (rpu_linearstep_device.h:66-80)."""

    _defaults = dict(gamma_up=1.0, gamma_down=1.0, gamma_up_dtod=0.0, gamma_down_dtod=0.0,
                     mean_bound_reference=False)
    _kind = 3

    def _fill_c(self, p):
        if not (self.gamma_up == 1.0 and self.gamma_down == 1.0 and self.gamma_up_dtod == 0.0
                and self.gamma_down_dtod == 0.0 and not self.allow_increasing
                and not self.mean_bound_reference):
            raise RuntimeError("SoftBounds set to wrong values!")  # rpu_linearstep_device.h:81-87
        super()._fill_c(p)


class VectorResistiveDeviceParameter(AbstractResistiveDeviceParameter):
    """rpu_base_devices.cpp:686-714 over VectorRPUDeviceMetaParameter: a list of device parameters.
    Only its transfer subclass can be turned into a tile on this path."""

    _defaults = dict(gamma_vec=None, update_policy=0, first_update_idx=0)

    def __init__(self):
        super().__init__()
        object.__setattr__(self, "gamma_vec", [])
        object.__setattr__(self, "_vec_par", [])

    def append_parameter(self, parameter) -> bool:
        """VectorRPUDeviceMetaParameter::appendVecPar (rpu_vector_device.cpp:74-91): pulsed devices only."""
        if not isinstance(parameter, PulsedResistiveDeviceParameter):
            return False
        self._vec_par.append(parameter)
        return True

    def calc_weight_granularity(self) -> float:
        return float(self._vec_par[0].calc_weight_granularity()) if self._vec_par else 0.0


class TransferResistiveDeviceParameter(VectorResistiveDeviceParameter):
    """rpu_base_devices.cpp:742-777 over TransferRPUDeviceMetaParameter (rpu_transfer_device.h:52-127)."""

    _defaults = dict(
        gamma=0.0, transfer_every=1.0, no_self_transfer=True, transfer_every_vec=None, units_in_mbatch=False,
        n_reads_per_transfer=1, with_reset_prob=0.0, random_selection=False, transfer_columns=True,
        transfer_lr=1.0, fast_lr=0.0, transfer_lr_vec=None, scale_transfer_lr=True, scale_fast_lr=True,
        transfer_forward=None, transfer_update=None,
    )
    _kind = 4

    def __init__(self):
        super().__init__()
        object.__setattr__(self, "transfer_every_vec", [])
        object.__setattr__(self, "transfer_lr_vec", [])
        object.__setattr__(self, "transfer_forward", AnalogTileInputOutputParameter())
        object.__setattr__(self, "transfer_update", AnalogTileUpdateParameter())

    def _to_transfer_c(self) -> TransferParams:
        n_dev = len(self._vec_par)
        if n_dev < 2:
            raise RuntimeError("Need at least 2 devices")
        if n_dev > MAX_VECTOR_DEVICES:
            raise RuntimeError(f"At most {MAX_VECTOR_DEVICES} devices in a transfer chain.")
        rest = self._vec_par[1]
        for other in self._vec_par[2:]:
            if type(other) is not type(rest) or other._all_values() != rest._all_values():
                raise RuntimeError("Only the first device can be a different RPU device. ")
        p = TransferParams()
        p.n_devices = n_dev
        p.construction_seed = int(self.construction_seed)
        for name in ("units_in_mbatch", "no_self_transfer", "random_selection", "scale_transfer_lr",
                     "scale_fast_lr", "transfer_columns"):
            setattr(p, name, int(bool(getattr(self, name))))
        p.n_reads_per_transfer = int(self.n_reads_per_transfer)
        for name in ("gamma", "transfer_every", "with_reset_prob", "fast_lr", "transfer_lr"):
            setattr(p, name, float(getattr(self, name)))
        for name in ("gamma_vec", "transfer_lr_vec", "transfer_every_vec"):
            values = list(getattr(self, name) or [])
            if len(values) > MAX_VECTOR_DEVICES:
                raise RuntimeError(f"{name} is longer than {MAX_VECTOR_DEVICES}")
            setattr(p, "n_" + name, len(values))
            for k, v in enumerate(values):
                getattr(p, name)[k] = float(v)
        p.transfer_io = self.transfer_forward._to_c()
        p.transfer_up = self.transfer_update._to_c()
        p.fast_device = self._vec_par[0]._to_c()
        p.rest_device = rest._to_c()
        return p


class AnalogTileParameter(_Struct):
    """rpu_base_devices.cpp:453-467 over PulsedMetaParameter (rpu_pulsed.h:127-151)."""

    _defaults = dict(forward_io=None, backward_io=None, update=None)

    def __init__(self):
        super().__init__()
        self.forward_io = AnalogTileInputOutputParameter()
        self.backward_io = AnalogTileInputOutputParameter()
        self.update = AnalogTileUpdateParameter()

    def _config(self, device_param) -> TileConfig:
        cfg = TileConfig()
        cfg.f_io = self.forward_io._to_c()
        cfg.b_io = self.backward_io._to_c()
        cfg.up = self.update._to_c()
        cfg.device = device_param._to_c()
        return cfg

    def create_array(self, x_size: int, d_size: int, device_param):
        """Build the host-side analog tile (device parameters are sampled here, on the CPU)."""
        from .tiles import AnalogTile

        if not isinstance(device_param, AbstractResistiveDeviceParameter) or device_param._kind is None:
            raise TypeError("device_param must be one of the *ResistiveDeviceParameter classes")
        import copy

        if isinstance(device_param, TransferResistiveDeviceParameter):
            transfer = device_param._to_transfer_c()
            config = self._config(device_param._vec_par[0])
            tile = AnalogTile._create_transfer(int(x_size), int(d_size), config, transfer)
        else:
            tile = AnalogTile._create(int(x_size), int(d_size), self._config(device_param))
        tile._meta_parameters, tile._parameters = copy.deepcopy(self), copy.deepcopy(device_param)
        return tile


class FloatingPointTileParameter(_Struct):
    """rpu_base_devices.cpp:436-451: floating-point tile = ideal device with perfect IO and no pulses."""

    _defaults = dict(diffusion=0.0, lifetime=0.0, drift=DriftParameter())

    def create_array(self, x_size: int, d_size: int):
        import copy

        from .tiles import FloatingPointTile

        meta = AnalogTileParameter()
        meta.forward_io.is_perfect = True
        meta.backward_io.is_perfect = True
        meta.update.pulse_type = PulseType.NONE
        device = IdealResistiveDeviceParameter()
        device.diffusion = float(self.diffusion)
        device.lifetime = float(self.lifetime)
        config = meta._config(device)
        if self.drift is not None:
            self.drift._fill_c(config.device, simple=True)  # RPUSimple::driftWeights (rpu.cpp:1581-1587)
        tile = FloatingPointTile._create(int(x_size), int(d_size), config)
        tile._meta_parameters, tile._parameters = copy.deepcopy(self), copy.deepcopy(self)
        return tile


__all__ = [name for name, obj in vars(sys.modules[__name__]).items()
           if isinstance(obj, type) and not name.startswith("_")]
