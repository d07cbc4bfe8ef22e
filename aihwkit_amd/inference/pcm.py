"""PCM noise model, global drift compensation and the inference tile that applies them.

Names and arguments follow the reference: ``PCMLikeNoiseModel`` (src/aihwkit/inference/noise/pcm.py:27-98, with the
single-pair conductance converter of converter/conductance.py:24-82), ``GlobalDriftCompensation``
(compensation/drift.py:21-41, base.py:25-62) and the ``program_weights`` / ``drift_weights`` / ``forward`` methods of
``InferenceTileWithPeriphery`` (src/aihwkit/simulator/tiles/inference.py:161-282).  The reference pulls the weights
to the host, perturbs them in torch and writes them back; here the perturbation runs on the tile's matrix in HBM.
"""
import ctypes as C
from typing import List, Optional

import torch

from .._cabi import PcmNoiseParams, check, lib
from ..rpu_base import devices, tiles


class PCMLikeNoiseModel:
    """Statistical PCM noise model (Nandakumar et al., ICECS 2019) with one pair of conductances per weight."""

    def __init__(self, prog_coeff: Optional[List[float]] = None, g_converter=None, g_max: Optional[float] = None,
                 t_read: float = 250.0e-9, t_0: float = 20.0, prog_noise_scale: float = 1.0,
                 read_noise_scale: float = 1.0, drift_scale: float = 1.0,
                 prog_coeff_g_max_reference: Optional[float] = None, g_min: Optional[float] = None):
        if g_converter is not None:
            raise NotImplementedError("only the single-pair conductance converter is provided")
        self.g_max = 25.0 if g_max is None else float(g_max)
        self.g_min = 0.0 if g_min is None else float(g_min)
        if self.g_max < 0.0:
            raise ValueError("g_max should be a positive value")
        if self.g_min < 0.0:
            raise ValueError("g_min should be a positive value")
        if self.g_min >= self.g_max:
            raise ValueError("g_min should be smaller than g_max")
        self.prog_coeff_g_max_reference = self.g_max if prog_coeff_g_max_reference is None \
            else float(prog_coeff_g_max_reference)
        if prog_coeff is None:
            # the standard coefficients were fitted at g_max = 25 uS (pcm.py:86-90)
            self.prog_coeff = [0.26348, 1.9650, -1.1731]
            self.prog_coeff_g_max_reference = 25.0
        else:
            if len(prog_coeff) != 3:
                raise NotImplementedError("a polynomial of degree 2 (three coefficients) is provided")
            self.prog_coeff = [float(c) for c in prog_coeff]
        self.t_0, self.t_read = float(t_0), float(t_read)
        self.prog_noise_scale = float(prog_noise_scale)
        self.read_noise_scale = float(read_noise_scale)
        self.drift_scale = float(drift_scale)

    def _to_c(self) -> PcmNoiseParams:
        p = PcmNoiseParams()
        check(lib().rpu_pcm_noise_params_default(C.byref(p)))
        for name in ("g_max", "g_min", "t_read", "t_0", "prog_noise_scale", "read_noise_scale", "drift_scale",
                     "prog_coeff_g_max_reference"):
            setattr(p, name, getattr(self, name))
        for k in range(3):
            p.prog_coeff[k] = self.prog_coeff[k]
        return p


class GlobalDriftCompensation:
    """One output scale for the whole tile: read-out of the unit vectors, mean absolute output."""

    @staticmethod
    def apply(current_value: float, ref_value: float) -> float:
        """compensation/base.py:53-62."""
        return ref_value / current_value


class InferenceTile:
    """GPU tile for inference: ideal device, analog forward pass, PCM weight pipeline, drift compensation."""

    def __init__(self, out_size: int, in_size: int, forward_io: Optional[devices.AnalogTileInputOutputParameter] = None,
                 noise_model: Optional[PCMLikeNoiseModel] = None,
                 drift_compensation: Optional[GlobalDriftCompensation] = GlobalDriftCompensation()):
        meta = devices.AnalogTileParameter()
        if forward_io is not None:
            meta.forward_io = forward_io
        meta.backward_io.is_perfect = True
        meta.update.pulse_type = devices.PulseType.NONE
        host = tiles.AnalogTile._create(int(in_size), int(out_size), meta._config(devices.IdealResistiveDeviceParameter()))
        self.host = host
        self.tile: Optional[tiles.CudaAnalogTile] = None
        self.noise_model = noise_model or PCMLikeNoiseModel()
        self.drift_compensation = drift_compensation
        self.drift_baseline: Optional[float] = None
        self.alpha = 1.0
        self._out_scale = float(meta.forward_io.out_scale)
        self._alpha_in_tile = False

    def set_weights(self, weights: torch.Tensor) -> None:
        (self.tile or self.host).set_weights(weights)

    def get_weights(self) -> torch.Tensor:
        return (self.tile or self.host).get_weights()

    def cuda(self) -> "InferenceTile":
        if self.tile is None:
            self.tile = tiles.CudaAnalogTile(self.host)
        return self

    def _gpu(self) -> tiles.CudaAnalogTile:
        if self.tile is None:
            raise RuntimeError("The inference tile computes on the GPU only: call .cuda() first.")
        return self.tile

    def _stream(self):
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def _readout(self) -> float:
        if self._alpha_in_tile:   # the read-out is of the uncompensated tile
            check(lib().rpu_tile_set_forward_out_scale(self._gpu()._h, float(self._out_scale)))
        value = C.c_float(0.0)
        check(lib().rpu_tile_drift_readout(self._gpu()._h, C.byref(value), self._stream()))
        return float(value.value)

    def program_weights(self, from_reference: bool = True, noise_model: Optional[PCMLikeNoiseModel] = None) -> None:
        """inference.py:161-213."""
        if noise_model is not None:
            self.noise_model = noise_model
        check(lib().rpu_tile_program_weights(self._gpu()._h, C.byref(self.noise_model._to_c()), int(from_reference),
                                             self._stream()))
        if self.drift_compensation is not None:
            self.drift_baseline = self._readout()
        self.alpha = 1.0
        if self._alpha_in_tile:
            self.compensate_in_tile(True)

    def drift_weights(self, t_inference: float = 0.0) -> None:
        """inference.py:215-262."""
        if self.drift_baseline is None and self.drift_compensation is not None:
            self.program_weights()
        check(lib().rpu_tile_drift_weights(self._gpu()._h, C.byref(self.noise_model._to_c()), float(t_inference),
                                           self._stream()))
        if self.drift_compensation is not None:
            self.alpha = self.drift_compensation.apply(self._readout(), self.drift_baseline)
        if self._alpha_in_tile:
            self.compensate_in_tile(True)

    def compensate_in_tile(self, enable: bool = True) -> None:
        """Let the drift-compensation factor ride on the tile's ADC stage (its forward ``out_scale``) instead of
        multiplying the output tensor afterwards; for callers that forward in evaluation mode only, e.g. through a
        ``TileGroup``.  Call again after ``drift_weights`` / ``program_weights`` changed the factor."""
        self._alpha_in_tile = bool(enable)
        scale = self._out_scale * (self.alpha if enable else 1.0)
        check(lib().rpu_tile_set_forward_out_scale(self._gpu()._h, float(scale)))

    def drift_state(self):
        """(programmed weights, drift coefficients of the positive and of the negative conductance), CPU tensors."""
        tile = self._gpu()
        shape = (tile.get_d_size(), tile.get_x_size())
        out = [torch.empty(shape, dtype=torch.float32) for _ in range(3)]
        check(lib().rpu_tile_get_drift_state(tile._h, out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr()))
        return tuple(out)

    def set_matrix_indices(self, indices: torch.Tensor) -> None:
        """Index matrix of a convolution layer (what ``AnalogConvNd`` computes once per input shape)."""
        self._gpu().set_matrix_indices(indices)

    def forward_indexed(self, x_input: torch.Tensor, d_tensor: torch.Tensor, is_test: bool = False) -> torch.Tensor:
        """Analog forward of a convolution through the index matrix, drift compensation as in ``forward``."""
        out = self._gpu().forward_indexed(x_input, d_tensor, is_test)
        if is_test and self.drift_compensation is not None and self.alpha != 1.0 and not self._alpha_in_tile:
            out.mul_(self.alpha)
        return out

    def forward(self, x_input: torch.Tensor, is_test: bool = False, bias: bool = False) -> torch.Tensor:
        """Analog forward; in evaluation mode the output is scaled by the drift compensation (inference.py:264-282).
        ``bias``: the tile's last input column is the bias column and ``x_input`` comes without it (the tile adds the
        column of ones, as the reference's ``forward(x_input, bias=True)`` does)."""
        out = self._gpu().forward(x_input, bias, False, False, is_test, False)
        if is_test and self.drift_compensation is not None and self.alpha != 1.0 and not self._alpha_in_tile:
            out = out * self.alpha
        return out
