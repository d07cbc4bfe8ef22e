"""Mirror of ``rpu_base.tiles``: tile classes with the call signatures of the reference bindings.

Reference: src/aihwkit/simulator/rpu_base_src/rpu_base_tiles.cpp (CPU tiles ``FloatingPointTile`` /
``AnalogTile``) and rpu_base_tiles_cuda.cpp (``CudaFloatingPointTile`` / ``CudaAnalogTile``).

The host tiles hold parameters, the sampled per-device arrays and the weights; they can be inspected
and copied to a GPU (``CudaAnalogTile(cpu_tile)``, as ``.cuda()`` does in the reference,
src/aihwkit/simulator/tiles/rpucuda.py:145-209) but they do not compute: ``forward`` / ``backward`` /
``update`` exist only on the GPU tiles and run hand-written HIP kernels through the C ABI.  Positional
argument order is the reference's; it is what its Python callers rely on
(src/aihwkit/simulator/tiles/periphery.py:1061,1165,1225).
"""
import ctypes as C
from typing import List

import torch

from .._cabi import MAX_MODIFIER_COEFFS, ModifierParams, RemapParams, check, lib
# the reference binds these parameter structs in its tiles module (rpu_base_utils.cpp:17-58)
from .devices import (WeightClipParameter, WeightClipType, WeightModifierParameter,  # noqa: F401
                      WeightModifierType, WeightRemapParameter, WeightRemapType)

_DTYPE = torch.float32


def _check_input(tensor: torch.Tensor, cuda: bool, name: str) -> torch.Tensor:
    # CHECK_TORCH_INPUT / CHECK_TORCH_CUDA_INPUT (rpu_base_tiles.cpp:15-22)
    if not isinstance(tensor, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    tensor = tensor.contiguous()
    if tensor.dtype != _DTYPE:
        raise RuntimeError(f"{name} must be a float32 tensor")
    if cuda and not tensor.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not cuda and tensor.is_cuda:
        raise RuntimeError(f"{name} must be a CPU tensor")
    return tensor


class _TileBase:
    """State surface shared by host and GPU tiles."""

    def __init__(self, handle):
        self._h = C.c_void_p(handle)

    def __del__(self):
        handle, self._h = getattr(self, "_h", None), None
        if handle:
            try:
                lib().rpu_tile_destroy(handle)
            except Exception:  # pylint: disable=broad-except
                pass

    @classmethod
    def _create(cls, x_size, d_size, config):
        handle = C.c_void_p()
        check(lib().rpu_tile_create(C.byref(handle), x_size, d_size, C.byref(config)))
        return cls(handle.value)

    @classmethod
    def _create_transfer(cls, x_size, d_size, config, transfer):
        handle = C.c_void_p()
        check(lib().rpu_tile_create_transfer(C.byref(handle), x_size, d_size, C.byref(config), C.byref(transfer)))
        return cls(handle.value)

    def get_transfer_state(self):
        """(number of update vectors since the weights were set, next column per device) of a transfer compound."""
        count = C.c_uint64(0)
        from .._cabi import MAX_VECTOR_DEVICES
        slices = (C.c_int32 * MAX_VECTOR_DEVICES)(*([-1] * MAX_VECTOR_DEVICES))
        check(lib().rpu_tile_get_transfer_state(self._h, C.byref(count), slices))
        return int(count.value), [v for v in slices if v >= 0]

    def _clone_handle(self):
        handle = C.c_void_p()
        check(lib().rpu_tile_clone(C.byref(handle), self._h))
        return handle.value

    def _copy_parameters_to(self, other):
        other._meta_parameters = getattr(self, "_meta_parameters", None)
        other._parameters = getattr(self, "_parameters", None)
        return other

    def __copy__(self):
        return self._copy_parameters_to(type(self)(self._clone_handle()))

    def __deepcopy__(self, memo):
        return self._copy_parameters_to(type(self)(self._clone_handle()))

    # -- parameter structs the tile was built from (rpu_base_tiles.cpp get_parameters / get_meta_parameters)
    def get_meta_parameters(self):
        return self._meta_parameters

    def get_parameters(self):
        return self._parameters

    def set_weights_uniform_random(self, min_value: float, max_value: float) -> None:
        """Uniform random weights in [min_value, max_value], clipped into the device bounds like ``set_weights``
        (RPUPulsed::setWeightsUniformRandom, src/rpucuda/rpu_pulsed.cpp:280-284); the draw uses torch's generator."""
        shape = (self.get_d_size(), self.get_x_size())
        self.set_weights(torch.rand(shape, dtype=_DTYPE) * (float(max_value) - float(min_value)) + float(min_value))

    # -- hardware-aware-training utilities of the reference bindings (rpu_base_tiles.cpp:292-371, 845-868): they work
    #    on the matrix in HBM and are methods of the GPU tiles
    def _needs_gpu(self, *args, **kwargs):
        raise RuntimeError("Host tiles do not compute: build a CudaAnalogTile(tile) / CudaFloatingPointTile(tile).")

    drift_weights = _needs_gpu
    remap_weights = _needs_gpu
    modify_weights = _needs_gpu

    def get_read_asymmetry(self, backward: bool = False) -> torch.Tensor:
        """[d_size, x_size] factors of the negative pass of PosNegSeparate (the reference's ``fwd.w_asymmetry`` /
        ``bwd.w_asymmetry`` state entries, rpu_forward_backward_pass.cpp:62-100)."""
        out = torch.empty(self.get_d_size(), self.get_x_size(), dtype=_DTYPE)
        check(lib().rpu_tile_get_read_asymmetry(self._h, int(bool(backward)), out.data_ptr()))
        return out

    def set_read_asymmetry(self, factors: torch.Tensor, backward: bool = False) -> None:
        factors = _check_input(factors, False, "factors")
        if tuple(factors.shape) != (self.get_d_size(), self.get_x_size()):
            raise RuntimeError("Invalid dimensions of the read asymmetry factors")
        check(lib().rpu_tile_set_read_asymmetry(self._h, int(bool(backward)), factors.data_ptr()))

    def get_pulse_counters(self) -> torch.Tensor:
        """int64 [2, d_size, x_size] (up-counting pulses where the signs of x and d agree, then where they differ)
        of a tile whose device has ``count_pulses`` set, else an empty tensor (rpu_base_tiles.cpp:845-868)."""
        if not lib().rpu_tile_pulse_counter_count(self._h):
            return torch.empty(0, dtype=torch.int64)
        out = torch.empty(2, self.get_d_size(), self.get_x_size(), dtype=torch.int64)
        check(lib().rpu_tile_get_pulse_counters(self._h, out.data_ptr()))
        return out

    # -- sizes / learning rate (rpu_base_tiles.cpp get_x_size, get_d_size, get/set_learning_rate)
    def get_x_size(self) -> int:
        return lib().rpu_tile_get_x_size(self._h)

    def get_d_size(self) -> int:
        return lib().rpu_tile_get_d_size(self._h)

    def get_learning_rate(self) -> float:
        return float(lib().rpu_tile_get_learning_rate(self._h))

    def set_learning_rate(self, learning_rate: float) -> None:
        check(lib().rpu_tile_set_learning_rate(self._h, float(learning_rate)))

    # -- weights: [d_size, x_size] CPU tensors (rpu_base_tiles.cpp:161-214)
    def get_weights(self) -> torch.Tensor:
        out = torch.empty(self.get_d_size(), self.get_x_size(), dtype=_DTYPE)
        check(lib().rpu_tile_get_weights(self._h, out.data_ptr()))
        return out

    def set_weights(self, weights: torch.Tensor) -> None:
        weights = _check_input(weights.detach().cpu() if weights.is_cuda else weights.detach(), False, "weights")
        if weights.dim() != 2 or weights.size(0) != self.get_d_size() or weights.size(1) != self.get_x_size():
            raise RuntimeError(
                f"Invalid weights dimensions: expected [{self.get_d_size()},{self.get_x_size()}] array")
        check(lib().rpu_tile_set_weights(self._h, weights.data_ptr()))

    # -- index matrix of the *_indexed methods (rpu_base_tiles.cpp:721-760)
    def set_matrix_indices(self, indices: torch.Tensor) -> None:
        """int32 tensor with x_size * patches entries, patch index fastest (what the conv layers produce)."""
        if indices.dtype != torch.int32:
            raise RuntimeError("indices must be an int32 tensor")
        indices = indices.detach().cpu().contiguous()
        x_size = self.get_x_size()
        if indices.numel() == 0 or indices.numel() % x_size != 0:
            raise RuntimeError("The number of indices must be a multiple of x_size")
        patches = indices.numel() // x_size
        check(lib().rpu_tile_set_matrix_indices(self._h, indices.data_ptr(), x_size, patches))

    def has_matrix_indices(self) -> bool:
        return lib().rpu_tile_has_matrix_indices(self._h) > 0

    # -- hidden per-device parameters (rpu_base_tiles.cpp:763-825)
    def get_hidden_parameter_names(self) -> List[str]:
        count = lib().rpu_tile_hidden_parameter_count(self._h)
        return [lib().rpu_tile_hidden_parameter_name(self._h, k).decode() for k in range(count)]

    def get_hidden_parameters(self) -> torch.Tensor:
        count = lib().rpu_tile_hidden_parameter_count(self._h)
        out = torch.empty(count, self.get_d_size(), self.get_x_size(), dtype=_DTYPE)
        if count:
            check(lib().rpu_tile_get_hidden_parameters(self._h, out.data_ptr()))
        return out

    def set_hidden_parameters(self, params: torch.Tensor) -> None:
        count = lib().rpu_tile_hidden_parameter_count(self._h)
        params = _check_input(params.detach(), False, "hidden parameters")
        if params.dim() != 3 or tuple(params.shape) != (count, self.get_d_size(), self.get_x_size()):
            raise RuntimeError(
                f"Invalid parameters dimensions: expected [{count},{self.get_d_size()},{self.get_x_size()}] array")
        if count:
            check(lib().rpu_tile_set_hidden_parameters(self._h, params.data_ptr()))

    def set_seed(self, seed: int) -> None:
        """Seed of the Philox generator behind every random draw of this tile on the GPU."""
        check(lib().rpu_tile_set_seed(self._h, int(seed) & 0xFFFFFFFFFFFFFFFF))

    def set_update_variant(self, variant: str = "exact", samples_per_step: int = 32) -> None:
        """Not in the reference: "exact" (default) applies the coincidences pulse by pulse like the reference;
        "aggregated" (opt-in, LinearStep / SoftBounds with multiplicative noise) counts them per group of
        `samples_per_step` samples and applies them in closed form with one noise draw per group."""
        codes = {"exact": 0, "aggregated": 1}
        if variant not in codes:
            raise RuntimeError("Unknown update variant: " + str(variant))
        check(lib().rpu_tile_set_update_variant(self._h, codes[variant], int(samples_per_step)))

    # -- state beyond weights and hidden parameters (rpu_base_tiles.cpp:89-113)
    def dump_extra(self) -> dict:
        count = lib().rpu_tile_extra_count(self._h)
        values = (C.c_int64 * count)()
        check(lib().rpu_tile_get_extra(self._h, values))
        return {"rpu." + lib().rpu_tile_extra_name(self._h, k).decode(): int(values[k]) for k in range(count)}

    def load_extra(self, state: dict, strict: bool) -> None:
        current = self.dump_extra()
        for name in current:
            if name in state:
                current[name] = int(state[name])
            elif strict:
                raise RuntimeError("Cannot find the key: '" + name + "' in state.")
        values = (C.c_int64 * len(current))(*current.values())
        check(lib().rpu_tile_set_extra(self._h, values, len(current)))

    def get_shared_weights_if(self) -> bool:
        return bool(lib().rpu_tile_get_shared_weights_if(self._h))

    def get_brief_info(self) -> str:
        where = "gfx950" if lib().rpu_tile_is_on_device(self._h) else "host"
        return f"{type(self).__name__}({self.get_d_size()},{self.get_x_size()}) [{where}]"

    # -- the hot path is not provided on host tiles
    def forward(self, *args, **kwargs):
        raise RuntimeError("Host tiles do not compute: build a CudaAnalogTile(tile) / CudaFloatingPointTile(tile).")

    backward = forward
    update = forward


class FloatingPointTile(_TileBase):
    """Host-side floating point tile (rpu_base_tiles.cpp ``FloatingPointTile``)."""


class AnalogTile(_TileBase):
    """Host-side analog tile (rpu_base_tiles.cpp ``AnalogTile``)."""


class _CudaTileMixin:
    def _init_cuda(self, tile: _TileBase):
        if not isinstance(tile, _TileBase):
            raise TypeError("expected a host tile")
        if not torch.cuda.is_available():
            raise RuntimeError("No GPU available: the analog tile kernels need a HIP device.")
        handle = tile._clone_handle()
        _TileBase.__init__(self, handle)
        tile._copy_parameters_to(self)
        check(lib().rpu_tile_to_device(self._h, torch.cuda.current_device()))
        self._device = torch.device("cuda", torch.cuda.current_device())

    @staticmethod
    def _stream_for(tensor: torch.Tensor):
        return C.c_void_p(torch.cuda.current_stream(tensor.device).cuda_stream)

    def _finish(self, tensor: torch.Tensor, non_blocking: bool):
        if not non_blocking:
            torch.cuda.current_stream(tensor.device).synchronize()

    @staticmethod
    def _out_dims(inp: torch.Tensor, in_trans: bool, out_trans: bool, m_batch: int, out_size: int):
        # The reference copies the input dims and replaces the first (transposed) or last entry
        # (rpu_base_tiles_cuda.cpp:170-189).  That is only a valid shape when both flags agree, which is
        # how its Python callers use it; with mixed flags the result is the plain 2-D matrix.
        if in_trans == out_trans:
            dims = list(inp.shape)
            dims[0 if out_trans else -1] = out_size
            return dims
        return [out_size, m_batch] if out_trans else [m_batch, out_size]

    # rpu_base_tiles_cuda.cpp:159-236
    def forward(self, x_input: torch.Tensor, bias: bool = False, x_trans: bool = False, d_trans: bool = False,
                is_test: bool = False, non_blocking: bool = False) -> torch.Tensor:
        x_input = _check_input(x_input, True, "x_input")
        if x_input.dim() < 1:
            raise RuntimeError("Invalid x_input dimensions: expected at least 1 dimensional tensor")
        in_size = x_input.size(0) if x_trans else x_input.size(-1)
        expected = self.get_x_size() - (1 if bias else 0)
        if in_size != expected:
            shape = f"[*, {expected}]" if x_trans else f"[{expected},*]"
            raise RuntimeError(f"Invalid x_input dimensions: expected {shape} tensor")
        m_batch = x_input.numel() // in_size
        d_output = torch.empty(self._out_dims(x_input, x_trans, d_trans, m_batch, self.get_d_size()),
                               dtype=x_input.dtype, device=x_input.device)
        check(lib().rpu_tile_forward(self._h, x_input.data_ptr(), d_output.data_ptr(), m_batch, int(bias),
                                     int(x_trans), int(d_trans), int(is_test), self._stream_for(x_input)))
        self._finish(x_input, non_blocking)
        return d_output

    # rpu_base_tiles_cuda.cpp:237-309
    def backward(self, d_input: torch.Tensor, bias: bool = False, d_trans: bool = False, x_trans: bool = False,
                 non_blocking: bool = False) -> torch.Tensor:
        d_input = _check_input(d_input, True, "d_input")
        if d_input.dim() < 1:
            raise RuntimeError("Invalid d_input dimensions: expected at least 1 dimensional tensor")
        in_size = d_input.size(0) if d_trans else d_input.size(-1)
        expected = self.get_d_size()
        if in_size != expected:
            shape = f"[*, {expected}]" if d_trans else f"[{expected},*]"
            raise RuntimeError(f"Invalid d_input dimensions: expected {shape} tensor")
        m_batch = d_input.numel() // in_size
        x_output = torch.empty(
            self._out_dims(d_input, d_trans, x_trans, m_batch, self.get_x_size() - (1 if bias else 0)),
            dtype=d_input.dtype, device=d_input.device)
        check(lib().rpu_tile_backward(self._h, d_input.data_ptr(), x_output.data_ptr(), m_batch, int(bias),
                                      int(d_trans), int(x_trans), self._stream_for(d_input)))
        self._finish(d_input, non_blocking)
        return x_output

    # rpu_base_tiles_cuda.cpp:310-397.  The keyword names of the 4th / 5th argument are swapped in the
    # reference (py::arg("d_trans") precedes py::arg("x_trans")); positions are what callers use.
    def update(self, x_input: torch.Tensor, d_input: torch.Tensor, bias: bool, x_trans: bool = False,
               d_trans: bool = False, non_blocking: bool = False) -> None:
        if self.get_learning_rate() == 0.0:
            return
        d_input = _check_input(d_input, True, "d_input")
        x_input = _check_input(x_input, True, "x_input")
        if x_input.dim() < 1 or d_input.dim() < 1:
            raise RuntimeError("Invalid x_input/d_input dimensions: expected at least 1 dimensional tensor")
        in_size = x_input.size(0) if x_trans else x_input.size(-1)
        expected_in = self.get_x_size() - (1 if bias else 0)
        m_batch = x_input.numel() // in_size
        out_size = d_input.size(0) if d_trans else d_input.size(-1)
        expected_out = self.get_d_size()
        m_batch_from_d = d_input.numel() // out_size
        if in_size != expected_in:
            shape = f"[*, {expected_in}]" if x_trans else f"[{expected_in}, *]"
            raise RuntimeError(f"Invalid x_input dimensions: expected {shape} tensor")
        if out_size != expected_out:
            shape = f"[*, {expected_out}]" if d_trans else f"[{expected_out}, *]"
            raise RuntimeError(f"Invalid d_input dimensions: expected {shape} tensor")
        if m_batch != m_batch_from_d:
            raise RuntimeError("Invalid x_input or d_input dimensions: batch dimensions mismatch!")
        entry = lib().rpu_tile_update_noalloc if self._update_without_allocation else lib().rpu_tile_update
        check(entry(self._h, x_input.data_ptr(), d_input.data_ptr(), m_batch, int(bias),
                    int(x_trans), int(d_trans), self._stream_for(x_input)))
        self._finish(x_input, non_blocking)

    _update_without_allocation = False

    def set_update_without_allocation(self, enable: bool) -> None:
        """Not in the reference: route `update` through the entry point that allocates nothing (scratch in a static
        device array of limited size, shared by all tiles of the GPU)."""
        self._update_without_allocation = bool(enable)

    # -- inspection hooks
    # -- indexed (convolution) interface (rpu_base_tiles.cpp:621-737)
    # -- weight maintenance between steps (rpu_base_tiles.cpp:276-404); the matrix in HBM is changed in place
    def _current_stream(self):
        return C.c_void_p(torch.cuda.current_stream(self._device).cuda_stream)

    def decay_weights(self, alpha: float = 1.0) -> None:
        check(lib().rpu_tile_decay_weights(self._h, float(alpha), 0, self._current_stream()))

    def diffuse_weights(self) -> None:
        check(lib().rpu_tile_diffuse_weights(self._h, self._current_stream()))

    def clip_weights(self, weight_clipper_params) -> None:
        par = weight_clipper_params
        check(lib().rpu_tile_clip_weights(self._h, int(par.type), float(par.fixed_value), float(par.sigma),
                                          self._current_stream()))

    def reset_columns(self, start_column_idx: int = 0, num_columns: int = 1, reset_prob: float = 1.0) -> None:
        check(lib().rpu_tile_reset_columns(self._h, int(start_column_idx), int(num_columns), float(reset_prob),
                                           self._current_stream()))

    def drift_weights(self, time_since_last_call: float) -> None:
        """Power-law drift of the weights that have not changed since the last call (rpu_base_tiles.cpp:293-313)."""
        check(lib().rpu_tile_drift_device_weights(self._h, float(time_since_last_call), self._current_stream()))

    def remap_weights(self, weight_remap_params, scales: torch.Tensor) -> torch.Tensor:
        """Rescales the rows of the weights, ``scales`` ([d_size], on the tile's GPU) takes the factors up in place
        and is returned (rpu_base_tiles.cpp:330-356)."""
        if isinstance(scales, torch.Tensor) and not scales.is_contiguous():
            raise RuntimeError("scales must be contiguous")
        scales = _check_input(scales, True, "scales")
        if scales.numel() != self.get_d_size() or scales.dim() != 1:
            raise RuntimeError("Invalid scales dimensions: expected [%d] tensor" % self.get_d_size())
        par = weight_remap_params
        c_par = RemapParams(int(par.type), int(bool(getattr(par, "clip_if", True))), float(par.max_scale_range),
                            float(par.max_scale_ref), float(getattr(par, "row_norm", 1.0)), float(par.remapped_wmax))
        check(lib().rpu_tile_remap_weights(self._h, C.byref(c_par), scales.data_ptr(), self._current_stream()))
        return scales

    def modify_weights(self, weight_modifier_params) -> None:
        """Makes the modified copy of the weights that forward and backward use from now on
        (rpu_base_tiles.cpp:357-371)."""
        par = weight_modifier_params
        coeffs = [float(c) for c in par.coeffs]
        if len(coeffs) > MAX_MODIFIER_COEFFS:
            raise RuntimeError("At most %d modifier coefficients." % MAX_MODIFIER_COEFFS)
        c_par = ModifierParams()
        c_par.type = int(par.type)
        for name in ("per_batch_sample", "sto_round", "enable_during_test", "copy_last_column", "rel_to_actual_wmax"):
            setattr(c_par, name, int(bool(getattr(par, name))))
        for name in ("std_dev", "res", "dorefa_clip", "pdrop", "assumed_wmax", "g_max"):
            setattr(c_par, name, float(getattr(par, name)))
        c_par.n_coeffs = len(coeffs)
        for k, c in enumerate(coeffs):
            c_par.coeffs[k] = c
        check(lib().rpu_tile_modify_weights(self._h, C.byref(c_par), self._current_stream()))

    def get_modified_weights(self) -> torch.Tensor:
        """[d_size, x_size] CPU tensor of the weights forward and backward contract with after ``modify_weights``."""
        out = torch.empty(self.get_d_size(), self.get_x_size(), dtype=_DTYPE)
        check(lib().rpu_tile_get_modified_weights(self._h, out.data_ptr()))
        return out

    # -- shared and delta weights as the reference's CUDA tiles bind them (rpu_base_tiles_cuda.cpp:88-130): the
    # tensors are [x_size, d_size] ("weight is d major for CUDA"), which is what the reference's Python allocates for
    # a tile whose class name contains "Cuda" and reads back through .t() (simulator/tiles/base.py:392-446)
    def _check_matrix(self, tensor: torch.Tensor, what: str) -> torch.Tensor:
        if isinstance(tensor, torch.Tensor) and not tensor.is_contiguous():
            raise RuntimeError(what + " must be contiguous")
        tensor = _check_input(tensor, True, what)
        if tensor.dim() != 2 or tensor.size(0) != self.get_x_size() or tensor.size(1) != self.get_d_size():
            raise RuntimeError("Invalid %s dimensions: expected [%d,%d] array" % (what, self.get_x_size(), self.get_d_size()))
        if tensor.device.index != self._device.index:
            raise RuntimeError("%s need to be on the same cuda device: expected %d, got %d"
                               % (what.capitalize(), self._device.index, tensor.device.index))
        return tensor

    def set_shared_weights(self, weights: torch.Tensor) -> None:
        """``weights``, a CUDA tensor ``[x_size, d_size]``, mirrors the weight matrix of the tile from now on (the
        tile's weights are copied into it; it is re-read before and re-written after every call) and must outlive it."""
        weights = self._check_matrix(weights, "weights")
        check(lib().rpu_tile_set_shared_weights_xd(self._h, weights.data_ptr()))
        self._shared_weights = weights

    def set_delta_weights(self, delta_weights: torch.Tensor) -> None:
        delta_weights = self._check_matrix(delta_weights, "delta weights")
        check(lib().rpu_tile_set_delta_weights_xd(self._h, delta_weights.data_ptr()))
        self._delta_weights = delta_weights

    def set_shared_weights_row_major(self, weights: torch.Tensor) -> None:
        """Not in the reference: the tile adopts a ``[d_size, x_size]`` CUDA tensor as its weight matrix itself (no
        copies between calls), for callers written against this library."""
        if not (isinstance(weights, torch.Tensor) and weights.is_cuda and weights.is_contiguous()
                and tuple(weights.shape) == (self.get_d_size(), self.get_x_size()) and weights.dtype == _DTYPE):
            raise RuntimeError("Invalid weights: expected a contiguous [%d,%d] CUDA tensor" % (self.get_d_size(), self.get_x_size()))
        check(lib().rpu_tile_set_shared_weights(self._h, weights.data_ptr()))
        self._shared_weights = weights

    def reset_delta_weights(self) -> None:
        check(lib().rpu_tile_set_delta_weights_xd(self._h, None))
        self._delta_weights = None

    def _patches(self) -> int:
        patches = lib().rpu_tile_has_matrix_indices(self._h)
        if patches <= 0:
            raise RuntimeError("The index matrix has not been set (set_matrix_indices).")
        return patches

    def forward_indexed(self, x_input: torch.Tensor, d_tensor: torch.Tensor, is_test: bool = False,
                        non_blocking: bool = False) -> torch.Tensor:
        """x_input: N, C, (D), H, W images; d_tensor: the output tensor N, C_out, (d_depth,) d_height, d_width."""
        x_input = _check_input(x_input, True, "x_input")
        d_tensor = _check_input(d_tensor, True, "d_tensor")
        n_images = x_input.size(0)
        patches = d_tensor.numel() // d_tensor.size(0) // d_tensor.size(1)
        if patches != self._patches() or d_tensor.size(1) != self.get_d_size() or d_tensor.size(0) != n_images:
            raise RuntimeError("Invalid d_tensor dimensions for the index matrix that is set")
        check(lib().rpu_tile_forward_indexed(self._h, x_input.data_ptr(), d_tensor.data_ptr(), n_images,
                                             x_input.numel() // n_images, int(is_test), self._stream_for(x_input)))
        self._finish(x_input, non_blocking)
        return d_tensor

    def backward_indexed(self, d_input: torch.Tensor, x_tensor: torch.Tensor, non_blocking: bool = False) -> torch.Tensor:
        d_input = _check_input(d_input, True, "d_input")
        x_tensor = _check_input(x_tensor, True, "x_tensor")
        n_images = d_input.size(0)
        patches = d_input.numel() // d_input.size(0) // d_input.size(1)
        if patches != self._patches() or d_input.size(1) != self.get_d_size() or x_tensor.size(0) != n_images:
            raise RuntimeError("Invalid d_input dimensions for the index matrix that is set")
        check(lib().rpu_tile_backward_indexed(self._h, d_input.data_ptr(), x_tensor.data_ptr(), n_images,
                                              x_tensor.numel() // n_images, self._stream_for(d_input)))
        self._finish(d_input, non_blocking)
        return x_tensor

    def update_indexed(self, x_input: torch.Tensor, d_input: torch.Tensor, non_blocking: bool = False) -> None:
        if self.get_learning_rate() == 0.0:
            return
        x_input = _check_input(x_input, True, "x_input")
        d_input = _check_input(d_input, True, "d_input")
        n_images = d_input.size(0)
        patches = d_input.numel() // d_input.size(0) // d_input.size(1)
        if patches != self._patches() or d_input.size(1) != self.get_d_size() or x_input.size(0) != n_images:
            raise RuntimeError("Invalid x_input or d_input dimensions for the index matrix that is set")
        check(lib().rpu_tile_update_indexed(self._h, x_input.data_ptr(), d_input.data_ptr(), n_images,
                                            x_input.numel() // n_images, self._stream_for(x_input)))
        self._finish(x_input, non_blocking)

    def get_update_words(self, m_batch: int):
        """Packed pulse words and per-sample BL of the last stochastic update (CPU tensors).  With bit lines beyond 31
        pulses a sample takes ``get_update_words_per_sample()`` consecutive rows of words."""
        rows = m_batch * self.get_update_words_per_sample()
        x_words = torch.empty(rows, self.get_x_size(), dtype=torch.int32)
        d_words = torch.empty(rows, self.get_d_size(), dtype=torch.int32)
        bl = torch.empty(m_batch, dtype=torch.int32)
        check(lib().rpu_tile_get_update_words(self._h, x_words.data_ptr(), d_words.data_ptr(), bl.data_ptr(), m_batch))
        return x_words, d_words, bl

    def set_fused_rounds(self, mode: int = -1) -> None:
        """Fewer launches for the bound-management rounds of the forward pass: 1 = rounds 0 and 1 in one launch, 2 = all
        rounds after round 0 in one launch, 3 = both (rounds 0 and 1, then all others), 5 / 7 = as 1 / 3 with round 2 in the
        first launch as well, 0 = one launch per round, -1 (default) = the tile decides by what its recent calls needed.  Outputs and round counts do not depend on it."""
        check(lib().rpu_tile_set_fused_rounds(self._h, int(mode)))

    def set_round_wait_test_hook(self, spin_limit: int = 0, extra_arrivals: int = 0) -> None:
        """For the test of the time-out path of the merged-round launches only: shorten their bounded waits to
        ``spin_limit`` polls and make them expect ``extra_arrivals`` workgroups more than the launch has."""
        check(lib().rpu_tile_set_round_wait_test_hook(self._h, int(spin_limit), int(extra_arrivals)))

    def get_update_words_per_sample(self) -> int:
        """Rows of pulse words per sample of the last stochastic update: ceil(longest possible BL / 31)."""
        n = C.c_int32(0)
        check(lib().rpu_tile_get_update_words_per_sample(self._h, C.byref(n)))
        return int(n.value)

    def get_update_ab(self, m_batch: int):
        """Per-sample probability scales (A for d, B for x) of the last pulsed update (CPU tensors)."""
        a = torch.empty(m_batch, dtype=torch.float32)
        b = torch.empty(m_batch, dtype=torch.float32)
        check(lib().rpu_tile_get_update_ab(self._h, a.data_ptr(), b.data_ptr(), m_batch))
        return a, b

    def update_with_words(self, x_words: torch.Tensor, d_words: torch.Tensor, non_blocking: bool = False) -> None:
        """Apply the device steps for given packed pulse words (int32 CUDA tensors [m, x_size], [m, d_size])."""
        if x_words.dtype != torch.int32 or d_words.dtype != torch.int32 or not x_words.is_cuda or not d_words.is_cuda:
            raise RuntimeError("pulse words must be int32 CUDA tensors")
        x_words, d_words = x_words.contiguous(), d_words.contiguous()
        m_batch = x_words.shape[0]
        if tuple(x_words.shape) != (m_batch, self.get_x_size()) or tuple(d_words.shape) != (m_batch, self.get_d_size()):
            raise RuntimeError("Invalid pulse word dimensions")
        check(lib().rpu_tile_update_with_words(self._h, x_words.data_ptr(), d_words.data_ptr(), m_batch,
                                               self._stream_for(x_words)))
        self._finish(x_words, non_blocking)

    def get_implicit_counts(self, m_batch: int) -> torch.Tensor:
        """Signed coincidence counts [m_batch, d_size, x_size] of the last deterministic-implicit update."""
        counts = torch.empty(m_batch, self.get_d_size(), self.get_x_size(), dtype=torch.int32)
        check(lib().rpu_tile_get_implicit_counts(self._h, counts.data_ptr(), m_batch))
        return counts

    def set_profiling(self, enable: bool) -> None:
        """Record HIP events around every kernel of the following compute calls."""
        check(lib().rpu_tile_set_profiling(self._h, int(enable)))

    def get_profile(self):
        """[(kernel name, milliseconds)] of the last compute call, in launch order."""
        count = C.c_int(0)
        buf = (C.c_float * 128)()
        check(lib().rpu_tile_get_profile(self._h, buf, 128, C.byref(count)))
        return [(lib().rpu_tile_profile_name(self._h, k).decode(), float(buf[k])) for k in range(count.value)]

    def get_bm_rounds(self, m_batch: int) -> torch.Tensor:
        """Number of bound-management rounds each sample of the last forward pass took."""
        rounds = torch.empty(m_batch, dtype=torch.int32)
        check(lib().rpu_tile_get_bm_rounds(self._h, rounds.data_ptr(), m_batch))
        return rounds


class CudaFloatingPointTile(_CudaTileMixin, _TileBase):
    """GPU floating point tile (rpu_base_tiles_cuda.cpp:45-58)."""

    def __init__(self, tile):  # pylint: disable=super-init-not-called
        if isinstance(tile, int):
            _TileBase.__init__(self, tile)
            self._device = torch.device("cuda", torch.cuda.current_device())
        else:
            self._init_cuda(tile)


class CudaAnalogTile(_CudaTileMixin, _TileBase):
    """GPU analog tile (rpu_base_tiles_cuda.cpp:524-543): built from a host tile.

    ``bind_shared_weights`` (class attribute, default off): allocate an ``[x_size, d_size]`` CUDA tensor for every new
    tile and bind it with ``set_shared_weights``, which is what the reference's Python does for every CUDA tile when a
    module is moved to the GPU (src/aihwkit/simulator/tiles/base.py:386-446).  Tiles that the library cannot bind
    (transfer compounds) stay as they are.
    """

    bind_shared_weights = False

    def __init__(self, tile):  # pylint: disable=super-init-not-called
        if isinstance(tile, int):
            _TileBase.__init__(self, tile)
            self._device = torch.device("cuda", torch.cuda.current_device())
        else:
            self._init_cuda(tile)
        if type(self).bind_shared_weights:
            shared = torch.empty(self.get_x_size(), self.get_d_size(), dtype=_DTYPE, device=self._device)
            try:
                self.set_shared_weights(shared)
            except RuntimeError as err:
                if "transfer compound" not in str(err):
                    raise


class TileGroup:
    """Forward pass of several GPU tiles in a few kernel launches.

    The reference runs the tiles of a tile array one after the other (TileModuleArray.forward,
    src/aihwkit/simulator/tiles/array.py:155-182); a group gives every tile the same result as its own
    ``forward(x, False, False, False, is_test)`` would, with one launch per kernel variant and round for all of them.
    """

    def __init__(self, tile_list):
        self._tiles = list(tile_list)
        if not self._tiles:
            raise RuntimeError("empty tile list")
        handles = (C.c_void_p * len(self._tiles))(*[t._h for t in self._tiles])
        self._g = C.c_void_p()
        check(lib().rpu_group_create(C.byref(self._g), handles, len(self._tiles)))

    def __del__(self):
        handle, self._g = getattr(self, "_g", None), None
        if handle:
            try:
                lib().rpu_group_destroy(handle)
            except Exception:  # pylint: disable=broad-except
                pass

    def set_round_wait_test_hook(self, spin_limit: int = 0, extra_arrivals: int = 0) -> None:
        """For the test of the time-out path of the group's merged-round launch only (see the tiles' method)."""
        check(lib().rpu_group_set_round_wait_test_hook(self._g, int(spin_limit), int(extra_arrivals)))

    @staticmethod
    def _rows(tensor: torch.Tensor, what: str) -> torch.Tensor:
        # dense rows or a column slice of a larger row-major matrix
        if not isinstance(tensor, torch.Tensor) or tensor.dtype != _DTYPE or not tensor.is_cuda:
            raise RuntimeError(what + " must be a float32 CUDA tensor")
        if tensor.dim() != 2 or (tensor.shape[1] > 1 and tensor.stride(1) != 1):
            raise RuntimeError(what + " must be a matrix with unit column stride")
        return tensor

    def update(self, x_inputs, d_inputs, non_blocking: bool = False) -> None:
        """Stochastic pulsed update of every tile with its own ``x_inputs[i]`` [m_batch, x_size_i] and ``d_inputs[i]``
        [m_batch, d_size_i] (column slices of larger matrices are read in place): what each tile's own ``update`` does,
        in three launches for the whole group."""
        if len(x_inputs) != len(self._tiles) or len(d_inputs) != len(self._tiles):
            raise RuntimeError("one input and one output gradient per tile expected")
        xs = [self._rows(x, "x_input") for x in x_inputs]
        ds = [self._rows(d, "d_input") for d in d_inputs]
        m_batch = xs[0].shape[0]
        for x, d, tile in zip(xs, ds, self._tiles):
            if x.shape[0] != m_batch or x.shape[1] != tile.get_x_size():
                raise RuntimeError("Invalid x_input dimensions")
            if d.shape[0] != m_batch or d.shape[1] != tile.get_d_size():
                raise RuntimeError("Invalid d_input dimensions")
        n = len(xs)
        x_ptrs = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
        d_ptrs = (C.c_void_p * n)(*[d.data_ptr() for d in ds])
        x_ld = (C.c_long * n)(*[x.stride(0) if x.shape[0] > 1 else x.shape[1] for x in xs])
        d_ld = (C.c_long * n)(*[d.stride(0) if d.shape[0] > 1 else d.shape[1] for d in ds])
        stream = torch.cuda.current_stream(xs[0].device)
        check(lib().rpu_group_update_strided(self._g, x_ptrs, x_ld, d_ptrs, d_ld, m_batch, C.c_void_p(stream.cuda_stream)))
        if not non_blocking:
            stream.synchronize()

    def get_shared_input_sets(self):
        """(sets, tiles) of the last call: sets of at least two tiles that were handed the same input and convert it the
        same way, so that its quantized rows were written once for the set, and the number of tiles in such sets."""
        n_sets, n_tiles = C.c_int(0), C.c_int(0)
        check(lib().rpu_group_get_shared_input_sets(self._g, C.byref(n_sets), C.byref(n_tiles)))
        return n_sets.value, n_tiles.value

    def backward(self, d_inputs, non_blocking: bool = False, outs=None):
        """d_inputs[i]: CUDA tensor [m_batch, d_size_i]; returns the input gradients [m_batch, x_size_i] of every tile
        (``outs``: tensors to fill, e.g. column slices), each what the tile's own ``backward`` gives."""
        if len(d_inputs) != len(self._tiles):
            raise RuntimeError("one input per tile expected")
        ds = [self._rows(d, "d_input") for d in d_inputs]
        m_batch = ds[0].shape[0]
        for d, tile in zip(ds, self._tiles):
            if d.shape[0] != m_batch or d.shape[1] != tile.get_d_size():
                raise RuntimeError("Invalid d_input dimensions")
        if outs is None:
            xs = [torch.empty(m_batch, tile.get_x_size(), dtype=_DTYPE, device=ds[0].device) for tile in self._tiles]
        else:
            if len(outs) != len(self._tiles):
                raise RuntimeError("one output per tile expected")
            xs = [self._rows(x, "output") for x in outs]
            for x, tile in zip(xs, self._tiles):
                if x.shape[0] != m_batch or x.shape[1] != tile.get_x_size():
                    raise RuntimeError("Invalid output dimensions")
        n = len(ds)
        d_ptrs = (C.c_void_p * n)(*[d.data_ptr() for d in ds])
        x_ptrs = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
        d_ld = (C.c_long * n)(*[d.stride(0) if d.shape[0] > 1 else d.shape[1] for d in ds])
        x_ld = (C.c_long * n)(*[x.stride(0) if x.shape[0] > 1 else x.shape[1] for x in xs])
        stream = torch.cuda.current_stream(ds[0].device)
        check(lib().rpu_group_backward_strided(self._g, d_ptrs, d_ld, x_ptrs, x_ld, m_batch, C.c_void_p(stream.cuda_stream)))
        if not non_blocking:
            stream.synchronize()
        return xs

    def forward(self, x_inputs, is_test: bool = False, non_blocking: bool = False, outs=None):
        """x_inputs[i]: CUDA tensor [m_batch, x_size_i] (column slices of one matrix are read in place); returns the
        list of outputs [m_batch, d_size_i].  ``outs`` may give the output tensors, e.g. column slices of one
        [m_batch, out_total] matrix, which the tiles then fill in place."""
        if len(x_inputs) != len(self._tiles):
            raise RuntimeError("one input per tile expected")
        xs = [self._rows(x, "x_input") for x in x_inputs]
        m_batch = xs[0].shape[0]
        for x, tile in zip(xs, self._tiles):
            if x.shape[0] != m_batch or x.shape[1] != tile.get_x_size():
                raise RuntimeError("Invalid x_input dimensions")
        if outs is None:
            ys = [torch.empty(m_batch, tile.get_d_size(), dtype=_DTYPE, device=xs[0].device) for tile in self._tiles]
        else:
            if len(outs) != len(self._tiles):
                raise RuntimeError("one output per tile expected")
            ys = [self._rows(y, "output") for y in outs]
            for y, tile in zip(ys, self._tiles):
                if y.shape[0] != m_batch or y.shape[1] != tile.get_d_size():
                    raise RuntimeError("Invalid output dimensions")
        n = len(xs)
        x_ptrs = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
        y_ptrs = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
        x_ld = (C.c_long * n)(*[x.stride(0) if x.shape[0] > 1 else x.shape[1] for x in xs])
        y_ld = (C.c_long * n)(*[y.stride(0) if y.shape[0] > 1 else y.shape[1] for y in ys])
        stream = torch.cuda.current_stream(xs[0].device)
        check(lib().rpu_group_forward_strided(self._g, x_ptrs, x_ld, y_ptrs, y_ld, m_batch, int(is_test),
                                              C.c_void_p(stream.cuda_stream)))
        if not non_blocking:
            stream.synchronize()
        return ys
