"""TEST INFRASTRUCTURE -- numpy restatement of the reference's hardware-aware-training helpers of a tile: weight
remapping, the weight modifier (forward / backward weights), device-level power-law drift and the pulse counters.
The shipped package never imports it.

Arrays are float32 [d_size, x_size]; every operation is rounded to float32 in the order of the reference's loops.
Random draws are arguments (standard normals / uniforms in [0, 1)), so a test can feed known values.
"""
import numpy as np

F = np.float32

# WeightRemapType (src/rpucuda/weight_remapper.h:14-22)
REMAP_NONE, REMAP_LAYERWISE_SYMMETRIC, REMAP_CHANNELWISE_SYMMETRIC, REMAP_CHANNELWISE_NORM = 0, 1, 2, 3
# WeightModifierType (src/rpucuda/weight_modifier.h:14-25)
(MOD_COPY, MOD_DISCRETIZE, MOD_MULT_NORMAL, MOD_ADD_NORMAL, MOD_DISCRETIZE_ADD_NORMAL, MOD_DOREFA, MOD_POLY,
 MOD_PCM_NOISE, MOD_DROP_CONNECT, MOD_PROG_NOISE) = range(10)


def remap(w, scales, kind, remapped_wmax=1.0, max_scale_range=0.0, max_scale_ref=0.0, row_norm=1.0, clip_if=True):
    """WeightRemapper::apply (src/rpucuda/weight_remapper.cpp:19-190).  Returns (weights, scales)."""
    w = w.astype(F).copy()
    scales = scales.astype(F).copy()
    if kind == REMAP_NONE:
        return w, scales
    if kind == REMAP_LAYERWISE_SYMMETRIC:                       # :24-48
        amax = F(np.abs(w).max()) / F(remapped_wmax)
        if amax > 0:
            scales = (scales * amax).astype(F)
            w = (w / amax).astype(F)
        return w, scales
    if kind == REMAP_CHANNELWISE_SYMMETRIC:                     # :49-135
        row_max = np.abs(w).max(axis=1).astype(F)
        if max_scale_range <= 0:
            if remapped_wmax != 1.0:
                row_max = (row_max / F(remapped_wmax)).astype(F)
            f = np.where(row_max > 0, row_max, F(1.0)).astype(F)
            return (w / f[:, None]).astype(F), (scales * f).astype(F)
        assert remapped_wmax == 1.0
        old = scales.copy()
        min_scale = max(F(old.min()), F(0.0))
        if min_scale > 0 and max_scale_ref:
            min_scale = max(min_scale, F(max_scale_ref))
        new = np.where(row_max > 0, (row_max * old).astype(F), old).astype(F)
        if min_scale > 0:
            ratio = (new / F(min_scale)).astype(F)
            new = np.where(ratio > F(max_scale_range), F(min_scale) * F(max_scale_range), new).astype(F)
        w = ((w * old[:, None]).astype(F) / new[:, None]).astype(F)
        return w, new
    if kind == REMAP_CHANNELWISE_NORM:                          # :137-178
        nm = np.sqrt((w.astype(np.float64) ** 2).sum(axis=1)).astype(F)
        nm = np.where(nm > 0, nm, F(1.0)).astype(F)
        nm = (nm / F(row_norm)).astype(F)
        nm = np.where(nm > 1, nm, F(1.0)).astype(F)
        if not clip_if:
            scales = (scales * nm).astype(F)
        return (w / nm[:, None]).astype(F), scales
    raise ValueError("Remapping type not implemented.")


def _round_half_away(v):
    """roundf of the C library."""
    return (np.sign(v) * np.floor(np.abs(v) + F(0.5))).astype(F)


def _discretize(v, res, sto_round, uniforms):
    """getDiscretizedValueRound (src/rpucuda/utility_functions.h:195-202)."""
    if res <= 0:
        return v
    q = (v / F(res)).astype(F)
    if sto_round:
        q = (q + (uniforms.astype(F) - F(0.5))).astype(F)
    return (_round_half_away(q) * F(res)).astype(F)


def modify(w, kind, normals=None, uniforms=None, drop_uniforms=None, std_dev=0.0, res=0.1, sto_round=False,
           dorefa_clip=0.6, pdrop=0.0, copy_last_column=False, rel_to_actual_wmax=True, assumed_wmax=1.0, g_max=25.0,
           coeffs=(0.26348 / 25.0, 0.0768, -0.001877 * 25.0)):
    """WeightModifier::apply (src/rpucuda/weight_modifier.cpp:28-224): the modified copy of w."""
    w = w.astype(F)
    out = w.copy()
    amax = F(assumed_wmax)
    if rel_to_actual_wmax and kind != MOD_COPY:                 # :50-62
        body = w[:, :-1] if copy_last_column else w
        amax = F(np.abs(body).max())
        amax = amax if amax > 0 else F(1.0)
    z = None if normals is None else normals.astype(F)
    if kind == MOD_DISCRETIZE:                                  # :73-84
        if res > 0:
            out = (amax * _discretize((out / amax).astype(F), res, sto_round, uniforms)).astype(F)
    elif kind == MOD_MULT_NORMAL:                               # :85-96
        if std_dev > 0:
            std = F(std_dev) * amax
            out = (out + ((out * std).astype(F) * z).astype(F)).astype(F)
    elif kind == MOD_ADD_NORMAL:                                # :97-107
        if std_dev > 0:
            out = (out + (F(std_dev) * amax * z).astype(F)).astype(F)
    elif kind in (MOD_POLY, MOD_PROG_NOISE):                    # :108-152
        if std_dev > 0 and len(coeffs) > 0:
            std = F(std_dev) if kind == MOD_POLY else F(std_dev) / F(g_max)
            aw = (np.abs(out) / amax).astype(F)
            paw = np.ones_like(aw)
            sig = np.full_like(aw, F(coeffs[0]))
            for c in coeffs[1:]:
                paw = (paw * aw).astype(F)
                sig = (sig + (F(c) * paw).astype(F)).astype(F)
            sig = (sig * std).astype(F)
            noisy = (out + ((amax * sig).astype(F) * z).astype(F)).astype(F)
            out = noisy if kind == MOD_POLY else np.where(out < 0, -np.abs(noisy), np.abs(noisy)).astype(F)
    elif kind == MOD_DOREFA:                                    # :153-166
        if res > 0:
            scale = F(abs(F(dorefa_clip) / F(np.tanh(np.float32(amax)))))
            out = _discretize((np.tanh(out).astype(F) * scale).astype(F), res, sto_round, uniforms)
    elif kind == MOD_DISCRETIZE_ADD_NORMAL:                     # :167-182
        std = F(std_dev) * amax
        if res > 0 or std > 0:
            out = (amax * _discretize((out / amax).astype(F), res, sto_round, uniforms)).astype(F)
            out = (out + (std * z).astype(F)).astype(F)
    elif kind not in (MOD_COPY, MOD_DROP_CONNECT):
        raise ValueError("Requested WeightModifierType not implemented in CPU version.")
    if pdrop > 0:                                               # :18-26, 193-195
        out = np.where(drop_uniforms < F(pdrop), F(0.0), out).astype(F)
    if copy_last_column:                                        # :42-48, 197-201
        out[:, -1] = w[:, -1]
    return out


class Drifter:
    """WeightDrifter (src/rpucuda/weight_drifter.cpp:41-150) with the saturation of a pulsed device
    (weight_drifter.cpp:98-106, rpu_pulsed_device.cpp:422-430)."""

    def __init__(self, nu, nu_std=0.0, wg_ratio=1.0, g_offset=0.0, w_offset=0.0, nu_k=0.0, log_g0=0.0, t0=1.0,
                 reset_tol=1e-7, w_read_std=0.0):
        self.nu = nu                       # scalar (simple drift) or an array per weight
        self.nu_std, self.wg_ratio, self.g_offset, self.w_offset = F(nu_std), F(wg_ratio), F(g_offset), F(w_offset)
        self.nu_k, self.log_g0, self.t0, self.reset_tol, self.w_read_std = F(nu_k), F(log_g0), F(t0), F(reset_tol), F(w_read_std)
        self.prev = self.w0 = self.t = None
        self.current_t = F(0.0)

    def apply(self, w, time_since_last_call, nu_normals=None, read_normals=None, w_min=None, w_max=None):
        w = w.astype(F).copy()
        if self.prev is None:                                   # initialize, :41-55
            self.prev, self.w0, self.t = w.copy(), w.copy(), np.zeros_like(w)
            self.current_t = F(0.0)
        self.current_t = F(self.current_t + F(time_since_last_call) / self.t0)
        a = F(self.g_offset * self.wg_ratio + self.w_offset)
        if abs(a) < self.reset_tol:
            a = F(0.0)
        changed = np.abs(self.prev - w) > self.reset_tol
        self.t = np.where(changed, self.current_t, self.t).astype(F)
        self.w0 = np.where(changed, w, self.w0).astype(F)
        nu = np.broadcast_to(np.asarray(self.nu, dtype=F), w.shape).astype(F)
        if self.nu_std > 0:
            nu = (nu + ((self.nu_std * nu).astype(F) * nu_normals.astype(F)).astype(F)).astype(F)
        if self.nu_k != 0:
            with np.errstate(invalid="ignore", divide="ignore"):
                g = ((w - self.w_offset) / self.wg_ratio + self.g_offset).astype(F)
                nu = (nu - self.nu_k * np.log(g).astype(F) + self.nu_k * self.log_g0).astype(F)
        delta_t = np.maximum(self.current_t - self.t, F(1.0)).astype(F)
        nu_scale = np.power(delta_t.astype(np.float64), -nu.astype(np.float64)).astype(F)
        drifted = (self.w0 * nu_scale).astype(F)
        if a != 0:
            drifted = (drifted + a * (nu_scale - F(1.0))).astype(F)
        out = np.where(changed, w, drifted).astype(F)
        if self.w_read_std > 0:
            out = (out + self.w_read_std * read_normals.astype(F)).astype(F)
        if w_min is not None:                                   # saturate, :98-106: MIN(MAX(min, w), max)
            out = np.minimum(np.maximum(out, w_min), w_max)
        self.prev = out.copy()
        return out


def pulse_counts(x_words, d_words):
    """kernelPulseCounter (src/rpucuda/cuda/pwu_kernel.h:1523-1627, getNfromCount :84-113) on packed pulse words
    (bit 0 = sign, bits 1.. = pulses): per cross-point the coincidences of the batch, [2, d_size, x_size] with the
    coincidences of equal sign first."""
    x_words = np.asarray(x_words, dtype=np.uint32)   # [B, X]
    d_words = np.asarray(d_words, dtype=np.uint32)   # [B, D]
    out = np.zeros((2, d_words.shape[1], x_words.shape[1]), dtype=np.int64)
    for xw, dw in zip(x_words, d_words):
        both = (dw[:, None] & xw[None, :]) & np.uint32(0xFFFFFFFE)
        n = np.zeros(both.shape, dtype=np.int64)
        for bit in range(1, 32):
            n += (both >> np.uint32(bit)) & np.uint32(1)
        negative = ((dw[:, None] ^ xw[None, :]) & np.uint32(1)).astype(bool)
        out[0] += np.where(negative, 0, n)
        out[1] += np.where(negative, n, 0)
    return out
