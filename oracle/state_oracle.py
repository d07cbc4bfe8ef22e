"""TEST INFRASTRUCTURE -- numpy restatement of the reference's weight maintenance between training steps (decay,
diffusion, clipping, column reset, delta weights).  The shipped package never imports it.

Every function works on float32 arrays shaped [d_size, x_size] and cites the reference lines it follows.
"""
import numpy as np

F = np.float32


def _bounds(w, w_min, w_max):
    w = np.minimum(w, w_max)
    return np.maximum(w, w_min)


def decay_device(w, decay_scale, reset_bias, w_min, w_max, alpha=1.0, bias_no_decay=False):
    """PulsedRPUDevice::decayWeights (src/rpucuda/rpu_pulsed_device.cpp:392-420)."""
    s = (F(1.0) + F(alpha) * (decay_scale - F(1.0))).astype(F)
    if bias_no_decay:
        s = s.copy()
        s[:, -1] = 1.0
    out = ((w - reset_bias) * s + reset_bias).astype(F)
    return _bounds(out, w_min, w_max)


def decay_simple(w, lifetime, alpha=1.0, bias_no_decay=False):
    """SimpleRPUDevice::decayWeights (src/rpucuda/rpu_simple_device.cpp:96-115)."""
    rate = F(1.0) / F(lifetime) if lifetime > 1.0 else F(0.0)
    scale = F(1.0) - F(alpha) * rate
    out = w.astype(F).copy()
    if 0.0 < scale < 1.0:
        if bias_no_decay:
            out[:, :-1] *= scale
        else:
            out *= scale
    return out


def diffuse(w, rates, normals, w_min=None, w_max=None):
    """rpu_pulsed_device.cpp:432-446 (with bounds), rpu_simple_device.cpp:124-134 (a scalar rate, no bounds)."""
    out = (w + F(1.0) * rates * normals).astype(F)
    return out if w_min is None else _bounds(out, w_min, w_max)


def clip_fixed(w, clip, w_min=None, w_max=None):
    """rpu_pulsed_device.cpp:448-467 with bounds (clip < 0: bounds only); rpu.cpp:1589-1599 without."""
    out = w.astype(F).copy()
    if w_min is None:
        return np.clip(out, -F(clip), F(clip)) if clip >= 0 else out
    if clip < 0:
        return _bounds(out, w_min, w_max)
    out = np.minimum(out, np.minimum(w_max, F(clip)))
    return np.maximum(out, np.maximum(w_min, -F(clip)))


def clip_value_layer_gaussian(w, sigma, fixed_value=-1.0):
    """WeightClipType::LayerGaussian (src/rpucuda/weight_clipper.cpp:68-93)."""
    flat = w.astype(np.float64).reshape(-1)
    mean = flat.sum() / flat.size
    std = np.sqrt(((flat - mean) ** 2 / (flat.size - 1)).sum())
    clip = std * sigma
    return min(clip, fixed_value) if fixed_value > 0 else clip


def clip_value_average_channel_max(w, fixed_value=-1.0):
    """WeightClipType::AverageChannelMax (weight_clipper.cpp:38-66)."""
    amax = np.zeros(w.shape[0], F)
    for i in range(w.shape[0]):
        for v in w[i]:
            amax[i] = max(amax[i], abs(v))
    clip = abs(float(amax.astype(np.float64).sum()) / w.shape[0])
    return min(clip, fixed_value) if fixed_value > 0 else clip


def clip_with_value(w, clip):
    """WeightClipper::apply tail (weight_clipper.cpp:101-104)."""
    return np.clip(w, -F(clip), F(clip)).astype(F) if clip > 0 else w.astype(F).copy()


def reset_column_mask(x_size, start_col, n_cols):
    """Columns hit by resetCols (rpu_pulsed_device.cpp:476-481), the condition as written there."""
    n = n_cols if n_cols >= 0 else x_size
    mask = np.zeros(x_size, bool)
    for j in range(x_size):
        if (start_col + n <= x_size and start_col <= j < start_col + n) or \
                (start_col + n > x_size and (j >= start_col or j < n - (x_size - start_col))):
            mask[j] = True
    return mask


def reset_cols(w, reset_bias, w_min, w_max, reset_std, start_col, n_cols, normals, lottery=None, reset_prob=1.0):
    """resetCols (rpu_pulsed_device.cpp:469-494); reset_bias / bounds None: rpu_simple_device.cpp:148-168."""
    out = w.astype(F).copy()
    cols = reset_column_mask(w.shape[1], start_col, n_cols)
    hit = np.broadcast_to(cols[None, :], w.shape).copy()
    if reset_prob < 1.0:
        hit &= lottery < reset_prob
    value = (0.0 if reset_bias is None else reset_bias) + (F(reset_std) * normals if reset_std > 0 else 0.0)
    value = np.broadcast_to(value, w.shape).astype(F)
    if w_min is not None:
        value = _bounds(value, w_min, w_max)
    out[hit] = value[hit]
    return out


def get_and_reset_weight_update(w_new, w_old, scale):
    """RPUSimple::getAndResetWeightUpdate (src/rpucuda/rpu.cpp:1432-1442): returns (restored weights, delta)."""
    return w_old.copy(), (F(scale) * (w_new - w_old)).astype(F)
