"""TEST INFRASTRUCTURE -- numpy restatement (float32) of the reference's PCM noise model and conductance
converter, used as checker for the GPU inference weight pipeline.  The shipped package never imports it.

Follows src/aihwkit/inference/noise/pcm.py:100-158 (programming noise, drift coefficients, drift + accumulated
read noise), src/aihwkit/inference/converter/conductance.py:51-82 (single pair of conductances) and
src/aihwkit/inference/noise/base.py:82-131 (how the two are combined); normals come from a numpy generator.
"""
import numpy as np

F = np.float32
ZERO_CLIP = F(1e-7)


class PcmOracle:
    def __init__(self, g_max=25.0, g_min=0.0, t_read=250.0e-9, t_0=20.0, prog_noise_scale=1.0, read_noise_scale=1.0,
                 drift_scale=1.0, prog_coeff=(0.26348, 1.9650, -1.1731), prog_coeff_g_max_reference=25.0, seed=0):
        self.g_max, self.g_min, self.t_read, self.t_0 = F(g_max), F(g_min), float(t_read), float(t_0)
        self.prog_noise_scale, self.read_noise_scale, self.drift_scale = F(prog_noise_scale), F(read_noise_scale), F(drift_scale)
        self.prog_coeff = [F(c) for c in prog_coeff]
        self.ref = F(prog_coeff_g_max_reference)
        self.rng = np.random.default_rng(seed)

    def _randn(self, like):
        return self.rng.standard_normal(like.shape).astype(F)

    # conductance.py:51-63
    def to_conductances(self, w):
        w = np.asarray(w, F)
        ratio = F((self.g_max - self.g_min) / max(F(np.abs(w).max()), ZERO_CLIP))
        sw = w * ratio
        return [np.clip(sw, 0, self.g_max) + self.g_min, np.clip(-sw, 0, self.g_max) + self.g_min], ratio

    # conductance.py:65-82
    def to_weights(self, conductances, ratio):
        return (((conductances[0] - self.g_min) - (conductances[1] - self.g_min)) / ratio).astype(F)

    # pcm.py:100-117
    def program_conductance(self, g):
        mat = F(1)
        sig = self.prog_coeff[0]
        for c in self.prog_coeff[1:]:
            mat = mat * (g / self.g_max)
            sig = sig + mat * c
        sig = sig * (self.g_max / self.ref)
        return np.maximum(g + self.prog_noise_scale * sig * self._randn(g), F(0)).astype(F)

    # pcm.py:119-131
    def drift_coefficients(self, g):
        rel = np.maximum(np.abs(g / self.g_max), ZERO_CLIP)
        mu = np.clip(F(-0.0155) * np.log(rel) + F(0.0244), F(0.049), F(0.1))
        sd = np.clip(F(-0.0125) * np.log(rel) - F(0.0059), F(0.008), F(0.045))
        return (np.maximum(np.abs(mu + sd * self._randn(g)), F(0)) * self.drift_scale).astype(F)

    # pcm.py:133-158
    def drift_conductance(self, g, nu, t_inference):
        t = t_inference + self.t_0
        g_drift = g * (F(t / self.t_0) ** (-nu)) if t > self.t_0 else g
        if t > 0:
            q = np.minimum(F(0.0088) / np.maximum((np.abs(g) / self.g_max) ** F(0.65), F(1e-3)), F(0.2))
            sig = q * F(np.sqrt(np.log((t + self.t_read) / (2 * self.t_read))))
            g_final = g_drift + np.abs(g_drift) * self.read_noise_scale * sig * self._randn(g)
        else:
            g_final = g
        return np.maximum(g_final, F(0)).astype(F)

    # base.py:82-103
    def apply_programming_noise(self, w):
        conductances, ratio = self.to_conductances(w)
        noisy = [self.program_conductance(g) for g in conductances]
        nu = [self.drift_coefficients(g) for g in conductances]
        return self.to_weights(noisy, ratio), nu

    # base.py:105-131
    def apply_drift_noise(self, w_prog, nu, t_inference):
        conductances, ratio = self.to_conductances(w_prog)
        noisy = [self.drift_conductance(g, n, t_inference) for g, n in zip(conductances, nu)]
        return self.to_weights(noisy, ratio)
