"""TEST INFRASTRUCTURE -- CPU restatement of the reference's transfer compound (Tiki-Taka) over the
oracle tile primitives of rpu_oracle.cpp.  The shipped package never imports it.

Follows src/rpucuda/rpu_transfer_device.cpp and rpu_vector_device.cpp of the reference, vector by vector as
its CPU path does (RPUPulsed::updateVector -> PulsedRPUWeightUpdater::updateVectorWithDevice ->
TransferRPUDevice::doSparseUpdate / finishUpdateCycle):

* one OracleTile per device of the chain holds that device's weights and arrays; device 0 is updated with the
  tile's update parameters, the others with transfer_up; all are read with transfer_io (noise and bound
  management off, rpu_transfer_device.cpp:198-213);
* after every update vector the counter advances and each device j whose period divides it transfers:
  the next n_reads_per_transfer unit vectors are forwarded through device j (scaled by -1) and written onto
  device j + 1 with learning rate transfer_lr (x current lr) (rpu_transfer_device.cpp:428-516,536-557);
* tile weights = sum_k gamma_k w_k, or the last device alone when gamma = 0 (rpu_transfer_device.cpp:596-602);
* random_selection: the first column of a transfer is floor(u * in_size) for a uniform u (rpu_transfer_device.cpp:486-488);
  with_reset_prob: with that probability per transfer the columns just read are reset on the source device, after all
  of them were read and written -- the order of the reference's GPU code (cuda/rpucuda_transfer_device.cu:320-324;
  its CPU code draws per vector inside the loop, rpu_transfer_device.cpp:464-470), because the tile under test
  stands in for that one.  Both uniforms come from callbacks (`select`, `reset_lottery`), so that a test feeds the
  draws of the tile under test.

This oracle samples nothing itself: tests copy the device arrays from the library through the hidden-parameter
interface, and the library's draw order for a chain (one generator walked device by device,
rpu_vector_device.cpp:398-418) is pinned against the raw libstdc++ stream in tests/test_draw_order_pins.py.
"""
import copy
import math

import numpy as np

from aihwkit_amd._cabi import TileConfig
from oracle_lib import OracleTile


class TransferOracle:
    def __init__(self, x_size, d_size, config: TileConfig, transfer):
        """config: f_io / b_io / up of the tile; transfer: aihwkit_amd._cabi.TransferParams."""
        self.X, self.D = x_size, d_size
        self.tp = transfer
        n = transfer.n_devices
        self.n = n
        self.cols = bool(transfer.transfer_columns)
        self.in_size = x_size if self.cols else d_size
        self.out_size = d_size if self.cols else x_size
        # rpu_transfer_device.cpp:146-196
        if transfer.n_gamma_vec:
            self.gamma_vec = [np.float32(transfer.gamma_vec[k]) for k in range(n)]
            gamma = float(sum(self.gamma_vec[:-1]))
        else:
            gamma = float(transfer.gamma)
            self.gamma_vec = [np.float32(0)] * n
            for i in range(n):
                self.gamma_vec[n - i - 1] = np.float32(np.float32(gamma) ** np.float32(i)) if i else np.float32(1.0)
        self.lr_vec = ([float(transfer.transfer_lr_vec[k]) for k in range(n)] if transfer.n_transfer_lr_vec
                       else [float(transfer.transfer_lr)] * n)
        self.n_reads = min(int(transfer.n_reads_per_transfer), self.in_size)
        if transfer.n_transfer_every_vec:
            self.every_vec = [np.float32(transfer.transfer_every_vec[k]) for k in range(n)]
        else:
            self.every_vec = []
            every = np.float32(transfer.transfer_every)
            for _ in range(n):
                self.every_vec.append(every)
                every = np.float32(every * (np.float32(self.out_size) / np.float32(self.n_reads)))
            if transfer.no_self_transfer:
                self.every_vec[-1] = np.float32(0)
        self.fully_hidden = (gamma == 0.0) and (float(self.gamma_vec[-1]) == 1.0)

        io = copy.copy(transfer.transfer_io)
        io.noise_management = 0
        io.bound_management = 0
        self.devices = []
        for k in range(n):
            cfg = TileConfig()
            cfg.f_io = io
            cfg.b_io = io
            cfg.up = config.up if k == 0 else transfer.transfer_up
            cfg.device = transfer.fast_device if k == 0 else transfer.rest_device
            self.devices.append(OracleTile(x_size, d_size, cfg))
        # rpu_vector_device.cpp:411-421: the compound's granularity is the average over its devices
        dw = [float(transfer.fast_device.dw_min)] + [float(transfer.rest_device.dw_min)] * (n - 1)
        self.devices[0].set_weight_granularity(np.float32(sum(np.float32(v) for v in dw) / np.float32(n)))
        # the visible tile: forward / backward with the tile's own IO on the reduced weights
        vis = TileConfig()
        vis.f_io, vis.b_io, vis.up = config.f_io, config.b_io, config.up
        vis.device = transfer.rest_device
        self.visible = OracleTile(x_size, d_size, vis)
        self._wide_open(self.visible)
        self.lr = 0.0
        self.update_idx = 0
        self.slice_idx = [0] * n
        self.select = None         # (update_idx, from) -> uniform in [0, 1) for random_selection
        self.reset_lottery = None  # (update_idx, from) -> uniform in [0, 1) for with_reset_prob
        self.set_weights(np.zeros((d_size, x_size), np.float32))

    @staticmethod
    def _wide_open(tile):
        hidden = tile.get_hidden()
        hidden[0] = np.float32(3.0e38)
        hidden[1] = np.float32(-3.0e38)
        tile.set_hidden(hidden)

    def set_seed(self, seed):
        for k, dev in enumerate(self.devices):
            dev.set_seed(seed + 17 * k)
        self.visible.set_seed(seed + 1000)

    def set_learning_rate(self, lr):
        self.lr = float(lr)

    def set_device_hidden(self, k, arrays):
        """Per-device arrays [n, D, X] in the single-device order; the weights are re-clipped by set_hidden."""
        self.devices[k].set_hidden(arrays)

    def device_weights(self, k):
        return self.devices[k].get_weights()

    def set_device_weights(self, k, w):
        self.devices[k].set_weights(w)
        self._reduce()

    # rpu_transfer_device.cpp:559-594
    def set_weights(self, w):
        w = np.asarray(w, np.float32)
        zero = np.zeros_like(w)
        for dev in self.devices[:-1]:
            dev.set_weights(zero)
        last = w if self.fully_hidden else (w / self.gamma_vec[-1]).astype(np.float32)
        self.devices[-1].set_weights(last)  # clipped into the device bounds
        self.update_idx = 0
        self.slice_idx = [0] * self.n
        self._reduce()

    def _reduce(self):
        if self.fully_hidden:
            w = self.devices[-1].get_weights()
        else:
            w = np.zeros((self.D, self.X), np.float32)
            for g, dev in zip(self.gamma_vec, self.devices):
                w = (w + g * dev.get_weights()).astype(np.float32)
        self.visible.set_weights(w)

    def get_weights(self):
        return self.visible.get_weights()

    def forward(self, x, **kw):
        return self.visible.forward(x, **kw)

    def backward(self, d, **kw):
        return self.visible.backward(d, **kw)

    # rpu_transfer_device.cpp:394-403
    def _every(self, j, m_batch):
        if self.tp.units_in_mbatch:
            return max(int(math.ceil(float(np.float32(self.every_vec[j] * np.float32(m_batch))))), 0)
        return max(int(math.floor(float(self.every_vec[j]) + 0.5)), 0)  # roundf of a non-negative value

    def _transfer(self, to, frm, m_batch):
        start = self.slice_idx[frm]
        if self.tp.random_selection:  # rpu_transfer_device.cpp:486-488
            u = np.float32(self.select(self.update_idx, frm))
            start = max(min(int(math.floor(float(np.float32(u * np.float32(self.in_size))))), self.in_size - 1), 0)
        self.slice_idx[frm] = (start + self.n_reads) % self.in_size
        lr = self.lr_vec[frm] * self.lr if self.tp.scale_transfer_lr else self.lr_vec[frm]
        lr = float(np.float32(lr))
        src, dst = self.devices[frm], self.devices[to]
        if lr != 0.0 and to != frm:
            for v in range(self.n_reads):
                unit = np.zeros((1, self.in_size), np.float32)
                unit[0, (start + v) % self.in_size] = 1.0
                dst.set_learning_rate(lr)
                if self.cols:
                    read = (-src.forward(unit)).astype(np.float32)
                    dst.update(unit, read)
                else:
                    read = (-src.backward(unit)).astype(np.float32)
                    dst.update(read, unit)
        # cuda/rpucuda_transfer_device.cu:320-324 (every element of the columns: device-wise probability 1)
        if self.cols and self.tp.with_reset_prob > 0.0 and \
                np.float32(self.reset_lottery(self.update_idx, frm)) < np.float32(self.tp.with_reset_prob):
            from state_oracle import reset_cols
            if float(self.tp.fast_device.reset_std if frm == 0 else self.tp.rest_device.reset_std) > 0.0:
                raise NotImplementedError("the transfer oracle resets without noise (reset_std = 0)")
            hidden = src.get_hidden()
            w = reset_cols(src.get_weights(), hidden[6], hidden[1], hidden[0], 0.0, start, self.n_reads, None)
            src.set_weights(w)

    def update(self, x, d):
        """Row-major batches x [B, X], d [B, D]."""
        x = np.asarray(x, np.float32)
        d = np.asarray(d, np.float32)
        if self.lr == 0.0:
            return
        m_batch = x.shape[0]
        tp = self.tp
        fast = self.lr
        if tp.fast_lr > 0.0:
            fast = float(np.float32(np.float32(tp.fast_lr) * np.float32(self.lr))) if tp.scale_fast_lr else float(tp.fast_lr)
        self.devices[0].set_learning_rate(fast)
        every = [self._every(j, m_batch) for j in range(self.n)]
        for b in range(m_batch):
            self.devices[0].update(x[b:b + 1], d[b:b + 1])
            self.update_idx += 1
            for j in range(self.n):
                if every[j] > 0 and self.update_idx % every[j] == 0:
                    self._transfer(min(j + 1, self.n - 1), j, m_batch)
        self._reduce()
