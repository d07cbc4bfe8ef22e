"""TEST INFRASTRUCTURE -- numpy restatement of the reference's indexed (convolution) interface around an oracle
tile.  The shipped package never imports it.

Follows RPUSimple::forwardIndexed / backwardIndexed / updateIndexed with trans = true (src/rpucuda/rpu.cpp:1117-1239),
copyIndexedInput / copyIndexedOutput (rpu.cpp:1017-1115) and permute132 (math_util.cpp:319-346), which is how the
bindings call them (src/aihwkit/simulator/rpu_base_src/rpu_base_tiles.cpp:621-720: m_batch = patches per image,
dim3 = number of images).
"""
import numpy as np


def copy_indexed_input(images, indices, x_size, patches):
    """images [N, image_size] -> x_tensor in the transposed layout [x_size, N * patches] (rpu.cpp:1072-1083)."""
    n_images, image_size = images.shape
    m, dim3 = patches, n_images
    big_l, big_m = m * dim3, m * x_size
    flat = images.reshape(-1)
    out = np.zeros(x_size * m * dim3, np.float32)
    for idx in range(out.size):
        i = (idx % big_l) // m * big_m + (idx % m) + idx // big_l * m
        j = indices[i % big_m]
        out[idx] = np.float32(j) if j <= 1 else flat[(j - 2) + i // big_m * image_size]
    return out.reshape(x_size, big_l)


def copy_indexed_output(x_tensor, indices, x_size, patches, n_images, image_size):
    """x_tensor [x_size, N * patches] -> images [N, image_size], overlapping patches add up (rpu.cpp:1130-1141)."""
    m, dim3 = patches, n_images
    big_l, big_m = m * dim3, m * x_size
    src = x_tensor.reshape(-1)
    out = np.zeros(n_images * image_size, np.float32)
    for idx in range(src.size):
        i = (idx % big_l) // m * big_m + (idx % m) + idx // big_l * m
        j = indices[i % big_m]
        if j > 1:
            out[(j - 2) + i // big_m * image_size] += src[idx]
    return out.reshape(n_images, image_size)


def permute132(x_in, d1, d2, d3):
    """math_util.cpp:319-346 without bias: in [d3][d2][d1] -> out [d2][d3][d1]."""
    return np.ascontiguousarray(x_in.reshape(d3, d2, d1).transpose(1, 0, 2))


class IndexedOracle:
    def __init__(self, tile, indices, patches):
        self.tile, self.indices, self.patches = tile, np.asarray(indices, np.int64).reshape(-1), patches

    def forward(self, images):
        """images [N, ...] -> [N, d_size, patches]"""
        n = images.shape[0]
        flat = np.ascontiguousarray(images, np.float32).reshape(n, -1)
        x_t = copy_indexed_input(flat, self.indices, self.tile.X, self.patches)          # [X, N P]
        d_t = self.tile.forward(x_t, x_trans=True, d_trans=True)                          # [D, N P]
        return permute132(np.ascontiguousarray(d_t), self.patches, n, self.tile.D)      # [N, D, P]

    def backward(self, d_images, image_size):
        n = d_images.shape[0]
        d_in = np.ascontiguousarray(d_images, np.float32).reshape(n, self.tile.D, self.patches)
        d_t = permute132(d_in, self.patches, self.tile.D, n)                             # [D, N, P]
        x_t = self.tile.backward(d_t.reshape(self.tile.D, -1), d_trans=True, x_trans=True)
        return copy_indexed_output(np.ascontiguousarray(x_t), self.indices, self.tile.X, self.patches, n, image_size)

    def update(self, images, d_images):
        n = images.shape[0]
        flat = np.ascontiguousarray(images, np.float32).reshape(n, -1)
        x_t = copy_indexed_input(flat, self.indices, self.tile.X, self.patches)
        d_in = np.ascontiguousarray(d_images, np.float32).reshape(n, self.tile.D, self.patches)
        d_t = permute132(d_in, self.patches, self.tile.D, n).reshape(self.tile.D, -1)
        self.tile.update(x_t, d_t, x_trans=True, d_trans=True)
