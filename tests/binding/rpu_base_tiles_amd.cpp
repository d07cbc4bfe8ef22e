// A compiled instance of the binding a maintainer of the reference would add beside
// src/aihwkit/simulator/rpu_base_src/rpu_base_tiles_cuda.cpp: a pybind11 + libtorch module whose CudaAnalogTile
// forwards the reference's lambdas (rpu_base_tiles_cuda.cpp:88-130 set_shared_weights / set_delta_weights, :159-236
// forward, :238-308 backward, :310-375 update, :524-543 the constructor from the CPU tile) to the C entry points of
// rpu_amd.h.  Torch tensors stay at this layer; the library sees pointers, sizes and the stream.
//
// One difference from the file that would live in the reference's tree: there the constructor takes the CPU tile
// (RPU::RPUPulsed<float> &) and copies its meta parameters field by field into rpu_tile_config; the reference's C++
// classes cannot be compiled here (they need a BLAS header this image lacks), so this instance is constructed from
// the address of a host tile that the C library already holds (rpu_tile_create) and clones it.  Everything after
// the constructor is what the reference-side file would contain.
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "rpu_amd.h"

namespace py = pybind11;

namespace {

void check(int rc) {
  if (rc != 0) throw std::runtime_error(rpu_last_error());
}

void check_device_input(const torch::Tensor &t, const char *name) {
  if (!t.is_cuda()) throw std::runtime_error(std::string(name) + " must be a CUDA tensor");
  if (t.scalar_type() != torch::kFloat32) throw std::runtime_error(std::string(name) + " must be float32");
  if (!t.is_contiguous()) throw std::runtime_error(std::string(name) + " must be contiguous");
}

struct AmdAnalogTile {
  rpu_tile_t *h = nullptr;
  std::mutex mutex;
  std::vector<torch::Tensor> bound; // tensors the tile works on in place: kept alive with it

  explicit AmdAnalogTile(rpu_tile_t *host_tile) {
    check(rpu_tile_clone(&h, host_tile));
    const int rc = rpu_tile_to_device(h, -1);
    if (rc != 0) {
      const std::string message = rpu_last_error();
      rpu_tile_destroy(h);
      throw std::runtime_error(message);
    }
  }
  ~AmdAnalogTile() { rpu_tile_destroy(h); }
  AmdAnalogTile(const AmdAnalogTile &) = delete;
  AmdAnalogTile &operator=(const AmdAnalogTile &) = delete;

  int x_size() const { return rpu_tile_get_x_size(h); }
  int d_size() const { return rpu_tile_get_d_size(h); }
};

// batch size and output shape of a call: the vector index is the last dimension, or the first with `trans`
int batch_of(const torch::Tensor &t, bool trans, int expected, const char *name) {
  if (t.dim() < 1) throw std::runtime_error(std::string("Invalid ") + name + " dimensions: expected at least 1 dimensional array");
  const int size = trans ? t.size(0) : t.size(-1);
  if (size != expected) {
    const std::string shape = trans ? ("[*, " + std::to_string(expected) + "]") : ("[" + std::to_string(expected) + ", *]");
    throw std::runtime_error(std::string("Invalid ") + name + " dimensions: expected " + shape + " array");
  }
  return (int)(t.numel() / size);
}

torch::Tensor output_like(const torch::Tensor &in, bool trans, int out_size) {
  std::vector<int64_t> dims(in.sizes().begin(), in.sizes().end());
  dims[trans ? 0 : dims.size() - 1] = out_size;
  return torch::empty(dims, in.options());
}

} // namespace

PYBIND11_MODULE(rpu_base_tiles_amd, m) {
  m.doc() = "CudaAnalogTile of the reference's rpu_base.tiles, on the MI355X library";
  py::class_<AmdAnalogTile>(m, "CudaAnalogTile")
      .def(py::init([](uintptr_t host_tile_address) {
             if (!host_tile_address) throw std::runtime_error("null tile");
             return std::make_unique<AmdAnalogTile>(reinterpret_cast<rpu_tile_t *>(host_tile_address));
           }),
           py::arg("tile"))
      .def("get_x_size", &AmdAnalogTile::x_size)
      .def("get_d_size", &AmdAnalogTile::d_size)
      .def("get_learning_rate", [](AmdAnalogTile &self) { return rpu_tile_get_learning_rate(self.h); })
      .def("set_learning_rate",
           [](AmdAnalogTile &self, float learning_rate) {
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_set_learning_rate(self.h, learning_rate));
           },
           py::arg("learning_rate"))
      .def("set_seed",
           [](AmdAnalogTile &self, uint64_t seed) {
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_set_seed(self.h, seed));
           },
           py::arg("seed"))
      .def("get_weights",
           [](AmdAnalogTile &self) {
             torch::Tensor weights = torch::empty({self.d_size(), self.x_size()}, torch::kFloat32);
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_get_weights(self.h, weights.data_ptr<float>()));
             return weights;
           })
      .def("set_weights",
           [](AmdAnalogTile &self, const torch::Tensor &weights_) {
             auto weights = weights_.cpu().contiguous().to(torch::kFloat32);
             if (weights.dim() != 2 || weights.size(0) != self.d_size() || weights.size(1) != self.x_size()) {
               throw std::runtime_error("Invalid weights dimensions: expected [" + std::to_string(self.d_size()) + "," +
                                        std::to_string(self.x_size()) + "] array");
             }
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_set_weights(self.h, weights.data_ptr<float>()));
           },
           py::arg("weights"))
      .def("set_shared_weights",
           [](AmdAnalogTile &self, torch::Tensor weights) {
             check_device_input(weights, "weights");
             // the weight tensor of a CUDA tile is [x_size, d_size]
             if (weights.dim() != 2 || weights.size(1) != self.d_size() || weights.size(0) != self.x_size()) {
               throw std::runtime_error("Invalid weights dimensions: expected [" + std::to_string(self.x_size()) + "," +
                                        std::to_string(self.d_size()) + "] array");
             }
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_set_shared_weights_xd(self.h, weights.data_ptr<float>()));
             self.bound.push_back(weights);
           },
           py::arg("weights"))
      .def("set_delta_weights",
           [](AmdAnalogTile &self, torch::Tensor delta_weights) {
             check_device_input(delta_weights, "delta_weights");
             if (delta_weights.dim() != 2 || delta_weights.size(1) != self.d_size() || delta_weights.size(0) != self.x_size()) {
               throw std::runtime_error("Invalid delta weights dimensions: expected [" + std::to_string(self.x_size()) +
                                        "," + std::to_string(self.d_size()) + "] array");
             }
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_set_delta_weights_xd(self.h, delta_weights.data_ptr<float>()));
             self.bound.push_back(delta_weights);
           },
           py::arg("delta_weights"))
      .def("forward",
           [](AmdAnalogTile &self, const torch::Tensor &x_input_, bool bias, bool x_trans, bool d_trans, bool is_test,
              bool non_blocking) {
             auto x_input = x_input_.contiguous();
             check_device_input(x_input, "x_input");
             const int m_batch = batch_of(x_input, x_trans, self.x_size() - (bias ? 1 : 0), "x_input");
             torch::Tensor d_output = output_like(x_input, d_trans, self.d_size());
             auto stream = c10::hip::getCurrentHIPStream(x_input.device().index());
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_forward(self.h, x_input.data_ptr<float>(), d_output.data_ptr<float>(), m_batch, bias, x_trans,
                                    d_trans, is_test, stream.stream()));
             if (!non_blocking) stream.synchronize();
             return d_output;
           },
           py::arg("x_input"), py::arg("bias") = false, py::arg("x_trans") = false, py::arg("d_trans") = false,
           py::arg("is_test") = false, py::arg("non_blocking") = false)
      .def("backward",
           [](AmdAnalogTile &self, const torch::Tensor &d_input_, bool bias, bool d_trans, bool x_trans, bool non_blocking) {
             auto d_input = d_input_.contiguous();
             check_device_input(d_input, "d_input");
             const int m_batch = batch_of(d_input, d_trans, self.d_size(), "d_input");
             torch::Tensor x_output = output_like(d_input, x_trans, self.x_size() - (bias ? 1 : 0));
             auto stream = c10::hip::getCurrentHIPStream(d_input.device().index());
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_backward(self.h, d_input.data_ptr<float>(), x_output.data_ptr<float>(), m_batch, bias, d_trans,
                                     x_trans, stream.stream()));
             if (!non_blocking) stream.synchronize();
             return x_output;
           },
           py::arg("d_input"), py::arg("bias") = false, py::arg("d_trans") = false, py::arg("x_trans") = false,
           py::arg("non_blocking") = false)
      .def("update",
           [](AmdAnalogTile &self, const torch::Tensor &x_input_, const torch::Tensor &d_input_, bool bias, bool x_trans,
              bool d_trans, bool non_blocking) {
             if (rpu_tile_get_learning_rate(self.h) == 0.0f) return;
             auto x_input = x_input_.contiguous();
             auto d_input = d_input_.contiguous();
             check_device_input(x_input, "x_input");
             check_device_input(d_input, "d_input");
             const int m_batch = batch_of(x_input, x_trans, self.x_size() - (bias ? 1 : 0), "x_input");
             const int m_batch_from_d = batch_of(d_input, d_trans, self.d_size(), "d_input");
             if (m_batch != m_batch_from_d) {
               throw std::runtime_error("Invalid x_input or d_input dimensions: batch dimensions mismatch!");
             }
             auto stream = c10::hip::getCurrentHIPStream(x_input.device().index());
             std::lock_guard<std::mutex> lock(self.mutex);
             check(rpu_tile_update(self.h, x_input.data_ptr<float>(), d_input.data_ptr<float>(), m_batch, bias, x_trans,
                                   d_trans, stream.stream()));
             if (!non_blocking) stream.synchronize();
           },
           // (the reference names the fourth and fifth argument d_trans, x_trans while its lambda takes them as
           //  x_trans, d_trans, rpu_base_tiles_cuda.cpp:312-314,373-374; positional calls mean the lambda's order)
           py::arg("x_input"), py::arg("d_input"), py::arg("bias") = false, py::arg("x_trans") = false,
           py::arg("d_trans") = false, py::arg("non_blocking") = false);
}
