// The third device branch of the binding layer, written without nanobind so that it compiles anywhere: the body of
// `gqa_decode_attention` (axono/python/src/nanobind_module.cpp:1016-1028 of the reference), of `add_rms_norm`
// (:977-992) and of the graph class (capture :1267-1297, replay, reset) with a hip arm.
#include <stdexcept>
#include <string>
#include <utility>

#include "axhip.h"
#include "hip_ops.h"

namespace axono_binding_sketch {

using axono::core::Context;
using axono::core::Status;
using axono::core::Tensor;
namespace hip = axono::ops::hip;

Tensor gqa_decode_attention(const Tensor &q, const Tensor &k, const Tensor &v) {
  Tensor result(q.dtype(), q.shape(), q.device());
  Status st = Status::DEVICE_MISMATCH;
  if (hip::IsHip(q)) st = hip::GqaDecodeAttention(Context(), q, k, v, result);
  // else: the existing CUDA branch
  if (st != Status::OK)
    throw std::runtime_error("gqa_decode_attention failed, status " + std::to_string(static_cast<int>(st)));
  return result;
}

std::pair<Tensor, Tensor> add_rms_norm(const Tensor &x, const Tensor &residual, const Tensor &weight, float eps) {
  Tensor y(x.dtype(), x.shape(), x.device()), out(x.dtype(), x.shape(), x.device());
  Status st = Status::DEVICE_MISMATCH;
  if (hip::IsHip(x)) st = hip::AddRmsNorm(Context(), x, residual, weight, eps, y, out);
  if (st != Status::OK) throw std::runtime_error("add_rms_norm failed, status " + std::to_string(static_cast<int>(st)));
  return {y, out};
}

bool hip_available() {
  int n = 0;
  return axhip_device_count(&n) == AXHIP_OK && n > 0;
}

// storage of a hip tensor (Tensor::InitializeStorage, src/core/tensor.cpp:217-234): the block comes from the caching
// allocator; a block the capture pool owns gets the reference's no-op deleter (src/core/cuda/detail.cu:196-199)
std::shared_ptr<void> allocate_storage(const std::string &device, size_t bytes) {
  if (axhip_set_device(hip::DeviceIndex(device)) != AXHIP_OK) throw std::runtime_error("no such hip device");
  void *p = nullptr;
  if (axhip_alloc(bytes, /*zero=*/1, &p) != AXHIP_OK) throw std::bad_alloc();
  int pool_owned = 0;
  axhip_block_is_capture_owned(p, &pool_owned);
  return std::shared_ptr<void>(p, [pool_owned](void *q) {
    if (!pool_owned) axhip_free(q);
  });
}

class HipGraph {
 public:
  template <typename Fn>
  void capture(Fn &&fn) {
    axhip_capture_pool_reset();
    axhip_capture_pool_set_recording(1);
    fn();  // warm-up run: its allocations become the addresses of the recorded run
    axhip_capture_pool_set_recording(0);
    axhip_stream s = nullptr;
    if (axhip_graph_begin_capture(&s) != AXHIP_OK) throw std::runtime_error("begin_capture failed");
    try {
      fn();
    } catch (...) {
      axhip_graph_abort_capture(s);
      throw;
    }
    size_t nodes = 0;
    const int rc = axhip_graph_end_capture(s, &graph_, &nodes);
    if (rc == AXHIP_INVALID_ARGUMENT) throw std::runtime_error("empty graph");
    if (rc != AXHIP_OK) throw std::runtime_error("end_capture failed");
    nodes_ = nodes;
  }
  void replay() {
    if (axhip_graph_replay(graph_) != AXHIP_OK) throw std::runtime_error("replay failed");
  }
  void reset() {
    if (graph_) axhip_graph_destroy(graph_);
    graph_ = nullptr;
    nodes_ = 0;
  }
  size_t num_nodes() const { return nodes_; }
  ~HipGraph() { reset(); }

 private:
  axhip_graph graph_ = nullptr;
  size_t nodes_ = 0;
};

// one use of the class so that every member is compiled
size_t capture_one_norm(const Tensor &x, const Tensor &r, const Tensor &w) {
  HipGraph g;
  g.capture([&] { (void)add_rms_norm(x, r, w, 1e-6f); });
  g.replay();
  const size_t n = g.num_nodes();
  g.reset();
  return n;
}

}  // namespace axono_binding_sketch
