// See hip_ops.h.  Every function checks what its CUDA counterpart checks (same Status for the same mistake), sizes
// the result like it, and forwards to libaxhip.so; the C ABI's return value is the reference's Status integer.
#include "hip_ops.h"

#include <cstdlib>

#include "axhip.h"

namespace axono {
namespace ops {
namespace hip {

namespace {
using core::DataType;
using core::Status;
using core::Tensor;

inline Status S(int rc) { return static_cast<Status>(rc); }
inline int DT(const Tensor &t) { return static_cast<int>(t.dtype()); }
inline bool IsFloat(const Tensor &t) { return t.dtype() == DataType::FLOAT32 || t.dtype() == DataType::FLOAT16; }

// the values of the two enumerations must stay aligned: the C ABI passes them through as integers
static_assert(static_cast<int>(DataType::INT32) == AXHIP_INT32 && static_cast<int>(DataType::INT64) == AXHIP_INT64 &&
                  static_cast<int>(DataType::FLOAT16) == AXHIP_FLOAT16 &&
                  static_cast<int>(DataType::FLOAT32) == AXHIP_FLOAT32,
              "DataType codes of axhip.h follow include/axono/core/types.h:18-27");
static_assert(static_cast<int>(Status::OK) == AXHIP_OK && static_cast<int>(Status::INVALID_ARGUMENT) == AXHIP_INVALID_ARGUMENT &&
                  static_cast<int>(Status::OUT_OF_MEMORY) == AXHIP_OUT_OF_MEMORY &&
                  static_cast<int>(Status::UNSUPPORTED_TYPE) == AXHIP_UNSUPPORTED_TYPE &&
                  static_cast<int>(Status::SHAPE_MISMATCH) == AXHIP_SHAPE_MISMATCH &&
                  static_cast<int>(Status::DEVICE_ERROR) == AXHIP_DEVICE_ERROR &&
                  static_cast<int>(Status::INVALID_PTR) == AXHIP_INVALID_PTR &&
                  static_cast<int>(Status::DEVICE_MISMATCH) == AXHIP_DEVICE_MISMATCH,
              "Status codes of axhip.h follow include/axono/core/types.h:54-64");
}  // namespace

int DeviceIndex(const std::string &device) {
  const size_t colon = device.find(':');
  return colon == std::string::npos ? 0 : std::atoi(device.c_str() + colon + 1);
}

// src/ops/cuda/gqa.cu:139-182.  The reference call is one sequence with token-major K/V (L, Hkv, D): in the
// batched C ABI that is B = 1, stride_h = D, stride_s = Hkv * D.
Status GqaDecodeAttention(const core::Context &, const Tensor &q, const Tensor &k, const Tensor &v, Tensor &result) {
  if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || !IsFloat(q)) return Status::UNSUPPORTED_TYPE;
  const size_t sq = q.shape()[0], hq = q.shape()[1], d = q.shape()[2];
  const size_t skv = k.shape()[0], hkv = k.shape()[1];
  if (sq != 1) return Status::INVALID_ARGUMENT;
  if (k.shape()[2] != d || v.shape()[0] != skv || v.shape()[1] != hkv || v.shape()[2] != d || hkv == 0 ||
      hq % hkv != 0)
    return Status::SHAPE_MISMATCH;
  Status st = result.Resize({1, hq, d});
  if (st != Status::OK) return st;
  const int H = static_cast<int>(hq), HK = static_cast<int>(hkv), D = static_cast<int>(d), L = static_cast<int>(skv);
  const size_t wsb = axhip_gqa_decode_workspace_bytes(1, H, HK, D, L);
  Tensor ws(DataType::INT8, {wsb > 0 ? wsb : 256}, q.device());  // from the caching allocator, like gqa.cu:166-168
  return S(axhip_gqa_decode(q.data(), k.data(), v.data(), /*seq_lens=*/nullptr, result.data(), ws.data(), wsb, DT(q),
                            /*B=*/1, H, HK, D, /*max_len=*/L, /*stride_b=*/0, /*stride_h=*/D,
                            /*stride_s=*/static_cast<int64_t>(hkv) * D, axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:451-472
Status ScaledDotProductAttention(const core::Context &, const Tensor &q, const Tensor &k, const Tensor &v,
                                 bool is_causal, Tensor &result) {
  if (q.ndim() != 3 || k.ndim() != 3 || v.ndim() != 3 || !IsFloat(q)) return Status::UNSUPPORTED_TYPE;
  const size_t sq = q.shape()[0], hq = q.shape()[1], d = q.shape()[2];
  const size_t skv = k.shape()[0], hkv = k.shape()[1];
  if (k.shape()[2] != d || v.shape()[0] != skv || v.shape()[1] != hkv || v.shape()[2] != d || hkv == 0 ||
      hq % hkv != 0)
    return Status::SHAPE_MISMATCH;
  Status st = result.Resize({sq, hq, d});
  if (st != Status::OK) return st;
  return S(axhip_sdpa(q.data(), k.data(), v.data(), result.data(), DT(q), static_cast<int>(sq), static_cast<int>(hq),
                      static_cast<int>(hkv), static_cast<int>(d), static_cast<int>(skv), is_causal ? 1 : 0,
                      axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:318-342
Status Rope(const core::Context &, const Tensor &x, const Tensor &pos_ids, float theta, Tensor &result) {
  if (x.ndim() != 3 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  const size_t rows = x.shape()[0], heads = x.shape()[1], dim = x.shape()[2];
  if (dim % 2 != 0) return Status::INVALID_ARGUMENT;
  if (pos_ids.num_elements() != rows || pos_ids.dtype() != DataType::INT64) return Status::UNSUPPORTED_TYPE;
  Status st = result.Resize(x.shape());
  if (st != Status::OK) return st;
  return S(axhip_rope(x.data(), pos_ids.data<int64_t>(), theta, result.data(), DT(x), static_cast<int64_t>(rows),
                      static_cast<int64_t>(heads), static_cast<int64_t>(dim), axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:344-367
Status RopeWithCosSin(const core::Context &, const Tensor &x, const Tensor &cos, const Tensor &sin, Tensor &result) {
  if (x.ndim() != 3 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  const size_t rows = x.shape()[0], heads = x.shape()[1], dim = x.shape()[2];
  if (dim % 2 != 0) return Status::INVALID_ARGUMENT;
  if (cos.ndim() != 2 || sin.ndim() != 2 || cos.shape()[0] != rows || cos.shape()[1] != dim ||
      sin.shape()[0] != rows || sin.shape()[1] != dim || cos.dtype() != DataType::FLOAT32 ||
      sin.dtype() != DataType::FLOAT32)
    return Status::SHAPE_MISMATCH;
  Status st = result.Resize(x.shape());
  if (st != Status::OK) return st;
  return S(axhip_rope_with_cos_sin(x.data(), cos.data<float>(), sin.data<float>(), result.data(), DT(x),
                                   static_cast<int64_t>(rows), static_cast<int64_t>(heads), static_cast<int64_t>(dim),
                                   axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:421-449
Status RopeThd(const core::Context &, const Tensor &x, const Tensor &pos, const Tensor &inv_freq, int t_sec, int h_sec,
               int w_sec, Tensor &result) {
  if (x.ndim() != 3 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  const size_t rows = x.shape()[0], heads = x.shape()[1], dim = x.shape()[2];
  if (dim % 2 != 0) return Status::INVALID_ARGUMENT;
  if (pos.ndim() != 2 || pos.shape()[0] != 3 || pos.shape()[1] != rows || pos.dtype() != DataType::INT64)
    return Status::SHAPE_MISMATCH;
  if (inv_freq.ndim() != 1 || inv_freq.shape()[0] != dim / 2 || inv_freq.dtype() != DataType::FLOAT32)
    return Status::SHAPE_MISMATCH;
  Status st = result.Resize(x.shape());
  if (st != Status::OK) return st;
  return S(axhip_rope_thd(x.data(), pos.data<int64_t>(), inv_freq.data<float>(), t_sec, h_sec, w_sec, result.data(),
                          DT(x), static_cast<int64_t>(rows), static_cast<int64_t>(heads), static_cast<int64_t>(dim),
                          axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:399-419
Status MropeCosSin(const core::Context &, const Tensor &pos, const Tensor &inv_freq, int h_sec, int w_sec,
                   Tensor &cos_out, Tensor &sin_out) {
  if (pos.ndim() != 2 || pos.shape()[0] != 3 || pos.dtype() != DataType::INT64) return Status::SHAPE_MISMATCH;
  const size_t rows = pos.shape()[1];
  const size_t half = inv_freq.ndim() ? inv_freq.shape()[0] : 0;
  if (half == 0) return Status::INVALID_ARGUMENT;
  Status st = cos_out.Resize({rows, 2 * half});
  if (st != Status::OK) return st;
  st = sin_out.Resize({rows, 2 * half});
  if (st != Status::OK) return st;
  return S(axhip_mrope_cos_sin(pos.data<int64_t>(), inv_freq.data<float>(), h_sec, w_sec, cos_out.data<float>(),
                               sin_out.data<float>(), static_cast<int64_t>(rows), static_cast<int64_t>(half),
                               axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:474-521: the KV-cache append of the reference (DynamicKVCache.update concatenates along
// axis 0, axono/python/axono/nn/kv_cache.py:96-107)
Status Concat(const core::Context &, const Tensor &a, const Tensor &b, int axis, Tensor &result) {
  if (a.ndim() != b.ndim() || a.ndim() == 0 || a.dtype() != b.dtype()) return Status::SHAPE_MISMATCH;
  const int nd = static_cast<int>(a.ndim());
  if (axis < 0) axis += nd;
  if (axis < 0 || axis >= nd) return Status::INVALID_ARGUMENT;
  size_t outer = 1, inner = core::GetDataTypeSize(a.dtype());
  core::Shape out_shape = a.shape();
  for (int i = 0; i < nd; ++i) {
    if (i != axis && a.shape()[i] != b.shape()[i]) return Status::SHAPE_MISMATCH;
    if (i < axis) outer *= a.shape()[i];
    if (i > axis) inner *= a.shape()[i];
  }
  out_shape[axis] = a.shape()[axis] + b.shape()[axis];
  Status st = result.Resize(out_shape);
  if (st != Status::OK) return st;
  return S(axhip_concat(a.data(), b.data(), result.data(), static_cast<int64_t>(outer),
                        static_cast<int64_t>(a.shape()[axis] * inner), static_cast<int64_t>(b.shape()[axis] * inner),
                        axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:296-316
Status Embedding(const core::Context &, const Tensor &ids, const Tensor &table, Tensor &result) {
  if (ids.ndim() < 1 || table.ndim() != 2) return Status::INVALID_ARGUMENT;
  if (!IsFloat(table)) return Status::UNSUPPORTED_TYPE;
  core::Shape out_shape = ids.shape();
  out_shape.push_back(table.shape()[1]);
  Status st = result.Resize(out_shape);
  if (st != Status::OK) return st;
  if (ids.dtype() != DataType::INT64 && ids.dtype() != DataType::INT32) return Status::UNSUPPORTED_TYPE;
  return S(axhip_embedding(ids.data(), DT(ids), table.data(), result.data(), DT(table),
                           static_cast<int64_t>(ids.num_elements()), static_cast<int64_t>(table.shape()[0]),
                           static_cast<int64_t>(table.shape()[1]), axhip_current_stream()));
}

// src/ops/cuda/sequence.cu:262-292 (result INT64, the last dimension dropped)
Status ArgmaxLastDim(const core::Context &, const Tensor &x, Tensor &result) {
  if (x.ndim() < 1 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  const size_t cols = x.shape().back();
  if (cols == 0) return Status::INVALID_ARGUMENT;
  core::Shape out_shape(x.shape().begin(), x.shape().end() - 1);
  if (out_shape.empty()) out_shape.push_back(1);
  Status st = result.Resize(out_shape);
  if (st != Status::OK) return st;
  return S(axhip_argmax(x.data(), result.data<int64_t>(), DT(x), static_cast<int64_t>(x.num_elements() / cols),
                        static_cast<int64_t>(cols), axhip_current_stream()));
}

// src/ops/cuda/fused.cu:76-89
Status SiluMul(const core::Context &, const Tensor &gate, const Tensor &up, Tensor &result) {
  if (!IsFloat(gate) || gate.dtype() != up.dtype() || gate.shape() != up.shape() || gate.device() != up.device())
    return Status::SHAPE_MISMATCH;
  Status st = result.Resize(gate.shape());
  if (st != Status::OK) return st;
  return S(axhip_silu_mul(gate.data(), up.data(), result.data(), DT(gate), static_cast<int64_t>(gate.num_elements()),
                          axhip_current_stream()));
}

// src/ops/cuda/fused.cu:91-110
Status AddRmsNorm(const core::Context &, const Tensor &x, const Tensor &residual, const Tensor &weight, float eps,
                  Tensor &y, Tensor &out) {
  if (!IsFloat(x) || x.dtype() != residual.dtype() || x.shape() != residual.shape()) return Status::SHAPE_MISMATCH;
  if (x.ndim() < 1) return Status::INVALID_ARGUMENT;
  const size_t hidden = x.shape().back();
  if (weight.ndim() != 1 || weight.shape()[0] != hidden) return Status::SHAPE_MISMATCH;
  Status st = y.Resize(x.shape());
  if (st != Status::OK) return st;
  st = out.Resize(x.shape());
  if (st != Status::OK) return st;
  return S(axhip_add_rms_norm(x.data(), residual.data(), weight.data(), eps, y.data(), out.data(), DT(x), DT(weight),
                              static_cast<int64_t>(x.num_elements() / hidden), static_cast<int64_t>(hidden),
                              axhip_current_stream()));
}

// src/ops/cuda/llm.cu:140-158 and its host wrapper (an empty weight tensor means no weight)
Status RmsNorm(const core::Context &, const Tensor &x, const Tensor &weight, float eps, Tensor &result) {
  if (x.ndim() < 1 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  const size_t cols = x.shape().back();
  const bool has_w = weight.num_elements() != 0;
  if (has_w && (weight.ndim() != 1 || weight.shape()[0] != cols)) return Status::SHAPE_MISMATCH;
  Status st = result.Resize(x.shape());
  if (st != Status::OK) return st;
  return S(axhip_rms_norm(x.data(), has_w ? weight.data() : nullptr, eps, result.data(), DT(x),
                          has_w ? DT(weight) : AXHIP_FLOAT32, static_cast<int64_t>(x.num_elements() / cols),
                          static_cast<int64_t>(cols), axhip_current_stream()));
}

// src/ops/cuda/linear.cu:76-176, the fp16-weight branch: x FLOAT32 (rounded to fp16 on load, linear.cu:110) or
// FLOAT16, weight FLOAT16 [out_f, k], bias FLOAT16 (or empty), result FLOAT32; FLOAT32 weights go to the plain fp32
// operator.  FLOAT64 weights have no hip counterpart.
Status Linear(const core::Context &, const Tensor &x, const Tensor &weight, const Tensor &bias, Tensor &result) {
  if (x.ndim() < 1 || weight.ndim() != 2) return Status::INVALID_ARGUMENT;
  const size_t k = x.shape().back(), out_f = weight.shape()[0];
  if (weight.shape()[1] != k) return Status::SHAPE_MISMATCH;
  const bool has_bias = bias.num_elements() != 0;
  if (has_bias && (bias.ndim() != 1 || bias.shape()[0] != out_f)) return Status::SHAPE_MISMATCH;
  core::Shape out_shape = x.shape();
  out_shape.back() = out_f;
  const int64_t rows = static_cast<int64_t>(x.num_elements() / k);
  if (weight.dtype() == DataType::FLOAT32) {
    // the FLOAT32 branch (linear.cu:178-251): x and bias of the weight's type
    if (x.dtype() != DataType::FLOAT32 || (has_bias && bias.dtype() != DataType::FLOAT32)) return Status::UNSUPPORTED_TYPE;
    Status st32 = result.Resize(out_shape);
    if (st32 != Status::OK) return st32;
    return S(axhip_linear_f32(x.data<float>(), weight.data<float>(), has_bias ? bias.data<float>() : nullptr,
                              result.data<float>(), rows, static_cast<int64_t>(k), static_cast<int64_t>(out_f),
                              axhip_current_stream()));
  }
  if (weight.dtype() != DataType::FLOAT16 || !IsFloat(x)) return Status::UNSUPPORTED_TYPE;
  if (has_bias && bias.dtype() != DataType::FLOAT16) return Status::UNSUPPORTED_TYPE;
  Status st = result.Resize(out_shape);
  if (st != Status::OK) return st;
  return S(axhip_linear_f16(x.data(), DT(x), weight.data(), has_bias ? bias.data() : nullptr, result.data(), DT(result),
                            rows, static_cast<int64_t>(k), static_cast<int64_t>(out_f), /*workspace=*/nullptr, 0,
                            axhip_current_stream()));
}

// src/ops/cuda/add.cu:17-24 (equal shapes)
Status Add(const core::Context &, const Tensor &a, const Tensor &b, Tensor &result) {
  if (a.shape() != b.shape() || a.dtype() != b.dtype()) return Status::SHAPE_MISMATCH;
  Status st = result.Resize(a.shape());
  if (st != Status::OK) return st;
  return S(axhip_add(a.data(), b.data(), result.data(), DT(a), static_cast<int64_t>(a.num_elements()),
                     axhip_current_stream()));
}

// src/core/tensor.cpp:437-489 (FLOAT16 <-> FLOAT32 arm of Tensor::CastTo)
Status CastTo(const Tensor &src, DataType target, Tensor &result) {
  if (result.dtype() != target || result.num_elements() != src.num_elements()) return Status::SHAPE_MISMATCH;
  return S(axhip_cast(src.data(), DT(src), result.data(), static_cast<int>(target),
                      static_cast<int64_t>(src.num_elements()), axhip_current_stream()));
}

}  // namespace hip
}  // namespace ops
}  // namespace axono
