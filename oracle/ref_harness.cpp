// C entry points around the REFERENCE's own CPU operators, compiled together with the reference's
// sources where they lie (see oracle/Makefile, target `ref`).  Test infrastructure only: it exists
// to check the restatement in axono_cpu_oracle.c bit for bit and, optionally, to serve as the CPU
// baseline.  Nothing here is shipped and no reference source is copied into this repository.
//
// Each wrapper borrows the caller's buffers as axono::core::Tensor objects
// (include/axono/core/tensor.h:24-129), calls the reference operator, and copies the result out.
#include <cstdint>
#include <cstring>
#include <vector>

#include "axono/core/half.h"
#include "axono/core/tensor.h"
#include "axono/core/types.h"
#include "axono/ops/cpu/fused.h"
#include "axono/ops/cpu/linear.h"
#include "axono/ops/cpu/llm.h"
#include "axono/ops/cpu/sequence.h"

using axono::core::Context;
using axono::core::DataType;
using axono::core::Shape;
using axono::core::Status;
using axono::core::Tensor;

namespace {
Tensor Borrow(DataType dt, const Shape &shape, const void *p) {
  return Tensor::FromBorrowed(dt, shape, p);
}
int Emit(Status st, const Tensor &t, void *dst) {
  if (st == Status::OK && dst != nullptr && t.num_bytes() > 0)
    std::memcpy(dst, t.data(), t.num_bytes());
  return static_cast<int>(st);
}
Shape S(std::initializer_list<int64_t> dims) {
  Shape s;
  for (int64_t d : dims) s.push_back(static_cast<size_t>(d));
  return s;
}
}  // namespace

extern "C" {

#define REF_API __attribute__((visibility("default")))

// ops::cpu::ScaledDotProductAttention, src/ops/cpu/sequence.cpp:236-301
REF_API int axref_sdpa(const float *q, const float *k, const float *v, float *out, int64_t sq,
                       int64_t hq, int64_t hkv, int64_t d, int64_t skv, int is_causal) {
  Tensor tq = Borrow(DataType::FLOAT32, S({sq, hq, d}), q);
  Tensor tk = Borrow(DataType::FLOAT32, S({skv, hkv, d}), k);
  Tensor tv = Borrow(DataType::FLOAT32, S({skv, hkv, d}), v);
  Tensor r(DataType::FLOAT32, S({sq, hq, d}));
  Status st = axono::ops::cpu::ScaledDotProductAttention(Context(), tq, tk, tv, is_causal != 0, r);
  return Emit(st, r, out);
}

// ops::cpu::SiluMul, src/ops/cpu/fused.cpp:16-35
REF_API int axref_silu_mul(const float *gate, const float *up, float *y, int64_t n) {
  Tensor g = Borrow(DataType::FLOAT32, S({n}), gate);
  Tensor u = Borrow(DataType::FLOAT32, S({n}), up);
  Tensor r(DataType::FLOAT32, S({n}));
  return Emit(axono::ops::cpu::SiluMul(Context(), g, u, r), r, y);
}

// ops::cpu::AddRmsNorm, src/ops/cpu/fused.cpp:37-76
REF_API int axref_add_rms_norm(const float *x, const float *res, const float *w, float eps,
                               float *y, float *out, int64_t rows, int64_t hidden) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, hidden}), x);
  Tensor tr = Borrow(DataType::FLOAT32, S({rows, hidden}), res);
  Tensor tw = Borrow(DataType::FLOAT32, S({hidden}), w);
  Tensor ty(DataType::FLOAT32, S({rows, hidden}));
  Tensor to(DataType::FLOAT32, S({rows, hidden}));
  Status st = axono::ops::cpu::AddRmsNorm(Context(), tx, tr, tw, eps, ty, to);
  Emit(st, ty, y);
  return Emit(st, to, out);
}

// ops::cpu::RmsNorm, src/ops/cpu/llm.cpp:240-264
REF_API int axref_rms_norm(const float *x, const float *w, float eps, float *out, int64_t rows,
                           int64_t cols) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, cols}), x);
  Tensor tw = w ? Borrow(DataType::FLOAT32, S({cols}), w) : Tensor();
  Tensor r(DataType::FLOAT32, S({rows, cols}));
  return Emit(axono::ops::cpu::RmsNorm(Context(), tx, tw, eps, r), r, out);
}

// ops::cpu::Rope, src/ops/cpu/sequence.cpp:54-93
REF_API int axref_rope(const float *x, const int64_t *pos, float theta, float *out, int64_t rows,
                       int64_t heads, int64_t dim) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, heads, dim}), x);
  Tensor tp = Borrow(DataType::INT64, S({rows}), pos);
  Tensor r(DataType::FLOAT32, S({rows, heads, dim}));
  return Emit(axono::ops::cpu::Rope(Context(), tx, tp, theta, r), r, out);
}

// ops::cpu::RopeWithCosSin, src/ops/cpu/sequence.cpp:96-135
REF_API int axref_rope_with_cos_sin(const float *x, const float *cs, const float *sn, float *out,
                                    int64_t rows, int64_t heads, int64_t dim) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, heads, dim}), x);
  Tensor tc = Borrow(DataType::FLOAT32, S({rows, dim}), cs);
  Tensor ts = Borrow(DataType::FLOAT32, S({rows, dim}), sn);
  Tensor r(DataType::FLOAT32, S({rows, heads, dim}));
  return Emit(axono::ops::cpu::RopeWithCosSin(Context(), tx, tc, ts, r), r, out);
}

// ops::cpu::MropeCosSin, src/ops/cpu/sequence.cpp:140-182
REF_API int axref_mrope_cos_sin(const int64_t *pos, const float *inv_freq, int h_sec, int w_sec,
                                float *cos_out, float *sin_out, int64_t rows, int64_t half) {
  Tensor tp = Borrow(DataType::INT64, S({3, rows}), pos);
  Tensor tf = Borrow(DataType::FLOAT32, S({half}), inv_freq);
  Tensor c(DataType::FLOAT32), s(DataType::FLOAT32);
  Status st = axono::ops::cpu::MropeCosSin(Context(), tp, tf, h_sec, w_sec, c, s);
  Emit(st, c, cos_out);
  return Emit(st, s, sin_out);
}

// ops::cpu::RopeThd, src/ops/cpu/sequence.cpp:184-234
REF_API int axref_rope_thd(const float *x, const int64_t *pos, const float *inv_freq, int t_sec,
                           int h_sec, int w_sec, float *out, int64_t rows, int64_t heads,
                           int64_t dim) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, heads, dim}), x);
  Tensor tp = Borrow(DataType::INT64, S({3, rows}), pos);
  Tensor tf = Borrow(DataType::FLOAT32, S({dim / 2}), inv_freq);
  Tensor r(DataType::FLOAT32, S({rows, heads, dim}));
  return Emit(axono::ops::cpu::RopeThd(Context(), tx, tp, tf, t_sec, h_sec, w_sec, r), r, out);
}

// ops::cpu::Linear, src/ops/cpu/linear.cpp:48-126
REF_API int axref_linear(const float *x, const float *w, const float *bias, float *out,
                         int64_t rows, int64_t k, int64_t out_f) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, k}), x);
  Tensor tw = Borrow(DataType::FLOAT32, S({out_f, k}), w);
  Tensor tb = bias ? Borrow(DataType::FLOAT32, S({out_f}), bias) : Tensor();
  Tensor r(DataType::FLOAT32, S({rows, out_f}));
  return Emit(axono::ops::cpu::Linear(Context(), tx, tw, tb, r), r, out);
}

// ops::cpu::Concat, src/ops/cpu/sequence.cpp:303-338, on raw bytes (INT8 tensors), axis 0
REF_API int axref_concat_axis0(const void *a, const void *b, void *out, int64_t a_rows,
                               int64_t b_rows, int64_t row_bytes) {
  Tensor ta = Borrow(DataType::INT8, S({a_rows, row_bytes}), a);
  Tensor tb = Borrow(DataType::INT8, S({b_rows, row_bytes}), b);
  Tensor r(DataType::INT8);
  return Emit(axono::ops::cpu::Concat(Context(), ta, tb, 0, r), r, out);
}

// ops::cpu::Embedding, src/ops/cpu/sequence.cpp:18-52
REF_API int axref_embedding(const int64_t *ids, const float *table, float *out, int64_t n,
                            int64_t vocab, int64_t hidden) {
  Tensor ti = Borrow(DataType::INT64, S({n}), ids);
  Tensor tt = Borrow(DataType::FLOAT32, S({vocab, hidden}), table);
  Tensor r(DataType::FLOAT32, S({n, hidden}));
  return Emit(axono::ops::cpu::Embedding(Context(), ti, tt, r), r, out);
}

// ops::cpu::ArgmaxLastDim, src/ops/cpu/sequence.cpp:372-404
REF_API int axref_argmax(const float *x, int64_t *out, int64_t rows, int64_t cols) {
  Tensor tx = Borrow(DataType::FLOAT32, S({rows, cols}), x);
  Tensor r(DataType::INT64, S({rows}));
  return Emit(axono::ops::cpu::ArgmaxLastDim(Context(), tx, r), r, out);
}

// detail::Float2Half / Half2Float, include/axono/core/half.h:14-79 (the CPU bit-level helpers,
// kept to document where they depart from IEEE; the device path follows IEEE RNE instead).
REF_API void axref_float2half(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = axono::core::detail::Float2Half(src[i]);
}
REF_API void axref_half2float(const uint16_t *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = axono::core::detail::Half2Float(src[i]);
}

}  // extern "C"
