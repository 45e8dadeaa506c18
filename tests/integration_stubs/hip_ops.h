// Operator layer a maintainer of the reference would add for a `hip:<id>` device: one function per operator of
// the decode path, with the signature of its CUDA counterpart (include/axono/ops/cuda/{gqa,fused,llm,sequence,
// linear,add}.h of the reference), forwarding to one C-ABI call of libaxhip.so.  Host C++ only.
//
// This directory is compiled by tests/test_integration_stubs.py against the reference's own headers
// (include/axono/core/tensor.h, types.h) and this repository's include/axhip.h, so that a signature change on
// either side fails on a machine without a GPU.  It is not part of the product library.
#pragma once

#include "axono/core/tensor.h"
#include "axono/core/types.h"

namespace axono {
namespace ops {
namespace hip {

// device predicate next to Tensor::is_cuda() (include/axono/core/tensor.h:56-57)
inline bool IsHip(const core::Tensor &t) { return t.device().compare(0, 3, "hip") == 0; }
// "hip" -> 0, "hip:3" -> 3
int DeviceIndex(const std::string &device);

// ops/cuda/gqa.h:16-20
core::Status GqaDecodeAttention(const core::Context &ctx, const core::Tensor &q, const core::Tensor &k,
                                const core::Tensor &v, core::Tensor &result);
// ops/cuda/sequence.h (ScaledDotProductAttention, Rope, RopeWithCosSin, RopeThd, MropeCosSin, Concat, Embedding,
// ArgmaxLastDim)
core::Status ScaledDotProductAttention(const core::Context &ctx, const core::Tensor &q, const core::Tensor &k,
                                       const core::Tensor &v, bool is_causal, core::Tensor &result);
core::Status Rope(const core::Context &ctx, const core::Tensor &x, const core::Tensor &pos_ids, float theta,
                  core::Tensor &result);
core::Status RopeWithCosSin(const core::Context &ctx, const core::Tensor &x, const core::Tensor &cos,
                            const core::Tensor &sin, core::Tensor &result);
core::Status RopeThd(const core::Context &ctx, const core::Tensor &x, const core::Tensor &pos,
                     const core::Tensor &inv_freq, int t_sec, int h_sec, int w_sec, core::Tensor &result);
core::Status MropeCosSin(const core::Context &ctx, const core::Tensor &pos, const core::Tensor &inv_freq, int h_sec,
                         int w_sec, core::Tensor &cos_out, core::Tensor &sin_out);
core::Status Concat(const core::Context &ctx, const core::Tensor &a, const core::Tensor &b, int axis,
                    core::Tensor &result);
core::Status Embedding(const core::Context &ctx, const core::Tensor &ids, const core::Tensor &table,
                       core::Tensor &result);
core::Status ArgmaxLastDim(const core::Context &ctx, const core::Tensor &x, core::Tensor &result);
// ops/cuda/fused.h
core::Status SiluMul(const core::Context &ctx, const core::Tensor &gate, const core::Tensor &up,
                     core::Tensor &result);
core::Status AddRmsNorm(const core::Context &ctx, const core::Tensor &x, const core::Tensor &residual,
                        const core::Tensor &weight, float eps, core::Tensor &y, core::Tensor &out);
// ops/cuda/llm.h
core::Status RmsNorm(const core::Context &ctx, const core::Tensor &x, const core::Tensor &weight, float eps,
                     core::Tensor &result);
// ops/cuda/linear.h (fp16-weight branch, src/ops/cuda/linear.cu:105-176)
core::Status Linear(const core::Context &ctx, const core::Tensor &x, const core::Tensor &weight,
                    const core::Tensor &bias, core::Tensor &result);
// ops/cuda/add.h (equal shapes)
core::Status Add(const core::Context &ctx, const core::Tensor &a, const core::Tensor &b, core::Tensor &result);
// Tensor::CastTo for FLOAT16 <-> FLOAT32 (src/core/tensor.cpp:437-489)
core::Status CastTo(const core::Tensor &src, core::DataType target, core::Tensor &result);

}  // namespace hip
}  // namespace ops
}  // namespace axono
