// fp32 Linear: out[M,N] = x[M,K] . W[N,K]^T (+ bias), every operand FLOAT32 - what a Linear computes before
// cast_linear_fp16() has been called on it (the reference's fp32 branch, src/ops/cuda/linear.cu:178-251, a
// cublasSgemm).  Not on the decode path, so this is a plain tiled kernel on the fp32 matrix instruction
// (v_mfma_f32_16x16x4_f32), written for correctness and a reasonable rate, not tuned: a workgroup of four
// wavefronts owns 64 rows of x by 64 rows of W, K advances 32 per step through LDS, a wavefront owns 16 rows of x.
// Every output element sums its products in K order (fp32 products and sums).
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kTile = 64, kStep = 32, kPad = 4;

struct LinearF32Args {
  const float *x, *w, *bias;
  float *out;
  int M, K, N;
};

__global__ __launch_bounds__(256) void linear_f32_kernel(LinearF32Args a) {
  __shared__ __attribute__((aligned(16))) float xs[kTile][kStep + kPad];
  __shared__ __attribute__((aligned(16))) float ws[kTile][kStep + kPad];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * kTile, m0 = blockIdx.y * kTile;
  const bool vec = (a.K & 3) == 0;  // rows start on 16-byte boundaries: whole float4 loads

  float4_t acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

  for (int k0 = 0; k0 < a.K; k0 += kStep) {
    // stage 64 x 32 of x and of W: 512 float4 each, two per thread and matrix
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int v = p * 256 + tid;
      const int row = v >> 3, q = (v & 7) * 4;
      const int k = k0 + q;
      float4_t xv{0.f, 0.f, 0.f, 0.f}, wv{0.f, 0.f, 0.f, 0.f};
      if (vec && k + 4 <= a.K) {
        if (m0 + row < a.M) xv = *reinterpret_cast<const float4_t *>(a.x + static_cast<int64_t>(m0 + row) * a.K + k);
        if (n0 + row < a.N) wv = *reinterpret_cast<const float4_t *>(a.w + static_cast<int64_t>(n0 + row) * a.K + k);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (k + e < a.K && m0 + row < a.M) xv[e] = a.x[static_cast<int64_t>(m0 + row) * a.K + k + e];
          if (k + e < a.K && n0 + row < a.N) wv[e] = a.w[static_cast<int64_t>(n0 + row) * a.K + k + e];
        }
      }
      *reinterpret_cast<float4_t *>(&xs[row][q]) = xv;
      *reinterpret_cast<float4_t *>(&ws[row][q]) = wv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStep; kk += 4) {
      // A: x row (wave's 16 rows) c, K element kk + g; B: W row (tile t) c, the same K element
      const float af = xs[wave * 16 + c][kk + g];
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(af, ws[t * 16 + c][kk + g], acc[t], 0, 0, 0);
    }
    __syncthreads();
  }
  // C: this lane holds output column n = c of the tile for rows m = 4g .. 4g + 3 of the wavefront's 16
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = n0 + t * 16 + c;
    if (n >= a.N) continue;
    const float bv = a.bias ? a.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + wave * 16 + 4 * g + i;
      if (m < a.M) a.out[static_cast<int64_t>(m) * a.N + n] = acc[t][i] + bv;
    }
  }
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API int axhip_linear_f32(const float *x, const float *w, const float *bias, float *out, int64_t M,
                               int64_t K, int64_t N, axhip_stream stream) {
  if (M < 0 || K <= 0 || N <= 0) return AXHIP_INVALID_ARGUMENT;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
  if (M == 0) return AXHIP_OK;
  if (!x || !w || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) & 15)
    return AXHIP_INVALID_PTR;
  const int64_t gy = (M + kTile - 1) / kTile;
  if (gy > 65535) return AXHIP_INVALID_ARGUMENT;
  LinearF32Args a{x, w, bias, out, static_cast<int>(M), static_cast<int>(K), static_cast<int>(N)};
  hipLaunchKernelGGL(linear_f32_kernel, dim3(static_cast<unsigned>((N + kTile - 1) / kTile), static_cast<unsigned>(gy)),
                     dim3(256), 0, as_stream(stream), a);
  return launch_status();
}

}  // extern "C"
