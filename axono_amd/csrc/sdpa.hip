// General scaled-dot-product attention (prefill, short contexts): q [Sq,Hq,D], k/v [Skv,Hkv,D].
//
// fp16 with head size 64 or 128 and at least 32 query rows runs the tiled prefill kernel on the matrix
// cores.  Otherwise, for head sizes the decode kernel supports (64/128/256) every query row is treated
// as one "sequence" of the split-K decode kernel that shares the same K/V (batch stride 0) and sees
// len[t] keys: t+1 under the causal rule, Skv otherwise.  K/V are then re-read per query row, mostly
// from L2.
// Other head sizes take a plain three-phase kernel (scores to a workspace, softmax, weighted sum).
#include "common.hpp"

extern "C" int axhip_internal_fill_zero(void *dst, int64_t n, hipStream_t st);
extern "C" int axhip_internal_sdpa_f16_mfma(const void *q, const void *k, const void *v, void *out, int Sq,
                                            int Hq, int Hkv, int D, int Skv, int is_causal, hipStream_t st);

namespace axhip {
namespace {

constexpr int kBlock = 256;
constexpr int kRowsPerCall = 32768;  // grid.z limit of the decode launch
constexpr int kMfmaMinRows = 32;     // fewer query rows than this stay on the split-K decode kernel

__global__ void visible_len_kernel(int32_t *len, int t0, int n, int skv, int causal) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int t = t0 + i;
  len[i] = (causal && skv >= t + 1) ? t + 1 : skv;
}

// Fallback for arbitrary D: one workgroup per (query row, head).
template <typename T>
__global__ __launch_bounds__(kBlock) void sdpa_generic_kernel(const T *__restrict__ q,
                                                              const T *__restrict__ k,
                                                              const T *__restrict__ v,
                                                              T *__restrict__ out,
                                                              float *__restrict__ scores, int Hq,
                                                              int Hkv, int D, int Skv, int causal) {
  __shared__ float red[kBlock / 64];
  const int t = blockIdx.x, h = blockIdx.y;
  const int hk = h / (Hq / Hkv);
  const int visible = (causal && Skv >= t + 1) ? t + 1 : Skv;
  const T *qr = q + (static_cast<int64_t>(t) * Hq + h) * D;
  float *sc = scores + (static_cast<int64_t>(t) * Hq + h) * Skv;
  const float scale = 1.0f / sqrtf(static_cast<float>(D));
  float mx = -INFINITY;
  for (int s = threadIdx.x; s < visible; s += kBlock) {
    const T *kr = k + (static_cast<int64_t>(s) * Hkv + hk) * D;
    float acc = 0.f;
    for (int i = 0; i < D; ++i) acc = __builtin_fmaf(ldf(qr + i), ldf(kr + i), acc);
    acc *= scale;
    sc[s] = acc;
    mx = fmaxf(mx, acc);
  }
  mx = group_max<64>(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.f;
  for (int s = threadIdx.x; s < visible; s += kBlock) {
    const float p = expf(sc[s] - mx);
    sc[s] = p;
    sum += p;
  }
  sum = block_sum<kBlock / 64>(sum, red);  // also orders the sc[] writes before the reads below
  const float inv = 1.0f / sum;
  for (int d = threadIdx.x; d < D; d += kBlock) {
    float acc = 0.f;
    for (int s = 0; s < visible; ++s)
      acc = __builtin_fmaf(sc[s] * inv, ldf(v + (static_cast<int64_t>(s) * Hkv + hk) * D + d), acc);
    stf(out + (static_cast<int64_t>(t) * Hq + h) * D + d, acc);
  }
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API int axhip_sdpa(const void *q, const void *k, const void *v, void *out, int dtype, int Sq,
                         int Hq, int Hkv, int D, int Skv, int is_causal, axhip_stream stream) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (Sq < 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || Skv <= 0) return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (Sq == 0) return AXHIP_OK;
  if (!q || !k || !v || !out) return AXHIP_INVALID_PTR;
  hipStream_t st = as_stream(stream);
  const int64_t esz = dtype == AXHIP_FLOAT16 ? 2 : 4;

  // fp16 with enough query rows to fill 16-row tiles: the causal prefill kernel on the matrix cores
  const uintptr_t ptr_bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
                             reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out);
  if (dtype == AXHIP_FLOAT16 && (D == 64 || D == 128) && Sq >= kMfmaMinRows && Hq <= 65535 &&
      (ptr_bits & 15) == 0)
    return axhip_internal_sdpa_f16_mfma(q, k, v, out, Sq, Hq, Hkv, D, Skv, is_causal, st);

  if (D == 64 || D == 128 || D == 256) {
    const int rows_max = Sq < kRowsPerCall ? Sq : kRowsPerCall;
    const size_t ws_bytes = axhip_gqa_decode_workspace_bytes(rows_max, Hq, Hkv, D, Skv);
    void *ws = nullptr, *lens = nullptr;
    int rc = axhip_alloc(ws_bytes, 0, &ws);
    if (rc != AXHIP_OK) return rc;
    rc = axhip_alloc(static_cast<size_t>(rows_max) * sizeof(int32_t), 0, &lens);
    if (rc != AXHIP_OK) {
      axhip_free(ws);
      return rc;
    }
    for (int t0 = 0; t0 < Sq && rc == AXHIP_OK; t0 += kRowsPerCall) {
      const int n = Sq - t0 < kRowsPerCall ? Sq - t0 : kRowsPerCall;
      hipLaunchKernelGGL(visible_len_kernel, dim3((n + 255) / 256), dim3(256), 0, st,
                         static_cast<int32_t *>(lens), t0, n, Skv, is_causal);
      // under the causal rule rows t0..t0+n-1 never see more than t0+n keys
      const int max_len = (is_causal && Skv >= t0 + n) ? t0 + n : Skv;
      rc = axhip_gqa_decode(static_cast<const char *>(q) + static_cast<int64_t>(t0) * Hq * D * esz, k, v,
                            static_cast<const int32_t *>(lens),
                            static_cast<char *>(out) + static_cast<int64_t>(t0) * Hq * D * esz, ws,
                            ws_bytes, dtype, n, Hq, Hkv, D, max_len, /*stride_b=*/0,
                            /*stride_h=*/D, /*stride_s=*/static_cast<int64_t>(Hkv) * D, stream);
    }
    // stream order keeps the blocks valid until the kernels above have run
    axhip_free(lens);
    axhip_free(ws);
    return rc;
  }

  if (Sq > 65535 * 32 || Hq > 65535) return AXHIP_INVALID_ARGUMENT;
  const size_t sc_bytes = static_cast<size_t>(Sq) * Hq * Skv * sizeof(float);
  if (sc_bytes > (size_t(4) << 30)) return AXHIP_INVALID_ARGUMENT;
  void *sc = nullptr;
  int rc = axhip_alloc(sc_bytes, 0, &sc);
  if (rc != AXHIP_OK) return rc;
  const dim3 grid(Sq, Hq);
  if (dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((sdpa_generic_kernel<__half>), grid, dim3(kBlock), 0, st,
                       static_cast<const __half *>(q), static_cast<const __half *>(k),
                       static_cast<const __half *>(v), static_cast<__half *>(out),
                       static_cast<float *>(sc), Hq, Hkv, D, Skv, is_causal);
  else
    hipLaunchKernelGGL((sdpa_generic_kernel<float>), grid, dim3(kBlock), 0, st,
                       static_cast<const float *>(q), static_cast<const float *>(k),
                       static_cast<const float *>(v), static_cast<float *>(out),
                       static_cast<float *>(sc), Hq, Hkv, D, Skv, is_causal);
  rc = launch_status();
  axhip_free(sc);
  return rc;
}

}  // extern "C"
