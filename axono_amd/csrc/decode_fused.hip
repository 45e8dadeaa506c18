// Glue kernels of the captured decode step: per-head q/k RMSNorm + M-RoPE + fp16 store of q + KV
// append in one launch; SiLU-mul over a fused [gate | up] projection; in-place integer increments
// for device-resident lengths and positions.  Each equals the composition of the single operators
// (rms_norm, rope_thd, cast, kv_append; silu_mul; an integer add) and is tested against that
// composition of the oracle.
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kBlock = 256;

struct QkvArgs {
  const float *q, *k, *v;   // rows of the projection output; row strides in elements
  int64_t q_stride, k_stride, v_stride;
  const void *qw, *kw;      // per-head norm weights [D] (may be null), dtype w_f16 ? half : float
  int w_f16;
  float eps;
  const int64_t *pos;       // [3, B]
  const float *inv_freq;    // [D/2]
  int h_lim, w_lim;
  const int32_t *seq_lens;  // [B]: append position
  void *q_out;              // [B, Hq, D]   cache dtype
  void *k_cache, *v_cache;  // [B, Hkv, Lmax, D]
  int B, Hq, Hkv, D, Lmax;
  int S;  // tokens per sequence (1 in a decode step); token r belongs to sequence r / S
};

__device__ __forceinline__ float wload(const void *w, int f16, int i) {
  return f16 ? __half2float(static_cast<const __half *>(w)[i]) : static_cast<const float *>(w)[i];
}

// One wavefront per token and group of `hpw` consecutive heads; heads [0,Hq) are q, [Hq,Hq+Hkv) are k,
// the rest v.  The rotation angles depend on the token and the pair only, so a wavefront computes its
// sincosf values once and applies them to every q / k head of its group (with many tokens hpw grows,
// up to 8: the accurate sincosf is most of this kernel's arithmetic).
// PAIRS = ceil(D/2/64): rotate-half pairs (i, i + D/2) owned by each lane.
template <typename CT, int PAIRS>
__global__ __launch_bounds__(kBlock) void qkv_norm_rope_append_kernel(QkvArgs a, int hpw) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * (kBlock / 64) + (threadIdx.x >> 6);
  const int heads = a.Hq + 2 * a.Hkv;
  const int groups = (heads + hpw - 1) / hpw;
  const int64_t tokens = static_cast<int64_t>(a.B) * a.S;
  if (unit >= tokens * groups) return;  // whole wavefront leaves together
  const int64_t r = unit / groups;      // token
  const int h_begin = static_cast<int>(unit % groups) * hpw, h_end = min(h_begin + hpw, heads);
  const int b = static_cast<int>(r / a.S);
  const int half = a.D / 2;
  const int64_t len = (a.seq_lens ? a.seq_lens[b] : 0) + r % a.S;  // append position of this token
  const bool can_append = len >= 0 && len < a.Lmax;

  float cs[PAIRS], sn[PAIRS];
  if (h_begin < a.Hq + a.Hkv) {  // some head of this group is rotated
    const float pt = static_cast<float>(a.pos[r]);
    const float ph = static_cast<float>(a.pos[tokens + r]);
    const float pw = static_cast<float>(a.pos[2 * tokens + r]);
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
      const int i = lane + p * 64;
      cs[p] = 1.f;
      sn[p] = 0.f;
      if (i >= half) continue;
      const float f = a.inv_freq[i];
      float ang = pt * f;
      if (i % 3 == 1 && i < a.h_lim)
        ang = ph * f;
      else if (i % 3 == 2 && i < a.w_lim)
        ang = pw * f;
      sincosf(ang, &sn[p], &cs[p]);
    }
  }

  for (int h = h_begin; h < h_end; ++h) {
    if (h >= a.Hq + a.Hkv) {  // v: convert and append
      if (!can_append) continue;
      const int hv = h - a.Hq - a.Hkv;
      const float *src = a.v + r * a.v_stride + static_cast<int64_t>(hv) * a.D;
      CT *dst = static_cast<CT *>(a.v_cache) + ((static_cast<int64_t>(b) * a.Hkv + hv) * a.Lmax + len) * a.D;
      for (int i = lane; i < a.D; i += 64) stf(dst + i, src[i]);
      continue;
    }
    const bool is_q = h < a.Hq;
    const int hh = is_q ? h : h - a.Hq;
    const float *src = is_q ? a.q + r * a.q_stride + static_cast<int64_t>(hh) * a.D
                            : a.k + r * a.k_stride + static_cast<int64_t>(hh) * a.D;
    const void *w = is_q ? a.qw : a.kw;
    float lo[PAIRS], hi[PAIRS];
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
      const int i = lane + p * 64;
      lo[p] = i < half ? src[i] : 0.f;
      hi[p] = i < half ? src[i + half] : 0.f;
      ss = __builtin_fmaf(lo[p], lo[p], ss);
      ss = __builtin_fmaf(hi[p], hi[p], ss);
    }
    ss = group_sum<64>(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(a.D) + a.eps);
    CT *dst;
    if (is_q) {
      dst = static_cast<CT *>(a.q_out) + (r * a.Hq + hh) * a.D;
    } else {
      if (!can_append) continue;
      dst = static_cast<CT *>(a.k_cache) + ((static_cast<int64_t>(b) * a.Hkv + hh) * a.Lmax + len) * a.D;
    }
#pragma unroll
    for (int p = 0; p < PAIRS; ++p) {
      const int i = lane + p * 64;
      if (i >= half) continue;
      // same evaluation order as rms_norm then rope_thd: (x * inv) * w, then the rotation
      float x0 = lo[p] * inv, x1 = hi[p] * inv;
      if (w) {
        x0 *= wload(w, a.w_f16, i);
        x1 *= wload(w, a.w_f16, i + half);
      }
      stf(dst + i, x0 * cs[p] - x1 * sn[p]);
      stf(dst + i + half, x1 * cs[p] + x0 * sn[p]);
    }
  }
}

// First operators of a decode step in one launch: h[i, :] = float(table[ids[i], :]) (the embedding row
// widened to the fp32 residual stream) and xn[i, :] = fp16((h * rms) * w), the first RMSNorm.  Same
// arithmetic, in the same order, as axhip_embedding -> axhip_cast -> axhip_rms_norm_ex: 8 elements per
// thread and pass, per-thread fused multiply-add sum of squares, block sum, 1 / sqrt(mean + eps).
constexpr int kEmbedChunks = 4;  // 8-element chunks a thread keeps: dim <= 256 * 8 * 4
template <typename I, typename WT>
__global__ __launch_bounds__(kBlock) void embed_norm_kernel(const I *__restrict__ ids, const __half *__restrict__ table,
                                                            const WT *__restrict__ w, float eps, float *__restrict__ h,
                                                            __half *__restrict__ xn, int64_t vocab, int dim) {
  __shared__ float red[kBlock / 64];
  const int64_t row = blockIdx.x;
  const int64_t id = static_cast<int64_t>(ids[row]);
  const bool valid = id >= 0 && id < vocab;  // out-of-range ids give a zero row, as the gather alone does
  const __half *src = table + (valid ? id : 0) * dim;
  const int nvec = dim / 8;
  float keep[kEmbedChunks][8];
  float ss = 0.f;
  int c = 0;
  for (int i = threadIdx.x; i < nvec; i += kBlock, ++c) {
    float a[8];
    Row8<__half>::load(src + i * 8, a);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      a[j] = valid ? a[j] : 0.f;
      ss = __builtin_fmaf(a[j], a[j], ss);
      keep[c][j] = a[j];
    }
    Row8<float>::store(h + row * dim + i * 8, a);
  }
  ss = block_sum<kBlock / 64>(ss, red);
  const float rms = 1.0f / sqrtf(ss / static_cast<float>(dim) + eps);
  c = 0;
  for (int i = threadIdx.x; i < nvec; i += kBlock, ++c) {
    float wv[8], o[8];
    Row8<WT>::load(w + i * 8, wv);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = keep[c][j] * rms * wv[j];
    Row8<__half>::store(xn + row * dim + i * 8, o);
  }
}

// Last operators of a greedy decode step in one launch (one workgroup): the chosen tokens become the
// next step's input ids, positions and sequence lengths advance by one, and the tokens are appended
// to a device-side log at the row a device-side counter names.
__global__ __launch_bounds__(kBlock) void decode_advance_kernel(const int64_t *__restrict__ next_ids,
                                                                int64_t *__restrict__ ids, int64_t *__restrict__ pos,
                                                                int pos_rows, int32_t *__restrict__ seq_lens,
                                                                int64_t *__restrict__ log, int64_t log_rows,
                                                                unsigned long long *__restrict__ counter, int B) {
  const unsigned long long step = counter ? *counter : 0ull;
  for (int t = threadIdx.x; t < B; t += kBlock) {
    const int64_t id = next_ids[t];
    if (ids) ids[t] = id;
    for (int r = 0; r < pos_rows; ++r) pos[static_cast<int64_t>(r) * B + t] += 1;
    if (seq_lens) seq_lens[t] += 1;
    if (log && step < static_cast<unsigned long long>(log_rows)) log[step * B + t] = id;
  }
  __syncthreads();  // every thread has read the counter
  if (threadIdx.x == 0 && counter) *counter = step + 1;
}

template <typename T, typename OT>
__global__ __launch_bounds__(kBlock) void silu_mul_fused_kernel(const T *__restrict__ gu,
                                                                OT *__restrict__ y, int64_t rows,
                                                                int cols) {
  // gu [rows, 2*cols] = [gate | up]; 8 elements per thread (cols % 8 == 0)
  const int vec_per_row = cols / 8;
  const int64_t total = rows * vec_per_row;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < total; t += stride) {
    const int64_t r = t / vec_per_row;
    const int c = static_cast<int>(t % vec_per_row) * 8;
    float g[8], u[8], o[8];
    Row8<T>::load(gu + r * 2 * cols + c, g);
    Row8<T>::load(gu + r * 2 * cols + cols + c, u);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = g[j] / (1.0f + expf(-g[j])) * u[j];
    Row8<OT>::store(y + r * cols + c, o);
  }
}

template <typename I>
__global__ void index_add_kernel(I *x, int64_t n, int64_t delta) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) x[i] += static_cast<I>(delta);
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API int axhip_qkv_norm_rope_append(const float *q, int64_t q_stride, const float *k,
                                         int64_t k_stride, const float *v, int64_t v_stride,
                                         const void *q_weight, const void *k_weight, int w_dtype,
                                         float eps, const int64_t *pos, const float *inv_freq,
                                         int h_sec, int w_sec, const int32_t *seq_lens, void *q_out,
                                         void *k_cache, void *v_cache, int cache_dtype, int B, int S,
                                         int Hq, int Hkv, int D, int Lmax, axhip_stream stream) {
  if (!is_float_dtype(cache_dtype) || ((q_weight || k_weight) && !is_float_dtype(w_dtype)))
    return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || S <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || D % 2 != 0 || D > 512 || Lmax <= 0)
    return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (!q || !k || !v || !pos || !inv_freq || !q_out || !k_cache || !v_cache)
    return AXHIP_INVALID_PTR;
  QkvArgs a{q, k, v, q_stride, k_stride, v_stride, q_weight, k_weight, w_dtype == AXHIP_FLOAT16, eps,
            pos, inv_freq, h_sec * 3, w_sec * 3, seq_lens, q_out, k_cache, v_cache, B, Hq, Hkv, D, Lmax, S};
  // heads per wavefront: as many (up to 8) as still leave 16384 wavefronts
  const int heads = Hq + 2 * Hkv;
  int hpw = 1;
  while (hpw < 8 && static_cast<int64_t>(B) * S * ((heads + 2 * hpw - 1) / (2 * hpw)) >= 16384) hpw *= 2;
  const int64_t rows = static_cast<int64_t>(B) * S * ((heads + hpw - 1) / hpw);
  const dim3 grid(static_cast<unsigned>((rows + kBlock / 64 - 1) / (kBlock / 64)));
  hipStream_t st = as_stream(stream);
  const int pairs = (D / 2 + 63) / 64;
  const bool f16 = cache_dtype == AXHIP_FLOAT16;
#define AXHIP_QKV_LAUNCH(P)                                                                          \
  do {                                                                                               \
    if (f16)                                                                                         \
      hipLaunchKernelGGL((qkv_norm_rope_append_kernel<__half, P>), grid, dim3(kBlock), 0, st, a, hpw); \
    else                                                                                             \
      hipLaunchKernelGGL((qkv_norm_rope_append_kernel<float, P>), grid, dim3(kBlock), 0, st, a, hpw);  \
  } while (0)
  switch (pairs) {
    case 1: AXHIP_QKV_LAUNCH(1); break;
    case 2: AXHIP_QKV_LAUNCH(2); break;
    default: AXHIP_QKV_LAUNCH(4); break;
  }
#undef AXHIP_QKV_LAUNCH
  return launch_status();
}

AXHIP_API int axhip_silu_mul_fused(const void *gate_up, void *y, int dtype, int out_dtype, int64_t rows,
                                   int64_t cols, axhip_stream stream) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (out_dtype != dtype && !(dtype == AXHIP_FLOAT32 && out_dtype == AXHIP_FLOAT16)) return AXHIP_UNSUPPORTED_TYPE;
  if (rows < 0 || cols <= 0 || cols % 8 != 0) return AXHIP_INVALID_ARGUMENT;
  if (rows == 0) return AXHIP_OK;
  if (!gate_up || !y) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(y)) & 15) return AXHIP_INVALID_ARGUMENT;
  const int64_t total = rows * (cols / 8);
  unsigned grid = static_cast<unsigned>((total + kBlock - 1) / kBlock);
  if (grid > 256u * 16u) grid = 256u * 16u;
  hipStream_t st = as_stream(stream);
  if (dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((silu_mul_fused_kernel<__half, __half>), dim3(grid), dim3(kBlock), 0, st,
                       static_cast<const __half *>(gate_up), static_cast<__half *>(y), rows,
                       static_cast<int>(cols));
  else if (out_dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((silu_mul_fused_kernel<float, __half>), dim3(grid), dim3(kBlock), 0, st,
                       static_cast<const float *>(gate_up), static_cast<__half *>(y), rows,
                       static_cast<int>(cols));
  else
    hipLaunchKernelGGL((silu_mul_fused_kernel<float, float>), dim3(grid), dim3(kBlock), 0, st,
                       static_cast<const float *>(gate_up), static_cast<float *>(y), rows,
                       static_cast<int>(cols));
  return launch_status();
}

AXHIP_API int axhip_embedding_rms_norm(const void *ids, int ids_dtype, const void *table, const void *weight,
                                       int w_dtype, float eps, void *h, void *xn, int64_t n_ids, int64_t vocab,
                                       int64_t dim, axhip_stream stream) {
  if (ids_dtype != AXHIP_INT32 && ids_dtype != AXHIP_INT64) return AXHIP_UNSUPPORTED_TYPE;
  if (w_dtype != AXHIP_FLOAT32 && w_dtype != AXHIP_FLOAT16) return AXHIP_UNSUPPORTED_TYPE;
  if (n_ids < 0 || vocab <= 0 || dim <= 0 || dim % 8 != 0 || dim > kBlock * 8 * kEmbedChunks) return AXHIP_INVALID_ARGUMENT;
  if (n_ids == 0) return AXHIP_OK;
  if (!ids || !table || !weight || !h || !xn) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(h) |
       reinterpret_cast<uintptr_t>(xn)) & 15)
    return AXHIP_INVALID_ARGUMENT;
  const dim3 grid(static_cast<unsigned>(n_ids));
  hipStream_t st = as_stream(stream);
#define AXHIP_EMBED_LAUNCH(I, WT)                                                                      \
  hipLaunchKernelGGL((embed_norm_kernel<I, WT>), grid, dim3(kBlock), 0, st, static_cast<const I *>(ids), \
                     static_cast<const __half *>(table), static_cast<const WT *>(weight), eps,          \
                     static_cast<float *>(h), static_cast<__half *>(xn), vocab, static_cast<int>(dim))
  if (ids_dtype == AXHIP_INT64) {
    if (w_dtype == AXHIP_FLOAT16) AXHIP_EMBED_LAUNCH(int64_t, __half); else AXHIP_EMBED_LAUNCH(int64_t, float);
  } else {
    if (w_dtype == AXHIP_FLOAT16) AXHIP_EMBED_LAUNCH(int32_t, __half); else AXHIP_EMBED_LAUNCH(int32_t, float);
  }
#undef AXHIP_EMBED_LAUNCH
  return launch_status();
}

AXHIP_API int axhip_decode_advance(const int64_t *next_ids, int64_t *ids, int64_t *pos, int pos_rows,
                                   int32_t *seq_lens, int64_t *log, int64_t log_rows, uint64_t *counter, int B,
                                   axhip_stream stream) {
  if (B < 0 || pos_rows < 0 || log_rows < 0) return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (!next_ids || (pos_rows > 0 && !pos)) return AXHIP_INVALID_PTR;
  hipLaunchKernelGGL(decode_advance_kernel, dim3(1), dim3(kBlock), 0, as_stream(stream), next_ids, ids, pos, pos_rows,
                     seq_lens, log, log_rows, reinterpret_cast<unsigned long long *>(counter), B);
  return launch_status();
}

AXHIP_API int axhip_index_add(void *x, int dtype, int64_t n, int64_t delta, axhip_stream stream) {
  if (dtype != AXHIP_INT32 && dtype != AXHIP_INT64) return AXHIP_UNSUPPORTED_TYPE;
  if (n < 0) return AXHIP_INVALID_ARGUMENT;
  if (n == 0) return AXHIP_OK;
  if (!x) return AXHIP_INVALID_PTR;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  hipStream_t st = as_stream(stream);
  if (dtype == AXHIP_INT32)
    hipLaunchKernelGGL((index_add_kernel<int32_t>), grid, dim3(256), 0, st, static_cast<int32_t *>(x), n, delta);
  else
    hipLaunchKernelGGL((index_add_kernel<int64_t>), grid, dim3(256), 0, st, static_cast<int64_t *>(x), n, delta);
  return launch_status();
}

}  // extern "C"
