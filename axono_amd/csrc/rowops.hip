// Bandwidth-bound row-wise and elementwise operators of the decode step: add_rms_norm, rms_norm,
// silu_mul, add, fp16<->fp32 cast, the rotary family, KV-cache append, concat, embedding, argmax.
//
// All of them move each byte once with 16-byte accesses (8 fp16 or 2x4 fp32 elements per lane),
// compute in fp32 and round once at the final store.  At decode sizes (tens of rows) they are
// launch-latency bound; the layouts are chosen so the same kernels stream at HBM speed when the
// row count is large (prefill).
#include <cmath>

#include "common.hpp"

namespace axhip {
namespace {

constexpr int kBlock = 256;

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

inline unsigned blocks_for(int64_t items, int per_block) {
  return static_cast<unsigned>((items + per_block - 1) / per_block);
}

// ------------------------------------------------------------------------------------------------
// add_rms_norm / rms_norm.  TPR threads cooperate on one row (64: one wavefront, for short rows
// such as per-head q/k norm; 256: the whole workgroup).  Each thread owns 8-element chunks at
// stride TPR*8 and keeps up to kRegChunks of them in registers between the two passes.
// ------------------------------------------------------------------------------------------------
constexpr int kRegChunks = 4;

template <typename T, typename WT, typename OT, int TPR, bool ADD>
__global__ __launch_bounds__(kBlock) void rms_norm_kernel(const T *__restrict__ x,
                                                          const T *__restrict__ res,
                                                          const WT *__restrict__ w, float eps,
                                                          T *__restrict__ y, OT *__restrict__ out,
                                                          int64_t rows, int hidden, int vec_ok) {
  constexpr int RPB = kBlock / TPR;
  __shared__ float red[kBlock / 64];
  const int lane = threadIdx.x % TPR;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * RPB + threadIdx.x / TPR;
  const bool live = row < rows;
  const int64_t off = (live ? row : 0) * hidden;
  // whole 8-element chunks (only when rows start on 16-byte boundaries); the rest goes element by element
  const int nvec = vec_ok ? hidden / 8 : 0;

  float keep[kRegChunks][8];
  float ss = 0.0f;
  if (live) {
    int c = 0;
    for (int i = lane; i < nvec; i += TPR, ++c) {
      float a[8];
      Row8<T>::load_stream(x + off + i * 8, a);
      if (ADD) {
        float r[8];
        Row8<T>::load_stream(res + off + i * 8, r);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] += r[j];
        Row8<T>::store_stream(y + off + i * 8, a);  // the only rounding of y; the norm uses the fp32 sum
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(a[j], a[j], ss);
      if (c < kRegChunks) {
#pragma unroll
        for (int j = 0; j < 8; ++j) keep[c][j] = a[j];
      }
    }
    for (int i = nvec * 8 + lane; i < hidden; i += TPR) {
      float a = ldf(x + off + i);
      if (ADD) {
        a += ldf(res + off + i);
        stf(y + off + i, a);
      }
      ss = __builtin_fmaf(a, a, ss);
    }
  }
  if (TPR == 64)
    ss = group_sum<64>(ss);
  else
    ss = block_sum<kBlock / 64>(ss, red);
  if (!live) return;
  const float rms = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
  int c = 0;
  for (int i = lane; i < nvec; i += TPR, ++c) {
    float a[8], o[8];
    if (c < kRegChunks) {
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] = keep[c][j];
    } else {  // recompute the fp32 sum rather than read back the rounded y
      Row8<T>::load(x + off + i * 8, a);
      if (ADD) {
        float r[8];
        Row8<T>::load(res + off + i * 8, r);
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] += r[j];
      }
    }
    if (w) {
      float wv[8];
      Row8<WT>::load(w + i * 8, wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = a[j] * rms * wv[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = a[j] * rms;
    }
    Row8<OT>::store_stream(out + off + i * 8, o);
  }
  for (int i = nvec * 8 + lane; i < hidden; i += TPR) {
    float a = ldf(x + off + i);
    if (ADD) a += ldf(res + off + i);
    stf(out + off + i, w ? a * rms * ldf(w + i) : a * rms);
  }
}

template <typename T, typename WT, typename OT, bool ADD>
int launch_rms(const void *x, const void *res, const void *w, float eps, void *y, void *out,
               int64_t rows, int64_t hidden, hipStream_t st) {
  // rows of both element sizes must start on 16-byte boundaries, else every element goes through
  // the scalar path
  const int vec_ok = (hidden * sizeof(T)) % 16 == 0 && (hidden * sizeof(OT)) % 16 == 0;
  const T *xp = static_cast<const T *>(x), *rp = static_cast<const T *>(res);
  const WT *wp = static_cast<const WT *>(w);
  T *yp = static_cast<T *>(y);
  OT *op = static_cast<OT *>(out);
  if (hidden <= 512) {
    hipLaunchKernelGGL((rms_norm_kernel<T, WT, OT, 64, ADD>), dim3(blocks_for(rows, kBlock / 64)),
                       dim3(kBlock), 0, st, xp, rp, wp, eps, yp, op, rows, static_cast<int>(hidden), vec_ok);
  } else {
    hipLaunchKernelGGL((rms_norm_kernel<T, WT, OT, kBlock, ADD>), dim3(static_cast<unsigned>(rows)),
                       dim3(kBlock), 0, st, xp, rp, wp, eps, yp, op, rows, static_cast<int>(hidden), vec_ok);
  }
  return launch_status();
}

template <bool ADD>
int dispatch_rms(const void *x, const void *res, const void *w, float eps, void *y, void *out,
                 int dtype, int w_dtype, int out_dtype, int64_t rows, int64_t hidden, hipStream_t st) {
  if (!is_float_dtype(dtype) || (w && !is_float_dtype(w_dtype))) return AXHIP_UNSUPPORTED_TYPE;
  // the normalised output may be FLOAT16 while the activations are FLOAT32 (it feeds an fp16 Linear)
  if (out_dtype != dtype && !(dtype == AXHIP_FLOAT32 && out_dtype == AXHIP_FLOAT16)) return AXHIP_UNSUPPORTED_TYPE;
  if (rows < 0 || hidden <= 0 || hidden > (1 << 24)) return AXHIP_INVALID_ARGUMENT;
  if (rows == 0) return AXHIP_OK;
  if (!x || !out || (ADD && (!res || !y))) return AXHIP_INVALID_PTR;
  // 16-byte row accesses need aligned bases and rows that start on 16-byte boundaries
  const int64_t esz = dtype == AXHIP_FLOAT16 ? 2 : 4;
  if (!aligned16(x) || !aligned16(out) || (ADD && (!aligned16(res) || !aligned16(y))) ||
      (w && !aligned16(w)))
    return AXHIP_INVALID_ARGUMENT;
  (void)esz;
  const bool wh = w && w_dtype == AXHIP_FLOAT16;
  if (dtype == AXHIP_FLOAT16)
    return wh ? launch_rms<__half, __half, __half, ADD>(x, res, w, eps, y, out, rows, hidden, st)
              : launch_rms<__half, float, __half, ADD>(x, res, w, eps, y, out, rows, hidden, st);
  if (out_dtype == AXHIP_FLOAT16)
    return wh ? launch_rms<float, __half, __half, ADD>(x, res, w, eps, y, out, rows, hidden, st)
              : launch_rms<float, float, __half, ADD>(x, res, w, eps, y, out, rows, hidden, st);
  return wh ? launch_rms<float, __half, float, ADD>(x, res, w, eps, y, out, rows, hidden, st)
            : launch_rms<float, float, float, ADD>(x, res, w, eps, y, out, rows, hidden, st);
}

// ------------------------------------------------------------------------------------------------
// Flat elementwise kernels: 8 elements per thread, scalar tail.
// ------------------------------------------------------------------------------------------------
struct SiluMulOp {
  static __device__ __forceinline__ float apply(float g, float u) { return g / (1.0f + expf(-g)) * u; }
};
struct AddOp {
  static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};

// STREAM: operands larger than the caches are read and written once with streaming accesses.
template <typename T, typename OP, bool STREAM>
__global__ __launch_bounds__(kBlock) void binary_kernel(const T *__restrict__ a,
                                                        const T *__restrict__ b,
                                                        T *__restrict__ y, int64_t n) {
  constexpr int UN = 4;  // independent 16-byte groups per thread and pass
  const int64_t nvec = n / 8;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock * UN;
  int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock * UN + threadIdx.x;
  for (; i + (UN - 1) * kBlock < nvec; i += stride) {
    float fa[UN][8], fb[UN][8];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (STREAM) {
        Row8<T>::load_stream(a + (i + u * kBlock) * 8, fa[u]);
        Row8<T>::load_stream(b + (i + u * kBlock) * 8, fb[u]);
      } else {
        Row8<T>::load(a + (i + u * kBlock) * 8, fa[u]);
        Row8<T>::load(b + (i + u * kBlock) * 8, fb[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      float fy[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) fy[j] = OP::apply(fa[u][j], fb[u][j]);
      if (STREAM)
        Row8<T>::store_stream(y + (i + u * kBlock) * 8, fy);
      else
        Row8<T>::store(y + (i + u * kBlock) * 8, fy);
    }
  }
  // the last, incomplete pass: i is this thread's first group of it (or lies past the end)
  for (int u = 0; u < UN; ++u) {
    const int64_t idx = i + u * kBlock;
    if (idx >= nvec) break;
    float fa[8], fb[8], fy[8];
    Row8<T>::load(a + idx * 8, fa);
    Row8<T>::load(b + idx * 8, fb);
#pragma unroll
    for (int j = 0; j < 8; ++j) fy[j] = OP::apply(fa[j], fb[j]);
    Row8<T>::store(y + idx * 8, fy);
  }
  if (blockIdx.x == 0) {
    for (int64_t e = nvec * 8 + threadIdx.x; e < n; e += kBlock)
      stf(y + e, OP::apply(ldf(a + e), ldf(b + e)));
  }
}

template <typename OP>
int launch_binary(const void *a, const void *b, void *y, int dtype, int64_t n, hipStream_t st) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (n < 0) return AXHIP_INVALID_ARGUMENT;
  if (n == 0) return AXHIP_OK;
  if (!a || !b || !y) return AXHIP_INVALID_PTR;
  if (!aligned16(a) || !aligned16(b) || !aligned16(y)) return AXHIP_INVALID_ARGUMENT;
  const int64_t nvec = n / 8;
  unsigned grid = blocks_for(nvec > 0 ? (nvec + 3) / 4 : 1, kBlock);  // four groups per thread and pass
  if (grid > 256u * 16u) grid = 256u * 16u;
  // three arrays that together exceed the 256 MB memory-side cache are touched once: streaming accesses
  const bool stream = 3 * n * (dtype == AXHIP_FLOAT16 ? 2 : 4) > (int64_t(256) << 20);
#define AXHIP_BINARY_LAUNCH(T, S)                                                                      \
  hipLaunchKernelGGL((binary_kernel<T, OP, S>), dim3(grid), dim3(kBlock), 0, st, static_cast<const T *>(a), \
                     static_cast<const T *>(b), static_cast<T *>(y), n)
  if (dtype == AXHIP_FLOAT16) {
    if (stream) AXHIP_BINARY_LAUNCH(__half, true); else AXHIP_BINARY_LAUNCH(__half, false);
  } else {
    if (stream) AXHIP_BINARY_LAUNCH(float, true); else AXHIP_BINARY_LAUNCH(float, false);
  }
#undef AXHIP_BINARY_LAUNCH
  return launch_status();
}

template <typename S, typename Dt>
__global__ __launch_bounds__(kBlock) void cast_kernel(const S *__restrict__ src,
                                                      Dt *__restrict__ dst, int64_t n) {
  const int64_t nvec = n / 8;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < nvec; i += stride) {
    float f[8];
    Row8<S>::load_stream(src + i * 8, f);
    Row8<Dt>::store_stream(dst + i * 8, f);
  }
  if (blockIdx.x == 0) {
    for (int64_t i = nvec * 8 + threadIdx.x; i < n; i += kBlock) stf(dst + i, ldf(src + i));
  }
}

// Plain 16-byte copy / fill (graph-capturable replacements for memcpy / memset nodes).
__global__ __launch_bounds__(kBlock) void copy_bytes_kernel(const uint8_t *__restrict__ src,
                                                            uint8_t *__restrict__ dst, int64_t n,
                                                            int vec_ok) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (vec_ok) {
    const int64_t nvec = n / 16;
    for (int64_t i = t; i < nvec; i += stride) st16_stream(dst + i * 16, ld16_stream(src + i * 16));
    for (int64_t i = nvec * 16 + t; i < n; i += stride) dst[i] = src[i];
  } else {
    for (int64_t i = t; i < n; i += stride) dst[i] = src[i];
  }
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(uint8_t *__restrict__ dst, int64_t n,
                                                           int64_t head) {
  // `head` unaligned leading bytes, then 16-byte stores, then the tail
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t < head) dst[t] = 0;
  uint8_t *body = dst + head;
  const int64_t nb = n - head, nvec = nb / 16;
  Vec16 z;
  z.w[0] = z.w[1] = z.w[2] = z.w[3] = 0u;
  for (int64_t i = t; i < nvec; i += stride) st16(body + i * 16, z);
  for (int64_t i = nvec * 16 + t; i < nb; i += stride) body[i] = 0;
}

int launch_copy(const void *src, void *dst, int64_t n, hipStream_t st) {
  if (n <= 0) return AXHIP_OK;
  const int vec_ok = aligned16(src) && aligned16(dst);
  unsigned grid = blocks_for((n + 15) / 16, kBlock);
  if (grid > 256u * 16u) grid = 256u * 16u;
  hipLaunchKernelGGL(copy_bytes_kernel, dim3(grid), dim3(kBlock), 0, st,
                     static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), n, vec_ok);
  return launch_status();
}

// ------------------------------------------------------------------------------------------------
// Rotary embeddings.  One thread rotates 8 pairs (i, i + dim/2) of one (row, head).
// ------------------------------------------------------------------------------------------------
constexpr int kMaxHalf = 256;
struct FreqTable {
  float f[kMaxHalf];
};

enum RopeMode { kRopeTheta = 0, kRopeThd = 1, kRopeTable = 2 };

struct RopeArgs {
  const void *x;
  void *out;
  const int64_t *pos;     // [rows] (theta) or [3, rows] (thd)
  const float *inv_freq;  // device [half] (thd)
  const float *cos_t;     // device [rows, dim] (table)
  const float *sin_t;
  int64_t rows;
  int heads, dim, h_lim, w_lim;
};

// One thread rotates 8 pairs (i, i + dim/2) of `hpt` consecutive heads of one row: the angles depend on
// (row, i) only, so the accurate sincosf - most of this kernel's arithmetic - is paid once per hpt heads.
template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void rope_kernel(RopeArgs a, FreqTable ft, int hpt) {
  const int half = a.dim / 2;
  const int chunks = (half + 7) / 8;  // 8-pair chunks per (row, head)
  const int hgroups = a.heads / hpt;
  const int64_t total = a.rows * hgroups * chunks;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t >= total) return;
  const int ch = static_cast<int>(t % chunks);
  const int64_t rg = t / chunks;
  const int64_t row = rg / hgroups;
  const int64_t rh0 = row * a.heads + (rg % hgroups) * hpt;  // first (row, head) of this thread
  float pt = 0.f, ph = 0.f, pw = 0.f;
  if (MODE == kRopeTheta) pt = static_cast<float>(a.pos[row]);
  if (MODE == kRopeThd) {
    pt = static_cast<float>(a.pos[row]);
    ph = static_cast<float>(a.pos[a.rows + row]);
    pw = static_cast<float>(a.pos[2 * a.rows + row]);
  }
  const int i0 = ch * 8;
  const bool full = (i0 + 8 <= half) && (half % 8 == 0) && (sizeof(T) * a.dim % 16 == 0);
  float c_lo[8], s_lo[8], c_hi[8], s_hi[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = i0 + j;
    if (MODE == kRopeTable) {
      const bool in = i < half;
      const float *cr = a.cos_t + row * a.dim, *sr = a.sin_t + row * a.dim;
      c_lo[j] = in ? cr[i] : 1.f;
      s_lo[j] = in ? sr[i] : 0.f;
      c_hi[j] = in ? cr[i + half] : 1.f;
      s_hi[j] = in ? sr[i + half] : 0.f;
    } else {
      float f, ang;
      if (MODE == kRopeTheta) {
        f = ft.f[i < kMaxHalf ? i : 0];
        ang = pt * f;
      } else {
        f = i < half ? a.inv_freq[i] : 0.f;
        ang = pt * f;
        if (i % 3 == 1 && i < a.h_lim)
          ang = ph * f;
        else if (i % 3 == 2 && i < a.w_lim)
          ang = pw * f;
      }
      sincosf(ang, &s_lo[j], &c_lo[j]);
      c_hi[j] = c_lo[j];
      s_hi[j] = s_lo[j];
    }
  }
  for (int hh = 0; hh < hpt; ++hh) {
    const T *src = static_cast<const T *>(a.x) + (rh0 + hh) * a.dim;
    T *dst = static_cast<T *>(a.out) + (rh0 + hh) * a.dim;
    float lo[8], hi[8];
    if (full) {
      Row8<T>::load(src + i0, lo);
      Row8<T>::load(src + i0 + half, hi);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        lo[j] = (i0 + j < half) ? ldf(src + i0 + j) : 0.f;
        hi[j] = (i0 + j < half) ? ldf(src + i0 + j + half) : 0.f;
      }
    }
    float olo[8], ohi[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      olo[j] = lo[j] * c_lo[j] - hi[j] * s_lo[j];
      ohi[j] = hi[j] * c_hi[j] + lo[j] * s_hi[j];
    }
    if (full) {
      Row8<T>::store(dst + i0, olo);
      Row8<T>::store(dst + i0 + half, ohi);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (i0 + j < half) {
          stf(dst + i0 + j, olo[j]);
          stf(dst + i0 + j + half, ohi[j]);
        }
      }
    }
  }
}

// Row-blocked form for the common case (dim/2 a multiple of 8, at most 256, rows 16-byte aligned): a
// workgroup takes RPW = 256 / (dim/2) rows (at least one), first evaluates each row's dim/2 angles once -
// one accurate sincosf per thread - into LDS, then rotates every head of those rows, of one tensor or of
// two that share the positions (q and k of a layer: one launch), 16 bytes per access.  The angle
// arithmetic, which bounds the per-thread form above (one sincosf per 8 elements of a head), is paid
// once per row instead of once per head.
struct RopeRowsArgs {
  const void *x1, *x2;   // [rows, heads1, dim], [rows, heads2, dim] (x2 may be null with heads2 = 0)
  void *out1, *out2;
  const int64_t *pos;
  const float *inv_freq;
  int64_t rows;
  int heads1, heads2, dim, h_lim, w_lim;
};

template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void rope_rows_kernel(RopeRowsArgs a, FreqTable ft) {
  const int half = a.dim / 2;
  const int rpw = half >= kBlock ? 1 : kBlock / half;  // rows per workgroup
  __shared__ float s_cos[kBlock], s_sin[kBlock];
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * rpw;
  const int tid = threadIdx.x;
  if (tid < rpw * half) {
    const int r = tid / half, i = tid - r * half;
    const int64_t row = row0 + r;
    float sn = 0.f, cs = 1.f;
    if (row < a.rows) {
      float ang;
      if (MODE == kRopeTheta) {
        ang = static_cast<float>(a.pos[row]) * ft.f[i];
      } else {
        const float f = a.inv_freq[i];
        const int64_t *p = a.pos + row;
        if (i % 3 == 1 && i < a.h_lim) p += a.rows;
        else if (i % 3 == 2 && i < a.w_lim) p += 2 * a.rows;
        ang = static_cast<float>(*p) * f;
      }
      sincosf(ang, &sn, &cs);
    }
    s_cos[tid] = cs;
    s_sin[tid] = sn;
  }
  __syncthreads();
  const int chunks = half / 8;
  const int heads = a.heads1 + a.heads2;
  const int per_row = heads * chunks;
  const int items = rpw * per_row;
  for (int it = tid; it < items; it += kBlock) {
    const int r = it / per_row, rem = it - r * per_row;
    const int64_t row = row0 + r;
    if (row >= a.rows) break;
    const int hd = rem / chunks, ch = rem - hd * chunks;
    const bool second = hd >= a.heads1;
    const int64_t off = second ? (row * a.heads2 + (hd - a.heads1)) * a.dim : (row * a.heads1 + hd) * a.dim;
    const T *src = static_cast<const T *>(second ? a.x2 : a.x1) + off + ch * 8;
    T *dst = static_cast<T *>(second ? a.out2 : a.out1) + off + ch * 8;
    float lo[8], hi[8], olo[8], ohi[8];
    Row8<T>::load_stream(src, lo);
    Row8<T>::load_stream(src + half, hi);
    const float *c = s_cos + r * half + ch * 8, *sn = s_sin + r * half + ch * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      olo[j] = lo[j] * c[j] - hi[j] * sn[j];
      ohi[j] = hi[j] * c[j] + lo[j] * sn[j];
    }
    Row8<T>::store_stream(dst, olo);
    Row8<T>::store_stream(dst + half, ohi);
  }
}

template <int MODE>
int launch_rope_rows(const RopeRowsArgs &a, const FreqTable &ft, int dtype, hipStream_t st) {
  const int half = a.dim / 2;
  const int rpw = half >= kBlock ? 1 : kBlock / half;
  const unsigned grid = static_cast<unsigned>((a.rows + rpw - 1) / rpw);
  if (dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((rope_rows_kernel<__half, MODE>), dim3(grid), dim3(kBlock), 0, st, a, ft);
  else
    hipLaunchKernelGGL((rope_rows_kernel<float, MODE>), dim3(grid), dim3(kBlock), 0, st, a, ft);
  return launch_status();
}

// Whether the row-blocked kernel applies: whole 8-pair chunks, 16-byte aligned head rows.
inline bool rope_rows_ok(int dtype, int64_t dim, const void *x, const void *out) {
  const int64_t half = dim / 2, esz = dtype == AXHIP_FLOAT16 ? 2 : 4;
  return half % 8 == 0 && half <= kMaxHalf && (dim * esz) % 16 == 0 && (half * esz) % 16 == 0 && aligned16(x) && aligned16(out);
}

template <int MODE>
int launch_rope(const RopeArgs &a, const FreqTable &ft, int dtype, hipStream_t st) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (a.dim % 2 != 0 || a.dim <= 0 || a.heads <= 0 || a.rows < 0) return AXHIP_INVALID_ARGUMENT;
  if (a.rows == 0) return AXHIP_OK;
  if (!a.x || !a.out) return AXHIP_INVALID_PTR;
  if (!aligned16(a.x) || !aligned16(a.out)) return AXHIP_INVALID_ARGUMENT;
  if (MODE != kRopeTable && rope_rows_ok(dtype, a.dim, a.x, a.out) && a.rows < (int64_t(1) << 31)) {
    RopeRowsArgs r{a.x, nullptr, a.out, nullptr, a.pos, a.inv_freq, a.rows, a.heads, 0, a.dim, a.h_lim, a.w_lim};
    return launch_rope_rows<(MODE == kRopeTable ? kRopeTheta : MODE)>(r, ft, dtype, st);
  }
  const int chunks = (a.dim / 2 + 7) / 8;
  // heads per thread: as many as still leave about a thousand workgroups
  int hpt = 1;
  while (hpt < 8 && a.heads % (hpt * 2) == 0 && a.rows * (a.heads / (hpt * 2)) * chunks >= (1 << 18)) hpt *= 2;
  const unsigned grid = blocks_for(a.rows * (a.heads / hpt) * chunks, kBlock);
  if (dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((rope_kernel<__half, MODE>), dim3(grid), dim3(kBlock), 0, st, a, ft, hpt);
  else
    hipLaunchKernelGGL((rope_kernel<float, MODE>), dim3(grid), dim3(kBlock), 0, st, a, ft, hpt);
  return launch_status();
}

__global__ __launch_bounds__(kBlock) void mrope_cos_sin_kernel(const int64_t *__restrict__ pos,
                                                               const float *__restrict__ inv_freq,
                                                               int h_lim, int w_lim,
                                                               float *__restrict__ cos_out,
                                                               float *__restrict__ sin_out,
                                                               int64_t rows, int half) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t >= rows * half) return;
  const int i = static_cast<int>(t % half);
  const int64_t r = t / half;
  const float f = inv_freq[i];
  float ang = static_cast<float>(pos[r]) * f;
  if (i % 3 == 1 && i < h_lim)
    ang = static_cast<float>(pos[rows + r]) * f;
  else if (i % 3 == 2 && i < w_lim)
    ang = static_cast<float>(pos[2 * rows + r]) * f;
  float s, c;
  sincosf(ang, &s, &c);
  float *cr = cos_out + r * 2 * half, *sr = sin_out + r * 2 * half;
  cr[i] = c;
  cr[i + half] = c;
  sr[i] = s;
  sr[i + half] = s;
}

// ------------------------------------------------------------------------------------------------
// KV-cache append: cache[b, hk, pos[b], :] = new[b, hk, :] for K and V, 16 bytes per thread.
// ------------------------------------------------------------------------------------------------
template <typename P>
__global__ __launch_bounds__(kBlock) void kv_append_kernel(const uint8_t *__restrict__ k_new,
                                                           const uint8_t *__restrict__ v_new,
                                                           uint8_t *__restrict__ k_cache,
                                                           uint8_t *__restrict__ v_cache,
                                                           const P *__restrict__ pos, int B, int Hkv,
                                                           int Lmax, int row_bytes) {
  const int vec_per_row = row_bytes / 16;
  const int64_t total = static_cast<int64_t>(B) * Hkv * vec_per_row;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t >= total) return;
  const int vi = static_cast<int>(t % vec_per_row);
  const int64_t bh = t / vec_per_row;
  const int b = static_cast<int>(bh / Hkv);
  const int64_t p = static_cast<int64_t>(pos[b]);
  if (p < 0 || p >= Lmax) return;
  const int64_t src = bh * row_bytes + vi * 16;
  const int64_t dst = (bh * Lmax + p) * row_bytes + vi * 16;
  st16(k_cache + dst, ld16(k_new + src));
  st16(v_cache + dst, ld16(v_new + src));
}

// Paged form: token t of sequence b (rows [B, S, Hkv, row_bytes], token-major) goes to key position
// start[b] + t, i.e. row (position % 128) of page page_table[b, position / 128] of pools
// [n_pages, Hkv, 128, row_bytes].  Positions past the table and page numbers outside the pool are skipped.
template <typename P>
__global__ __launch_bounds__(kBlock) void kv_append_paged_kernel(const uint8_t *__restrict__ k_new,
                                                                 const uint8_t *__restrict__ v_new,
                                                                 uint8_t *__restrict__ k_pool, uint8_t *__restrict__ v_pool,
                                                                 const int32_t *__restrict__ page_table,
                                                                 const P *__restrict__ start, int B, int S, int Hkv,
                                                                 int row_bytes, int max_pages, int n_pages) {
  const int vec_per_row = row_bytes / 16;
  const int64_t total = static_cast<int64_t>(B) * S * Hkv * vec_per_row;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t >= total) return;
  const int vi = static_cast<int>(t % vec_per_row);
  const int64_t th = t / vec_per_row;       // (b, token, head)
  const int hk = static_cast<int>(th % Hkv);
  const int64_t bt = th / Hkv;
  const int b = static_cast<int>(bt / S);
  const int64_t p = (start ? static_cast<int64_t>(start[b]) : 0) + (bt - static_cast<int64_t>(b) * S);
  if (p < 0 || (p >> 7) >= max_pages) return;
  const int pid = page_table[static_cast<int64_t>(b) * max_pages + (p >> 7)];
  if (pid < 0 || pid >= n_pages) return;
  const int64_t src = th * row_bytes + vi * 16;
  const int64_t dst = ((static_cast<int64_t>(pid) * Hkv + hk) * 128 + (p & 127)) * row_bytes + vi * 16;
  st16(k_pool + dst, ld16(k_new + src));
  st16(v_pool + dst, ld16(v_new + src));
}

// Dense cache [B, Hkv, rows, row_bytes] -> pages: key positions 0 .. lens[b]-1 (all `rows` when lens is null) of
// every sequence are copied to row (position % 128) of page page_table[b, position / 128].
__global__ __launch_bounds__(kBlock) void kv_dense_to_paged_kernel(const uint8_t *__restrict__ k_dense,
                                                                   const uint8_t *__restrict__ v_dense,
                                                                   uint8_t *__restrict__ k_pool, uint8_t *__restrict__ v_pool,
                                                                   const int32_t *__restrict__ page_table,
                                                                   const int32_t *__restrict__ lens, int B, int Hkv, int rows,
                                                                   int row_bytes, int max_pages, int n_pages) {
  const int vec_per_row = row_bytes / 16;
  const int64_t total = static_cast<int64_t>(B) * Hkv * rows * vec_per_row;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; t < total; t += stride) {
    const int vi = static_cast<int>(t % vec_per_row);
    const int64_t r = t / vec_per_row;                 // (b, head, position)
    const int p = static_cast<int>(r % rows);
    const int64_t bh = r / rows;
    const int hk = static_cast<int>(bh % Hkv), b = static_cast<int>(bh / Hkv);
    if (lens && p >= lens[b]) continue;
    if ((p >> 7) >= max_pages) continue;
    const int pid = page_table[static_cast<int64_t>(b) * max_pages + (p >> 7)];
    if (pid < 0 || pid >= n_pages) continue;
    const int64_t src = r * row_bytes + vi * 16;
    const int64_t dst = ((static_cast<int64_t>(pid) * Hkv + hk) * 128 + (p & 127)) * row_bytes + vi * 16;
    st16(k_pool + dst, ld16(k_dense + src));
    st16(v_pool + dst, ld16(v_dense + src));
  }
}

// ------------------------------------------------------------------------------------------------
// Embedding gather and argmax.
// ------------------------------------------------------------------------------------------------
template <typename I>
__global__ __launch_bounds__(kBlock) void embedding_kernel(const I *__restrict__ ids,
                                                           const uint8_t *__restrict__ table,
                                                           uint8_t *__restrict__ out, int64_t vocab,
                                                           int64_t row_bytes, int vec_ok) {
  const int64_t i = blockIdx.x;
  int64_t id = static_cast<int64_t>(ids[i]);
  const bool valid = id >= 0 && id < vocab;  // out-of-range ids give a zero row instead of a fault
  const uint8_t *src = table + (valid ? id : 0) * row_bytes;
  uint8_t *dst = out + i * row_bytes;
  if (vec_ok) {
    Vec16 z;
    z.w[0] = z.w[1] = z.w[2] = z.w[3] = 0u;
    for (int64_t o = threadIdx.x * 16; o < row_bytes; o += kBlock * 16)
      st16(dst + o, valid ? ld16(src + o) : z);
  } else {
    for (int64_t o = threadIdx.x; o < row_bytes; o += kBlock) dst[o] = valid ? src[o] : 0;
  }
}

constexpr int kArgmaxBlock = 1024;

template <typename T>
__global__ __launch_bounds__(kArgmaxBlock) void argmax_kernel(const T *__restrict__ x,
                                                              int64_t *__restrict__ out,
                                                              int64_t cols) {
  __shared__ float s_val[kArgmaxBlock / 64];
  __shared__ int64_t s_idx[kArgmaxBlock / 64];
  const T *row = x + static_cast<int64_t>(blockIdx.x) * cols;
  float best = -INFINITY;
  int64_t bi = INT64_MAX;
  // strided scan keeps indices increasing per thread, so `>` keeps the first maximum
  for (int64_t c = threadIdx.x; c < cols; c += kArgmaxBlock) {
    const float v = ldf(row + c);
    if (v > best || bi == INT64_MAX) {
      best = v;
      bi = c;
    }
  }
  // wavefront then block reduction; ties go to the smaller index
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int64_t oi = __shfl_xor(bi, off, 64);
    if (oi != INT64_MAX && (bi == INT64_MAX || ov > best || (ov == best && oi < bi))) {
      best = ov;
      bi = oi;
    }
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    s_val[wave] = best;
    s_idx[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxBlock / 64; ++w) {
      const float ov = s_val[w];
      const int64_t oi = s_idx[w];
      if (oi != INT64_MAX && (bi == INT64_MAX || ov > best || (ov == best && oi < bi))) {
        best = ov;
        bi = oi;
      }
    }
    out[blockIdx.x] = bi == INT64_MAX ? 0 : bi;
  }
}

// Wide rows (a vocabulary): kArgmaxParts workgroups scan one row's column ranges, park their
// (value, index) candidates in device scratch, and the workgroup that takes the last ticket of the row
// picks the winner.  Ties go to the smaller index, as in the single-workgroup kernel.
constexpr int kArgmaxParts = 64;
constexpr int kArgmaxMaxRows = 1024;  // per ticket lane
__device__ float g_argmax_val[AXHIP_TICKET_LANES * kArgmaxMaxRows * kArgmaxParts];
__device__ long long g_argmax_idx[AXHIP_TICKET_LANES * kArgmaxMaxRows * kArgmaxParts];
__device__ unsigned int g_argmax_ticket[AXHIP_TICKET_LANES * kArgmaxMaxRows];
// Atomics on one 128-byte line are served one after the other (about 10 ns each on MI355X; 64 workgroups x 16
// rows on one line cost 10 us): neighbouring rows take counters 128 bytes apart, the words in between belong to
// rows 32, 64, ... further on.
__device__ __forceinline__ unsigned int *argmax_ticket_of(int lane_row0, int row) {
  return &g_argmax_ticket[lane_row0 + (((row & 31) << 5) | (row >> 5))];
}
}  // namespace
int reset_argmax_tickets() {
  void *p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_argmax_ticket)) != hipSuccess || !p) return AXHIP_DEVICE_ERROR;
  if (hipDeviceSynchronize() != hipSuccess) return AXHIP_DEVICE_ERROR;
  return hipMemset(p, 0, sizeof(unsigned int) * AXHIP_TICKET_LANES * kArgmaxMaxRows) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}
namespace {

__device__ __forceinline__ bool better(float ov, int64_t oi, float v, int64_t i) {
  return oi != INT64_MAX && (i == INT64_MAX || ov > v || (ov == v && oi < i));
}

template <typename T>
__global__ __launch_bounds__(kBlock) void argmax_parts_kernel(const T *__restrict__ x,
                                                              int64_t *__restrict__ out, int64_t cols, int vec_ok,
                                                              int lane_row0) {
  __shared__ float s_val[kBlock / 64];
  __shared__ int64_t s_idx[kBlock / 64];
  __shared__ int s_last;
  const int row = blockIdx.y, part = blockIdx.x;
  const int trow = lane_row0 + row;  // this row's place in the caller's ticket lane
  const T *xr = x + static_cast<int64_t>(row) * cols;
  // parts start on multiples of 8 elements, so that a row whose length is a multiple of 8 can be read
  // with 16-byte loads; the first maximum wins inside a thread as it does across threads
  const int64_t per = ((cols + kArgmaxParts - 1) / kArgmaxParts + 7) & ~static_cast<int64_t>(7);
  const int64_t c0 = part * per < cols ? part * per : cols, c1 = c0 + per < cols ? c0 + per : cols;
  float best = -INFINITY;
  int64_t bi = INT64_MAX;
  if (vec_ok) {
    // whole 8-element groups, four per thread in flight
    const int64_t groups = (c1 - c0) / 8;
    for (int64_t g0 = 0; g0 < groups; g0 += 4 * kBlock) {
      float v[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t g = g0 + u * kBlock + threadIdx.x;
        Row8<T>::load(xr + c0 + (g < groups ? g : groups - 1) * 8, v[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t g = g0 + u * kBlock + threadIdx.x;
        if (g < groups) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (v[u][j] > best || bi == INT64_MAX) {
              best = v[u][j];
              bi = c0 + g * 8 + j;
            }
        }
      }
    }
    for (int64_t c = c0 + groups * 8 + threadIdx.x; c < c1; c += kBlock) {
      const float v = ldf(xr + c);
      if (better(v, c, best, bi)) {
        best = v;
        bi = c;
      }
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += kBlock) {
      const float v = ldf(xr + c);
      if (v > best || bi == INT64_MAX) {
        best = v;
        bi = c;
      }
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int64_t oi = __shfl_xor(bi, off, 64);
    if (better(ov, oi, best, bi)) {
      best = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    s_val[threadIdx.x >> 6] = best;
    s_idx[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlock / 64; ++w)
      if (better(s_val[w], s_idx[w], best, bi)) {
        best = s_val[w];
        bi = s_idx[w];
      }
    // agent-scope stores: written through, visible to a workgroup on another XCD (no L2 write-back)
    __hip_atomic_store(&g_argmax_val[trow * kArgmaxParts + part], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(&g_argmax_idx[trow * kArgmaxParts + part], static_cast<long long>(bi), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);  // both stores have completed before the ticket is taken
    unsigned int *ticket = argmax_ticket_of(lane_row0, row);
    const unsigned int t = atomicAdd(ticket, 1u);
    s_last = (t == kArgmaxParts - 1);
    if (s_last) atomicExch(ticket, 0u);
  }
  __syncthreads();
  if (!s_last || threadIdx.x >= 64) return;
  // one wavefront: lane p takes part p (kArgmaxParts == 64)
  best = __hip_atomic_load(&g_argmax_val[trow * kArgmaxParts + threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  bi = __hip_atomic_load(&g_argmax_idx[trow * kArgmaxParts + threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int64_t oi = __shfl_xor(bi, off, 64);
    if (better(ov, oi, best, bi)) {
      best = ov;
      bi = oi;
    }
  }
  if (threadIdx.x == 0) out[row] = bi == INT64_MAX ? 0 : bi;
}


// dst = src with two dimensions exchanged.  The contiguous source is seen as [outer, A, mid, B, inner]
// and the destination as [outer, B, mid, A, inner]; one element per thread step, stores coalesced.
template <typename E>
__global__ __launch_bounds__(kBlock) void transpose_kernel(const E *__restrict__ src, E *__restrict__ dst, int64_t n,
                                                            int64_t A, int64_t mid, int64_t Bd, int64_t inner) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
    int64_t t = i / inner;
    const int64_t in = i - t * inner;
    const int64_t a = t % A;
    t /= A;
    const int64_t m = t % mid;
    t /= mid;
    const int64_t b = t % Bd;
    const int64_t o = t / Bd;
    dst[i] = src[(((o * A + a) * mid + m) * Bd + b) * inner + in];
  }
}

template <typename E>
int launch_transpose(const void *src, void *dst, int64_t n, int64_t A, int64_t mid, int64_t Bd, int64_t inner,
                     hipStream_t st) {
  unsigned grid = blocks_for(n, kBlock);
  if (grid > 65536u) grid = 65536u;
  hipLaunchKernelGGL((transpose_kernel<E>), dim3(grid), dim3(kBlock), 0, st, static_cast<const E *>(src),
                     static_cast<E *>(dst), n, A, mid, Bd, inner);
  return launch_status();
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API int axhip_add_rms_norm(const void *x, const void *residual, const void *weight, float eps,
                                 void *y, void *out, int dtype, int w_dtype, int64_t rows,
                                 int64_t hidden, axhip_stream stream) {
  if (!weight) return AXHIP_INVALID_PTR;
  return dispatch_rms<true>(x, residual, weight, eps, y, out, dtype, w_dtype, dtype, rows, hidden,
                            as_stream(stream));
}

AXHIP_API int axhip_add_rms_norm_ex(const void *x, const void *residual, const void *weight, float eps,
                                    void *y, void *out, int dtype, int w_dtype, int out_dtype,
                                    int64_t rows, int64_t hidden, axhip_stream stream) {
  if (!weight) return AXHIP_INVALID_PTR;
  return dispatch_rms<true>(x, residual, weight, eps, y, out, dtype, w_dtype, out_dtype, rows, hidden,
                            as_stream(stream));
}

AXHIP_API int axhip_rms_norm_ex(const void *x, const void *weight, float eps, void *out, int dtype,
                                int w_dtype, int out_dtype, int64_t rows, int64_t cols,
                                axhip_stream stream) {
  return dispatch_rms<false>(x, nullptr, weight, eps, nullptr, out, dtype, w_dtype, out_dtype, rows, cols,
                             as_stream(stream));
}

AXHIP_API int axhip_rms_norm(const void *x, const void *weight, float eps, void *out, int dtype,
                             int w_dtype, int64_t rows, int64_t cols, axhip_stream stream) {
  return dispatch_rms<false>(x, nullptr, weight, eps, nullptr, out, dtype, w_dtype, dtype, rows, cols,
                             as_stream(stream));
}

AXHIP_API int axhip_silu_mul(const void *gate, const void *up, void *y, int dtype, int64_t n,
                             axhip_stream stream) {
  return launch_binary<SiluMulOp>(gate, up, y, dtype, n, as_stream(stream));
}

AXHIP_API int axhip_add(const void *a, const void *b, void *out, int dtype, int64_t n,
                        axhip_stream stream) {
  return launch_binary<AddOp>(a, b, out, dtype, n, as_stream(stream));
}

AXHIP_API int axhip_transpose(const void *src, void *dst, int elem_bytes, int64_t outer, int64_t dim_a, int64_t mid,
                              int64_t dim_b, int64_t inner, axhip_stream stream) {
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return AXHIP_UNSUPPORTED_TYPE;
  if (outer < 0 || dim_a < 0 || mid < 0 || dim_b < 0 || inner < 0) return AXHIP_INVALID_ARGUMENT;
  const int64_t n = outer * dim_a * mid * dim_b * inner;
  if (n == 0) return AXHIP_OK;
  if (!src || !dst) return AXHIP_INVALID_PTR;
  if (src == dst) return AXHIP_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  switch (elem_bytes) {
    case 1: return launch_transpose<uint8_t>(src, dst, n, dim_a, mid, dim_b, inner, st);
    case 2: return launch_transpose<uint16_t>(src, dst, n, dim_a, mid, dim_b, inner, st);
    case 4: return launch_transpose<uint32_t>(src, dst, n, dim_a, mid, dim_b, inner, st);
    default: return launch_transpose<uint64_t>(src, dst, n, dim_a, mid, dim_b, inner, st);
  }
}

AXHIP_API int axhip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n,
                         axhip_stream stream) {
  if (!is_float_dtype(src_dtype) || !is_float_dtype(dst_dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (n < 0) return AXHIP_INVALID_ARGUMENT;
  if (n == 0) return AXHIP_OK;
  if (!src || !dst) return AXHIP_INVALID_PTR;
  if (!aligned16(src) || !aligned16(dst)) return AXHIP_INVALID_ARGUMENT;
  hipStream_t st = as_stream(stream);
  if (src_dtype == dst_dtype)
    return launch_copy(src, dst, n * (src_dtype == AXHIP_FLOAT16 ? 2 : 4), st);
  unsigned grid = blocks_for(n / 8 > 0 ? n / 8 : 1, kBlock);
  if (grid > 256u * 16u) grid = 256u * 16u;
  if (src_dtype == AXHIP_FLOAT32)
    hipLaunchKernelGGL((cast_kernel<float, __half>), dim3(grid), dim3(kBlock), 0, st,
                       static_cast<const float *>(src), static_cast<__half *>(dst), n);
  else
    hipLaunchKernelGGL((cast_kernel<__half, float>), dim3(grid), dim3(kBlock), 0, st,
                       static_cast<const __half *>(src), static_cast<float *>(dst), n);
  return launch_status();
}

AXHIP_API int axhip_rope(const void *x, const int64_t *pos, float theta, void *out, int dtype,
                         int64_t rows, int64_t heads, int64_t dim, axhip_stream stream) {
  if (dim <= 0 || dim % 2 != 0 || dim / 2 > kMaxHalf) return AXHIP_INVALID_ARGUMENT;
  if (!pos && rows > 0) return AXHIP_INVALID_PTR;
  FreqTable ft;
  // same expression, in fp32 on the host, as the CPU operator evaluates per element
  for (int64_t i = 0; i < dim / 2; ++i)
    ft.f[i] = std::pow(theta, -2.0f * static_cast<float>(i) / static_cast<float>(dim));
  RopeArgs a{x, out, pos, nullptr, nullptr, nullptr, rows, static_cast<int>(heads),
             static_cast<int>(dim), 0, 0};
  return launch_rope<kRopeTheta>(a, ft, dtype, as_stream(stream));
}

AXHIP_API int axhip_rope_qk(const void *q, const void *k, const int64_t *pos, float theta, void *q_out, void *k_out,
                            int dtype, int64_t rows, int64_t q_heads, int64_t k_heads, int64_t dim, axhip_stream stream) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (dim <= 0 || dim % 2 != 0 || dim / 2 > kMaxHalf || q_heads <= 0 || k_heads <= 0 || rows < 0) return AXHIP_INVALID_ARGUMENT;
  if (rows == 0) return AXHIP_OK;
  if (!q || !k || !q_out || !k_out || !pos) return AXHIP_INVALID_PTR;
  if (!rope_rows_ok(dtype, dim, q, q_out) || !rope_rows_ok(dtype, dim, k, k_out) || rows >= (int64_t(1) << 31)) {
    // odd head sizes: the general kernel, one launch per tensor
    const int rc = axhip_rope(q, pos, theta, q_out, dtype, rows, q_heads, dim, stream);
    return rc != AXHIP_OK ? rc : axhip_rope(k, pos, theta, k_out, dtype, rows, k_heads, dim, stream);
  }
  FreqTable ft;
  for (int64_t i = 0; i < dim / 2; ++i)
    ft.f[i] = std::pow(theta, -2.0f * static_cast<float>(i) / static_cast<float>(dim));
  RopeRowsArgs r{q, k, q_out, k_out, pos, nullptr, rows, static_cast<int>(q_heads), static_cast<int>(k_heads),
                 static_cast<int>(dim), 0, 0};
  return launch_rope_rows<kRopeTheta>(r, ft, dtype, as_stream(stream));
}

AXHIP_API int axhip_rope_thd(const void *x, const int64_t *pos, const float *inv_freq, int t_sec,
                             int h_sec, int w_sec, void *out, int dtype, int64_t rows,
                             int64_t heads, int64_t dim, axhip_stream stream) {
  (void)t_sec;
  if ((!pos || !inv_freq) && rows > 0) return AXHIP_INVALID_PTR;
  RopeArgs a{x, out, pos, inv_freq, nullptr, nullptr, rows, static_cast<int>(heads),
             static_cast<int>(dim), h_sec * 3, w_sec * 3};
  FreqTable ft{};
  return launch_rope<kRopeThd>(a, ft, dtype, as_stream(stream));
}

AXHIP_API int axhip_rope_with_cos_sin(const void *x, const float *cos_t, const float *sin_t,
                                      void *out, int dtype, int64_t rows, int64_t heads,
                                      int64_t dim, axhip_stream stream) {
  if ((!cos_t || !sin_t) && rows > 0) return AXHIP_INVALID_PTR;
  RopeArgs a{x, out, nullptr, nullptr, cos_t, sin_t, rows, static_cast<int>(heads),
             static_cast<int>(dim), 0, 0};
  FreqTable ft{};
  return launch_rope<kRopeTable>(a, ft, dtype, as_stream(stream));
}

AXHIP_API int axhip_mrope_cos_sin(const int64_t *pos, const float *inv_freq, int h_sec, int w_sec,
                                  float *cos_out, float *sin_out, int64_t rows, int64_t half,
                                  axhip_stream stream) {
  if (half <= 0 || rows < 0) return AXHIP_INVALID_ARGUMENT;
  if (rows == 0) return AXHIP_OK;
  if (!pos || !inv_freq || !cos_out || !sin_out) return AXHIP_INVALID_PTR;
  hipLaunchKernelGGL(mrope_cos_sin_kernel, dim3(blocks_for(rows * half, kBlock)), dim3(kBlock), 0,
                     as_stream(stream), pos, inv_freq, h_sec * 3, w_sec * 3, cos_out, sin_out, rows,
                     static_cast<int>(half));
  return launch_status();
}

AXHIP_API int axhip_kv_append(const void *k_new, const void *v_new, void *k_cache, void *v_cache,
                              const void *pos, int pos_dtype, int elem_bytes, int B, int Hkv,
                              int Lmax, int D, axhip_stream stream) {
  if (pos_dtype != AXHIP_INT32 && pos_dtype != AXHIP_INT64) return AXHIP_UNSUPPORTED_TYPE;
  if (elem_bytes != 2 && elem_bytes != 4) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hkv <= 0 || Lmax <= 0 || D <= 0) return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (!k_new || !v_new || !k_cache || !v_cache || !pos) return AXHIP_INVALID_PTR;
  const int row_bytes = D * elem_bytes;
  if (row_bytes % 16 != 0 || !aligned16(k_new) || !aligned16(v_new) || !aligned16(k_cache) ||
      !aligned16(v_cache))
    return AXHIP_INVALID_ARGUMENT;
  const int64_t total = static_cast<int64_t>(B) * Hkv * (row_bytes / 16);
  const dim3 grid(blocks_for(total, kBlock));
  hipStream_t st = as_stream(stream);
  const uint8_t *kn = static_cast<const uint8_t *>(k_new), *vn = static_cast<const uint8_t *>(v_new);
  uint8_t *kc = static_cast<uint8_t *>(k_cache), *vc = static_cast<uint8_t *>(v_cache);
  if (pos_dtype == AXHIP_INT32)
    hipLaunchKernelGGL((kv_append_kernel<int32_t>), grid, dim3(kBlock), 0, st, kn, vn, kc, vc,
                       static_cast<const int32_t *>(pos), B, Hkv, Lmax, row_bytes);
  else
    hipLaunchKernelGGL((kv_append_kernel<int64_t>), grid, dim3(kBlock), 0, st, kn, vn, kc, vc,
                       static_cast<const int64_t *>(pos), B, Hkv, Lmax, row_bytes);
  return launch_status();
}

AXHIP_API int axhip_kv_append_paged(const void *k_new, const void *v_new, void *k_pool, void *v_pool,
                                    const int32_t *page_table, const void *start, int start_dtype, int elem_bytes, int B,
                                    int S, int Hkv, int D, int max_pages, int n_pages, axhip_stream stream) {
  if (start && start_dtype != AXHIP_INT32 && start_dtype != AXHIP_INT64) return AXHIP_UNSUPPORTED_TYPE;
  if (elem_bytes != 2 && elem_bytes != 4) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || S < 0 || Hkv <= 0 || D <= 0 || max_pages <= 0 || n_pages <= 0) return AXHIP_INVALID_ARGUMENT;
  if (B == 0 || S == 0) return AXHIP_OK;
  if (!k_new || !v_new || !k_pool || !v_pool || !page_table) return AXHIP_INVALID_PTR;
  const int row_bytes = D * elem_bytes;
  if (row_bytes % 16 != 0 || !aligned16(k_new) || !aligned16(v_new) || !aligned16(k_pool) || !aligned16(v_pool))
    return AXHIP_INVALID_ARGUMENT;
  const int64_t total = static_cast<int64_t>(B) * S * Hkv * (row_bytes / 16);
  const dim3 grid(blocks_for(total, kBlock));
  hipStream_t st = as_stream(stream);
  const uint8_t *kn = static_cast<const uint8_t *>(k_new), *vn = static_cast<const uint8_t *>(v_new);
  uint8_t *kp = static_cast<uint8_t *>(k_pool), *vp = static_cast<uint8_t *>(v_pool);
  if (start && start_dtype == AXHIP_INT64)
    hipLaunchKernelGGL((kv_append_paged_kernel<int64_t>), grid, dim3(kBlock), 0, st, kn, vn, kp, vp, page_table,
                       static_cast<const int64_t *>(start), B, S, Hkv, row_bytes, max_pages, n_pages);
  else
    hipLaunchKernelGGL((kv_append_paged_kernel<int32_t>), grid, dim3(kBlock), 0, st, kn, vn, kp, vp, page_table,
                       static_cast<const int32_t *>(start), B, S, Hkv, row_bytes, max_pages, n_pages);
  return launch_status();
}

AXHIP_API int axhip_kv_dense_to_paged(const void *k_dense, const void *v_dense, void *k_pool, void *v_pool,
                                      const int32_t *page_table, const int32_t *lens, int elem_bytes, int B, int Hkv,
                                      int rows, int D, int max_pages, int n_pages, axhip_stream stream) {
  if (elem_bytes != 2 && elem_bytes != 4) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hkv <= 0 || rows < 0 || D <= 0 || max_pages <= 0 || n_pages <= 0) return AXHIP_INVALID_ARGUMENT;
  if (B == 0 || rows == 0) return AXHIP_OK;
  if (!k_dense || !v_dense || !k_pool || !v_pool || !page_table) return AXHIP_INVALID_PTR;
  const int row_bytes = D * elem_bytes;
  if (row_bytes % 16 != 0 || !aligned16(k_dense) || !aligned16(v_dense) || !aligned16(k_pool) || !aligned16(v_pool))
    return AXHIP_INVALID_ARGUMENT;
  const int64_t total = static_cast<int64_t>(B) * Hkv * rows * (row_bytes / 16);
  unsigned grid = blocks_for(total, kBlock);
  if (grid > 256u * 32u) grid = 256u * 32u;
  hipLaunchKernelGGL(kv_dense_to_paged_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream),
                     static_cast<const uint8_t *>(k_dense), static_cast<const uint8_t *>(v_dense),
                     static_cast<uint8_t *>(k_pool), static_cast<uint8_t *>(v_pool), page_table, lens, B, Hkv, rows, row_bytes,
                     max_pages, n_pages);
  return launch_status();
}

AXHIP_API int axhip_concat(const void *a, const void *b, void *out, int64_t outer, int64_t a_bytes,
                           int64_t b_bytes, axhip_stream stream) {
  if (outer < 0 || a_bytes < 0 || b_bytes < 0) return AXHIP_INVALID_ARGUMENT;
  if (outer == 0 || a_bytes + b_bytes == 0) return AXHIP_OK;
  if ((a_bytes && !a) || (b_bytes && !b) || !out) return AXHIP_INVALID_PTR;
  hipStream_t st = as_stream(stream);
  uint8_t *dst = static_cast<uint8_t *>(out);
  for (int64_t o = 0; o < outer; ++o) {
    int rc = launch_copy(static_cast<const uint8_t *>(a) + o * a_bytes, dst, a_bytes, st);
    if (rc != AXHIP_OK) return rc;
    dst += a_bytes;
    rc = launch_copy(static_cast<const uint8_t *>(b) + o * b_bytes, dst, b_bytes, st);
    if (rc != AXHIP_OK) return rc;
    dst += b_bytes;
  }
  return AXHIP_OK;
}

AXHIP_API int axhip_embedding(const void *ids, int ids_dtype, const void *table, void *out,
                              int dtype, int64_t n_ids, int64_t vocab, int64_t hidden,
                              axhip_stream stream) {
  if (ids_dtype != AXHIP_INT32 && ids_dtype != AXHIP_INT64) return AXHIP_UNSUPPORTED_TYPE;
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (n_ids < 0 || vocab <= 0 || hidden <= 0) return AXHIP_INVALID_ARGUMENT;
  if (n_ids == 0) return AXHIP_OK;
  if (!ids || !table || !out) return AXHIP_INVALID_PTR;
  const int64_t row_bytes = hidden * (dtype == AXHIP_FLOAT16 ? 2 : 4);
  const int vec_ok = aligned16(table) && aligned16(out) && row_bytes % 16 == 0;
  const dim3 grid(static_cast<unsigned>(n_ids));
  hipStream_t st = as_stream(stream);
  if (ids_dtype == AXHIP_INT64)
    hipLaunchKernelGGL((embedding_kernel<int64_t>), grid, dim3(kBlock), 0, st,
                       static_cast<const int64_t *>(ids), static_cast<const uint8_t *>(table),
                       static_cast<uint8_t *>(out), vocab, row_bytes, vec_ok);
  else
    hipLaunchKernelGGL((embedding_kernel<int32_t>), grid, dim3(kBlock), 0, st,
                       static_cast<const int32_t *>(ids), static_cast<const uint8_t *>(table),
                       static_cast<uint8_t *>(out), vocab, row_bytes, vec_ok);
  return launch_status();
}

AXHIP_API int axhip_argmax(const void *x, int64_t *out, int dtype, int64_t rows, int64_t cols,
                           axhip_stream stream) {
  if (!is_float_dtype(dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (rows < 0 || cols <= 0) return AXHIP_INVALID_ARGUMENT;
  if (rows == 0) return AXHIP_OK;
  if (!x || !out) return AXHIP_INVALID_PTR;
  hipStream_t st = as_stream(stream);
  if (cols >= 16384 && rows <= kArgmaxMaxRows) {
    const dim3 pgrid(kArgmaxParts, static_cast<unsigned>(rows));
    const int vec_ok = (cols % 8 == 0 && aligned16(x)) ? 1 : 0;  // every part of every row then starts 16-byte aligned
    const int lane_row0 = axhip_ticket_lane() * kArgmaxMaxRows;
    if (dtype == AXHIP_FLOAT16)
      hipLaunchKernelGGL((argmax_parts_kernel<__half>), pgrid, dim3(kBlock), 0, st,
                         static_cast<const __half *>(x), out, cols, vec_ok, lane_row0);
    else
      hipLaunchKernelGGL((argmax_parts_kernel<float>), pgrid, dim3(kBlock), 0, st,
                         static_cast<const float *>(x), out, cols, vec_ok, lane_row0);
    return launch_status();
  }
  const dim3 grid(static_cast<unsigned>(rows));
  if (dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((argmax_kernel<__half>), grid, dim3(kArgmaxBlock), 0, st,
                       static_cast<const __half *>(x), out, cols);
  else
    hipLaunchKernelGGL((argmax_kernel<float>), grid, dim3(kArgmaxBlock), 0, st,
                       static_cast<const float *>(x), out, cols);
  return launch_status();
}

// Device-to-device copy and zero fill as kernels (used by the runtime; capturable).
int axhip_internal_copy(const void *src, void *dst, int64_t n, hipStream_t st) {
  return launch_copy(src, dst, n, st);
}
int axhip_internal_fill_zero(void *dst, int64_t n, hipStream_t st) {
  if (n <= 0) return AXHIP_OK;
  const int64_t mis = reinterpret_cast<uintptr_t>(dst) & 15;
  int64_t head = mis ? 16 - mis : 0;
  if (head > n) head = n;
  unsigned grid = blocks_for((n + 15) / 16, kBlock);
  if (grid > 256u * 16u) grid = 256u * 16u;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(kBlock), 0, st, static_cast<uint8_t *>(dst),
                     n, head);
  return launch_status();
}

}  // extern "C"
