// Shared device/host helpers for the gfx950 kernels of libaxhip.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstddef>
#include <cstdint>

#include "axhip_experimental.h"  // includes axhip.h

namespace axhip {

constexpr int kWave = 64;  // CDNA wavefront width

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

inline hipStream_t as_stream(axhip_stream s) { return reinterpret_cast<hipStream_t>(s); }

// Maps a launch error to a Status value.
inline int launch_status() {
  return hipGetLastError() == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}

// Raises a kernel's dynamic LDS limit above the 64 KB default, once per device (the attribute belongs
// to the kernel's code object on one device).  `done` holds one bit per device.
inline int raise_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return AXHIP_DEVICE_ERROR;
  const uint64_t bit = uint64_t(1) << dev;
  if (done.load(std::memory_order_acquire) & bit) return AXHIP_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
    return AXHIP_INTERNAL_ERROR;
  done.fetch_or(bit, std::memory_order_release);
  return AXHIP_OK;
}

// Compute units of the current device (hipDeviceProp_t::multiProcessorCount), read once per device;
// 256 (an MI355X) when no device can be asked, so that host-only callers of the planners get the
// plans of the part the kernels are written for.
inline int device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return 256;
  }
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return 256;
  }
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

// Zeroes the static ticket counters of the current device (defined beside the counters; see
// axhip_reset_tickets).  Host-side, synchronous.
int reset_attention_tickets();
int reset_argmax_tickets();

inline bool is_float_dtype(int dt) { return dt == AXHIP_FLOAT16 || dt == AXHIP_FLOAT32; }

// Workgroup barrier that waits for this wavefront's LDS traffic only.  __syncthreads() also waits for every
// outstanding global load (s_waitcnt vmcnt(0)), i.e. it drains whatever a kernel has requested ahead across the
// barrier.  Use where the barrier orders LDS writes and reads and nothing else.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- 16-byte vector access ---------------------------------------------------------------------
struct alignas(16) Vec16 {
  uint32_t w[4];
};

__device__ __forceinline__ Vec16 ld16(const void *p) { return *reinterpret_cast<const Vec16 *>(p); }
__device__ __forceinline__ void st16(void *p, const Vec16 &v) { *reinterpret_cast<Vec16 *>(p) = v; }
// Streaming form for data that is read once (KV cache rows, weight fragments): a non-temporal load.
// Measured on MI355X with a checksum kernel over 1 GiB: 6.9-7.0 TB/s against 6.1-6.2 TB/s for plain
// 16-byte loads.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Vec16 ld16_stream(const void *p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
  Vec16 r;
  r.w[0] = v[0];
  r.w[1] = v[1];
  r.w[2] = v[2];
  r.w[3] = v[3];
  return r;
}

__device__ __forceinline__ half2_t as_half2(uint32_t w) { return __builtin_bit_cast(half2_t, w); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

__device__ __forceinline__ void st16_stream(void *p, const Vec16 &v) {
  const u32x4_t x = {v.w[0], v.w[1], v.w[2], v.w[3]};
  __builtin_nontemporal_store(x, reinterpret_cast<u32x4_t *>(p));
}

// Eight consecutive elements of T as fp32.  The *_stream forms are for global memory that a kernel
// touches once (a read-and-write copy kernel over 1 GiB: 4.96 TB/s with both, 4.51 TB/s with neither).
template <typename T>
struct Row8;

template <>
struct Row8<__half> {
  // 8 halves = one 16-byte load
  static __device__ __forceinline__ void load(const __half *p, float (&f)[8]) {
    const Vec16 v = ld16(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = as_half2(v.w[i]);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  static __device__ __forceinline__ Vec16 pack(const float (&f)[8]) {
    Vec16 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t h;
      h.x = static_cast<_Float16>(f[2 * i]);  // round-to-nearest-even
      h.y = static_cast<_Float16>(f[2 * i + 1]);
      v.w[i] = as_u32(h);
    }
    return v;
  }
  static __device__ __forceinline__ void store(__half *p, const float (&f)[8]) { st16(p, pack(f)); }
  static __device__ __forceinline__ void store_stream(__half *p, const float (&f)[8]) { st16_stream(p, pack(f)); }
  static __device__ __forceinline__ void load_stream(const __half *p, float (&f)[8]) {
    const Vec16 v = ld16_stream(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = as_half2(v.w[i]);
      f[2 * i] = static_cast<float>(h.x);
      f[2 * i + 1] = static_cast<float>(h.y);
    }
  }
};

template <>
struct Row8<float> {
  static __device__ __forceinline__ void load(const float *p, float (&f)[8]) {
    const Vec16 a = ld16(p), b = ld16(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = __builtin_bit_cast(float, a.w[i]);
      f[4 + i] = __builtin_bit_cast(float, b.w[i]);
    }
  }
  static __device__ __forceinline__ void store(float *p, const float (&f)[8]) {
    Vec16 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a.w[i] = __builtin_bit_cast(uint32_t, f[i]);
      b.w[i] = __builtin_bit_cast(uint32_t, f[4 + i]);
    }
    st16(p, a);
    st16(p + 4, b);
  }
  static __device__ __forceinline__ void load_stream(const float *p, float (&f)[8]) {
    const Vec16 a = ld16_stream(p), b = ld16_stream(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = __builtin_bit_cast(float, a.w[i]);
      f[4 + i] = __builtin_bit_cast(float, b.w[i]);
    }
  }
  static __device__ __forceinline__ void store_stream(float *p, const float (&f)[8]) {
    Vec16 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a.w[i] = __builtin_bit_cast(uint32_t, f[i]);
      b.w[i] = __builtin_bit_cast(uint32_t, f[4 + i]);
    }
    st16_stream(p, a);
    st16_stream(p + 4, b);
  }
};

// Scalar element access as fp32 (tails, odd sizes).
__device__ __forceinline__ float ldf(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ float ldf(const float *p) { return *p; }
__device__ __forceinline__ void stf(__half *p, float v) { *p = __float2half_rn(v); }
__device__ __forceinline__ void stf(float *p, float v) { *p = v; }

// ---- cross-lane sums with DPP (no LDS traffic) -------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

// Across the 16-lane rows of a wavefront: the value of lane l and that of lane l ^ 16 (l ^ 32), in an order
// that depends on the lane - for sums, maxima and other symmetric operations.  One swap on the vector ALU
// (v_permlane16_swap / v_permlane32_swap of gfx950: odd rows of the first operand change places with even
// rows of the second, the upper half with the lower half) instead of a trip through the LDS crossbar.
__device__ __forceinline__ void pair_xor16(unsigned x, unsigned &a, unsigned &b) {
  const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  a = r[0];
  b = r[1];
}
__device__ __forceinline__ void pair_xor32(unsigned x, unsigned &a, unsigned &b) {
  const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  a = r[0];
  b = r[1];
}
__device__ __forceinline__ float sum_xor16(float x) {
  unsigned a, b;
  pair_xor16(__builtin_bit_cast(unsigned, x), a, b);
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}
__device__ __forceinline__ float sum_xor32(float x) {
  unsigned a, b;
  pair_xor32(__builtin_bit_cast(unsigned, x), a, b);
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}
__device__ __forceinline__ float max_xor16(float x) {
  unsigned a, b;
  pair_xor16(__builtin_bit_cast(unsigned, x), a, b);
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}
__device__ __forceinline__ float max_xor32(float x) {
  unsigned a, b;
  pair_xor32(__builtin_bit_cast(unsigned, x), a, b);
  return fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}

// Sum over aligned groups of LANES consecutive lanes (LANES in {1,2,4,8,16,32,64}); every lane of a
// group ends with the same bits because each step adds the same two partner values.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
  if constexpr (LANES >= 2) x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
  if constexpr (LANES >= 4) x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) x += dpp_f32<0x141>(x);  // row_half_mirror
  if constexpr (LANES >= 16) x += dpp_f32<0x140>(x); // row_mirror
  if constexpr (LANES >= 32) x = sum_xor16(x);
  if constexpr (LANES >= 64) x = sum_xor32(x);
  return x;
}

template <int LANES>
__device__ __forceinline__ float group_max(float x) {
  if constexpr (LANES >= 2) x = fmaxf(x, dpp_f32<0xB1>(x));
  if constexpr (LANES >= 4) x = fmaxf(x, dpp_f32<0x4E>(x));
  if constexpr (LANES >= 8) x = fmaxf(x, dpp_f32<0x141>(x));
  if constexpr (LANES >= 16) x = fmaxf(x, dpp_f32<0x140>(x));
  if constexpr (LANES >= 32) x = max_xor16(x);
  if constexpr (LANES >= 64) x = max_xor32(x);
  return x;
}

// The same for integers over the whole wavefront, and an inclusive prefix sum over its lanes (shifts within a
// row, then the last lane of a row broadcast into the rows after it): a handful of vector instructions each.
template <int CTRL, int ROW_MASK = 0xF, bool ZERO_FILL = true>
__device__ __forceinline__ int dpp_i32(int x) {
  return __builtin_amdgcn_update_dpp(0, x, CTRL, ROW_MASK, 0xF, ZERO_FILL);
}
__device__ __forceinline__ int wave_sum_i32(int v) {
  v += dpp_i32<0xB1>(v);
  v += dpp_i32<0x4E>(v);
  v += dpp_i32<0x141>(v);
  v += dpp_i32<0x140>(v);
  unsigned a, b;
  pair_xor16(static_cast<unsigned>(v), a, b);
  v = static_cast<int>(a + b);
  pair_xor32(static_cast<unsigned>(v), a, b);
  return static_cast<int>(a + b);
}
__device__ __forceinline__ int wave_max_i32(int v) {
  v = max(v, dpp_i32<0xB1>(v));
  v = max(v, dpp_i32<0x4E>(v));
  v = max(v, dpp_i32<0x141>(v));
  v = max(v, dpp_i32<0x140>(v));
  unsigned a, b;
  pair_xor16(static_cast<unsigned>(v), a, b);
  v = max(static_cast<int>(a), static_cast<int>(b));
  pair_xor32(static_cast<unsigned>(v), a, b);
  return max(static_cast<int>(a), static_cast<int>(b));
}
__device__ __forceinline__ int wave_prefix_i32(int v) {
  v += dpp_i32<0x111>(v);  // row_shr:1 (lanes without a source add 0)
  v += dpp_i32<0x112>(v);  // row_shr:2
  v += dpp_i32<0x114>(v);  // row_shr:4
  v += dpp_i32<0x118>(v);  // row_shr:8
  v += dpp_i32<0x142, 0xA, false>(v);  // row_bcast:15 into rows 1 and 3: the total of the row before
  v += dpp_i32<0x143, 0xC, false>(v);  // row_bcast:31 into rows 2 and 3: the total of rows 0 and 1
  return v;
}

// Block-wide sum for blocks of NWAVES wavefronts; `smem` holds NWAVES floats.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float x, float *smem) {
  x = group_sum<64>(x);
  if constexpr (NWAVES == 1) return x;
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) smem[wave] = x;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) t += smem[i];
  __syncthreads();
  return t;
}

// ---- LDS reads of MFMA operands (attention kernels) ------------------------------------------------
__device__ __forceinline__ half8_t lds_h8(const _Float16 *p) { return *reinterpret_cast<const half8_t *>(p); }

// 4 keys x 16 d of row-major V, delivered transposed: this lane gets V[key0 .. key0+3][d0 + lane%16].
// `row_base` points at V[key0][0] of the stage in LDS for this lane's group; rows are 2*D bytes.
template <int D>
__device__ __forceinline__ half4_t lds_v_tr(const _Float16 *stage, int key0, int d0, int c) {
  const int key = key0 + (c >> 2);           // the row this lane addresses
  const int unit = (d0 >> 3) + ((c & 3) >> 1);  // 16-byte unit within the row
  const _Float16 *p = stage + key * D + ((unit ^ (key & (D / 8 - 1))) << 3) + ((c & 1) << 2);
  typedef __fp16 fp16x4_t __attribute__((__vector_size__(4 * sizeof(__fp16))));
  const fp16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((fp16x4_t __attribute__((address_space(3))) *)(p));
  return __builtin_bit_cast(half4_t, r);
}

}  // namespace axhip
