// Everything of a decoder layer that follows the attention, for decode-sized batches (M <= 16 rows),
// in ONE persistent launch:
//
//   phase 1   h1  = attn . Wo^T + h                      (o_proj + residual add)
//   phase 2   act = silu(g) * u,  [g | u] = rmsnorm(h1, w_post) . Wgu^T
//   phase 3   h2  = act . Wd^T + h1                      (down_proj + residual add)
//   phase 4   y   = rmsnorm(h2, w_next) . Wn^T           (the next layer's qkv projection, or the
//                                                         final norm + lm_head after the last layer)
//
// The same arithmetic as the single operators (fp16 Linear with fp32 accumulation, add_rms_norm
// with evaluation order (x * rstd) * w, SiLU-mul) - only the five kernel boundaries between them are
// replaced by barriers across the resident workgroups.
//
// Measured on MI355X at the 2B shape (16 rows, H 2048, I 6144, next N 4096, cold weights): 61 us per
// launch - 16 us for the launch and its three barriers (2.5 us each plus 1.5 us for the cache
// invalidate behind it), 6 / 20 / 10 / 9 us for the four phases - against about 51 us for the seven
// launches it replaces inside a captured graph.  A phase still pays what a small kernel pays (one
// HBM round trip for its weights, one write-through drain), and a kernel boundary inside a graph
// turns out to be as cheap as a barrier, so the example model keeps this path switched off.
//
// One workgroup per CU (1024 threads = 16 wavefronts), workgroups stride over 16-row tiles of the
// weight matrix; the wavefronts of a team split K and add their fragments through LDS (as in the
// skinny Linear kernels).  x reaches the MFMA B operand through LDS: for the two phases that start
// with a norm the workgroup normalises all rows once (wavefront w takes row w) into a full [16, K]
// fp16 copy; the other two stage wave-private strips.
//
// Data written in one phase and read in the next crosses XCDs, whose L2 caches are not coherent:
// it is written with agent-scope (write-through) stores, and every workgroup invalidates its
// non-coherent cache lines (agent-scope acquire fence) after each barrier.  The barrier is two-level
// (16 workgroups per counter, then one counter for the groups), counts monotonically within a
// launch, is put back to zero by the last workgroup to leave the kernel, and spins a bounded number
// of times: if the workgroups are not all resident it gives up, flags the failure and every
// wavefront still exits.
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kTailThreads = 1024;
constexpr int kTailWaves = 16;
constexpr int kTailRows = 16;        // rows of x (M <= 16)
constexpr int kTailMaxNormK = 2048;  // K of the phases that hold all of x in LDS
constexpr int kU = 4;                // chunks of 32 K per loop iteration
constexpr int kBarGroup = 16;
constexpr int kBarMaxGroups = 64;
constexpr int kSpinLimit = 1 << 21;

struct TailBarrier {
  unsigned cnt[kBarMaxGroups * 32];  // one counter per group of workgroups, 128 bytes apart
  unsigned top, pad0[31];
  unsigned flag, pad1[31];
  unsigned done, pad2[31];
  unsigned fail, pad3[31];
};
__device__ TailBarrier g_tail_bar;

#define TAIL_LD(p) __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TAIL_ST(p, v) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TAIL_ADD(p, v) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// k-th barrier of this launch (k = 1, 2, ...).  Returns false when the wait ran out.
__device__ __forceinline__ bool grid_sync(unsigned k, int *s_ok, bool fence = true) {
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned n_wg = gridDim.x, wg = blockIdx.x;
    const unsigned grp = wg / kBarGroup, n_grp = (n_wg + kBarGroup - 1) / kBarGroup;
    const unsigned in_grp = min(static_cast<unsigned>(kBarGroup), n_wg - grp * kBarGroup);
    int ok = 1;
    bool released = false;
    if (TAIL_ADD(&g_tail_bar.cnt[grp * 32], 1u) == k * in_grp - 1) {
      if (TAIL_ADD(&g_tail_bar.top, 1u) == k * n_grp - 1) {
        TAIL_ST(&g_tail_bar.flag, k);
        released = true;
      }
    }
    if (!released) {
      int limit = kSpinLimit;
      while (TAIL_LD(&g_tail_bar.flag) < k && --limit > 0) __builtin_amdgcn_s_sleep(1);
      if (limit <= 0) {
        ok = 0;
        TAIL_ADD(&g_tail_bar.fail, 1u);
      }
    }
    // one invalidate per workgroup (the vector L1 belongs to the CU, the non-coherent L2 lines to the
    // XCD): later loads of any wavefront see the other workgroups' stores.  Issued by every wavefront
    // it costs about 2 us apiece.
    if (fence) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    *s_ok = ok;
  }
  __syncthreads();
  return *s_ok != 0;
}

struct TailArgs {
  const __half *attn;   // [M, K1] merged attention output
  const float *h_in;    // [M, H]  residual stream entering the layer
  const __half *w_o;    // packed [H, K1]
  const float *w_post;  // [H] post-attention norm weight
  const __half *w_gu;   // packed, gate / up tiles interleaved [2I, H]
  const __half *w_down; // packed [H, I]
  const float *w_next;  // [H] the norm in front of the next Linear
  const __half *w_nl;   // packed [N_next, H]
  float *h_mid;         // [M, H]  out: residual stream after the attention block
  __half *act;          // [M, I]  scratch
  float *h_out;         // [M, H]  out: residual stream leaving the layer
  float *y;             // [M, N_next] out
  int M, H, K1, I, N_next;
  float eps;
  int skip;  // measurement: bit p set = phase p + 1 does no work (results are then meaningless)
};

// Loads through pointers known to be global memory: the phase functions are not inlined, so their
// pointer arguments are generic, and a generic (flat) load also occupies the LDS counter, which
// would make every LDS wait in the loop wait for the weight loads as well.
#define TAIL_GLOBAL __attribute__((address_space(1)))
template <typename V, typename T>
__device__ __forceinline__ V gload(const T *p) {
  return *(const TAIL_GLOBAL V *)(p);
}
__device__ __forceinline__ half8_t tail_ld8(const __half *p) { return gload<half8_t>(p); }

// LDS (dynamic, so that the phase functions below - kept out of line to bound register use - address
// it as LDS): region X (64 KiB: the normalised x, or 16 wave-private strips) + region R (reduction).
constexpr int kXBytes = kTailRows * kTailMaxNormK * 2;
constexpr int kRBytes = 28 * 1024;
extern __shared__ __attribute__((aligned(16))) unsigned char tail_smem[];

// All rows of h (fp32 [M, K]) -> rmsnorm -> fp16 into xs[16][K] (16-byte units XOR-ed with the row).
__device__ __attribute__((noinline)) void stage_norm(const float *h, const float *w, int M, int K, float eps) {
  _Float16 *xs = reinterpret_cast<_Float16 *>(tail_smem);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n4 = K / 256;  // float4 per lane
  float4_t v[kTailMaxNormK / 256];
  float ss = 0.f;
  const float *row = h + static_cast<int64_t>(min(wave, M - 1)) * K;
#pragma unroll
  for (int i = 0; i < kTailMaxNormK / 256; ++i) {
    v[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (i < n4 && wave < M) v[i] = gload<float4_t>(row + (i * 64 + lane) * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) ss = __builtin_fmaf(v[i][e], v[i][e], ss);
  }
  ss = group_sum<64>(ss);
  const float rstd = 1.0f / sqrtf(ss / static_cast<float>(K) + eps);
#pragma unroll
  for (int i = 0; i < kTailMaxNormK / 256; ++i) {
    if (i >= n4) break;
    const int e0 = (i * 64 + lane) * 4;
    const float4_t wv = gload<float4_t>(w + e0);
    const float4_t y = (v[i] * rstd) * wv;
    const half4_t hv = {static_cast<_Float16>(y[0]), static_cast<_Float16>(y[1]), static_cast<_Float16>(y[2]),
                        static_cast<_Float16>(y[3])};
    const int unit = e0 >> 3;
    *reinterpret_cast<half4_t *>(xs + wave * K + ((unit ^ wave) << 3) + (e0 & 4)) = hv;
  }
}

// One Linear phase.  NT 16-row tiles of W per unit, TEAM wavefronts split K for a unit; XLDS: x is the
// normalised copy in LDS, otherwise fp16 rows in global memory staged through wave-private strips.
// EPI 0: + residual, fp32, write-through stores; 1: SiLU(gate) * up of a tile pair, fp16,
// write-through stores; 2: plain fp32 stores (nothing in this launch reads them).
template <int NT, int TEAM, bool XLDS, int EPI>
__device__ __attribute__((noinline)) void linear_phase(const __half *xg, int M, int K, const __half *wp, int N,
                                             const float *residual, void *out, int ld_out) {
  unsigned char *smem = tail_smem;
  constexpr int TEAMS = kTailWaves / TEAM;
  static_assert(TEAMS * (TEAM - 1) * NT * 1024 <= kRBytes, "reduction buffer");
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int team = wave / TEAM, tw = wave % TEAM;
  const int KC = K / 32;
  const int cpw = KC / TEAM;  // the host checks KC % (TEAM * kU) == 0
  const int c_begin = tw * cpw, c_end = c_begin + cpw;
  const int n_tiles = N / 16, n_units = (n_tiles + NT - 1) / NT;
  const int per_round = gridDim.x * TEAMS;
  const int rounds = (n_units + per_round - 1) / per_round;
  _Float16 *xs = reinterpret_cast<_Float16 *>(smem);
  _Float16 *strip = xs + wave * (kTailRows * kU * 32);
  float4_t *red = reinterpret_cast<float4_t *>(smem + kXBytes) + team * ((TEAM - 1) * NT * 64);

  for (int round = 0; round < rounds; ++round) {
    const int unit = (round * static_cast<int>(gridDim.x) + static_cast<int>(blockIdx.x)) * TEAMS + team;
    const bool valid = unit < n_units;
    const int tile0 = valid ? unit * NT : 0;
    float4_t acc[NT];
    const __half *wt[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
      wt[t] = wp + (static_cast<int64_t>(min(tile0 + t, n_tiles - 1)) * KC) * 512 + lane * 8;
    }
    for (int c = c_begin; c < c_end; c += kU) {
      half8_t af[NT][kU], bf[kU];
#pragma unroll
      for (int j = 0; j < kU; ++j)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          af[t][j] = __builtin_nontemporal_load((const TAIL_GLOBAL half8_t *)(wt[t] + static_cast<int64_t>(c + j) * 512));
      if constexpr (XLDS) {
#pragma unroll
        for (int j = 0; j < kU; ++j) {
          const int un = (c + j) * 4 + g;
          bf[j] = *reinterpret_cast<const half8_t *>(xs + r * K + ((un ^ r) << 3));
        }
      } else {
        // stage x[0..16)[32c .. 32(c+kU)) into this wavefront's strip: 16 rows x 16 units, 4 per lane
        half8_t xv[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int v = p * 64 + lane;
          const int row = v >> 4, un = v & 15;
          xv[p] = tail_ld8(xg + static_cast<int64_t>(min(row, M - 1)) * K + c * 32 + un * 8);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int v = p * 64 + lane;
          const int row = v >> 4, un = v & 15;
          *reinterpret_cast<half8_t *>(strip + row * (kU * 32) + ((un ^ row) << 3)) = xv[p];
        }
#pragma unroll
        for (int j = 0; j < kU; ++j) {
          const int un = j * 4 + g;
          bf[j] = *reinterpret_cast<const half8_t *>(strip + r * (kU * 32) + ((un ^ r) << 3));
        }
      }
#pragma unroll
      for (int j = 0; j < kU; ++j)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t][j], bf[j], acc[t], 0, 0, 0);
    }
    // add the K slices of the team
    if (tw > 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t) red[((tw - 1) * NT + t) * 64 + lane] = acc[t];
    }
    __syncthreads();
    if (tw == 0 && valid) {
      float4_t tot[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float4_t s = acc[t];
#pragma unroll
        for (int w = 0; w < TEAM - 1; ++w) s += red[(w * NT + t) * 64 + lane];
        tot[t] = s;
      }
      const int m = r;  // C layout: lane holds row m = lane % 16 of x, columns 4g .. 4g+3 of the tile
      if (m < M) {
        if constexpr (EPI == 1) {
          static_assert(EPI != 1 || NT == 2, "a unit is one (gate, up) tile pair");
          _Float16 hv[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float gt = tot[0][q];
            hv[q] = static_cast<_Float16>(gt / (1.0f + expf(-gt)) * tot[NT - 1][q]);
          }
          unsigned *dst = reinterpret_cast<unsigned *>(static_cast<__half *>(out) + static_cast<int64_t>(m) * ld_out +
                                                       unit * 16 + 4 * g);
          TAIL_ST(dst, __builtin_bit_cast(unsigned, half2_t{hv[0], hv[1]}));
          TAIL_ST(dst + 1, __builtin_bit_cast(unsigned, half2_t{hv[2], hv[3]}));
        } else {
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            if (tile0 + t >= n_tiles) continue;
            const int64_t o = static_cast<int64_t>(m) * ld_out + (tile0 + t) * 16 + 4 * g;
            if constexpr (EPI == 0) {
              const float4_t rv = gload<float4_t>(residual + o);
#pragma unroll
              for (int q = 0; q < 4; ++q) TAIL_ST(static_cast<float *>(out) + o + q, tot[t][q] + rv[q]);
            } else {
              *(TAIL_GLOBAL float4_t *)(static_cast<float *>(out) + o) = tot[t];
            }
          }
        }
      }
    }
    __syncthreads();  // the reduction buffer and the strips are free again
  }
}

__global__ __launch_bounds__(kTailThreads) void decode_tail_kernel(TailArgs a) {
  __shared__ int s_ok;

  // phase 1: o_proj + residual
  if (!(a.skip & 1)) linear_phase<1, 16, false, 0>(a.attn, a.M, a.K1, a.w_o, a.H, a.h_in, a.h_mid, a.H);
  __builtin_amdgcn_s_waitcnt(0);  // this thread's write-through stores have completed
  if (!grid_sync(1, &s_ok, !(a.skip & 64))) return;

  // phase 2: post-attention norm, gate+up, SiLU-mul
  if (!(a.skip & 16)) stage_norm(a.h_mid, a.w_post, a.M, a.H, a.eps);
  __syncthreads();
  if (!(a.skip & 2)) linear_phase<2, 8, true, 1>(nullptr, a.M, a.H, a.w_gu, 2 * a.I, nullptr, a.act, a.I);
  __builtin_amdgcn_s_waitcnt(0);
  if (!grid_sync(2, &s_ok, !(a.skip & 64))) return;

  // phase 3: down_proj + residual
  if (!(a.skip & 4)) linear_phase<1, 16, false, 0>(a.act, a.M, a.I, a.w_down, a.H, a.h_mid, a.h_out, a.H);
  __builtin_amdgcn_s_waitcnt(0);
  if (!grid_sync(3, &s_ok, !(a.skip & 64))) return;

  // phase 4: the next norm and the Linear behind it
  if (!(a.skip & 16)) stage_norm(a.h_out, a.w_next, a.M, a.H, a.eps);
  __syncthreads();
  if (a.skip & 8) {
  } else if (a.N_next >= 8192)
    linear_phase<2, 8, true, 2>(nullptr, a.M, a.H, a.w_nl, a.N_next, nullptr, a.y, a.N_next);
  else
    linear_phase<1, 16, true, 2>(nullptr, a.M, a.H, a.w_nl, a.N_next, nullptr, a.y, a.N_next);

  // the last workgroup out puts the barrier back to zero for the next launch
  if (threadIdx.x == 0) {
    if (TAIL_ADD(&g_tail_bar.done, 1u) == gridDim.x - 1) {
      const unsigned n_grp = (gridDim.x + kBarGroup - 1) / kBarGroup;
      for (unsigned i = 0; i < n_grp; ++i) TAIL_ST(&g_tail_bar.cnt[i * 32], 0u);
      TAIL_ST(&g_tail_bar.top, 0u);
      TAIL_ST(&g_tail_bar.flag, 0u);
      TAIL_ST(&g_tail_bar.done, 0u);
    }
  }
}

int g_tail_wgs = 0;  // resident workgroups to launch (0: one per CU, at most 256)
int g_tail_skip = 0;

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API int axhip_decode_layer_tail(const void *attn, const float *h_in, const void *w_o, const float *w_post,
                                      const void *w_gate_up, const void *w_down, const float *w_next,
                                      const void *w_next_linear, float *h_mid, void *act, float *h_out, float *y,
                                      int M, int H, int K1, int I, int N_next, float eps, axhip_stream stream) {
  if (M < 0 || M > kTailRows || H <= 0 || K1 <= 0 || I <= 0 || N_next <= 0) return AXHIP_INVALID_ARGUMENT;
  // shapes the phases are written for: K slices of whole 128-column steps per wavefront, whole tiles
  if (H % 256 != 0 || H > kTailMaxNormK || (H / 32) % (16 * kU) != 0) return AXHIP_INVALID_ARGUMENT;
  if ((K1 / 32) % (16 * kU) != 0 || K1 % 32 != 0 || (I / 32) % (16 * kU) != 0 || I % 32 != 0) return AXHIP_INVALID_ARGUMENT;
  if (H % 16 != 0 || I % 16 != 0 || N_next % 16 != 0) return AXHIP_INVALID_ARGUMENT;
  if (M == 0) return AXHIP_OK;
  if (!attn || !h_in || !w_o || !w_post || !w_gate_up || !w_down || !w_next || !w_next_linear || !h_mid || !act ||
      !h_out || !y)
    return AXHIP_INVALID_PTR;
  const uintptr_t all = reinterpret_cast<uintptr_t>(attn) | reinterpret_cast<uintptr_t>(h_in) |
                        reinterpret_cast<uintptr_t>(w_post) | reinterpret_cast<uintptr_t>(w_next) |
                        reinterpret_cast<uintptr_t>(h_mid) | reinterpret_cast<uintptr_t>(act) |
                        reinterpret_cast<uintptr_t>(h_out) | reinterpret_cast<uintptr_t>(y) |
                        reinterpret_cast<uintptr_t>(w_o) | reinterpret_cast<uintptr_t>(w_gate_up) |
                        reinterpret_cast<uintptr_t>(w_down) | reinterpret_cast<uintptr_t>(w_next_linear);
  if (all & 15) return AXHIP_INVALID_PTR;
  int wgs = g_tail_wgs;
  if (wgs <= 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      return AXHIP_INTERNAL_ERROR;
    wgs = cus < 256 ? cus : 256;
  }
  if (wgs > kBarGroup * kBarMaxGroups) wgs = kBarGroup * kBarMaxGroups;
  TailArgs a;
  a.attn = static_cast<const __half *>(attn);
  a.h_in = h_in;
  a.w_o = static_cast<const __half *>(w_o);
  a.w_post = w_post;
  a.w_gu = static_cast<const __half *>(w_gate_up);
  a.w_down = static_cast<const __half *>(w_down);
  a.w_next = w_next;
  a.w_nl = static_cast<const __half *>(w_next_linear);
  a.h_mid = h_mid;
  a.act = static_cast<__half *>(act);
  a.h_out = h_out;
  a.y = y;
  a.M = M;
  a.H = H;
  a.K1 = K1;
  a.I = I;
  a.N_next = N_next;
  a.eps = eps;
  a.skip = g_tail_skip;
  static std::atomic<uint64_t> lds_set{0};  // more dynamic LDS than the default limit
  const int lds_rc = raise_dynamic_lds(reinterpret_cast<const void *>(decode_tail_kernel), kXBytes + kRBytes, lds_set);
  if (lds_rc != AXHIP_OK) return lds_rc;
  hipLaunchKernelGGL(decode_tail_kernel, dim3(wgs), dim3(kTailThreads), kXBytes + kRBytes, as_stream(stream), a);
  return launch_status();
}

// Barrier bookkeeping of axhip_decode_layer_tail: number of barrier waits that ran out since the
// last reset (0 in a healthy process); reset != 0 also puts the counters back to zero (call it only
// while no such launch is in flight).
AXHIP_API int axhip_decode_layer_tail_status(int reset, unsigned *failed_waits) {
  TailBarrier h;
  if (hipMemcpyFromSymbol(&h, HIP_SYMBOL(g_tail_bar), sizeof(h)) != hipSuccess) return AXHIP_INTERNAL_ERROR;
  if (failed_waits) *failed_waits = h.fail;
  if (reset) {
    TailBarrier z = {};
    if (hipMemcpyToSymbol(HIP_SYMBOL(g_tail_bar), &z, sizeof(z)) != hipSuccess) return AXHIP_INTERNAL_ERROR;
  }
  return AXHIP_OK;
}

AXHIP_API void axhip_decode_layer_tail_tune(int workgroups, int skip_phases) {
  g_tail_wgs = workgroups > 0 ? workgroups : 0;
  g_tail_skip = skip_phases;
}

}  // extern "C"
