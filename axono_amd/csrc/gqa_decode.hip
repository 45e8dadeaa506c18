// Split-K flash-decoding attention for one query token per sequence (grouped-query heads).
//
// Work decomposition.  One workgroup (256 threads = 4 wavefronts) owns one (sequence, kv-head
// group, key range) and serves G query heads that share that kv head, so every K/V byte is read
// from HBM once.  A row of D elements is spread over D/8 lanes, 8 consecutive elements (one or
// two 16-byte loads) per lane; a wavefront therefore reads 64*16 B of consecutive memory per load
// instruction and the 256 threads cover RG = 256/(D/8) consecutive key rows at a time.  Each lane
// keeps its own running (max, sum, 8 output elements) per query head for the rows of its row
// group; nothing crosses row groups until the epilogue, where the RG partial states are merged
// through LDS.  Dot products are reduced over the D/8 lanes of a row with DPP adds.
//
// The kernel is HBM-bound: per key it moves 2*D*sizeof(T) bytes and issues about a dozen vector
// instructions per wavefront, so the arithmetic stays on the vector ALUs (packed-fp16 dot
// products with fp32 accumulation); the matrix cores would add nothing.
//
// Scores are kept in the log2 domain (q.k * scale * log2 e) so that the exponentials are single
// v_exp_f32 instructions.  Per-split results (unnormalised output, running max, running sum) go to
// a workspace and a second small kernel merges them; with one split the first kernel normalises
// and writes the result itself.  (A single-launch form, in which the workgroup that takes the last
// ticket of a (sequence, head group) merges, is kept behind the tuning hook: it measured no faster.)
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kThreads = 256;
constexpr float kNegBig = -1.0e30f;   // "no key seen yet" in the log2 domain (finite: no inf-inf)
constexpr int kMaxSplits = 128;
constexpr int kChunkAlign = 128;      // key ranges start on multiples of this
constexpr int kMinChunk = 256;
constexpr int kLongChunk = 1024;

struct Tuning {
  int target_workgroups = 1024;  // 256 CUs x 4 resident workgroups
  int force_splits = 0;          // > 0: fixed split count (measurement sweeps)
  int separate_merge = 1;        // 1: merge in a second kernel; 0: the last workgroup merges
};
Tuning g_tuning;

// Ticket counters of the in-kernel merge, one per (sequence, head group).  They start at zero and
// the merging workgroup puts its counter back to zero, so no launch ever has to clear them.
// Launches that overlap in time on one device must not share (sequence, head group) slots; calls on
// one stream, and replays of a captured graph, never overlap.
constexpr int kTicketSlots = 1 << 16;
__device__ unsigned int g_tickets[kTicketSlots];

struct SplitPlan {
  int n_splits;
  int chunk;
};

// The key axis is cut into `n_splits` ranges of `chunk` keys.  The plan depends only on host-side
// sizes so that a captured graph stays valid while the device-side lengths change.
SplitPlan plan_splits(int B, int head_groups, int max_len) {
  const long pairs = static_cast<long>(B) * head_groups > 0 ? static_cast<long>(B) * head_groups : 1;
  long s;
  if (g_tuning.force_splits > 0) {
    s = g_tuning.force_splits;
  } else {
    // Measured on MI355X: a workgroup streams best over >= 1024 keys (prologue, LDS merge and the
    // partial write are per workgroup), so aim for target_workgroups with chunks that long ...
    s = (g_tuning.target_workgroups + pairs - 1) / pairs;
    const long cap_long = max_len / kLongChunk > 0 ? max_len / kLongChunk : 1;
    if (s > cap_long) s = cap_long;
    // ... unless that leaves most of the 256 CUs idle: then shorter chunks, down to kMinChunk keys
    if (pairs * s < g_tuning.target_workgroups / 2) {
      s = (g_tuning.target_workgroups / 2 + pairs - 1) / pairs;
      const long cap = (max_len + kMinChunk - 1) / kMinChunk;
      if (s > cap) s = cap;
    }
  }
  if (s > kMaxSplits) s = kMaxSplits;
  if (s < 1) s = 1;
  long chunk = (max_len + s - 1) / s;
  chunk = (chunk + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
  if (chunk < kChunkAlign) chunk = kChunkAlign;
  s = (max_len + chunk - 1) / chunk;
  if (s < 1) s = 1;
  return {static_cast<int>(s), static_cast<int>(chunk)};
}

// ---- 8 consecutive K or V elements as they come from memory --------------------------------------
template <typename T>
struct Frag8;

template <>
struct Frag8<__half> {
  Vec16 v;
  __device__ __forceinline__ void load(const __half *p) { v = ld16(p); }
  __device__ __forceinline__ void zero() { v.w[0] = v.w[1] = v.w[2] = v.w[3] = 0u; }
  // sum_i q[i]*k[i]: four packed fp16 dot-2 with an fp32 accumulator (products are exact in fp32)
  __device__ __forceinline__ float dot(const Frag8 &k) const {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_fdot2(as_half2(v.w[i]), as_half2(k.v.w[i]), s, false);
    return s;
  }
  __device__ __forceinline__ void axpy(float p, float (&acc)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = as_half2(v.w[i]);
      acc[2 * i] = __builtin_fmaf(p, static_cast<float>(h.x), acc[2 * i]);
      acc[2 * i + 1] = __builtin_fmaf(p, static_cast<float>(h.y), acc[2 * i + 1]);
    }
  }
};

template <>
struct Frag8<float> {
  float f[8];
  __device__ __forceinline__ void load(const float *p) {
    const Vec16 a = ld16(p), b = ld16(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = __builtin_bit_cast(float, a.w[i]);
      f[4 + i] = __builtin_bit_cast(float, b.w[i]);
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = 0.0f;
  }
  __device__ __forceinline__ float dot(const Frag8 &k) const {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = __builtin_fmaf(f[i], k.f[i], s);
    return s;
  }
  __device__ __forceinline__ void axpy(float p, float (&acc)[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(p, f[i], acc[i]);
  }
};

struct DecodeArgs {
  const void *q, *k, *v;
  const int32_t *seq_lens;
  void *out;
  float *part_acc;  // [B, Hq, n_splits, D]
  float *part_ml;   // [B, Hq, n_splits, 2]  (running max in log2 units, running sum)
  int Hq, group, max_len, chunk, n_splits;
  int64_t stride_b, stride_h, stride_s;
  float scale_log2e;
  int fused_merge;  // the last workgroup of a (sequence, head group) merges the splits
};

// Split partials travel between workgroups that may sit on different XCDs, whose L2 caches are not
// coherent with each other.  They are written and read with agent-scope atomic accesses (stores
// written through, loads served past the local caches), which costs nothing for these few bytes; a
// device-scope release fence instead would write back the whole L2 from every workgroup and was
// measured to triple the kernel's time.
__device__ __forceinline__ float ld_agent(const float *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float *p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Keys per split for a sequence of `len` keys: the sequence is cut into n_splits nearly equal
// ranges (rounded up to 16 keys, at least kMinDevChunk), so that the workgroups of one sequence
// finish together whatever its current length is; a range cut from the host-side upper bound would
// leave the last split short (4100 keys in 4 splits: 1040/1040/1040/980 instead of 1152/1152/1152/644).
constexpr int kMinDevChunk = 128;
__device__ __forceinline__ int balanced_chunk(int len, int n_splits) {
  int c = (len + n_splits - 1) / n_splits;
  c = (c + 15) & ~15;
  return c < kMinDevChunk ? kMinDevChunk : c;
}

__device__ __forceinline__ int clamped_len(const int32_t *seq_lens, int b, int max_len) {
  int len = seq_lens ? seq_lens[b] : max_len;
  len = len < 0 ? 0 : len;
  return len > max_len ? max_len : len;
}

// One tile: U load instructions per lane for K and for V (U*RG key rows per workgroup).
template <typename T, int D, int G, int U, bool CHECK>
__device__ __forceinline__ void decode_tile(const T *kb, const T *vb, int64_t stride_s, int base,
                                            int rg, int s1, float scale_log2e,
                                            const Frag8<T> (&qf)[G], float (&m)[G], float (&l)[G],
                                            float (&acc)[G][8]) {
  constexpr int LPR = D / 8;
  constexpr int RG = kThreads / LPR;
  Frag8<T> kr[U], vr[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int row = base + u * RG + rg;
    if (!CHECK || row < s1) {
      kr[u].load(kb + row * stride_s);
      vr[u].load(vb + row * stride_s);
    } else {
      kr[u].zero();
      vr[u].zero();
    }
  }
  float sc[G][U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const bool ok = !CHECK || (base + u * RG + rg) < s1;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const float d = group_sum<LPR>(qf[g].dot(kr[u])) * scale_log2e;
      sc[g][u] = ok ? d : kNegBig;
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mt = sc[g][0];
#pragma unroll
    for (int u = 1; u < U; ++u) mt = fmaxf(mt, sc[g][u]);
    const float mn = fmaxf(m[g], mt);
    const float corr = __builtin_amdgcn_exp2f(m[g] - mn);
    m[g] = mn;
    l[g] *= corr;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] *= corr;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float p = __builtin_amdgcn_exp2f(sc[g][u] - mn);
      if (CHECK && (base + u * RG + rg) >= s1) p = 0.0f;
      l[g] += p;
      vr[u].axpy(p, acc[g]);
    }
  }
}

template <typename T, int D, int G, int U>
__global__ __launch_bounds__(kThreads, 4) void gqa_decode_split_kernel(DecodeArgs a) {
  constexpr int LPR = D / 8;
  constexpr int RG = kThreads / LPR;
  const int split = blockIdx.x, hg = blockIdx.y, b = blockIdx.z;
  const int len = clamped_len(a.seq_lens, b, a.max_len);
  const int chunk = balanced_chunk(len, a.n_splits);
  const int s0 = split * chunk;
  const int tid = threadIdx.x;
  const int h0 = hg * G;            // first query head of this workgroup
  if (s0 >= len) {
    // An empty split is never read by the merge.  A sequence without keys gets zeros, written by
    // its split-0 workgroup when no separate merge kernel will do it.
    if (len == 0 && split == 0 && (a.n_splits == 1 || a.fused_merge)) {
      for (int o = tid; o < G * D; o += kThreads)
        stf(static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.Hq + h0) * D + o, 0.0f);
    }
    return;
  }
  const int s1 = min(s0 + chunk, len);

  const int rg = tid / LPR, dl = tid % LPR;
  const int hk = h0 / a.group;      // the kv head those G query heads share

  const T *q = static_cast<const T *>(a.q);
  Frag8<T> qf[G];
#pragma unroll
  for (int g = 0; g < G; ++g) qf[g].load(q + (static_cast<int64_t>(b) * a.Hq + h0 + g) * D + dl * 8);

  const int64_t kv_off = b * a.stride_b + hk * a.stride_h + dl * 8;
  const T *kb = static_cast<const T *>(a.k) + kv_off;
  const T *vb = static_cast<const T *>(a.v) + kv_off;

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegBig;
    l[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }

  int base = s0;
  for (; base + U * RG <= s1; base += U * RG)
    decode_tile<T, D, G, U, false>(kb, vb, a.stride_s, base, rg, s1, a.scale_log2e, qf, m, l, acc);
  for (; base < s1; base += U * RG)
    decode_tile<T, D, G, U, true>(kb, vb, a.stride_s, base, rg, s1, a.scale_log2e, qf, m, l, acc);

  // ---- merge the RG row-group states of this workgroup ----------------------------------------
  __shared__ float s_m[G][RG];
  __shared__ float s_l[G][RG];
  __shared__ __attribute__((aligned(16))) float s_acc[G][RG][D];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (dl == 0) {
      s_m[g][rg] = m[g];
      s_l[g][rg] = l[g];
    }
    Row8<float>::store(&s_acc[g][rg][dl * 8], acc[g]);
  }
  __syncthreads();
  for (int o = tid; o < G * D; o += kThreads) {
    const int g = o / D, d = o % D;
    float mx = kNegBig;
#pragma unroll
    for (int r = 0; r < RG; ++r) mx = fmaxf(mx, s_m[g][r]);
    float lsum = 0.0f, asum = 0.0f;
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      const float w = __builtin_amdgcn_exp2f(s_m[g][r] - mx);
      lsum = __builtin_fmaf(s_l[g][r], w, lsum);
      asum = __builtin_fmaf(s_acc[g][r][d], w, asum);
    }
    const int64_t bh = static_cast<int64_t>(b) * a.Hq + h0 + g;
    if (a.n_splits == 1) {
      stf(static_cast<T *>(a.out) + bh * D + d, lsum > 0.0f ? asum / lsum : 0.0f);
    } else {
      st_agent(&a.part_acc[(bh * a.n_splits + split) * D + d], asum);
      if (d == 0) {
        st_agent(&a.part_ml[(bh * a.n_splits + split) * 2], mx);
        st_agent(&a.part_ml[(bh * a.n_splits + split) * 2 + 1], lsum);
      }
    }
  }
  if (a.n_splits == 1 || !a.fused_merge) return;

  // ---- in-kernel merge: the workgroup that takes the last ticket combines all splits ------------
  const int n_valid = (len + chunk - 1) / chunk;  // splits that run for this sequence
  __shared__ int s_last;
  __syncthreads();  // every wavefront's partial stores have completed before the ticket is taken
  if (tid == 0) {
    unsigned int *ticket = &g_tickets[b * gridDim.y + hg];
    const unsigned int t = atomicAdd(ticket, 1u);
    s_last = (t == static_cast<unsigned int>(n_valid - 1));
    if (s_last) atomicExch(ticket, 0u);  // ready for the next launch
  }
  __syncthreads();
  if (!s_last) return;
  for (int o = tid; o < G * D; o += kThreads) {
    const int g = o / D, d = o % D;
    const int64_t bh = static_cast<int64_t>(b) * a.Hq + h0 + g;
    const float *ml = a.part_ml + bh * a.n_splits * 2;
    const float *pa = a.part_acc + bh * a.n_splits * D + d;
    float mx = kNegBig;
    for (int s = 0; s < n_valid; ++s) mx = fmaxf(mx, ld_agent(ml + 2 * s));
    float lsum = 0.0f, asum = 0.0f;
    for (int s = 0; s < n_valid; ++s) {
      const float w = __builtin_amdgcn_exp2f(ld_agent(ml + 2 * s) - mx);
      lsum = __builtin_fmaf(ld_agent(ml + 2 * s + 1), w, lsum);
      asum = __builtin_fmaf(ld_agent(pa + static_cast<int64_t>(s) * D), w, asum);
    }
    stf(static_cast<T *>(a.out) + bh * D + d, lsum > 0.0f ? asum / lsum : 0.0f);
  }
}

// Cross-split merge: one workgroup of D threads per (sequence, query head).
template <typename T, int D>
__global__ __launch_bounds__(D) void gqa_decode_merge_kernel(DecodeArgs a) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int len = clamped_len(a.seq_lens, b, a.max_len);
  const int chunk = balanced_chunk(len, a.n_splits);
  const int n_valid = (len + chunk - 1) / chunk;  // splits that wrote a partial
  const int64_t bh = static_cast<int64_t>(b) * a.Hq + h;
  T *out = static_cast<T *>(a.out) + bh * D + d;
  if (n_valid == 0) {
    stf(out, 0.0f);
    return;
  }
  const float *ml = a.part_ml + bh * a.n_splits * 2;
  const float *pa = a.part_acc + bh * a.n_splits * D + d;
  float mx = kNegBig;
  for (int s = 0; s < n_valid; ++s) mx = fmaxf(mx, ml[2 * s]);
  float lsum = 0.0f, asum = 0.0f;
  for (int s = 0; s < n_valid; ++s) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * s] - mx);
    lsum = __builtin_fmaf(ml[2 * s + 1], w, lsum);
    asum = __builtin_fmaf(pa[static_cast<int64_t>(s) * D], w, asum);
  }
  stf(out, lsum > 0.0f ? asum / lsum : 0.0f);
}

template <typename T, int D, int G>
int launch_decode(const DecodeArgs &a, int B, hipStream_t st) {
  constexpr int U = (sizeof(T) == 2 ? 8 : 4) / (G >= 4 ? 2 : 1);
  const dim3 grid(a.n_splits, a.Hq / G, B);
  hipLaunchKernelGGL((gqa_decode_split_kernel<T, D, G, U>), grid, dim3(kThreads), 0, st, a);
  if (a.n_splits > 1 && !a.fused_merge)
    hipLaunchKernelGGL((gqa_decode_merge_kernel<T, D>), dim3(a.Hq, B), dim3(D), 0, st, a);
  return launch_status();
}

template <typename T, int D>
int dispatch_group(const DecodeArgs &a, int G, int B, hipStream_t st) {
  switch (G) {
    case 4: return launch_decode<T, D, 4>(a, B, st);
    case 2: return launch_decode<T, D, 2>(a, B, st);
    default: return launch_decode<T, D, 1>(a, B, st);
  }
}

template <typename T>
int dispatch_dim(const DecodeArgs &a, int D, int G, int B, hipStream_t st) {
  switch (D) {
    case 64: return dispatch_group<T, 64>(a, G, B, st);
    case 128: return dispatch_group<T, 128>(a, G, B, st);
    case 256: return dispatch_group<T, 256>(a, G, B, st);
    default: return AXHIP_INVALID_ARGUMENT;
  }
}

// Query heads served per workgroup: the largest of 4, 2, 1 that divides the group size.
int heads_per_workgroup(int group) { return group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1); }

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

// Measurement hook: overrides the split heuristics (0 restores the default).
AXHIP_API void axhip_gqa_decode_tune(int target_workgroups, int force_splits) {
  // a negative target selects the single-launch form (the last workgroup merges); measured no
  // faster than the second kernel (ticket + write-through latency at the tail), so not the default
  g_tuning.separate_merge = target_workgroups < 0 ? 0 : 1;
  g_tuning.target_workgroups = target_workgroups > 0 ? target_workgroups : Tuning().target_workgroups;
  g_tuning.force_splits = force_splits > 0 ? force_splits : 0;
}

// Reports the plan the launcher will use (tests and benchmarks print it).
AXHIP_API void axhip_gqa_decode_plan(int B, int Hq, int Hkv, int max_len, int *n_splits, int *chunk) {
  const int group = (Hkv > 0 && Hq % Hkv == 0) ? Hq / Hkv : 1;
  const SplitPlan p = plan_splits(B, Hq / heads_per_workgroup(group), max_len);
  if (n_splits) *n_splits = p.n_splits;
  if (chunk) *chunk = p.chunk;
}

AXHIP_API size_t axhip_gqa_decode_workspace_bytes(int B, int Hq, int Hkv, int D, int max_len) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || max_len <= 0 || Hq % Hkv != 0) return 0;
  // sized for the largest split count any tuning can choose
  return static_cast<size_t>(B) * Hq * kMaxSplits * (D + 2) * sizeof(float);
}

AXHIP_API int axhip_gqa_decode(const void *q, const void *k, const void *v, const int32_t *seq_lens,
                               void *out, void *workspace, size_t workspace_bytes, int dtype, int B,
                               int Hq, int Hkv, int D, int max_len, int64_t stride_b,
                               int64_t stride_h, int64_t stride_s, axhip_stream stream) {
  if (dtype != AXHIP_FLOAT16 && dtype != AXHIP_FLOAT32) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || max_len <= 0) return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (D != 64 && D != 128 && D != 256) return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (B > 65535) return AXHIP_INVALID_ARGUMENT;
  if (!q || !k || !v || !out) return AXHIP_INVALID_PTR;
  // rows must allow 16-byte loads
  const int64_t esz = dtype == AXHIP_FLOAT16 ? 2 : 4;
  if ((stride_s * esz) % 16 || (stride_h * esz) % 16 || (stride_b * esz) % 16) return AXHIP_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 15)
    return AXHIP_INVALID_PTR;

  const int group = Hq / Hkv;
  const int G = heads_per_workgroup(group);
  const SplitPlan plan = plan_splits(B, Hq / G, max_len);

  DecodeArgs a;
  a.q = q;
  a.k = k;
  a.v = v;
  a.seq_lens = seq_lens;
  a.out = out;
  a.Hq = Hq;
  a.group = group;
  a.max_len = max_len;
  a.chunk = plan.chunk;
  a.n_splits = plan.n_splits;
  a.stride_b = stride_b;
  a.stride_h = stride_h;
  a.stride_s = stride_s;
  a.scale_log2e = 1.4426950408889634f / sqrtf(static_cast<float>(D));
  a.part_acc = nullptr;
  a.part_ml = nullptr;
  a.fused_merge = (!g_tuning.separate_merge && static_cast<long>(B) * (Hq / G) <= kTicketSlots) ? 1 : 0;
  if (plan.n_splits > 1) {
    const size_t acc_elems = static_cast<size_t>(B) * Hq * plan.n_splits * D;
    const size_t need = (acc_elems + static_cast<size_t>(B) * Hq * plan.n_splits * 2) * sizeof(float);
    if (!workspace || workspace_bytes < need) return AXHIP_INVALID_ARGUMENT;
    a.part_acc = static_cast<float *>(workspace);
    a.part_ml = a.part_acc + acc_elems;
  }
  hipStream_t st = as_stream(stream);
  return dtype == AXHIP_FLOAT16 ? dispatch_dim<__half>(a, D, G, B, st)
                                : dispatch_dim<float>(a, D, G, B, st);
}

}  // extern "C"
