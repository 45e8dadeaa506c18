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
// v_exp_f32 instructions.  A sequence that is one key range is normalised and written by its
// workgroup.  Otherwise the per-range results (unnormalised output, running max, running sum) go to
// a workspace, and the workgroup that takes the last ticket of a (sequence, head group) merges them
// in the same launch; a second small merge kernel is kept behind the tuning hook for comparison.
#include "common.hpp"

#include <type_traits>

namespace axhip {
namespace {

constexpr int kThreads = 256;
constexpr float kNegBig = -1.0e30f;   // "no key seen yet" in the log2 domain (finite: no inf-inf)
constexpr int kMaxSplits = 128;
constexpr int kChunkAlign = 128;      // key ranges start on multiples of this
constexpr int kMinChunk = 256;

struct Tuning {
  int target_workgroups = 0;    // workgroups that stream at a time; 0 = one per compute unit of the
                                // device, which keeps HBM busy with streaming loads (measured on the
                                // 256 CUs of an MI355X: 256 workgroups 153 us, 1024 163 us at B=32
                                // L=8192), and nothing has to be merged when a sequence is one
  int force_splits = 0;         // > 0: fixed split count for every sequence (measurement sweeps)
  int mfma_groups = 1;          // 0: head groups of four and more stay on the vector path (measurement sweeps)
  int separate_merge = 0;       // 1: merge in a second kernel; 0: the last workgroup of a sequence merges
};
Tuning g_tuning;

// Ticket counters of the in-kernel merge, one per (sequence, head group).  They start at zero and
// the merging workgroup puts its counter back to zero, so no launch ever has to clear them.
// Launches that overlap in time on one device must not share (sequence, head group) slots; calls on
// one stream, and replays of a captured graph, never overlap.  Launches that do overlap (graphs replayed
// side by side) come from different ticket lanes: a lane is a region of its own in this array.
constexpr int kTicketSlots = 1 << 16;  // per ticket lane
__device__ unsigned int g_tickets[AXHIP_TICKET_LANES * kTicketSlots];
// What the slots of a length-dealt launch found, kept for the later launches of the same step
// (axhip_set_plan_reuse): 8 ints per slot, per ticket lane.
constexpr int kPlanSlots = 4096;
__device__ int g_plan_cache[AXHIP_TICKET_LANES * kPlanSlots * 8];

// Atomics on one 128-byte line are served one after the other (about 10 ns each on MI355X), and the workgroups
// of a launch finish together: neighbouring (sequence, head group) pairs therefore take counters 128 bytes
// apart; the words in between belong to pairs 2048, 4096, ... further on.
__device__ __forceinline__ unsigned int *ticket_of(int lane_base, int pair) {
  return &g_tickets[lane_base + (((pair & 2047) << 5) | (pair >> 11))];
}

// Scratch of the entry point that allocates nothing (axhip_gqa_decode_static): the split partials live here
// instead of in a caller's workspace.  Every device the library runs on holds its own copy of this array
// until the process ends.  In host code the array's name is only a stand-in for the symbol: the address
// on a device comes from hipGetSymbolAddress (static_scratch_on_this_device below) and kernels get that
// pointer as an argument, exactly as they get a caller's workspace.
static __device__ __align__(256) unsigned char scratch[AXHIP_GQA_DECODE_STATIC_SCRATCH_BYTES];

}  // namespace
int reset_attention_tickets() {
  void *p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_tickets)) != hipSuccess || !p) return AXHIP_DEVICE_ERROR;
  if (hipDeviceSynchronize() != hipSuccess) return AXHIP_DEVICE_ERROR;
  return hipMemset(p, 0, sizeof(unsigned int) * AXHIP_TICKET_LANES * kTicketSlots) == hipSuccess ? AXHIP_OK : AXHIP_DEVICE_ERROR;
}
namespace {

constexpr int kMaxDynBatch = 64;  // batches up to this size deal their workgroups by sequence length

// How the key axis is cut.  The plan depends only on host-side sizes, so that a captured launch stays
// valid while the device-side lengths change.
//   dynamic (B <= kMaxDynBatch, no forced split count): the grid holds `active` workgroups per head
//     group (one workgroup per CU over all head groups); on the device they are dealt to the
//     sequences in proportion to their current lengths, so that every workgroup streams about
//     (sum of lengths) / active keys whatever the mix of lengths is.  A batch of equal lengths gets
//     active / B splits per sequence.  The launch is one-dimensional with the slot index slowest, so
//     that the slots a launch leaves unused are the last workgroups dispatched: measured, a CU that
//     gets two streaming workgroups while another gets none costs 28 % (B=8, L=8192: 56 us against
//     44 us) - the memory pipeline of a CU holds about one workgroup's worth of loads in flight.
//   static: every sequence is cut into n_splits ranges.
struct SplitPlan {
  int n_splits;  // grid.x: workgroups per (sequence, head group) slot
  int chunk;     // nominal keys per workgroup for max_len (reporting only)
  int dynamic;
  int active;    // dynamic: streaming workgroups per head group
  int stride;    // splits a sequence can have at most (workspace stride)
};

SplitPlan plan_splits(int B, int head_groups, int max_len) {
  SplitPlan p{};
  const long target_workgroups = g_tuning.target_workgroups > 0 ? g_tuning.target_workgroups : device_cu_count();
  const long hgs = head_groups > 0 ? head_groups : 1;
  const long Bc = B > 0 ? B : 1;
  if (g_tuning.force_splits == 0 && Bc <= kMaxDynBatch) {
    long active = (target_workgroups + hgs - 1) / hgs;
    // no point in ranges shorter than kMinChunk - except that up to eight ranges per sequence may go down
    // to half of that: a short single sequence is all latency, and one tile per workgroup instead of two
    // saves a memory round trip (B=1, L=1024: 8.0 -> 6.9 us; with more ranges the merge eats the gain)
    long cap = (Bc * max_len + kMinChunk - 1) / kMinChunk;
    const long cap_half = (Bc * max_len + kMinChunk / 2 - 1) / (kMinChunk / 2);
    if (cap < (cap_half < 8 * Bc ? cap_half : 8 * Bc)) cap = cap_half < 8 * Bc ? cap_half : 8 * Bc;
    if (active > cap) active = cap;
    if (active < 1) active = 1;
    if (active < Bc) active = Bc;  // every sequence needs a workgroup of its own
    p.dynamic = 1;
    p.active = static_cast<int>(active);
    p.n_splits = static_cast<int>((active + Bc - 1) / Bc);  // reporting: splits of a sequence when all are equal
    p.stride = static_cast<int>(active < kMaxSplits ? active : kMaxSplits);
    long c = (Bc * max_len + active - 1) / active;
    p.chunk = static_cast<int>(c);
    return p;
  }
  long s;
  if (g_tuning.force_splits > 0) {
    s = g_tuning.force_splits;
  } else {
    const long pairs = Bc * hgs;
    s = (target_workgroups + pairs - 1) / pairs;
    const long cap = (max_len + kMinChunk - 1) / kMinChunk;
    if (s > cap) s = cap;
  }
  if (s > kMaxSplits) s = kMaxSplits;
  if (s < 1) s = 1;
  long chunk = (max_len + s - 1) / s;
  chunk = (chunk + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
  if (chunk < kChunkAlign) chunk = kChunkAlign;
  s = (max_len + chunk - 1) / chunk;
  if (s < 1) s = 1;
  p.n_splits = static_cast<int>(s);
  p.chunk = static_cast<int>(chunk);
  p.stride = p.n_splits;
  return p;
}

// ---- 8 consecutive K or V elements as they come from memory --------------------------------------
template <typename T>
struct Frag8;

template <>
struct Frag8<__half> {
  Vec16 v;
  template <int SECOND>
  __device__ __forceinline__ void load(const __half *p) { v = ld16(p); }
  template <int SECOND>
  __device__ __forceinline__ void load_stream(const __half *p) { v = ld16_stream(p); }
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
  // elements 4..7 sit SECOND elements behind p (see FragMap)
  template <int SECOND>
  __device__ __forceinline__ void load(const float *p) {
    const Vec16 a = ld16(p), b = ld16(p + SECOND);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = __builtin_bit_cast(float, a.w[i]);
      f[4 + i] = __builtin_bit_cast(float, b.w[i]);
    }
  }
  template <int SECOND>
  __device__ __forceinline__ void load_stream(const float *p) {
    const Vec16 a = ld16_stream(p), b = ld16_stream(p + SECOND);
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

// Which 8 of a row's D elements lane `dl` of a row group holds.  fp16: 8 consecutive ones (one
// 16-byte load).  fp32 takes two 16-byte loads; 4 elements from each half of the row, so that the
// lanes of a row group read a contiguous half row per load instruction (with 8 consecutive elements
// per lane each instruction would touch every cache line of the row and use half of it).
template <typename T, int D>
struct FragMap {
  static constexpr int kLane = sizeof(T) == 4 ? 4 : 8;        // first element = dl * kLane
  static constexpr int kSecond = sizeof(T) == 4 ? D / 2 : 4;  // offset of elements 4..7 from there
};

// Writes a lane's 8 accumulators to their places in an fp32 row of D elements.
template <typename T, int D>
__device__ __forceinline__ void store_lane_acc(float *row, int dl, const float (&acc)[8]) {
  float *p = row + dl * FragMap<T, D>::kLane;
  *reinterpret_cast<float4 *>(p) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  *reinterpret_cast<float4 *>(p + FragMap<T, D>::kSecond) = make_float4(acc[4], acc[5], acc[6], acc[7]);
}

struct DecodeArgs {
  const void *q, *k, *v;
  const int32_t *seq_lens;
  void *out;
  float *part_acc;  // [B, Hq, n_splits, D]
  float *part_ml;   // [B, Hq, n_splits, 2]  (running max in log2 units, running sum)
  int Hq, group, max_len, chunk, n_splits;
  int dynamic, active, split_stride, B, n_hg;  // see SplitPlan; split_stride = partial slots per (sequence, head)
  int wg_heads;  // query heads per workgroup (the template parameter G on the vector path)
  int ticket_base;  // first ticket counter of the caller's ticket lane
  int64_t stride_b, stride_h, stride_s;
  float scale_log2e;
  int fused_merge;  // the last workgroup of a (sequence, head group) merges the splits
  // Decode-step form (template parameter QKV): q, and the key / value row of the token being decoded,
  // come straight from the fp32 output of the qkv projection; seq_lens holds the lengths before the
  // append.  a.k / a.v are then the caches [B, Hkv, Lmax, D] and are written at row seq_lens[b].
  int len_add;              // 1 in that form: the attended length is seq_lens[b] + 1
  const float *pq, *pk, *pv;
  int64_t pq_stride, pk_stride, pv_stride;
  const void *qw, *kw;      // per-head RMSNorm weights [D] or null
  int w_f16;
  float eps;
  const int64_t *pos;       // [3, B]
  const float *inv_freq;    // [D/2]
  int h_lim, w_lim, cache_rows;
  // Paged cache (template parameter PAGED): a.k / a.v are pools [n_pages, Hkv, kPageKeys, D]; key s of
  // sequence b is row s % kPageKeys of page page_table[b * max_pages + s / kPageKeys].
  const int32_t *page_table;
  int max_pages, n_pages;
  int64_t page_stride;  // elements per page: Hkv * kPageKeys * D
  // Decode-step form with lengths dealt in the kernel: the attention launches of a step (one per layer) deal the
  // same lengths the same way.  plan_mode 1: a launch leaves what every slot found (8 ints per slot) in plan_cache; 2: a launch
  // reads that instead of the lengths and the dealing.  plan_check marks the entries of a launch of this shape.
  int *plan_cache;
  int plan_mode, plan_check;
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
constexpr int kNoLength = INT32_MIN;  // "read the length yourself"
__device__ __forceinline__ int balanced_chunk(int len, int n_splits) {
  int c = (len + n_splits - 1) / n_splits;
  c = (c + 15) & ~15;
  return c < kMinDevChunk ? kMinDevChunk : c;
}

__device__ __forceinline__ int clamped_len(const int32_t *seq_lens, int b, int max_len, int len_add = 0) {
  int len = seq_lens ? seq_lens[b] : max_len;
  len = len < 0 ? 0 : len;
  if (len_add && len < max_len) len += len_add;
  return len > max_len ? max_len : len;
}

__device__ __forceinline__ int dyn_splits_of(int len, int c, int stride) {
  const int n = len > 0 ? (len + c - 1) / c : 1;
  return n < stride ? n : stride;
}
__device__ __forceinline__ int wave_sum_i(int v) { return wave_sum_i32(v); }
__device__ __forceinline__ int wave_max_i(int v) { return wave_max_i32(v); }
__device__ __forceinline__ int wave_prefix_i(int v, int) { return wave_prefix_i32(v); }  // inclusive, over the lanes
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// One head row of the qkv projection -> RMSNorm over the head (weights optional) -> interleaved
// M-RoPE at this sequence's (t, h, w) position, in the evaluation order of the single operators
// (rms_norm: (x * inv) * w; rope_thd: x0*c - x1*s, x1*c + x0*s).  One wavefront per row; the result
// goes to `dst` (LDS) in the cache dtype and, when `gdst` is set, to the cache row as well.
template <typename T, int D>
__device__ __forceinline__ void norm_rope_row(const DecodeArgs &a, const float *src, const void *w, int b,
                                              int B, int lane, T *dst, T *gdst) {
  constexpr int HALF = D / 2;
  float ss = 0.f;
  for (int i = lane; i < HALF; i += 64) {
    const float x0 = src[i], x1 = src[i + HALF];
    ss = __builtin_fmaf(x0, x0, ss);
    ss = __builtin_fmaf(x1, x1, ss);
  }
  ss = group_sum<64>(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(D) + a.eps);
  const float pt = static_cast<float>(a.pos[b]);
  const float ph = static_cast<float>(a.pos[B + b]);
  const float pw = static_cast<float>(a.pos[2 * B + b]);
  for (int i = lane; i < HALF; i += 64) {
    float x0 = src[i] * inv, x1 = src[i + HALF] * inv;
    if (w) {
      x0 *= a.w_f16 ? __half2float(static_cast<const __half *>(w)[i]) : static_cast<const float *>(w)[i];
      x1 *= a.w_f16 ? __half2float(static_cast<const __half *>(w)[i + HALF]) : static_cast<const float *>(w)[i + HALF];
    }
    const float f = a.inv_freq[i];
    float ang = pt * f;
    if (i % 3 == 1 && i < a.h_lim)
      ang = ph * f;
    else if (i % 3 == 2 && i < a.w_lim)
      ang = pw * f;
    float sn, cs;
    sincosf(ang, &sn, &cs);
    const float y0 = x0 * cs - x1 * sn, y1 = x1 * cs + x0 * sn;
    stf(dst + i, y0);
    stf(dst + i + HALF, y1);
    if (gdst) {
      stf(gdst + i, y0);
      stf(gdst + i + HALF, y1);
    }
  }
}

// Where key row `row` of the workgroup's (sequence, kv head) starts, as an element offset from the
// workgroup's base pointers.  Dense: rows lie stride_s elements apart.  Paged: the sequence's keys live in
// pages of kPageKeys rows scattered over a pool [n_pages, Hkv, kPageKeys, D]; the page numbers of the
// workgroup's key range sit in LDS (filled from the page table before the first tile).
constexpr int kPageShift = 7;
constexpr int kPageKeys = 1 << kPageShift;      // keys per page: one tile of the fp16 D=128 kernel
constexpr int kMaxRangePages = 1025;            // page numbers a workgroup can hold: ranges of up to 131072 keys
struct DenseRows {
  int64_t stride_s;
  __device__ __forceinline__ int64_t operator()(int row) const { return row * stride_s; }
};
typedef const int __attribute__((address_space(3))) *lds_cint_ptr;
struct PagedRows {
  lds_cint_ptr pages;   // page numbers of pages first_page, first_page + 1, ... of this sequence
  int first_page;
  int row_elems;        // D
  int64_t page_stride;  // Hkv * kPageKeys * D
  __device__ __forceinline__ int64_t operator()(int row) const {
    return pages[(row >> kPageShift) - first_page] * page_stride + (row & (kPageKeys - 1)) * row_elems;
  }
};

// One tile: U load instructions per lane for K and for V (U*RG key rows per workgroup).
template <typename T, int D, int U, bool CHECK, typename ROWS>
__device__ __forceinline__ void tile_load(const T *kb, const T *vb, const ROWS &rows, int base, int rg, int s1,
                                          Frag8<T> (&kr)[U], Frag8<T> (&vr)[U]) {
  constexpr int RG = kThreads / (D / 8);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int row = base + u * RG + rg;
    if (!CHECK || row < s1) {
      const int64_t off = rows(row);
      kr[u].template load_stream<FragMap<T, D>::kSecond>(kb + off);  // read once: streaming loads
      vr[u].template load_stream<FragMap<T, D>::kSecond>(vb + off);
    } else {
      kr[u].zero();
      vr[u].zero();
    }
  }
}

template <typename T, int D, int G, int U, bool CHECK>
__device__ __forceinline__ void tile_update(const Frag8<T> (&kr)[U], const Frag8<T> (&vr)[U], int base, int rg,
                                            int s1, float scale_log2e, const Frag8<T> (&qf)[G], float (&m)[G],
                                            float (&l)[G], float (&acc)[G][8]) {
  constexpr int LPR = D / 8;
  constexpr int RG = kThreads / LPR;
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

template <typename T, int D, int G, int U, bool CHECK, typename ROWS>
__device__ __forceinline__ void decode_tile(const T *kb, const T *vb, const ROWS &rows, int base,
                                            int rg, int s1, float scale_log2e,
                                            const Frag8<T> (&qf)[G], float (&m)[G], float (&l)[G],
                                            float (&acc)[G][8]) {
  Frag8<T> kr[U], vr[U];
  tile_load<T, D, U, CHECK>(kb, vb, rows, base, rg, s1, kr, vr);
  tile_update<T, D, G, U, CHECK>(kr, vr, base, rg, s1, scale_log2e, qf, m, l, acc);
}

// A sequence without keys: its output rows are zeros.
template <typename T, int D, int G, bool MFMA = false>
__device__ __forceinline__ void write_zero_rows(const DecodeArgs &a, int b, int hg) {
  if constexpr (MFMA) {
    for (int o = threadIdx.x; o < a.wg_heads * D; o += kThreads)
      stf(static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.Hq + hg * a.wg_heads) * D + o, 0.0f);
    return;
  }
  for (int o = threadIdx.x; o < G * D; o += kThreads)
    stf(static_cast<T *>(a.out) + (static_cast<int64_t>(b) * a.Hq + hg * G) * D + o, 0.0f);
}

// The merge of the n_valid partial states a (sequence, head) was cut into, for output element d of the head:
//   out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M),  M = max_s m_s,
// summed in range order - the arithmetic of gqa_decode_merge_kernel, so both forms of the merge give the same bits.
// The partials were written past the local caches by other workgroups and are read the same way: a load costs
// a trip to the memory side, so all loads of up to NB ranges are in flight before the first is used (one trip
// for the 32 ranges a single long sequence is cut into; ranges beyond NB follow in further rounds of NB loads).
template <int NB>
__device__ __forceinline__ float merge_ranges(const float *ml, const float *pa, int n_valid, int D) {
  float pm[NB], pl[NB], pv[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int sidx = min(i, n_valid - 1);
    pm[i] = ld_agent(ml + 2 * sidx);
    pl[i] = ld_agent(ml + 2 * sidx + 1);
    pv[i] = ld_agent(pa + static_cast<int64_t>(sidx) * D);
  }
  float mx = kNegBig;
#pragma unroll
  for (int i = 0; i < NB; ++i)
    if (i < n_valid) mx = fmaxf(mx, pm[i]);
  // more ranges than NB: their maxima, again NB loads at a time
  for (int s0 = NB; s0 < n_valid; s0 += NB) {
    float qm[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) qm[i] = ld_agent(ml + 2 * min(s0 + i, n_valid - 1));
#pragma unroll
    for (int i = 0; i < NB; ++i) mx = fmaxf(mx, qm[i]);  // (a repeated last range changes no maximum)
  }
  float lsum = 0.0f, asum = 0.0f;
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if (i >= n_valid) continue;
    const float w = __builtin_amdgcn_exp2f(pm[i] - mx);
    lsum = __builtin_fmaf(pl[i], w, lsum);
    asum = __builtin_fmaf(pv[i], w, asum);
  }
  for (int s0 = NB; s0 < n_valid; s0 += NB) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int sidx = min(s0 + i, n_valid - 1);
      pm[i] = ld_agent(ml + 2 * sidx);
      pl[i] = ld_agent(ml + 2 * sidx + 1);
      pv[i] = ld_agent(pa + static_cast<int64_t>(sidx) * D);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      if (s0 + i >= n_valid) continue;
      const float w = __builtin_amdgcn_exp2f(pm[i] - mx);
      lsum = __builtin_fmaf(pl[i], w, lsum);
      asum = __builtin_fmaf(pv[i], w, asum);
    }
  }
  return lsum > 0.0f ? asum / lsum : 0.0f;
}

// Keys [s0, s1) of sequence b for the G query heads of head group hg: range number `split` of the
// `n_valid` non-empty ranges this sequence is cut into in this launch.  The only range of a sequence
// writes the result itself when `direct_ok`; otherwise the range leaves a partial state and (fused
// merge) the workgroup that finishes last combines them.  A workgroup may call this several times:
// the caller puts a barrier between two calls, because the LDS arrays are the same.
template <typename T, int D, int G, int U, bool QKV, bool HOIST, bool PAGED = false>
__device__ __forceinline__ void process_range(const DecodeArgs &a, int b, int hg, int split, int n_valid,
                                              bool direct_ok, int s0, int s1, int p_raw = kNoLength) {
  constexpr int LPR = D / 8;
  constexpr int RG = kThreads / LPR;
  int tid = threadIdx.x;
  // opaque inside a caller's loop over pieces, so that nothing derived from it is computed ahead of
  // the loop and held in registers across the whole piece
  if constexpr (!HOIST) asm volatile("" : "+v"(tid));
  const int h0 = hg * G;            // first query head of this workgroup

  const int rg = tid / LPR, dl = tid % LPR;
  const int hk = h0 / a.group;      // the kv head those G query heads share

  constexpr int SEC = FragMap<T, D>::kSecond;
  const int lane_el = dl * FragMap<T, D>::kLane;  // this lane's first element of a row
  // paged: the pool is [page, kv head, key in page, D], so only the head and the lane are fixed here
  const int64_t kv_off = PAGED ? static_cast<int64_t>(hk) * (kPageKeys * D) + lane_el
                               : b * a.stride_b + hk * a.stride_h + lane_el;
  const T *kb = static_cast<const T *>(a.k) + kv_off;
  const T *vb = static_cast<const T *>(a.v) + kv_off;
  // the page numbers of keys [s0, s1) of this sequence, from the page table into LDS
  __shared__ int s_pages[PAGED ? kMaxRangePages : 1];
  const int first_page = s0 >> kPageShift;
  if constexpr (PAGED) {
    const int range_pages = ((s1 - 1) >> kPageShift) - first_page + 1;
    const int32_t *tbl = a.page_table + static_cast<int64_t>(b) * a.max_pages + first_page;
    // page numbers are clamped into the pool: a corrupt table gives wrong values, never an access outside it
    for (int i = tid; i < range_pages; i += kThreads) s_pages[i] = min(max(tbl[i], 0), a.n_pages - 1);
    __syncthreads();
  }
  using Rows = typename std::conditional<PAGED, PagedRows, DenseRows>::type;
  Rows rows;
  if constexpr (PAGED) {
    rows.pages = (lds_cint_ptr)s_pages;
    rows.first_page = first_page;
    rows.row_elems = D;
    rows.page_stride = a.page_stride;
  } else {
    rows.stride_s = a.stride_s;
  }

  Frag8<T> qf[G];
  // Decode-step form: the token being decoded sits at row p_new; the workgroup whose key range holds
  // that row prepares its key and value itself (from the projection output, rounded to the cache
  // dtype exactly as the cache stores them) and attends to them from LDS, because the cache row is
  // written in this same launch - by the first of the workgroups that share the kv head.
  __shared__ __attribute__((aligned(16))) T s_q[QKV ? G : 1][D];
  __shared__ __attribute__((aligned(16))) T s_kv[2][QKV ? D : 8];
  bool mine = false;
  int kv_end = s1;  // keys [s0, kv_end) come from the cache
  Frag8<T> kr0[QKV && HOIST ? U : 1], vr0[QKV && HOIST ? U : 1];
  if constexpr (QKV) {
    int p_new = p_raw != kNoLength ? p_raw : a.seq_lens[b];  // (the caller may have it from the plan cache)
    p_new = p_new < 0 ? 0 : p_new;
    mine = p_new < a.max_len && p_new < a.cache_rows && p_new >= s0 && p_new < s1;  // then p_new == s1 - 1
    if (mine) kv_end = p_new;
    // the first tile of cached keys is requested before q is prepared: those loads do not need it
    if constexpr (HOIST) tile_load<T, D, U, true>(kb, vb, rows, s0, rg, kv_end, kr0, vr0);
    const int wave = tid >> 6, lane = tid & 63;
    const int B = a.B;
    bool writer = mine && (h0 % a.group == 0);
    if constexpr (PAGED) {
      // The clamp above protects reads only.  The page the new row is written to must be one the table
      // really names: an entry outside the pool (a sequence whose pages were given back) skips the store,
      // as kv_append_paged_kernel does, instead of landing in another sequence's page.
      if (writer) {
        const int raw = a.page_table[static_cast<int64_t>(b) * a.max_pages + (p_new >> kPageShift)];
        writer = raw >= 0 && raw < a.n_pages;
      }
    }
    for (int job = wave; job < G + (mine ? 2 : 0); job += kThreads / 64) {
      if (job < G) {
        norm_rope_row<T, D>(a, a.pq + b * a.pq_stride + static_cast<int64_t>(h0 + job) * D, a.qw, b, B, lane, s_q[job],
                            static_cast<T *>(nullptr));
      } else {
        // the cache row of the new token: through the page numbers of this range when the cache is paged
        // (p_new lies in [s0, s1), so its page is among them)
        T *crow = const_cast<T *>(static_cast<const T *>(job == G ? a.k : a.v));
        if constexpr (PAGED)
          crow += s_pages[(p_new >> kPageShift) - first_page] * a.page_stride + static_cast<int64_t>(hk) * (kPageKeys * D) +
                  (p_new & (kPageKeys - 1)) * D;
        else
          crow += b * a.stride_b + hk * a.stride_h + static_cast<int64_t>(p_new) * a.stride_s;
        if (job == G) {
          norm_rope_row<T, D>(a, a.pk + b * a.pk_stride + static_cast<int64_t>(hk) * D, a.kw, b, B, lane, s_kv[0],
                              writer ? crow : static_cast<T *>(nullptr));
        } else {
          const float *src = a.pv + b * a.pv_stride + static_cast<int64_t>(hk) * D;
          for (int i = lane; i < D; i += 64) {
            stf(&s_kv[1][i], src[i]);
            if (writer) stf(crow + i, src[i]);
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < G; ++g) qf[g].template load<SEC>(&s_q[g][lane_el]);
  } else {
    const T *q = static_cast<const T *>(a.q);
#pragma unroll
    for (int g = 0; g < G; ++g)
      qf[g].template load<SEC>(q + (static_cast<int64_t>(b) * a.Hq + h0 + g) * D + lane_el);
  }

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegBig;
    l[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[g][i] = 0.0f;
  }

  int base = s0;
  if constexpr (QKV && HOIST) {
    tile_update<T, D, G, U, true>(kr0, vr0, base, rg, kv_end, a.scale_log2e, qf, m, l, acc);
    base += U * RG;
  }
  for (; base + U * RG <= kv_end; base += U * RG)
    decode_tile<T, D, G, U, false>(kb, vb, rows, base, rg, kv_end, a.scale_log2e, qf, m, l, acc);
  for (; base < kv_end; base += U * RG)
    decode_tile<T, D, G, U, true>(kb, vb, rows, base, rg, kv_end, a.scale_log2e, qf, m, l, acc);
  if constexpr (QKV) {
    if (mine) {  // the new token's key and value: one more row, taken by row group 0
      Frag8<T> kn, vn;
      kn.template load<SEC>(&s_kv[0][lane_el]);
      vn.template load<SEC>(&s_kv[1][lane_el]);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float d = group_sum<LPR>(qf[g].dot(kn)) * a.scale_log2e;
        if (rg == 0) {
          const float mn = fmaxf(m[g], d);
          const float corr = __builtin_amdgcn_exp2f(m[g] - mn);
          const float p = __builtin_amdgcn_exp2f(d - mn);
          m[g] = mn;
          l[g] = l[g] * corr + p;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[g][i] *= corr;
          vn.axpy(p, acc[g]);
        }
      }
    }
  }

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
    store_lane_acc<T, D>(s_acc[g][rg], dl, acc[g]);
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
    if (n_valid == 1 && direct_ok) {
      // the only range of this sequence: normalise and write the result, nothing to merge
      stf(static_cast<T *>(a.out) + bh * D + d, lsum > 0.0f ? asum / lsum : 0.0f);
    } else {
      st_agent(&a.part_acc[(bh * a.split_stride + split) * D + d], asum);
      if (d == 0) {
        st_agent(&a.part_ml[(bh * a.split_stride + split) * 2], mx);
        st_agent(&a.part_ml[(bh * a.split_stride + split) * 2 + 1], lsum);
      }
    }
  }
  if (n_valid == 1 || !a.fused_merge) return;

  // ---- in-kernel merge: the workgroup that takes the last ticket combines all splits ------------
  __shared__ int s_last;
  // A workgroup barrier orders the wavefronts but does not wait for their outstanding stores: every
  // thread drains its own write-through partial stores first, so that all of them have reached memory
  // when thread 0 takes the ticket behind the barrier.
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0) {
    unsigned int *ticket = ticket_of(a.ticket_base, b * a.n_hg + hg);
    const unsigned int t = atomicAdd(ticket, 1u);
    s_last = (t == static_cast<unsigned int>(n_valid - 1));
    if (s_last) atomicExch(ticket, 0u);  // ready for the next launch
  }
  __syncthreads();
  if (!s_last) return;
  for (int o = tid; o < G * D; o += kThreads) {
    const int g = o / D, d = o % D;
    const int64_t bh = static_cast<int64_t>(b) * a.Hq + h0 + g;
    const float *ml = a.part_ml + bh * a.split_stride * 2;
    const float *pa = a.part_acc + bh * a.split_stride * D + d;
    const float res = n_valid <= 8 ? merge_ranges<8>(ml, pa, n_valid, D) : merge_ranges<32>(ml, pa, n_valid, D);
    stf(static_cast<T *>(a.out) + bh * D + d, res);
  }
}

// The end of a range on the matrix-core path (the same steps as the tail of process_range, with the
// head count at run time): the workgroup's NS partial states (running
// maximum s_m[head][NS], sum s_l[head][NS], unnormalised output s_acc[head][NS][D], in LDS, complete
// and visible) are combined; the only range of a sequence writes the result when `direct_ok`, otherwise
// the range leaves its state in the workspace and (fused merge) the workgroup that takes the last
// ticket of the (sequence, head group) combines all ranges.
// The states are named through LDS pointers: as generic pointers they cost 64-bit addresses and flat loads.
typedef const float __attribute__((address_space(3))) *lds_cfloat_ptr;
typedef int __attribute__((address_space(3))) *lds_int_ptr;
template <typename T, int D, int NS>
__device__ __forceinline__ void finish_range(const DecodeArgs &a, int b, int hg, int h0, int heads, int split,
                                             int n_valid, bool direct_ok, lds_cfloat_ptr s_m, lds_cfloat_ptr s_l,
                                             lds_cfloat_ptr s_acc, lds_int_ptr s_last) {
  const int tid = threadIdx.x;
  for (int o = tid; o < heads * D; o += kThreads) {
    const int g = o / D, d = o % D;
    float mx = kNegBig;
#pragma unroll
    for (int r = 0; r < NS; ++r) mx = fmaxf(mx, s_m[g * NS + r]);
    float lsum = 0.0f, asum = 0.0f;
#pragma unroll
    for (int r = 0; r < NS; ++r) {
      const float w = __builtin_amdgcn_exp2f(s_m[g * NS + r] - mx);
      lsum = __builtin_fmaf(s_l[g * NS + r], w, lsum);
      asum = __builtin_fmaf(s_acc[(g * NS + r) * D + d], w, asum);
    }
    const int64_t bh = static_cast<int64_t>(b) * a.Hq + h0 + g;
    if (n_valid == 1 && direct_ok) {
      // the only range of this sequence: normalise and write the result, nothing to merge
      stf(static_cast<T *>(a.out) + bh * D + d, lsum > 0.0f ? asum / lsum : 0.0f);
    } else {
      st_agent(&a.part_acc[(bh * a.split_stride + split) * D + d], asum);
      if (d == 0) {
        st_agent(&a.part_ml[(bh * a.split_stride + split) * 2], mx);
        st_agent(&a.part_ml[(bh * a.split_stride + split) * 2 + 1], lsum);
      }
    }
  }
  if (n_valid == 1 || !a.fused_merge) return;

  // ---- in-kernel merge: the workgroup that takes the last ticket combines all splits ------------
  // every thread drains its own write-through partial stores before the barrier (the barrier alone
  // does not wait for outstanding stores), so all partials are in memory when the ticket is taken
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (tid == 0) {
    unsigned int *ticket = ticket_of(a.ticket_base, b * a.n_hg + hg);
    const unsigned int t = atomicAdd(ticket, 1u);
    *s_last = (t == static_cast<unsigned int>(n_valid - 1));
    if (*s_last) atomicExch(ticket, 0u);  // ready for the next launch
  }
  __syncthreads();
  if (!*s_last) return;
  for (int o = tid; o < heads * D; o += kThreads) {
    const int g = o / D, d = o % D;
    const int64_t bh = static_cast<int64_t>(b) * a.Hq + h0 + g;
    const float *ml = a.part_ml + bh * a.split_stride * 2;
    const float *pa = a.part_acc + bh * a.split_stride * D + d;
    const float res = n_valid <= 8 ? merge_ranges<8>(ml, pa, n_valid, D) : merge_ranges<32>(ml, pa, n_valid, D);
    stf(static_cast<T *>(a.out) + bh * D + d, res);
  }
}

// ---- large head groups: the matrix-core path ---------------------------------------------------------
// With four or more query heads per kv head the per-key arithmetic of the loop above (one dot product
// and one axpy of D elements per head and key on the vector ALUs) takes longer than the key's bytes take
// to arrive (Hq=32, Hkv=8: 65 % of HBM peak; Hq=64: 38 %).  Here the heads of a kv head - up to 16 - are
// the columns of one MFMA tile instead, exactly as the positions are in the prefill kernel:
//   S^T = K . Q^T (16 keys x 16 heads per tile), O^T += V^T . P^T,
// so a key costs the same whatever the group size, and K and V are read once per kv head.  One workgroup
// per (sequence, kv head, key range); a stage of 128 keys of K and V travels through LDS (coalesced
// streaming loads into registers one stage ahead, XOR-swizzled rows, V^T fragments by the transposing
// LDS read), each of the 4 wavefronts takes 32 of the 128 keys and keeps its own online-softmax state for
// the 16 columns; the four states are merged at the end like the row groups of the vector path.
constexpr int kMfmaStage = 128;  // keys per LDS stage (32 per wavefront)
constexpr int kMfmaHeads = 16;   // columns of the MFMA tile: heads per workgroup at most

// Decode-step form (QKV): the query heads are prepared (RMSNorm, M-RoPE) into LDS by the wavefronts
// before the first stage is stored there; the workgroup whose range ends with the token being decoded
// prepares its key and value as well, keeps them in two rows of LDS behind the stage, attends to them in
// one more step after the cached keys, and writes the cache row.
extern __shared__ __attribute__((aligned(16))) unsigned char mfma_smem[];

template <int D, bool PAGED = false>
constexpr int mfma_lds_bytes() {
  // one stage of K and of V (the per-wavefront states reuse it), two rows for a new token, the merge flag,
  // and for a paged cache the page numbers of the workgroup's key range
  return 2 * kMfmaStage * D * 2 + 2 * D * 2 + 16 + (PAGED ? (kMaxRangePages * 4 + 15) / 16 * 16 : 0);
}

template <int D, bool QKV, bool PAGED = false>
__device__ __forceinline__ void process_range_mfma(const DecodeArgs &a, int b, int hg, int split, int n_valid,
                                                   bool direct_ok, int s0, int s1, int p_raw = kNoLength) {
  constexpr int KK = D / 32;   // MFMA steps over d for S^T
  constexpr int DT = D / 16;   // d tiles of O^T
  constexpr int UPR = D / 8;   // 16-byte units per K/V row
  constexpr int VEC = kMfmaStage * UPR / kThreads;  // staging vectors per thread and tensor
  constexpr int kStageHalves = kMfmaStage * D;
  static_assert(kMfmaHeads * 4 * (D + 2) * 4 <= 2 * kStageHalves * 2, "the merge states fit the stage memory");
  unsigned char *smem = mfma_smem;
  _Float16 *ks = reinterpret_cast<_Float16 *>(smem), *vs = ks + kStageHalves;
  _Float16 *s_new = vs + kStageHalves;  // [2][D]: key and value of the token being decoded

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c = lane & 15, g = lane >> 4;
  const int heads = a.wg_heads;     // query heads of this workgroup: columns 0 .. heads-1
  const int h0 = hg * heads;
  const int hk = h0 / a.group;

  bool mine = false;
  int kv_end = s1;  // keys [s0, kv_end) come from the cache
  int p_new = 0;
  if constexpr (QKV) {
    p_new = p_raw != kNoLength ? p_raw : a.seq_lens[b];
    p_new = p_new < 0 ? 0 : p_new;
    mine = p_new < a.max_len && p_new < a.cache_rows && p_new >= s0 && p_new < s1;  // then p_new == s1 - 1
    if (mine) kv_end = p_new;
  }
  // paged: the pool is [page, kv head, key in page, D]; the page numbers of keys [s0, s1) come from the page
  // table into LDS first (clamped into the pool: a corrupt table gives wrong values, never an access outside it)
  const int64_t kv_off = PAGED ? static_cast<int64_t>(hk) * (kPageKeys * D) : b * a.stride_b + hk * a.stride_h;
  const __half *kbase = static_cast<const __half *>(a.k) + kv_off;
  const __half *vbase = static_cast<const __half *>(a.v) + kv_off;
  int *s_pages = reinterpret_cast<int *>(smem + 2 * kStageHalves * 2 + 2 * D * 2 + 16);
  const int first_page = s0 >> kPageShift;
  if constexpr (PAGED) {
    const int range_pages = ((s1 - 1) >> kPageShift) - first_page + 1;
    const int32_t *tbl = a.page_table + static_cast<int64_t>(b) * a.max_pages + first_page;
    for (int i = tid; i < range_pages; i += kThreads) s_pages[i] = min(max(tbl[i], 0), a.n_pages - 1);
    __syncthreads();
  }
  auto row_offset = [&](int key) -> int64_t {
    if constexpr (PAGED)
      return s_pages[(key >> kPageShift) - first_page] * a.page_stride + static_cast<int64_t>(key & (kPageKeys - 1)) * D;
    else
      return static_cast<int64_t>(key) * a.stride_s;
  };
  // one stage waits in registers while the previous one is used from LDS.  (Two stages in registers
  // measured no faster: at 255 registers the compiler parks loaded data in accumulator registers, which
  // makes it wait for the loads early.  Per stage the kernel takes about 0.35 us more than its bytes do.)
  half8_t kst[1][VEC], vst[1][VEC];
  auto load_stage = [&](int key0, half8_t (&kr)[VEC], half8_t (&vr)[VEC]) {
#pragma unroll
    for (int p = 0; p < VEC; ++p) {
      const int vi = p * kThreads + tid;
      const int row = vi / UPR, unit = vi % UPR;
      const int64_t off = row_offset(min(key0 + row, kv_end - 1)) + unit * 8;  // rows past the range: its last key again
      kr[p] = __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(kbase + off));
      vr[p] = __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(vbase + off));
    }
  };
  // V rows past the range are stored as zeros: their probabilities are zero, and 0 * finite stays 0
  auto store_stage = [&](int key0, const half8_t (&kr)[VEC], const half8_t (&vr)[VEC]) {
#pragma unroll
    for (int p = 0; p < VEC; ++p) {
      const int vi = p * kThreads + tid;
      const int row = vi / UPR, unit = vi % UPR;
      const int o = row * D + ((unit ^ (row & (UPR - 1))) << 3);
      *reinterpret_cast<half8_t *>(&ks[o]) = kr[p];
      half8_t vv = vr[p];
      if (key0 + row >= kv_end) vv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      *reinterpret_cast<half8_t *>(&vs[o]) = vv;
    }
  };

  float4_t o[DT];
  float m = kNegBig, lsum = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = float4_t{0.f, 0.f, 0.f, 0.f};

  const int n_stages = (kv_end - s0 + kMfmaStage - 1) / kMfmaStage;
  // the first stage is requested before the queries are prepared: those loads do not need them
  if (n_stages > 0) load_stage(s0, kst[0], vst[0]);

  // Q as the B operand: column c is head h0 + c (columns past the last head are zero and never stored)
  half8_t qf[KK];
  if constexpr (QKV) {
    _Float16 *s_q = ks;  // [heads][D], gone once the first stage is stored
    bool writer = mine && (h0 % a.group == 0);
    if constexpr (PAGED) {
      // reads are clamped into the pool, the store of the new row is not redirected: skipped when the
      // table entry of its page lies outside the pool
      if (writer) {
        const int raw = a.page_table[static_cast<int64_t>(b) * a.max_pages + (p_new >> kPageShift)];
        writer = raw >= 0 && raw < a.n_pages;
      }
    }
    for (int job = wave; job < heads + (mine ? 2 : 0); job += kThreads / 64) {
      if (job < heads) {
        norm_rope_row<__half, D>(a, a.pq + b * a.pq_stride + static_cast<int64_t>(h0 + job) * D, a.qw, b, a.B, lane,
                                 reinterpret_cast<__half *>(s_q + job * D), static_cast<__half *>(nullptr));
      } else {
        __half *crow = const_cast<__half *>(static_cast<const __half *>(job == heads ? a.k : a.v)) + kv_off + row_offset(p_new);
        if (job == heads) {
          norm_rope_row<__half, D>(a, a.pk + b * a.pk_stride + static_cast<int64_t>(hk) * D, a.kw, b, a.B, lane,
                                   reinterpret_cast<__half *>(s_new), writer ? crow : static_cast<__half *>(nullptr));
        } else {
          const float *src = a.pv + b * a.pv_stride + static_cast<int64_t>(hk) * D;
          for (int i = lane; i < D; i += 64) {
            stf(reinterpret_cast<__half *>(s_new + D) + i, src[i]);
            if (writer) stf(crow + i, src[i]);
          }
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      qf[kk] = lds_h8(s_q + min(c, heads - 1) * D + kk * 32 + g * 8);
      if (c >= heads) qf[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
    __syncthreads();  // everyone has its fragments before the first stage overwrites the rows
  } else {
    const __half *qrow = static_cast<const __half *>(a.q) + (static_cast<int64_t>(b) * a.Hq + h0 + min(c, heads - 1)) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      qf[kk] = *reinterpret_cast<const half8_t *>(qrow + kk * 32 + g * 8);
      if (c >= heads) qf[kk] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  // one wavefront's 32 keys kb .. kb + 31 (those below `limit` count), rows k_l / v_l of the stage in LDS
  auto attend = [&](int kb, int limit, const _Float16 *k_l, const _Float16 *v_l) __attribute__((always_inline)) {
    float4_t sc[2] = {float4_t{0.f, 0.f, 0.f, 0.f}, float4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int tk = 0; tk < 2; ++tk)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const int row = tk * 16 + c, unit = kk * 4 + g;
        const half8_t kf = lds_h8(k_l + row * D + ((unit ^ (row & (UPR - 1))) << 3));
        sc[tk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[kk], sc[tk], 0, 0, 0);
      }
    // this lane: head c, keys kb + 16 tk + 4 g + e
    const bool tail = kb + 32 > limit;
    float x[8];
#pragma unroll
    for (int tk = 0; tk < 2; ++tk)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = sc[tk][e] * a.scale_log2e;
        if (tail && kb + tk * 16 + 4 * g + e >= limit) v = kNegBig;
        x[tk * 4 + e] = v;
      }
    float mx = x[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) mx = fmaxf(mx, x[j]);
    mx = max_xor32(max_xor16(mx));
    const float mn = fmaxf(m, mx);
    half8_t pf;
    float ps = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float pr = __builtin_amdgcn_exp2f(x[j] - mn);
      if (tail && x[j] <= kNegBig) pr = 0.f;
      ps += pr;
      pf[j] = static_cast<_Float16>(pr);
    }
    if (__any(mn != m)) {
      const float corr = __builtin_amdgcn_exp2f(m - mn);
      lsum *= corr;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= corr;
    }
    m = mn;
    lsum += ps;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const half4_t lo = lds_v_tr<D>(v_l, 4 * g, dt * 16, c);
      const half4_t hi = lds_v_tr<D>(v_l, 16 + 4 * g, dt * 16, c);
      const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[dt], 0, 0, 0);
    }
  };
  for (int st = 0; st < n_stages; ++st) {
    const int key0 = s0 + st * kMfmaStage;
    store_stage(key0, kst[0], vst[0]);
    __syncthreads();
    // the next stage into the registers just emptied; the last stage fetches itself again: no branch
    load_stage(s0 + min(st + 1, n_stages - 1) * kMfmaStage, kst[0], vst[0]);
    __builtin_amdgcn_sched_barrier(0);
    const int kb = key0 + wave * 32;  // first of this wavefront's 32 keys
    if (kb < kv_end) attend(kb, kv_end, ks + wave * 32 * D, vs + wave * 32 * D);
    __syncthreads();  // every wavefront is done with the stage before the next one overwrites it
  }
  if constexpr (QKV) {
    if (mine) {
      // the token being decoded: its key and value become row 0 of a stage of their own (row 0 is not
      // swizzled; the other rows hold finite leftovers that the mask keeps out)
      if (n_stages == 0) {
        for (int i = tid; i < 2 * kStageHalves / 8; i += kThreads)
          *reinterpret_cast<half8_t *>(ks + i * 8) = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        __syncthreads();
      }
      if (tid < UPR) *reinterpret_cast<half8_t *>(ks + tid * 8) = *reinterpret_cast<const half8_t *>(s_new + tid * 8);
      else if (tid < 2 * UPR)
        *reinterpret_cast<half8_t *>(vs + (tid - UPR) * 8) = *reinterpret_cast<const half8_t *>(s_new + D + (tid - UPR) * 8);
      __syncthreads();
      if (wave == 0) attend(p_new, p_new + 1, ks, vs);
      __syncthreads();
    }
  }

  // the four per-wavefront states, [head][wavefront]: maximum, sum, output
  float *s_m = reinterpret_cast<float *>(smem), *s_l = s_m + kMfmaHeads * 4, *s_acc = s_l + kMfmaHeads * 4;
  int *s_flag = reinterpret_cast<int *>(smem + 2 * kStageHalves * 2 + 2 * D * 2);
  lsum = sum_xor32(sum_xor16(lsum));
  if (g == 0) {
    s_m[c * 4 + wave] = m;
    s_l[c * 4 + wave] = lsum;
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    *reinterpret_cast<float4_t *>(&s_acc[(c * 4 + wave) * D + dt * 16 + 4 * g]) = o[dt];
  __syncthreads();
  finish_range<__half, D, 4>(a, b, hg, h0, heads, split, n_valid, direct_ok, (lds_cfloat_ptr)s_m, (lds_cfloat_ptr)s_l,
                             (lds_cfloat_ptr)s_acc, (lds_int_ptr)s_flag);
}

// Which keys a workgroup streams.
//   Static plan: (range, head group, sequence) straight from the grid.
//   Length-dealt plan: workgroup id = slot * n_hg + head group, and the `active` slots of a head group
//   share the keys of the whole batch.  Every wavefront builds the table in its registers - lane i
//   holds sequence i (B <= 64): one vector load for the lengths, wave sums, a prefix sum, a ballot.
//   (1) Whole slots per sequence: with c keys per slot, sequence b takes max(1, ceil(len_b / c))
//       consecutive slots and is cut into that many equal ranges; c starts at
//       ceil(sum of lengths / active) and grows until the slots suffice (a few rounds: the count falls
//       as c grows, and c = max_len needs B <= active slots).  Slots left over exit at once.  A batch
//       of (nearly) equal lengths is cut exactly evenly this way, with one range per workgroup.
//   (2) When whole slots leave the longest range more than an eighth (and 256 keys) above the
//       average - a ragged batch, or fewer slots than it takes to follow the lengths - the sequences
//       are laid end to end instead and slot j takes keys [j*c, (j+1)*c) of that line, whichever
//       sequences they belong to: a workgroup then works through a piece of each sequence its range
//       touches, and every slot streams the same number of keys.  A sequence without keys gets its
//       zeros from the slot that holds its place on the line.
template <typename T, int D, int G, int U, bool QKV, bool MFMA = false, bool PAGED = false>
// (the decode-step form needs 161 registers: at four workgroups per CU, 128 registers, it spills 37 of them)
__global__ __launch_bounds__(kThreads, MFMA ? 1 : (QKV ? 3 : 4)) void gqa_decode_split_kernel(DecodeArgs a) {
  // the piece to work on: keys [s0, s1) of sequence b, range `split` of its n_valid ranges
  int b, hg, split, n_valid, s0, s1, p_raw = kNoLength;
  bool direct_ok = true;
  if (!a.dynamic) {
    split = blockIdx.x, hg = blockIdx.y, b = blockIdx.z;
    const int len_b = clamped_len(a.seq_lens, b, a.max_len, a.len_add);
    const int chunk = balanced_chunk(len_b, a.n_splits);
    n_valid = (len_b + chunk - 1) / chunk;  // ranges of this sequence that hold keys
    direct_ok = a.n_splits == 1 || a.fused_merge;
    s0 = split * chunk;
    s1 = min(s0 + chunk, len_b);
    if (s0 >= len_b) {
      // an empty range is never read by the merge; without a merge kernel the zeros of a sequence
      // without keys come from its first workgroup
      if (len_b == 0 && split == 0 && direct_ok) write_zero_rows<T, D, G, MFMA>(a, b, hg);
      return;
    }
  } else {
    const int lane = threadIdx.x & 63;
    const int j = static_cast<int>(blockIdx.x) / a.n_hg;
    hg = static_cast<int>(blockIdx.x) % a.n_hg;
    // What an earlier launch of the same step found for slot j, if the caller keeps a plan cache: kind (0 nothing
    // to do, 1 one range, 2 "deal again": ranges laid end to end, or rows of zeros to write), sequence, range,
    // ranges of the sequence, first key, end, the sequence's length before the append, the mark of the launch.
    // (not for four heads per workgroup on the vector units: the second way in costs that form registers it does
    // not have to spare at three workgroups per CU)
    constexpr bool kPlanTable = QKV && (MFMA || G <= 2);
    bool planned = false;
    if constexpr (kPlanTable) {
      if (a.plan_mode == 2) {
        // the same words in every lane; a launch that records stores to the table, so the loads are vector loads
        // whatever the address: say that the values are uniform, so that what follows lives in scalar registers
        const int4 *e = reinterpret_cast<const int4 *>(a.plan_cache + 8 * j);
        const int4 lo = e[0], hi = e[1];
        const int kind = uni(lo.x), mark = uni(hi.w);
        if (mark == a.plan_check && kind == 0) return;
        if (mark == a.plan_check && kind == 1) {
          b = uni(lo.y), split = uni(lo.z), n_valid = uni(lo.w), s0 = uni(hi.x), s1 = uni(hi.y), p_raw = uni(hi.z);
          planned = true;
        }
      }
    }
    if (!planned) {
    auto record = [&](int kind, int rb, int rsplit, int rn, int rs0, int rs1) {
      if constexpr (kPlanTable) {
        if (a.plan_mode == 1 && hg == 0 && threadIdx.x == 0) {
          int *e = a.plan_cache + 8 * j;
          e[0] = kind, e[1] = rb, e[2] = rsplit, e[3] = rn, e[4] = rs0, e[5] = rs1;
          e[6] = kind == 1 ? a.seq_lens[rb] : 0;
          e[7] = a.plan_check;
        }
      }
    };
    const bool live = lane < a.B;
    const int len = live ? clamped_len(a.seq_lens, lane, a.max_len, a.len_add) : 0;
    // sum of lengths in units of 64 keys (rounded up per sequence): fits an int for any supported size
    const int total64 = wave_sum_i((len + 63) >> 6);
    const long long c_even = (static_cast<long long>(total64) * 64 + a.active - 1) / a.active;
    int c = static_cast<int>(c_even < kMinDevChunk ? kMinDevChunk : (c_even > a.max_len ? a.max_len : c_even));
    int n = 0;
#pragma unroll 1
    for (int round = 0; round < 8; ++round) {
      n = live ? dyn_splits_of(len, c, a.split_stride) : 0;
      const int used = wave_sum_i(n);
      if (used <= a.active) break;
      // too many slots: grow c by the overshoot (at least one key), the last round takes one range each
      const long long grown = (static_cast<long long>(c) * used + a.active - 1) / a.active;
      c = round == 6 ? a.max_len : static_cast<int>(grown > a.max_len ? a.max_len : (grown > c ? grown : c + 1));
    }
    const int longest = wave_max_i(live && len > 0 ? balanced_chunk(len, n) : 0);
    const long long slack = c_even / 8 > 256 ? c_even / 8 : 256;
    // a slot can leave at most one piece per sequence, so `active` partial slots per sequence suffice
    const bool end_to_end = a.active <= a.split_stride && total64 < (1 << 24) && longest - c_even > slack;
    if (end_to_end) {
      record(2, 0, 0, 0, 0, 0);
      const int start = wave_prefix_i(len, lane) - len;  // where this lane's sequence begins on the line
      const int total = __builtin_amdgcn_readlane(start + len, 63);
      int cc = (total + a.active - 1) / a.active;
      cc = cc < kMinDevChunk ? kMinDevChunk : cc;
      cc = (cc + 15) & ~15;
      const int g0 = j * cc, g1 = min(g0 + cc, total);
      unsigned long long todo = __ballot(live && len > 0 && start < g1 && start + len > g0);
      // the place of an empty sequence belongs to the slot of the key before it (slot 0 at the start)
      unsigned long long empty = __ballot(live && len == 0 && (start > 0 ? (start - 1) / cc : 0) == j);
      for (bool again = false; todo; again = true) {
        b = uni(__ffsll(todo) - 1);
        todo &= todo - 1;
        // start and length of sequence b, from memory again: held in vector registers across the
        // piece they would push the streaming loop over its register budget
        const int lane2 = threadIdx.x & 63;
        const int before = lane2 < b ? clamped_len(a.seq_lens, lane2, a.max_len, a.len_add) : 0;
        const int start_b = uni(wave_sum_i(before));
        const int len_b = clamped_len(a.seq_lens, b, a.max_len, a.len_add);
        const int first_slot = start_b / cc, last_slot = (start_b + len_b - 1) / cc;
        if (again) __syncthreads();  // the previous piece is done with the LDS arrays
        if constexpr (MFMA)
          process_range_mfma<D, QKV, PAGED>(a, b, hg, j - first_slot, last_slot - first_slot + 1, true,
                                            max(g0 - start_b, 0), min(g1 - start_b, len_b));
        else
          process_range<T, D, G, U, QKV, false, PAGED>(a, b, hg, j - first_slot, last_slot - first_slot + 1, true,
                                                       max(g0 - start_b, 0), min(g1 - start_b, len_b));
      }
      while (empty) {
        const int e = uni(__ffsll(empty) - 1);
        empty &= empty - 1;
        write_zero_rows<T, D, G, MFMA>(a, e, hg);
      }
      return;
    }
    const int first = wave_prefix_i(n, lane) - n;
    const unsigned long long hit = __ballot(j >= first && j < first + n);
    if (hit == 0ull) {  // a slot the lengths of this launch leave unused
      record(0, 0, 0, 0, 0, 0);
      return;
    }
    // the same in every lane: say so, so that everything derived from it lives in scalar registers
    b = uni(__ffsll(hit) - 1);
    split = j - __builtin_amdgcn_readlane(first, b);
    const int n_b = __builtin_amdgcn_readlane(n, b);
    const int len_b = __builtin_amdgcn_readlane(len, b);
    const int chunk = balanced_chunk(len_b, n_b);
    n_valid = (len_b + chunk - 1) / chunk;
    s0 = split * chunk;
    s1 = min(s0 + chunk, len_b);
    if (s0 >= len_b) {
      record(len_b == 0 && split == 0 ? 2 : 0, 0, 0, 0, 0, 0);
      if (len_b == 0 && split == 0) write_zero_rows<T, D, G, MFMA>(a, b, hg);
      return;
    }
    record(1, b, split, n_valid, s0, s1);
    }
    b = uni(b), split = uni(split), n_valid = uni(n_valid), s0 = uni(s0), s1 = uni(s1), p_raw = uni(p_raw);
  }
  if constexpr (MFMA)
    process_range_mfma<D, QKV, PAGED>(a, b, hg, split, n_valid, direct_ok, s0, s1, p_raw);
  else
    process_range<T, D, G, U, QKV, true, PAGED>(a, b, hg, split, n_valid, direct_ok, s0, s1, p_raw);
}

// Cross-split merge: one workgroup of D threads per (sequence, query head).
template <typename T, int D>
__global__ __launch_bounds__(D) void gqa_decode_merge_kernel(DecodeArgs a) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const int len = clamped_len(a.seq_lens, b, a.max_len, a.len_add);
  const int chunk = balanced_chunk(len, a.n_splits);
  const int n_valid = (len + chunk - 1) / chunk;  // splits that wrote a partial
  const int64_t bh = static_cast<int64_t>(b) * a.Hq + h;
  T *out = static_cast<T *>(a.out) + bh * D + d;
  if (n_valid == 0) {
    stf(out, 0.0f);
    return;
  }
  const float *ml = a.part_ml + bh * a.split_stride * 2;
  const float *pa = a.part_acc + bh * a.split_stride * D + d;
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
  // static plan: (split, head group, sequence); length-dealt plan: one dimension, slot index slowest
  const dim3 grid(a.dynamic ? a.active * (a.Hq / G) : a.n_splits, a.dynamic ? 1 : a.Hq / G, a.dynamic ? 1 : B);
  if (a.page_table && a.len_add) {
    if constexpr (sizeof(T) == 2)  // the decode-step form over a paged cache: fp16 caches
      hipLaunchKernelGGL((gqa_decode_split_kernel<T, D, G, U, true, false, true>), grid, dim3(kThreads), 0, st, a);
    else
      return AXHIP_UNSUPPORTED_TYPE;
  } else if (a.page_table)
    hipLaunchKernelGGL((gqa_decode_split_kernel<T, D, G, U, false, false, true>), grid, dim3(kThreads), 0, st, a);
  else if (a.len_add)
    hipLaunchKernelGGL((gqa_decode_split_kernel<T, D, G, U, true>), grid, dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((gqa_decode_split_kernel<T, D, G, U, false>), grid, dim3(kThreads), 0, st, a);
  if (a.n_splits > 1 && !a.fused_merge)
    hipLaunchKernelGGL((gqa_decode_merge_kernel<T, D>), dim3(a.Hq, B), dim3(D), 0, st, a);
  return launch_status();
}

template <int D, bool QKV, bool PAGED>
int launch_decode_mfma_form(const DecodeArgs &a, int B, hipStream_t st) {
  const int n_hg = a.n_hg;
  const dim3 grid(a.dynamic ? a.active * n_hg : a.n_splits, a.dynamic ? 1 : n_hg, a.dynamic ? 1 : B);
  auto kernel = gqa_decode_split_kernel<__half, D, 1, 8, QKV, true, PAGED>;
  constexpr int lds = mfma_lds_bytes<D, PAGED>();
  if (lds > 64 * 1024) {  // more dynamic LDS than the default limit
    static std::atomic<uint64_t> lds_set{0};
    const int rc = raise_dynamic_lds(reinterpret_cast<const void *>(kernel), lds, lds_set);
    if (rc != AXHIP_OK) return rc;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), lds, st, a);
  if (a.n_splits > 1 && !a.fused_merge)
    hipLaunchKernelGGL((gqa_decode_merge_kernel<__half, D>), dim3(a.Hq, B), dim3(D), 0, st, a);
  return launch_status();
}

template <int D>
int launch_decode_mfma(const DecodeArgs &a, int B, hipStream_t st) {
  if (a.page_table)
    return a.len_add ? launch_decode_mfma_form<D, true, true>(a, B, st) : launch_decode_mfma_form<D, false, true>(a, B, st);
  return a.len_add ? launch_decode_mfma_form<D, true, false>(a, B, st) : launch_decode_mfma_form<D, false, false>(a, B, st);
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
// Matrix-core path: all heads of a kv head in one workgroup when there are at most 16 (the columns of a
// tile), otherwise the largest divisor of the group size that fits.
int mfma_heads_per_workgroup(int group) {
  int h = group < kMfmaHeads ? group : kMfmaHeads;
  while (group % h != 0) --h;
  return h;
}

}  // namespace
}  // namespace axhip

using namespace axhip;

namespace {
// Split plan, workspace carve-up and launch shared by the entry points.
// The device address of `scratch` on the current device, looked up once per device (with that device
// current) and kept: each device holds its own copy of the array at its own address.
int static_scratch_on_this_device(void **out) {
  static std::atomic<void *> addr[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return AXHIP_DEVICE_ERROR;
  void *p = addr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return AXHIP_DEVICE_ERROR;
    }
    addr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return AXHIP_OK;
}

// `static_ws`: the partials go to this device's static scratch instead of a caller's workspace; a plan that
// needs more than the array holds is refused with AXHIP_OUT_OF_MEMORY.
int plan_and_launch(DecodeArgs &a, void *workspace, size_t workspace_bytes, int dtype, int B, int Hq, int Hkv,
                    int D, int max_len, axhip_stream stream, bool static_ws = false) {
  const int group = Hq / Hkv;
  // four or more heads per kv head, fp16: the heads of a kv head become the columns of an MFMA tile
  const bool mfma = g_tuning.mfma_groups && dtype == AXHIP_FLOAT16 && group >= 4 && (D == 64 || D == 128) &&
                    a.stride_s % 8 == 0 && a.stride_h % 8 == 0 && a.stride_b % 8 == 0;
  const int G = mfma ? mfma_heads_per_workgroup(group) : heads_per_workgroup(group);
  a.wg_heads = G;
  a.ticket_base = axhip_ticket_lane() * kTicketSlots;
  const SplitPlan plan = plan_splits(B, Hq / G, max_len);
  a.Hq = Hq;
  a.group = group;
  a.max_len = max_len;
  a.chunk = plan.chunk;
  a.n_splits = plan.n_splits;
  a.dynamic = plan.dynamic;
  a.active = plan.active;
  a.split_stride = plan.stride;
  a.B = B;
  a.n_hg = Hq / G;
  a.scale_log2e = 1.4426950408889634f / sqrtf(static_cast<float>(D));
  a.part_acc = nullptr;
  a.part_ml = nullptr;
  a.plan_mode = 0;
  if (plan.dynamic && axhip_plan_reuse() != 0 && plan.active <= kPlanSlots && (mfma || G <= 2)) {
    static std::atomic<int *> cache[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return AXHIP_DEVICE_ERROR;
    int *p = cache[dev].load(std::memory_order_acquire);
    if (!p) {
      if (hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(g_plan_cache)) != hipSuccess || !p) {
        (void)hipGetLastError();
        return AXHIP_DEVICE_ERROR;
      }
      cache[dev].store(p, std::memory_order_release);
    }
    a.plan_cache = p + static_cast<size_t>(axhip_ticket_lane()) * kPlanSlots * 8;
    a.plan_mode = axhip_plan_reuse();
    // entries left by a launch of another shape, or dealt from another lengths array, are not taken
    unsigned h = 2166136261u;
    for (const long long v : {static_cast<long long>(B), static_cast<long long>(Hq), static_cast<long long>(G),
                              static_cast<long long>(max_len), static_cast<long long>(plan.active),
                              static_cast<long long>(plan.stride), static_cast<long long>(a.len_add),
                              static_cast<long long>(a.cache_rows),
                              static_cast<long long>(reinterpret_cast<uintptr_t>(a.seq_lens))})
      for (int i = 0; i < 8; ++i) h = (h ^ static_cast<unsigned>((v >> (8 * i)) & 255)) * 16777619u;
    a.plan_check = static_cast<int>(h | 1u);  // (never 0, which a cache nobody has written holds)
  }
  // the length-dealt plan always merges in the kernel (a second kernel could not be skipped when no
  // sequence needs it); the static plan does unless the two-kernel form was asked for
  a.fused_merge = ((plan.dynamic || !g_tuning.separate_merge) && static_cast<long>(B) * (Hq / G) <= kTicketSlots) ? 1 : 0;
  if (plan.dynamic && !a.fused_merge) return AXHIP_INTERNAL_ERROR;  // B <= 64: the ticket slots always suffice
  if (plan.stride > 1) {
    const size_t acc_elems = static_cast<size_t>(B) * Hq * plan.stride * D;
    const size_t need = (acc_elems + static_cast<size_t>(B) * Hq * plan.stride * 2) * sizeof(float);
    if (static_ws) {
      if (need > static_cast<size_t>(AXHIP_GQA_DECODE_STATIC_SCRATCH_BYTES)) return AXHIP_OUT_OF_MEMORY;
      const int rc = static_scratch_on_this_device(&workspace);
      if (rc != AXHIP_OK) return rc;
      workspace_bytes = AXHIP_GQA_DECODE_STATIC_SCRATCH_BYTES;
    }
    if (!workspace || workspace_bytes < need) return AXHIP_INVALID_ARGUMENT;
    a.part_acc = static_cast<float *>(workspace);
    a.part_ml = a.part_acc + acc_elems;
  }
  hipStream_t st = as_stream(stream);
  if (mfma) return D == 128 ? launch_decode_mfma<128>(a, B, st) : launch_decode_mfma<64>(a, B, st);
  return dtype == AXHIP_FLOAT16 ? dispatch_dim<__half>(a, D, G, B, st) : dispatch_dim<float>(a, D, G, B, st);
}
}  // namespace

extern "C" {

// Measurement hook: overrides the split heuristics (0 restores the default).
AXHIP_API void axhip_gqa_decode_tune(int target_workgroups, int force_splits) {
  // a negative target selects the two-kernel form for a forced split count (split kernel + merge kernel)
  g_tuning.separate_merge = target_workgroups < 0 ? 1 : 0;
  g_tuning.target_workgroups = target_workgroups > 0 ? target_workgroups : 0;
  // force_splits >= 1000: keep large head groups on the vector path (for comparison), splits = force_splits - 1000
  g_tuning.mfma_groups = force_splits >= 1000 ? 0 : 1;
  if (force_splits >= 1000) force_splits -= 1000;
  g_tuning.force_splits = force_splits > 0 ? force_splits : 0;
}

// Reports the plan the launcher will use (tests and benchmarks print it).
AXHIP_API void axhip_gqa_decode_plan(int B, int Hq, int Hkv, int max_len, int *n_splits, int *chunk) {
  const int group = (Hkv > 0 && Hq % Hkv == 0) ? Hq / Hkv : 1;
  // (as for fp16 and D <= 128; other launches of groups >= 4 use heads_per_workgroup)
  const int G = (g_tuning.mfma_groups && group >= 4) ? mfma_heads_per_workgroup(group) : heads_per_workgroup(group);
  const SplitPlan p = plan_splits(B, Hq / G, max_len);
  if (n_splits) *n_splits = p.n_splits;
  if (chunk) *chunk = p.chunk;
}

AXHIP_API size_t axhip_gqa_decode_workspace_bytes(int B, int Hq, int Hkv, int D, int max_len) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || max_len <= 0 || Hq % Hkv != 0) return 0;
  // sized for the largest split count any tuning can choose
  return static_cast<size_t>(B) * Hq * kMaxSplits * (D + 2) * sizeof(float);
}

}  // extern "C"

namespace {
int gqa_decode_entry(const void *q, const void *k, const void *v, const int32_t *seq_lens, void *out,
                     void *workspace, size_t workspace_bytes, int dtype, int B, int Hq, int Hkv, int D,
                     int max_len, int64_t stride_b, int64_t stride_h, int64_t stride_s, axhip_stream stream,
                     bool static_ws) {
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

  DecodeArgs a{};
  a.q = q;
  a.k = k;
  a.v = v;
  a.seq_lens = seq_lens;
  a.out = out;
  a.stride_b = stride_b;
  a.stride_h = stride_h;
  a.stride_s = stride_s;
  return plan_and_launch(a, workspace, workspace_bytes, dtype, B, Hq, Hkv, D, max_len, stream, static_ws);
}
}  // namespace

extern "C" {

AXHIP_API int axhip_gqa_decode(const void *q, const void *k, const void *v, const int32_t *seq_lens,
                               void *out, void *workspace, size_t workspace_bytes, int dtype, int B,
                               int Hq, int Hkv, int D, int max_len, int64_t stride_b,
                               int64_t stride_h, int64_t stride_s, axhip_stream stream) {
  return gqa_decode_entry(q, k, v, seq_lens, out, workspace, workspace_bytes, dtype, B, Hq, Hkv, D, max_len,
                          stride_b, stride_h, stride_s, stream, false);
}

// axhip_gqa_decode with the split partials in the library's static device scratch: no workspace argument,
// no allocation of any kind on the call path (the kernels, the plan and the results are the same).
AXHIP_API int axhip_gqa_decode_static(const void *q, const void *k, const void *v, const int32_t *seq_lens,
                                      void *out, int dtype, int B, int Hq, int Hkv, int D, int max_len,
                                      int64_t stride_b, int64_t stride_h, int64_t stride_s,
                                      axhip_stream stream) {
  return gqa_decode_entry(q, k, v, seq_lens, out, nullptr, 0, dtype, B, Hq, Hkv, D, max_len, stride_b,
                          stride_h, stride_s, stream, true);
}

// Paged cache: the same kernels, plan and merge as axhip_gqa_decode; only the address of a key row differs
// (looked up through the page table), so the result has the bits of the dense call on the same keys.
AXHIP_API int axhip_gqa_decode_paged(const void *q, const void *k_pool, const void *v_pool, const int32_t *page_table,
                                     const int32_t *seq_lens, void *out, void *workspace, size_t workspace_bytes,
                                     int dtype, int B, int Hq, int Hkv, int D, int max_len, int max_pages, int n_pages,
                                     axhip_stream stream) {
  if (dtype != AXHIP_FLOAT16 && dtype != AXHIP_FLOAT32) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || max_len <= 0 || max_pages <= 0 || n_pages <= 0) return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (D != 64 && D != 128 && D != 256) return AXHIP_INVALID_ARGUMENT;
  // every key up to max_len needs a table entry; a workgroup holds the page numbers of its range in LDS
  if (static_cast<int64_t>(max_pages) * kPageKeys < max_len || max_len > (kMaxRangePages - 1) * kPageKeys)
    return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (B > 65535) return AXHIP_INVALID_ARGUMENT;
  if (!q || !k_pool || !v_pool || !page_table || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool)) & 15)
    return AXHIP_INVALID_PTR;
  DecodeArgs a{};
  a.q = q;
  a.k = k_pool;
  a.v = v_pool;
  a.seq_lens = seq_lens;
  a.out = out;
  a.page_table = page_table;
  a.max_pages = max_pages;
  a.n_pages = n_pages;
  a.page_stride = static_cast<int64_t>(Hkv) * kPageKeys * D;
  a.stride_s = D;  // (unused by the paged addressing; kept sane for the alignment rule of the MFMA test)
  return plan_and_launch(a, workspace, workspace_bytes, dtype, B, Hq, Hkv, D, max_len, stream);
}

AXHIP_API int axhip_gqa_decode_qkv(const float *q, int64_t q_stride, const float *k, int64_t k_stride,
                                   const float *v, int64_t v_stride, const void *q_weight,
                                   const void *k_weight, int w_dtype, float eps, const int64_t *pos,
                                   const float *inv_freq, int h_sec, int w_sec, const int32_t *seq_lens,
                                   void *k_cache, void *v_cache, void *out, void *workspace,
                                   size_t workspace_bytes, int cache_dtype, int B, int Hq, int Hkv, int D,
                                   int cache_rows, int max_len, axhip_stream stream) {
  if (cache_dtype != AXHIP_FLOAT16 && cache_dtype != AXHIP_FLOAT32) return AXHIP_UNSUPPORTED_TYPE;
  if ((q_weight || k_weight) && !is_float_dtype(w_dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || max_len <= 0 || cache_rows <= 0 || max_len > cache_rows)
    return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (D != 64 && D != 128 && D != 256) return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (B > 65535) return AXHIP_INVALID_ARGUMENT;
  if (!q || !k || !v || !pos || !inv_freq || !seq_lens || !k_cache || !v_cache || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15) return AXHIP_INVALID_PTR;
  DecodeArgs a{};
  a.k = k_cache;
  a.v = v_cache;
  a.seq_lens = seq_lens;
  a.out = out;
  a.stride_b = static_cast<int64_t>(Hkv) * cache_rows * D;
  a.stride_h = static_cast<int64_t>(cache_rows) * D;
  a.stride_s = D;
  a.len_add = 1;
  a.pq = q;
  a.pk = k;
  a.pv = v;
  a.pq_stride = q_stride;
  a.pk_stride = k_stride;
  a.pv_stride = v_stride;
  a.qw = q_weight;
  a.kw = k_weight;
  a.w_f16 = w_dtype == AXHIP_FLOAT16;
  a.eps = eps;
  a.pos = pos;
  a.inv_freq = inv_freq;
  a.h_lim = h_sec * 3;
  a.w_lim = w_sec * 3;
  a.cache_rows = cache_rows;
  return plan_and_launch(a, workspace, workspace_bytes, cache_dtype, B, Hq, Hkv, D, max_len, stream);
}

// axhip_gqa_decode_qkv over a paged cache: the new token's k / v row goes to row seq_lens[b] % 128 of page
// page_table[b, seq_lens[b] / 128] (the page must have been reserved), the keys are read through the table.
AXHIP_API int axhip_gqa_decode_qkv_paged(const float *q, int64_t q_stride, const float *k, int64_t k_stride,
                                         const float *v, int64_t v_stride, const void *q_weight, const void *k_weight,
                                         int w_dtype, float eps, const int64_t *pos, const float *inv_freq, int h_sec,
                                         int w_sec, const int32_t *seq_lens, void *k_pool, void *v_pool,
                                         const int32_t *page_table, void *out, void *workspace, size_t workspace_bytes,
                                         int cache_dtype, int B, int Hq, int Hkv, int D, int max_len, int max_pages,
                                         int n_pages, axhip_stream stream) {
  if (cache_dtype != AXHIP_FLOAT16) return AXHIP_UNSUPPORTED_TYPE;
  if ((q_weight || k_weight) && !is_float_dtype(w_dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || Hq <= 0 || Hkv <= 0 || max_len <= 0 || max_pages <= 0 || n_pages <= 0) return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (D != 64 && D != 128 && D != 256) return AXHIP_INVALID_ARGUMENT;
  if (static_cast<int64_t>(max_pages) * kPageKeys < max_len || max_len > (kMaxRangePages - 1) * kPageKeys)
    return AXHIP_INVALID_ARGUMENT;
  if (B == 0) return AXHIP_OK;
  if (B > 65535) return AXHIP_INVALID_ARGUMENT;
  if (!q || !k || !v || !pos || !inv_freq || !seq_lens || !k_pool || !v_pool || !page_table || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool)) & 15) return AXHIP_INVALID_PTR;
  DecodeArgs a{};
  a.k = k_pool;
  a.v = v_pool;
  a.seq_lens = seq_lens;
  a.out = out;
  a.page_table = page_table;
  a.max_pages = max_pages;
  a.n_pages = n_pages;
  a.page_stride = static_cast<int64_t>(Hkv) * kPageKeys * D;
  a.stride_s = D;
  a.len_add = 1;
  a.pq = q;
  a.pk = k;
  a.pv = v;
  a.pq_stride = q_stride;
  a.pk_stride = k_stride;
  a.pv_stride = v_stride;
  a.qw = q_weight;
  a.kw = k_weight;
  a.w_f16 = w_dtype == AXHIP_FLOAT16;
  a.eps = eps;
  a.pos = pos;
  a.inv_freq = inv_freq;
  a.h_lim = h_sec * 3;
  a.w_lim = w_sec * 3;
  a.cache_rows = max_pages * kPageKeys;
  return plan_and_launch(a, workspace, workspace_bytes, cache_dtype, B, Hq, Hkv, D, max_len, stream);
}

}  // extern "C"
