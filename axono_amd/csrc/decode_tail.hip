// Everything of a decoder layer that follows the attention, for decode-sized batches (M <= 16 rows), in ONE
// persistent launch that also runs the next layer's q/k/v projection:
//
//   phase 1   h1  = attn . Wo^T + h                      (o_proj + residual add)
//   phase 2   act = silu(g) * u,  [g | u] = rmsnorm(h1, w_post) . Wgu^T
//   phase 3   h2  = act . Wd^T + h1                      (down_proj + residual add)
//   phase 4   y   = rmsnorm(h2, w_next) . Wn^T           (the next layer's qkv projection)
//
// The same arithmetic as the single operators (fp16 Linear with fp32 accumulation, RMSNorm evaluated as
// (x * rstd) * w, SiLU-mul); the sums of squares of a row are added in another order than add_rms_norm adds
// them, so rstd may differ in its last bit.
//
// What the launch is for: a small Linear is a chain of dependent round trips (launch, x, weights from HBM,
// write drain) during most of which HBM idles.  Here a phase's weights do not depend on the phase before it,
// so they are requested BEFORE the barrier that ends the previous phase and arrive while the workgroup waits:
// every phase has at most one unit of work per workgroup, and a unit's weight fragments fit the registers of
// its 16 wavefronts (<= 48 VGPRs each).
//
// One workgroup per CU (1024 threads = 16 wavefronts, 128 registers each).  The wavefronts of a workgroup split K
// and add their fragments through LDS, as in the skinny Linear kernels; wavefront 0 finishes a unit (epilogue,
// store), arrives at the barrier and waits there, the other 15 request their next weights meanwhile (wavefront 0
// right after its first look at the flag: a look that follows those loads also waits for them, the memory
// counter being in order).  Barriers inside the workgroup wait for LDS traffic only (lds_barrier): __syncthreads()
// would wait for the weights in flight.
//
// Data that crosses a barrier is written with agent-scope (write-through) stores into blocks that a single
// workgroup owns as whole 128-byte lines (the residual stream as [unit][16 rows][8 columns] + the rows' partial
// sums of squares; the activations in matrix-instruction fragment order, 256 bytes per 8 columns: both are what a
// lane of the consuming phase loads as contiguous bytes), and read with ordinary loads: a line that
// no workgroup of an XCD has touched in this launch is not in that XCD's L2, so the load fetches what the
// barrier made visible; no cache invalidate is needed.  Each such buffer is written in exactly one phase and
// first read after the barrier behind it.  Results for the next launch (h_out, y) are also stored row-major.
//
// The barrier is two-level (16 workgroups per counter, then one counter for the groups; the release writes
// one flag per group), every counter and flag on its own 128-byte line (atomics on one line are served one
// after the other), only ever counts upwards (a launch starts from where its flag stands, so nothing is put back
// between launches), and spins a bounded number of times: if the workgroups are not all resident it gives up,
// counts the failure (axhip_decode_layer_tail_status; the caller then resets the counters) and every wavefront
// still exits.
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kTailWaves = 16;
constexpr int kTailThreads = kTailWaves * 64;
constexpr int kTailRows = 16;
constexpr int kBarGroup = 16;
constexpr int kBarMaxGroups = 16;
constexpr int kTailMaxWgs = kBarGroup * kBarMaxGroups;  // 256
constexpr int kSpinLimit = 1 << 17;  // looks at the flag before a wait gives up: about a tenth of a second (a barrier takes microseconds)
constexpr int kHBlockBytes = 640;  // [16][8] fp32 + 16 partial sums of squares + padding: five whole lines

// Counters and flags only ever grow (a launch adds 3 to every flag), so nothing has to be put back between
// launches: a launch reads where its group's flag stands and counts from there.  All launches on a device use
// the same number of workgroups.
struct TailBarrier {
  unsigned cnt[kBarMaxGroups * 32];
  unsigned flag[kBarMaxGroups * 32];
  unsigned top[32];
  unsigned fail[32];
};
__device__ TailBarrier g_tail_bar;

#define TAIL_LD(p) __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TAIL_ST(p, v) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define TAIL_ADD(p, v) __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// k-th barrier of this launch (k = 1, 2, 3), called by every thread; `base` = the group's flag when the launch
// began.  Only wavefront 0 has stores in flight.  Wavefront 0 arrives, looks at the flag once and only then
// requests its share of the next phase's weights (`prefetch`): the memory counter is in order, so a look at the
// flag that follows those loads also waits for them - which costs nothing, the wavefront needs them anyway.
// Returns false when the wait ran out.
template <typename F>
__device__ __forceinline__ bool grid_sync(unsigned k, unsigned base, int *s_ok, F prefetch, int spin_limit,
                                          unsigned failed_before = 0) {
  if (threadIdx.x < 64 && failed_before != 0) {
    if (threadIdx.x == 0) *s_ok = 0;
  } else if (threadIdx.x < 64) {
    __builtin_amdgcn_s_waitcnt(0);  // the write-through stores of this wavefront have reached memory
    const unsigned n_wg = gridDim.x, wg = blockIdx.x;
    const unsigned grp = wg / kBarGroup, n_grp = (n_wg + kBarGroup - 1) / kBarGroup;
    const unsigned in_grp = min(static_cast<unsigned>(kBarGroup), n_wg - grp * kBarGroup);
    const unsigned want = base + k;
    if (threadIdx.x == 0) {
      if (TAIL_ADD(&g_tail_bar.cnt[grp * 32], 1u) == want * in_grp - 1) {
        if (TAIL_ADD(&g_tail_bar.top[0], 1u) == want * n_grp - 1) {
          for (unsigned i = 0; i < n_grp; ++i) TAIL_ST(&g_tail_bar.flag[i * 32], want);
        }
      }
    }
    unsigned f = TAIL_LD(&g_tail_bar.flag[grp * 32]);
    __builtin_amdgcn_sched_barrier(0);
    prefetch();
    __builtin_amdgcn_sched_barrier(0);
    int ok = 1, limit = spin_limit;
    while (static_cast<int>(f - want) < 0) {
      if (--limit <= 0) {
        ok = 0;
        break;
      }
      __builtin_amdgcn_s_sleep(1);
      f = TAIL_LD(&g_tail_bar.flag[grp * 32]);
    }
    if (threadIdx.x == 0) {
      if (!ok) TAIL_ADD(&g_tail_bar.fail[0], 1u);
      *s_ok = ok;
    }
  }
  lds_barrier();
  return *s_ok != 0;
}

struct TailArgs {
  const __half *attn;    // [M, K1] merged attention output
  const float *h_in;     // [M, H]  residual stream entering the layer
  const __half *w_o;     // packed [H, K1]
  const float *w_post;   // [H] post-attention norm weight
  const __half *w_gu;    // packed, every tile 8 gate rows + their 8 up rows [2I, H]
  const __half *w_down;  // packed [H, I]
  const float *w_next;   // [H] the norm in front of the next Linear
  const __half *w_nl;    // packed [N_next, H]
  unsigned char *hmid;   // blocks: residual stream after the attention part
  unsigned char *hout;   // blocks: residual stream leaving the layer
  unsigned char *act;    // activations in MFMA fragment order: 1 KiB per 32 columns, lane (r, g) = 8 halves of row r
  float *h_out;          // [M, H]  out, row-major
  float *y;              // [M, N_next] out, row-major
  __half *xn;            // N_next == 0 (nothing behind the last norm in this launch): [M, H] out, the normalised rows
  int M, H, K1, I, N_next;
  float eps;
  unsigned long long *dbg;  // measurement: 32 timestamps per workgroup (axhip_decode_layer_tail_trace), or null
  int skip;  // measurement: bits 0-3 = phase 1-4 computes nothing, 32 = no barriers, 256 = a barrier gives up after one look
};

extern __shared__ __attribute__((aligned(16))) unsigned char tail_smem[];
constexpr int kStripBytes = kTailRows * 4 * 32 * 2;                     // per wavefront: 16 rows x 128 halves
// LDS: [0, 64 KiB) the x strips of phase 1, later the transposed partial sums of squares; then the parked fragments
// of the K slices, their partial sums, the rows' rstd, both norm weights.
constexpr int kRedOffset = kTailWaves * kStripBytes;
constexpr int kRedBytes = kTailWaves * 3 * 64 * 16;                     // up to three tiles per unit
constexpr int kRed2Offset = kRedOffset + kRedBytes;                     // partial sums of four wavefronts each
constexpr int kRstdOffset = kRed2Offset + 3 * 4 * 64 * 16;
constexpr int kNormWOffset = kRstdOffset + kTailRows * 4 + 16;         // both norm weights, fp32
constexpr int kTailMaxH = 2048;
constexpr int kTailLds = kNormWOffset + 2 * kTailMaxH * 4;
constexpr int kSsqStride = 260;                                         // floats per row of the transposed partial sums

__device__ __forceinline__ half8_t ld_w(const __half *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(p));
}

// x fragments of SC chunks from this wavefront's strip (rows of SC*32 halves, 16-byte units XOR-ed with the row)
template <int SC>
__device__ __forceinline__ void read_frags(const _Float16 *strip, int r, int g, half8_t (&bf)[SC]) {
#pragma unroll
  for (int j = 0; j < SC; ++j) {
    const int un = j * 4 + g;
    bf[j] = *reinterpret_cast<const half8_t *>(strip + r * (SC * 32) + ((un ^ (r & (SC * 4 - 1))) << 3));
  }
}

// rstd of the 16 rows from the per-unit partial sums of squares.  Thread u reads the 16 sums of unit u (one
// line), the sums go through LDS transposed, wavefront w adds row w (every workgroup adds in the same order, so
// all of them normalise with the same bits).  Two workgroup barriers inside.
__device__ __forceinline__ void row_rstd(const unsigned char *blocks, int n_units, int K, float eps, float *s_rstd) {
  float *T = reinterpret_cast<float *>(tail_smem);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid < 256) {
    float4_t v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      v[q] = tid < n_units ? *reinterpret_cast<const float4_t *>(blocks + static_cast<size_t>(tid) * kHBlockBytes + 512 + q * 16)
                           : float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) T[(q * 4 + e) * kSsqStride + tid] = v[q][e];
  }
  lds_barrier();
  {
    const int row = wave;  // kTailWaves == kTailRows
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s += T[row * kSsqStride + lane + 64 * i];
    s = group_sum<64>(s);
    if (lane == 0) s_rstd[row] = 1.0f / sqrtf(s / static_cast<float>(K) + eps);
  }
  lds_barrier();
}
static_assert(kTailWaves == kTailRows && kTailWaves == 16, "one wavefront per row in row_rstd, four times four fragments in total()");

// x fragments of a norm phase, straight from the residual blocks (a block holds a unit's 8 columns of all 16 rows:
// lane (r, g) of chunk c reads 32 contiguous bytes of block 4c + g): request, then normalise.
template <int NC>
__device__ __forceinline__ void load_h_frags(const unsigned char *blocks, int chunk0, int r, int g, float4_t (&hv)[NC][2]) {
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const unsigned char *p = blocks + static_cast<size_t>((chunk0 + j) * 4 + g) * kHBlockBytes + r * 32;
    hv[j][0] = *reinterpret_cast<const float4_t *>(p);
    hv[j][1] = *reinterpret_cast<const float4_t *>(p + 16);
  }
}
// (w: the norm weight's copy in LDS)
__device__ __forceinline__ half8_t norm_frag(const float4_t (&hv)[2], const float *w, int col, float rs) {
  const float4_t w0 = *reinterpret_cast<const float4_t *>(w + col), w1 = *reinterpret_cast<const float4_t *>(w + col + 4);
  const float4_t y0 = (hv[0] * rs) * w0, y1 = (hv[1] * rs) * w1;
  return half8_t{static_cast<_Float16>(y0[0]), static_cast<_Float16>(y0[1]), static_cast<_Float16>(y0[2]),
                 static_cast<_Float16>(y0[3]), static_cast<_Float16>(y1[0]), static_cast<_Float16>(y1[1]),
                 static_cast<_Float16>(y1[2]), static_cast<_Float16>(y1[3])};
}

// Sum over the 16 wavefronts (the K slices): every wavefront parks its fragments; wavefront 4 t + q adds parked
// fragments 4 q .. 4 q + 3 of tile t; wavefront 0 adds the four partial sums of every tile.  Called by all
// wavefronts (two workgroup barriers inside); the totals are valid in wavefront 0.
template <int NT>
__device__ __forceinline__ void total(float4_t (&acc)[NT], int wave, int lane) {
  float4_t *red = reinterpret_cast<float4_t *>(tail_smem + kRedOffset);
  float4_t *red2 = reinterpret_cast<float4_t *>(tail_smem + kRed2Offset);
#pragma unroll
  for (int t = 0; t < NT; ++t) red[(wave * NT + t) * 64 + lane] = acc[t];
  lds_barrier();
  if (wave < 4 * NT) {
    const int t = wave >> 2, q = wave & 3;
    float4_t p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) p[i] = red[((q * 4 + i) * NT + t) * 64 + lane];
    red2[wave * 64 + lane] = ((p[0] + p[1]) + p[2]) + p[3];
  }
  lds_barrier();
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float4_t p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = red2[((t * 4 + i)) * 64 + lane];
      acc[t] = ((p[0] + p[1]) + p[2]) + p[3];
    }
  }
}

// Residual epilogue of phases 1 and 3 (wavefront 0): the unit's 8 columns of 16 rows + residual (`rv`: this
// lane's four values, requested earlier) -> block (+ the rows' partial sums of squares), optionally row-major too.
__device__ __forceinline__ void store_residual_unit(const float4_t &tot, const float4_t &rv, unsigned char *blocks, int unit,
                                                    int half, float *row_major, int H, int M, int lane) {
  const int r = lane & 15, g = lane >> 4;
  const bool mine = (g >> 1) == half;  // output rows 4g .. 4g+3 of the tile belong to this half
  float4_t hn = {0.f, 0.f, 0.f, 0.f};
  if (mine && r < M) hn = tot + rv;
  float s = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) s = __builtin_fmaf(hn[q], hn[q], s);
  s = sum_xor16(s);  // the two lanes that hold a row's 8 columns
  if (!mine || r >= M) return;
  float *blk = reinterpret_cast<float *>(blocks + static_cast<size_t>(unit) * kHBlockBytes);
#pragma unroll
  for (int q = 0; q < 4; ++q) TAIL_ST(blk + r * 8 + (g & 1) * 4 + q, hn[q]);
  if ((g & 1) == 0) TAIL_ST(blk + 128 + r, s);
  if (row_major) *reinterpret_cast<float4_t *>(row_major + static_cast<int64_t>(r) * H + unit * 8 + (g & 1) * 4) = hn;
}

// measurement: the 100 MHz clock at point i of wavefront 0 (slots 0-15) and wavefront 5 (16-31), kept in LDS (a
// store to memory at the point itself would enter the in-order memory counter and move what it measures)
#define STAMP(i) do { if (a.dbg && lane == 0 && (wave == 0 || wave == 5)) s_stamp[(wave ? 16 : 0) + (i)] = wall_clock64(); } while (0)
template <int CK1, int CH, int CI, int NT2>
__global__ __launch_bounds__(kTailThreads) void decode_tail_kernel(TailArgs a) {
  __shared__ int s_ok;
  __shared__ unsigned long long s_stamp[32];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  _Float16 *strip = reinterpret_cast<_Float16 *>(tail_smem) + wave * (kStripBytes / 2);
  float *s_rstd = reinterpret_cast<float *>(tail_smem + kRstdOffset);
  const int wg = blockIdx.x;
  const int units1 = a.H / 8;               // phases 1 and 3: half a row tile each
  const int tiles2 = a.I / 8;               // phase 2: (gate, up) tiles of 8 output columns
  const int units2 = tiles2 / NT2;
  const int tiles4 = a.N_next / 16;
  const bool on1 = wg < units1, on2 = wg < units2, on4 = wg < tiles4;
  const int half1 = wg & 1;
  const int src_lane = (lane & ~8) | (half1 << 3);  // both halves of the fragment hold this half's 8 rows
  const bool bars = !(a.skip & 32);
  const int spin_limit = (a.skip & 256) ? 1 : kSpinLimit;  // (256: a test of the path a wait that runs out takes)
  static_assert(CK1 <= 4 && CH <= 4, "one staging step per phase");

  STAMP(0);
  // where this group's barrier flag stands (wavefront 0 needs it at the first barrier)
  unsigned base = 0, failed_before = 0;
  if (wave == 0) {
    base = TAIL_LD(&g_tail_bar.flag[(wg / kBarGroup) * 32]);
    // a wait that ran out in an earlier launch has left the counters in disorder: until the caller has reset them
    // (axhip_decode_layer_tail_status) a launch gives up at its first barrier at once instead of spinning again
    failed_before = TAIL_LD(&g_tail_bar.fail[0]);
  }
  // both norm weights go to LDS (read there by every wavefront in phases 2 and 4), the residual of phase 1 to
  // wavefront 0: requested first, so that they are back before anything that follows
  float *s_wn = reinterpret_cast<float *>(tail_smem + kNormWOffset);
  float4_t wn4 = {0.f, 0.f, 0.f, 0.f}, res1 = {0.f, 0.f, 0.f, 0.f};
  if (tid * 4 < 2 * a.H) wn4 = *reinterpret_cast<const float4_t *>((tid * 4 < a.H ? a.w_post : a.w_next - a.H) + tid * 4);
  if (wave == 0 && on1 && r < a.M && (g >> 1) == half1)
    res1 = *reinterpret_cast<const float4_t *>(a.h_in + static_cast<int64_t>(r) * a.H + wg * 8 + (g & 1) * 4);
  __builtin_amdgcn_sched_barrier(0);

  // ---- weights of phases 1 and 2: no dependence on anything, requested at once; the x columns of phase 1 go in
  // between, so that waiting for them does not wait for the weights of phase 2 (the memory counter is in order)
  half8_t wA[CK1], wB[NT2][CH], xv1[CK1];
  {
    const __half *p = a.w_o + (static_cast<int64_t>(on1 ? wg >> 1 : 0) * (a.K1 / 32) + wave * CK1) * 512 + src_lane * 8;
#pragma unroll
    for (int j = 0; j < CK1; ++j) wA[j] = ld_w(p + j * 512);
    if (!(a.skip & 1)) {
#pragma unroll
      for (int q = 0; q < CK1; ++q) {
        const int v = q * 64 + lane;
        const int row = v / (CK1 * 4), un = v % (CK1 * 4);
        xv1[q] = *reinterpret_cast<const half8_t *>(a.attn + static_cast<int64_t>(min(row, a.M - 1)) * a.K1 + wave * CK1 * 32 + un * 8);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NT2; ++t) {
      const __half *q = a.w_gu + (static_cast<int64_t>(on2 ? wg * NT2 + t : 0) * (a.H / 32) + wave * CH) * 512 + lane * 8;
#pragma unroll
      for (int j = 0; j < CH; ++j) wB[t][j] = ld_w(q + j * 512);
    }
  }

  // ---- phase 1: o_proj + residual ----------------------------------------------------------------------------------
  {
    float4_t acc[1] = {float4_t{0.f, 0.f, 0.f, 0.f}};
    const int M = a.M;
    if (tid * 4 < 2 * a.H) *reinterpret_cast<float4_t *>(s_wn + tid * 4) = wn4;
    if (!(a.skip & 1)) {
      half8_t bf[CK1];
#pragma unroll
      for (int q = 0; q < CK1; ++q) {
        const int v = q * 64 + lane;
        const int row = v / (CK1 * 4), un = v % (CK1 * 4);
        *reinterpret_cast<half8_t *>(strip + row * (CK1 * 32) + ((un ^ (row & (CK1 * 4 - 1))) << 3)) = xv1[q];
      }
      read_frags<CK1>(strip, r, g, bf);
#pragma unroll
      for (int j = 0; j < CK1; ++j) acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wA[j], bf[j], acc[0], 0, 0, 0);
    }
    STAMP(1);
    total<1>(acc, wave, lane);
    if (wave == 0) {
      if (on1) store_residual_unit(acc[0], res1, a.hmid, wg, half1, nullptr, a.H, M, lane);
    }
  }
  STAMP(2);
  if (bars && !grid_sync(1, base, &s_ok, [] {}, spin_limit, failed_before)) return;
  STAMP(3);

  // ---- phase 2: post-attention norm, gate + up, SiLU-mul -------------------------------------------------------------
  half8_t wC[CI], wD[CH];
  const bool lin4 = a.N_next > 0;  // a Linear behind the last norm (else the launch ends with the normalised rows)
  const __half *pd = a.w_nl + (static_cast<int64_t>(on4 ? wg : 0) * (a.H / 32) + wave * CH) * 512 + lane * 8;
  const __half *pc = a.w_down + (static_cast<int64_t>(on1 ? wg >> 1 : 0) * (a.I / 32) + wave * CI) * 512 + src_lane * 8;
  {
    float4_t acc[NT2];
#pragma unroll
    for (int t = 0; t < NT2; ++t) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (!(a.skip & 2)) {
      float4_t hv[CH][2];
      load_h_frags<CH>(a.hmid, wave * CH, r, g, hv);  // in flight while the row sums are added
      row_rstd(a.hmid, units1, a.H, a.eps, s_rstd);
      const float rs = s_rstd[r];
      STAMP(4);
      half8_t bf[CH];
#pragma unroll
      for (int j = 0; j < CH; ++j) bf[j] = norm_frag(hv[j], s_wn, (wave * CH + j) * 32 + g * 8, rs);
#pragma unroll
      for (int j = 0; j < CH; ++j)
#pragma unroll
        for (int t = 0; t < NT2; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wB[t][j], bf[j], acc[t], 0, 0, 0);
    }
    STAMP(5);
    if (wave != 0) {
      // the weights of phase 3 travel while the unit is finished and the barrier is crossed
#pragma unroll
      for (int j = 0; j < CI; ++j) wC[j] = ld_w(pc + j * 512);
    }
    total<NT2>(acc, wave, lane);
    if (wave == 0) {
      if (on2) {
#pragma unroll
        for (int t = 0; t < NT2; ++t) {
          _Float16 hv[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float own = acc[t][q];
            unsigned lo, hi;
            pair_xor32(__builtin_bit_cast(unsigned, own), lo, hi);  // lower half: lo = own value, hi = that of lane + 32
            const float gt = __builtin_bit_cast(float, lo), up = __builtin_bit_cast(float, hi);
            hv[q] = static_cast<_Float16>(gt / (1.0f + expf(-gt)) * up);
          }
          if (g < 2 && r < a.M) {
            // columns 8 cg .. 8 cg + 7 are lanes (r, cg % 4) of chunk cg / 4: 256 bytes that this workgroup alone writes
            const int cg = wg * NT2 + t;
            unsigned *dst = reinterpret_cast<unsigned *>(a.act + static_cast<size_t>(cg >> 2) * 1024 + ((cg & 3) * 16 + r) * 16 + g * 8);
            TAIL_ST(dst, __builtin_bit_cast(unsigned, half2_t{hv[0], hv[1]}));
            TAIL_ST(dst + 1, __builtin_bit_cast(unsigned, half2_t{hv[2], hv[3]}));
          }
        }
      }
    }
  }
  {
    auto pf = [&] {
#pragma unroll
      for (int j = 0; j < CI; ++j) wC[j] = ld_w(pc + j * 512);
    };
    STAMP(6);
    if (bars) {
      if (!grid_sync(2, base, &s_ok, pf, spin_limit)) return;
    } else if (wave == 0) {
      pf();
    }
    STAMP(7);
  }

  // ---- phase 3: down_proj + residual -----------------------------------------------------------------------------------
  {
    float4_t acc[1] = {float4_t{0.f, 0.f, 0.f, 0.f}};
    float4_t res3 = {0.f, 0.f, 0.f, 0.f};  // this workgroup's own block of phase 1
    if (wave == 0 && on1 && r < a.M && (g >> 1) == half1)
      res3 = *reinterpret_cast<const float4_t *>(a.hmid + static_cast<size_t>(wg) * kHBlockBytes + r * 32 + (g & 1) * 16);
    if (!(a.skip & 4)) {
      const unsigned char *xf = a.act + static_cast<size_t>(wave * CI) * 1024 + lane * 16;
      half8_t bf[CI];
#pragma unroll
      for (int j = 0; j < CI; ++j) bf[j] = *reinterpret_cast<const half8_t *>(xf + j * 1024);
#pragma unroll
      for (int j = 0; j < CI; ++j) acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wC[j], bf[j], acc[0], 0, 0, 0);
    }
    STAMP(8);
    if (wave != 0 && lin4) {
#pragma unroll
      for (int j = 0; j < CH; ++j) wD[j] = ld_w(pd + j * 512);
    }
    total<1>(acc, wave, lane);
    if (wave == 0) {
      if (on1) store_residual_unit(acc[0], res3, a.hout, wg, half1, a.h_out, a.H, a.M, lane);
    }
  }
  {
    auto pf = [&] {
      if (!lin4) return;
#pragma unroll
      for (int j = 0; j < CH; ++j) wD[j] = ld_w(pd + j * 512);
    };
    STAMP(9);
    if (bars) {
      if (!grid_sync(3, base, &s_ok, pf, spin_limit)) return;
    } else if (wave == 0) {
      pf();
    }
    STAMP(10);
  }

  // ---- phase 4: the next norm and the Linear behind it -------------------------------------------------------------------
  {
    float4_t acc[1] = {float4_t{0.f, 0.f, 0.f, 0.f}};
    if (!(a.skip & 8)) {
      float4_t hv[CH][2];
      load_h_frags<CH>(a.hout, wave * CH, r, g, hv);
      row_rstd(a.hout, units1, a.H, a.eps, s_rstd);
      const float rs = s_rstd[r];
      half8_t bf[CH];
#pragma unroll
      for (int j = 0; j < CH; ++j) bf[j] = norm_frag(hv[j], s_wn + a.H, (wave * CH + j) * 32 + g * 8, rs);
      if (lin4) {
#pragma unroll
        for (int j = 0; j < CH; ++j) acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wD[j], bf[j], acc[0], 0, 0, 0);
      } else if (wg < kTailWaves && wave == wg && r < a.M) {
        // every workgroup holds all the normalised rows, 32 * CH columns per wavefront: workgroup w writes the
        // columns of its wavefront w
#pragma unroll
        for (int j = 0; j < CH; ++j)
          *reinterpret_cast<half8_t *>(a.xn + static_cast<int64_t>(r) * a.H + (wave * CH + j) * 32 + g * 8) = bf[j];
      }
    }
    STAMP(11);
    if (lin4) {
      total<1>(acc, wave, lane);
      if (wave == 0) {
        if (on4 && r < a.M)
          *reinterpret_cast<float4_t *>(a.y + static_cast<int64_t>(r) * a.N_next + wg * 16 + 4 * g) = acc[0];
      }
    }
    STAMP(12);
  }
  lds_barrier();
  if (a.dbg && tid < 32) a.dbg[blockIdx.x * 32 + tid] = s_stamp[tid];
}

int g_tail_skip = 0;
unsigned long long *g_tail_dbg = nullptr;

template <int CK1, int CH, int CI, int NT2>
int launch_tail(const TailArgs &a, int wgs, hipStream_t st) {
  static std::atomic<uint64_t> lds_set{0};
  const void *fn = reinterpret_cast<const void *>(decode_tail_kernel<CK1, CH, CI, NT2>);
  const int rc = raise_dynamic_lds(fn, kTailLds, lds_set);
  if (rc != AXHIP_OK) return rc;
  hipLaunchKernelGGL((decode_tail_kernel<CK1, CH, CI, NT2>), dim3(wgs), dim3(kTailThreads), kTailLds, st, a);
  return launch_status();
}

// The kernel instance for these widths on the current device: 0 = none (the caller uses the single operators),
// 1 = <4,4,12,3> (K1 = H = 2048, I = 6144), 2 = <1,1,2,1> (K1 = H = 512, I = 1024).  Every phase must have at most
// one unit per resident workgroup (one workgroup per compute unit, 256 at most).
int tail_instance(int M, int H, int K1, int I, int N_next, int *wgs_out) {
  if (M < 0 || M > kTailRows || H <= 0 || K1 <= 0 || I <= 0 || N_next < 0) return 0;  // N_next 0: no Linear behind
  if (H % 512 != 0 || K1 % 512 != 0 || I % 512 != 0 || N_next % 16 != 0 || H > kTailMaxH) return 0;
  const int cus = device_cu_count();
  const int wgs = cus < kTailMaxWgs ? cus : kTailMaxWgs;
  if (wgs_out) *wgs_out = wgs;
  const int ck1 = K1 / 512, ch = H / 512, ci = I / 512;
  int nt2 = 0;
  for (int t = 1; t <= 3; ++t)
    if ((I / 8) % t == 0 && (I / 8) / t <= wgs) {
      nt2 = t;
      break;
    }
  if (nt2 == 0 || H / 8 > wgs || N_next / 16 > wgs) return 0;
  if (N_next == 0 && wgs < kTailWaves) return 0;  // one workgroup per wavefront's columns writes the normalised rows
  if (ck1 == 4 && ch == 4 && ci == 12 && nt2 == 3) return 1;
  if (ck1 == 1 && ch == 1 && ci == 2 && nt2 == 1) return 2;
  return 0;
}

size_t tail_workspace_bytes(int H, int I) {
  return 2 * static_cast<size_t>(H / 8) * kHBlockBytes + static_cast<size_t>(I) * 32;
}

// The launch behind both entry points: N_next > 0 ends with y = norm(h_out) . w_next_linear^T, N_next == 0 with
// xn = norm(h_out) as fp16 rows.
int tail_entry(const void *attn, const float *h_in, const void *w_o, const float *w_post, const void *w_gate_up,
               const void *w_down, const float *w_next, const void *w_next_linear, float *h_out, float *y, void *xn,
               void *workspace, size_t workspace_bytes, int M, int H, int K1, int I, int N_next, float eps,
               axhip_stream stream) {
  int wgs = 0;
  const int instance = tail_instance(M, H, K1, I, N_next, &wgs);
  if (instance == 0) return AXHIP_INVALID_ARGUMENT;  // widths this launch is not built for: use the single operators
  if (M == 0) return AXHIP_OK;
  if (!attn || !h_in || !w_o || !w_post || !w_gate_up || !w_down || !w_next || !h_out || !workspace)
    return AXHIP_INVALID_PTR;
  if (N_next > 0 ? (!w_next_linear || !y) : !xn) return AXHIP_INVALID_PTR;
  if (h_in == h_out) return AXHIP_INVALID_ARGUMENT;  // lines of h_in are in the L2s when h_out is written
  const uintptr_t all = reinterpret_cast<uintptr_t>(attn) | reinterpret_cast<uintptr_t>(h_in) |
                        reinterpret_cast<uintptr_t>(w_post) | reinterpret_cast<uintptr_t>(w_next) |
                        reinterpret_cast<uintptr_t>(h_out) | reinterpret_cast<uintptr_t>(y) |
                        reinterpret_cast<uintptr_t>(xn) | reinterpret_cast<uintptr_t>(w_o) |
                        reinterpret_cast<uintptr_t>(w_gate_up) | reinterpret_cast<uintptr_t>(w_down) |
                        reinterpret_cast<uintptr_t>(w_next_linear);
  if (all & 15) return AXHIP_INVALID_PTR;
  if (reinterpret_cast<uintptr_t>(workspace) & 127) return AXHIP_INVALID_PTR;
  if (workspace_bytes < tail_workspace_bytes(H, I)) return AXHIP_INVALID_ARGUMENT;
  TailArgs a;
  a.attn = static_cast<const __half *>(attn);
  a.h_in = h_in;
  a.w_o = static_cast<const __half *>(w_o);
  a.w_post = w_post;
  a.w_gu = static_cast<const __half *>(w_gate_up);
  a.w_down = static_cast<const __half *>(w_down);
  a.w_next = w_next;
  a.w_nl = static_cast<const __half *>(w_next_linear);
  a.hmid = static_cast<unsigned char *>(workspace);
  a.hout = a.hmid + static_cast<size_t>(H / 8) * kHBlockBytes;
  a.act = a.hout + static_cast<size_t>(H / 8) * kHBlockBytes;
  a.h_out = h_out;
  a.y = y;
  a.xn = static_cast<__half *>(xn);
  a.M = M;
  a.H = H;
  a.K1 = K1;
  a.I = I;
  a.N_next = N_next;
  a.eps = eps;
  a.skip = g_tail_skip;
  a.dbg = g_tail_dbg;
  hipStream_t st = as_stream(stream);
  return instance == 1 ? launch_tail<4, 4, 12, 3>(a, wgs, st) : launch_tail<1, 1, 2, 1>(a, wgs, st);
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

AXHIP_API size_t axhip_decode_layer_tail_workspace_bytes(int H, int I) {
  if (H <= 0 || I <= 0) return 0;
  return tail_workspace_bytes(H, I);
}

AXHIP_API int axhip_decode_layer_tail(const void *attn, const float *h_in, const void *w_o, const float *w_post,
                                      const void *w_gate_up, const void *w_down, const float *w_next,
                                      const void *w_next_linear, float *h_out, float *y, void *workspace,
                                      size_t workspace_bytes, int M, int H, int K1, int I, int N_next, float eps,
                                      axhip_stream stream) {
  if (N_next <= 0) return AXHIP_INVALID_ARGUMENT;
  return tail_entry(attn, h_in, w_o, w_post, w_gate_up, w_down, w_next, w_next_linear, h_out, y, nullptr, workspace,
                    workspace_bytes, M, H, K1, I, N_next, eps, stream);
}

AXHIP_API int axhip_decode_layer_tail_last(const void *attn, const float *h_in, const void *w_o, const float *w_post,
                                           const void *w_gate_up, const void *w_down, const float *w_final_norm,
                                           float *h_out, void *xn_out, void *workspace, size_t workspace_bytes, int M,
                                           int H, int K1, int I, float eps, axhip_stream stream) {
  return tail_entry(attn, h_in, w_o, w_post, w_gate_up, w_down, w_final_norm, nullptr, h_out, nullptr, xn_out, workspace,
                    workspace_bytes, M, H, K1, I, 0, eps, stream);
}

AXHIP_API int axhip_decode_layer_tail_supported(int M, int H, int K1, int I, int N_next) {
  return tail_instance(M, H, K1, I, N_next, nullptr) != 0 ? 1 : 0;
}

// Barrier bookkeeping of axhip_decode_layer_tail: number of barrier waits that ran out since the last reset (0 in
// a healthy process); reset != 0 also puts the counters back to zero (only while no such launch is in flight).
AXHIP_API int axhip_decode_layer_tail_status(int reset, unsigned *failed_waits) {
  static TailBarrier h;
  if (hipMemcpyFromSymbol(&h, HIP_SYMBOL(g_tail_bar), sizeof(h)) != hipSuccess) return AXHIP_INTERNAL_ERROR;
  if (failed_waits) *failed_waits = h.fail[0];
  if (reset) {
    static const TailBarrier z = {};
    if (hipMemcpyToSymbol(HIP_SYMBOL(g_tail_bar), &z, sizeof(z)) != hipSuccess) return AXHIP_INTERNAL_ERROR;
  }
  return AXHIP_OK;
}

AXHIP_API void axhip_decode_layer_tail_tune(int skip_phases) { g_tail_skip = skip_phases; }
AXHIP_API void axhip_decode_layer_tail_trace(void *stamps) { g_tail_dbg = static_cast<unsigned long long *>(stamps); }

}  // extern "C"
