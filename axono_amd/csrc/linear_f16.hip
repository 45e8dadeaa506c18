// fp16 Linear: out[M,N] = x[M,K] . W[N,K]^T (+ bias), fp32 accumulation on the matrix cores.
//
// Both operands are K-contiguous, which is what the MFMA register layouts want: for
// v_mfma_f32_16x16x32_f16 every lane supplies 8 consecutive K elements of one row, i.e. exactly one
// 16-byte load.  Which 8 elements of the 32-wide K step a lane takes does not matter as long as the
// W fragment and the x fragment agree, so the lanes are assigned so that the four lanes serving a
// row read 64 consecutive bytes per load and 256 consecutive bytes per unrolled step.
//
// Skinny M (decode, M <= 32): the weight matrix is streamed from HBM exactly once and the work is
// HBM-bound.  A wavefront owns NT*16 rows of W and a K slice, with the W rows as the MFMA "A"
// operand and the (few) x rows as "B", so the output fragment holds out^T.  Nothing is staged
// through LDS: x is small and stays in L2.  The four wavefronts of a workgroup take four K slices
// of the same rows and add their fragments through LDS, so one launch finishes the product; small
// N gets up to 16 wavefronts (K slices) per workgroup so that the launch still fills 256 CUs.
//
//
// Larger M runs a tiled GEMM (128x128 output tile per workgroup, 32x32x16 MFMA, operands staged
// through LDS with register double buffering); it is MFMA-bound once M reaches a few hundred rows.
#include "common.hpp"

namespace axhip {
namespace {

constexpr int kThreads = 256;   // tiled GEMM workgroup
constexpr int kSkinnyMaxM = 32;
constexpr int kMaxWaves = 16;   // wavefronts per workgroup of the skinny kernel (K slices)

struct LinearTuning {
  int target_waves = 0;     // wavefronts to aim for in the skinny kernel; 0 = 8 per compute unit of the device
  int force_nt = 0;         // > 0: rows-of-16 per wavefront (1 to 4)
  int force_waves = 0;      // > 0: wavefronts (K slices) per workgroup (4, 8 or 16)
};
LinearTuning g_lin;

struct SkinnyPlan {
  int nt, mt, waves, k_per_wave;
  int half;  // packed weights: a workgroup takes 8 of the 16 rows of its tile (twice the workgroups)
};

// A workgroup owns NT*16 rows of W and all of K; its wavefronts split K and add their fragments
// through LDS, so one launch finishes the product.  Small N gets more wavefronts per workgroup
// (down to 128 of K each) so that the launch still fills the chip.
SkinnyPlan plan_skinny(int64_t M, int64_t K, int64_t N) {
  // Measured at M = 16 and 32 on MI355X (packed weights): two row tiles per wavefront win once N >= 8192
  // (lm_head 2048 -> 151936: 109 us with NT=2 / 8 wavefronts against 125 us with NT=4 / 4), one tile
  // with 8-16 K slices wins for the small matrices; every kernel costs about 3 us plus its bytes at
  // 5.5-5.7 TB/s.
  SkinnyPlan p;
  p.mt = M <= 16 ? 1 : 2;
  if (g_lin.force_nt > 0)
    p.nt = g_lin.force_nt;
  else
    p.nt = N >= 8192 ? 2 : 1;

  const int64_t ntiles = (N + p.nt * 16 - 1) / (p.nt * 16);
  const int64_t target_waves = g_lin.target_waves > 0 ? g_lin.target_waves : 8 * device_cu_count();
  int64_t want = g_lin.force_waves > 0 ? g_lin.force_waves : (target_waves + ntiles - 1) / ntiles;
  if (g_lin.force_waves == 0 && want < 8) want = 8;
  int waves = 4;
  while (waves < want && waves < kMaxWaves) waves *= 2;
  while (waves > 4 && K / waves < 128) waves /= 2;
  if (p.nt == 4 && waves > 4) waves = 4;   // LDS: the reduction buffer grows with NT * waves
  if (p.nt * p.mt >= 2 && waves > 8) waves = 8;
  // 32 rows of x double the LDS strip of a wavefront: with two row tiles of W, four wavefronts per
  // workgroup keep as many workgroups on a CU as at 16 rows (M = 32, 2048 -> 151936: 117 us against 134)
  if (g_lin.force_waves == 0 && p.mt == 2 && p.nt == 2 && waves > 4) waves = 4;
  p.waves = waves;
  // with one row tile per workgroup and at most 128 tiles half the CUs would idle: 8 rows per workgroup
  p.half = (p.nt == 1 && ntiles * ((M + p.mt * 16 - 1) / (p.mt * 16)) <= 128) ? 1 : 0;
  int64_t kpw = (K + waves - 1) / waves;
  p.k_per_wave = static_cast<int>((kpw + 127) / 128 * 128);
  return p;
}

__device__ __forceinline__ half8_t zero_h8() {
  half8_t z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<_Float16>(0.0f);
  return z;
}

__device__ __forceinline__ half8_t load_h8(const __half *p) {
  // a plain vector load: going through an integer struct makes the compiler touch the loaded
  // registers at once, which puts a wait right behind every load
  return *reinterpret_cast<const half8_t *>(p);
}

// weight fragments are read once per launch: streaming (non-temporal) loads
__device__ __forceinline__ half8_t load_h8_stream(const __half *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const half8_t *>(p));
}

// 8 fp32 activations -> fp16 round-to-nearest-even (the conversion the reference applies to x
// before its GEMM)
__device__ __forceinline__ half8_t load_h8(const float *p) {
  const Vec16 a = ld16(p), b = ld16(p + 4);
  half8_t h;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h[i] = static_cast<_Float16>(__builtin_bit_cast(float, a.w[i]));
    h[4 + i] = static_cast<_Float16>(__builtin_bit_cast(float, b.w[i]));
  }
  return h;
}

struct LinearArgs {
  const void *x;
  const __half *w;
  const __half *bias;
  void *out;
  int M, K, N;
  int k_per_wave, out_f16;
};

// Final store of 4 consecutive n for one m, bias added.
template <bool NT = false>
__device__ __forceinline__ void store_out4(const LinearArgs &a, int m, int n, const float (&v)[4]) {
  if (m >= a.M) return;
  const int64_t o = static_cast<int64_t>(m) * a.N + n;
  if (n + 3 < a.N && (a.N & 3) == 0) {
    float y[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) y[r] = v[r] + (a.bias ? __half2float(a.bias[n + r]) : 0.f);
    if (a.out_f16) {
      half4_t h;
#pragma unroll
      for (int r = 0; r < 4; ++r) h[r] = static_cast<_Float16>(y[r]);
      *reinterpret_cast<half4_t *>(static_cast<__half *>(a.out) + o) = h;
    } else {
      if constexpr (NT)
        __builtin_nontemporal_store(float4_t{y[0], y[1], y[2], y[3]}, reinterpret_cast<float4_t *>(static_cast<float *>(a.out) + o));
      else
        *reinterpret_cast<float4_t *>(static_cast<float *>(a.out) + o) = float4_t{y[0], y[1], y[2], y[3]};
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (n + r >= a.N) continue;
    float y = v[r];
    if (a.bias) y += __half2float(a.bias[n + r]);
    if (a.out_f16)
      static_cast<__half *>(a.out)[o + r] = __float2half_rn(y);
    else
      static_cast<float *>(a.out)[o + r] = y;
  }
}

// Gated epilogue of one 16-row tile that holds 8 gate rows (rows 0-7 of the tile) and their 8 up rows (rows
// 8-15).  A lane owns rows 4g .. 4g+3 of the tile for x row m: the lower half of the wavefront (g = 0, 1) has
// gate rows, fetches the up rows of the same columns from lane + 32 and stores silu(gate) * up for output
// columns 8 tile + 4g ..; the upper half stores nothing.  `o.N` is the number of output columns (N / 2).
__device__ __forceinline__ void store_glu_tile(const LinearArgs &o, int m, int tile, int g, const float4_t &acc) {
  float v[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float own = acc[q];  // (a copy: bit-casting the vector element itself reads element 0)
    unsigned lo, hi;
    pair_xor32(__builtin_bit_cast(unsigned, own), lo, hi);  // lower half: lo = own value, hi = that of lane + 32
    const float gt = __builtin_bit_cast(float, lo), up = __builtin_bit_cast(float, hi);
    v[q] = gt / (1.0f + expf(-gt)) * up;
  }
  if (g < 2) store_out4(o, m, tile * 8 + 4 * g, v);
}

template <int NT, int MT, int WAVES, typename XT>
__global__ __launch_bounds__(WAVES * 64) void linear_skinny_kernel(LinearArgs a) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * (NT * 16);
  const int m_base = blockIdx.y * (MT * 16);
  const int k_begin = wave * a.k_per_wave;
  const int k_end = min(k_begin + a.k_per_wave, a.K);
  const XT *x = static_cast<const XT *>(a.x);

  float4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};

  const __half *wrow[NT];
  bool wok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int row = n_base + t * 16 + r;
    wok[t] = row < a.N;
    wrow[t] = a.w + static_cast<int64_t>(wok[t] ? row : 0) * a.K;
  }
  const XT *xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int u = 0; u < MT; ++u) {
    const int m = m_base + u * 16 + r;
    xok[u] = m < a.M;
    xrow[u] = x + static_cast<int64_t>(xok[u] ? m : 0) * a.K;
  }

  for (int kk = k_begin; kk < k_end; kk += 128) {
    half8_t af[NT][4], bf[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kc = kk + (j * 4 + g) * 8;
      const bool kin = kc < k_end;
#pragma unroll
      for (int t = 0; t < NT; ++t) af[t][j] = (kin && wok[t]) ? load_h8_stream(wrow[t] + kc) : zero_h8();
#pragma unroll
      for (int u = 0; u < MT; ++u) bf[u][j] = (kin && xok[u]) ? load_h8(xrow[u] + kc) : zero_h8();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t][j], bf[u][j], acc[t][u], 0, 0, 0);
  }

  // add the K slices of this workgroup: wavefronts 1.. park their fragments in LDS, wavefront 0 sums
  __shared__ float4_t red[WAVES - 1][NT * MT][64];
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u) red[wave - 1][t * MT + u][lane] = acc[t][u];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      float4_t s = acc[t][u];
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) s += red[w][t * MT + u][lane];
      // fragment layout: this lane holds out[m = m_base + u*16 + r][n = n_base + t*16 + 4g + 0..3]
      const float v[4] = {s[0], s[1], s[2], s[3]};
      store_out4(a, m_base + u * 16 + r, n_base + t * 16 + 4 * g, v);
    }
  }
}

template <int NT, int MT, int WAVES, typename XT>
void launch_skinny(const LinearArgs &a, hipStream_t st) {
  const dim3 grid((a.N + NT * 16 - 1) / (NT * 16), (a.M + MT * 16 - 1) / (MT * 16));
  hipLaunchKernelGGL((linear_skinny_kernel<NT, MT, WAVES, XT>), grid, dim3(WAVES * 64), 0, st, a);
}

template <int NT, int MT, typename XT>
void dispatch_waves(const LinearArgs &a, int waves, hipStream_t st) {
  if constexpr (NT * MT == 1) {
    if (waves >= 16) return launch_skinny<NT, MT, 16, XT>(a, st);
  }
  if constexpr (NT < 4) {
    if (waves >= 8) return launch_skinny<NT, MT, 8, XT>(a, st);
  }
  launch_skinny<NT, MT, 4, XT>(a, st);
}

template <typename XT>
void dispatch_skinny(const LinearArgs &a, const SkinnyPlan &p, hipStream_t st) {
  if (p.mt == 1) {
    if (p.nt == 4)
      dispatch_waves<4, 1, XT>(a, p.waves, st);
    else if (p.nt == 2)
      dispatch_waves<2, 1, XT>(a, p.waves, st);
    else
      dispatch_waves<1, 1, XT>(a, p.waves, st);
  } else {
    if (p.nt == 2)
      dispatch_waves<2, 2, XT>(a, p.waves, st);
    else
      dispatch_waves<1, 2, XT>(a, p.waves, st);
  }
}

// ------------------------------------------------------------------------------------------------
// Tiled GEMM for M > 32.  Workgroup tile 128 (m) x 128 (n), K step 32; four wavefronts in a 2x2
// arrangement, each computing 64x64 with 2x2 MFMA 32x32x16 tiles.  Operands go global -> registers
// -> LDS (rows padded by 16 bytes against bank conflicts) -> MFMA fragments; the global loads of
// step k+1 are issued before the MFMAs of step k.
// ------------------------------------------------------------------------------------------------
constexpr int kTM = 128, kTN = 128, kTK = 32;
constexpr int kLdsRow = kTK + 8;  // halves per LDS row (64 B data + 16 B pad)

template <typename XT>
__global__ __launch_bounds__(kThreads) void linear_gemm_kernel(LinearArgs a) {
  __shared__ __attribute__((aligned(16))) _Float16 sx[kTM][kLdsRow];
  __shared__ __attribute__((aligned(16))) _Float16 sw[kTN][kLdsRow];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int m0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const XT *x = static_cast<const XT *>(a.x);

  // global -> register staging: 128 rows x 32 halves = 512 16-byte chunks per operand, 2 per thread
  const int lr = tid >> 2;        // 0..63 (+64 for the second chunk)
  const int lc = (tid & 3) * 8;   // k offset of the chunk
  half8_t gx[2], gw[2];
  auto load_global = [&](int kk) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = lr + h * 64;
      const int kc = kk + lc;
      const bool kin = kc < a.K;
      gx[h] = (kin && m0 + row < a.M) ? load_h8(x + static_cast<int64_t>(m0 + row) * a.K + kc) : zero_h8();
      gw[h] = (kin && n0 + row < a.N) ? load_h8(a.w + static_cast<int64_t>(n0 + row) * a.K + kc) : zero_h8();
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *reinterpret_cast<half8_t *>(&sx[lr + h * 64][lc]) = gx[h];
      *reinterpret_cast<half8_t *>(&sw[lr + h * 64][lc]) = gw[h];
    }
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int fr = lane & 31, fk = (lane >> 5) * 8;  // fragment row / k offset within a 16-wide K step
  load_global(0);
  for (int kk = 0; kk < a.K; kk += kTK) {
    __syncthreads();  // previous step's fragment reads are done
    store_lds();
    __syncthreads();
    if (kk + kTK < a.K) load_global(kk + kTK);
#pragma unroll
    for (int ks = 0; ks < kTK; ks += 16) {
      half8_t fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const half8_t *>(&sw[wn + i * 32 + fr][ks + fk]);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = *reinterpret_cast<const half8_t *>(&sx[wm + j * 32 + fr][ks + fk]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }
  // 32x32 fragment: rows are W rows (n), columns are x rows (m); lane holds column lane%32 and rows
  // 8*blk + 4*(lane/32)... : element e -> row 8*(e/4) + (lane/32)*4 + e%4
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = m0 + wm + j * 32 + (lane & 31);
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        const int n = n0 + wn + i * 32 + blk * 8 + (lane >> 5) * 4;
        const float v[4] = {acc[i][j][blk * 4], acc[i][j][blk * 4 + 1], acc[i][j][blk * 4 + 2],
                            acc[i][j][blk * 4 + 3]};
        store_out4(a, m, n, v);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// Packed weights.  W [N,K] row-major is re-ordered once into MFMA fragment order: the matrix is cut
// into tiles of 16 rows x 32 K, and a tile is stored as the 1 KiB block a wavefront loads for one
// v_mfma_f32_16x16x32_f16 (lane (r, g) = 8 halves W[16 t + r][32 c + 8 g ..]); the blocks of one
// row tile are consecutive in c.  A wavefront streaming a row tile then reads consecutive memory,
// 64 x 16 B per load instruction, the same pattern that lets the attention kernel run near HBM speed.
// Rows and K are zero-padded to whole tiles.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pack_weight_kernel(const __half *__restrict__ w,
                                                          __half *__restrict__ packed, int N, int K,
                                                          int KC, int64_t frags, int glu) {
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (f >= frags) return;
  const int lane = static_cast<int>(f & 63);
  const int64_t blk = f >> 6;
  const int c = static_cast<int>(blk % KC);
  const int64_t t = blk / KC;
  // glu: packed tile j takes rows [8j, 8j+8) of the first half of W (gate) as its rows 0-7 and the same rows of
  // the second half (up) as its rows 8-15: every tile holds the gate and up rows of its own 8 output columns
  const int r16 = lane & 15;
  const int64_t row = glu ? (r16 >> 3) * (N / 2) + t * 8 + (r16 & 7) : t * 16 + r16;
  const int k = c * 32 + (lane >> 4) * 8;
  Vec16 v;
  v.w[0] = v.w[1] = v.w[2] = v.w[3] = 0u;
  if (row < N && k + 8 <= K) v = ld16(w + row * K + k);
  st16(packed + f * 8, v);
}

struct PackedArgs {
  const void *x;
  const __half *wp;
  const __half *bias;
  void *out;
  int M, K, N, KC, chunks_per_wave, out_f16;
  int glu;  // every row tile holds 8 gate rows and their 8 up rows: the epilogue stores silu(gate) * up, N/2 columns
};

// x fragments.  Loading the MFMA "B" fragments straight from global memory is a 16-row gather (64
// bytes per row per instruction).  Instead, every iteration a wavefront copies the x columns it
// needs next (MT*16 rows x U*32 columns) into a private LDS strip with coalesced 16-byte loads,
// converting fp32 to fp16 on the way, and reads the fragments from LDS.  The strip has no padding;
// the 16-byte unit index is XOR-ed with the row so that the 16 rows of a fragment read fall into
// 16 different bank groups.
template <int NT, int MT, int WAVES, int U, bool HALF, typename XT>
__global__ __launch_bounds__(WAVES * 64) void linear_skinny_packed_kernel(PackedArgs a) {
  static_assert(!HALF || NT == 1, "half tiles come one per workgroup");
  constexpr int ROWS = MT * 16;
  constexpr int UNITS = U * 4;                 // 16-byte units per strip row
  constexpr int STRIP_HALVES = ROWS * U * 32;  // per wavefront
  constexpr int RED_BYTES = (WAVES - 1) * NT * MT * 64 * 16;
  constexpr int STRIP_BYTES = WAVES * STRIP_HALVES * 2;
  __shared__ __attribute__((aligned(16))) unsigned char smem[STRIP_BYTES > RED_BYTES ? STRIP_BYTES : RED_BYTES];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  // HALF: two workgroups per row tile.  Both run the full 16-row product, with the 8 rows of their half
  // loaded into both halves of the fragment (lane r and lane r ^ 8 read the same 16 bytes: no extra
  // memory traffic), and each stores the rows of its half only.
  const int tile0 = HALF ? blockIdx.x >> 1 : blockIdx.x * NT;
  const int half = blockIdx.x & 1;
  const int src_lane = HALF ? ((lane & ~8) | (half << 3)) : lane;
  const int n_tiles = (a.N + 15) / 16;
  const int m_base = blockIdx.y * ROWS;
  const int c_begin = wave * a.chunks_per_wave;
  const int c_end = min(c_begin + a.chunks_per_wave, a.KC);
  const XT *x = static_cast<const XT *>(a.x);
  _Float16 *strip = reinterpret_cast<_Float16 *>(smem) + wave * STRIP_HALVES;

  float4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};

  const __half *wt[NT];
  bool wok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    wok[t] = tile0 + t < n_tiles;
    wt[t] = a.wp + (static_cast<int64_t>(wok[t] ? tile0 + t : 0) * a.KC) * 512 + src_lane * 8;
  }

  for (int c = c_begin; c < c_end; c += U) {
    half8_t af[NT][U], bf[MT][U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const bool in = c + j < c_end;
#pragma unroll
      for (int t = 0; t < NT; ++t)
        af[t][j] = (in && wok[t]) ? load_h8_stream(wt[t] + static_cast<int64_t>(c + j) * 512) : zero_h8();
    }
    // stage x[m_base .. +ROWS)[32c .. 32(c+U)): ROWS*UNITS vectors, 64 per pass
    half8_t xv[ROWS * UNITS / 64];
#pragma unroll
    for (int p = 0; p < ROWS * UNITS / 64; ++p) {
      const int v = p * 64 + lane;
      const int row = v / UNITS, unit = v % UNITS;
      const int m = m_base + row, k = c * 32 + unit * 8;
      xv[p] = (m < a.M && k + 8 <= a.K && c + unit / 4 < c_end) ? load_h8(x + static_cast<int64_t>(m) * a.K + k)
                                                               : zero_h8();
    }
#pragma unroll
    for (int p = 0; p < ROWS * UNITS / 64; ++p) {
      const int v = p * 64 + lane;
      const int row = v / UNITS, unit = v % UNITS;
      *reinterpret_cast<half8_t *>(strip + row * (U * 32) + ((unit ^ (row & (UNITS - 1) & 15)) * 8)) = xv[p];
    }
#pragma unroll
    for (int j = 0; j < U; ++j)
#pragma unroll
      for (int u = 0; u < MT; ++u) {
        const int row = u * 16 + r, unit = j * 4 + g;
        bf[u][j] = *reinterpret_cast<const half8_t *>(strip + row * (U * 32) + ((unit ^ (row & (UNITS - 1) & 15)) * 8));
      }
#pragma unroll
    for (int j = 0; j < U; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t][j], bf[u][j], acc[t][u], 0, 0, 0);
  }

  // add the K slices: the x strips are dead by now, their LDS is reused for the fragments
  __syncthreads();
  float4_t *red = reinterpret_cast<float4_t *>(smem);  // [WAVES-1][NT*MT][64]
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u) red[((wave - 1) * NT * MT + t * MT + u) * 64 + lane] = acc[t][u];
  }
  __syncthreads();
  if (wave != 0) return;
  if (HALF && (g >> 1) != half) return;  // output rows 4g .. 4g+3 of the tile belong to the other workgroup
  LinearArgs o;  // only the fields store_out4 reads
  o.bias = a.bias;
  o.out = a.out;
  o.M = a.M;
  o.N = a.glu ? a.N / 2 : a.N;
  o.out_f16 = a.out_f16;
  float4_t tot[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      float4_t s = acc[t][u];
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) s += red[(w * NT * MT + t * MT + u) * 64 + lane];
      tot[t][u] = s;
    }
  }
  if (a.glu) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u) store_glu_tile(o, m_base + u * 16 + r, tile0 + t, g, tot[t][u]);
    return;
  }
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      const float v[4] = {tot[t][u][0], tot[t][u][1], tot[t][u][2], tot[t][u][3]};
      store_out4(o, m_base + u * 16 + r, (tile0 + t) * 16 + 4 * g, v);
    }
}

// Chunks of 32 K per loop iteration: bounded by the LDS the x strips take (WAVES * MT*16 * U*64 bytes
// must stay within 64 KiB).
template <int NT, int MT, int WAVES>
constexpr int packed_unroll() {
  return (WAVES * MT >= 16) ? 4 : ((NT == 1 && WAVES * MT <= 8) ? 8 : 4);
}

template <int NT, int MT, int WAVES, typename XT>
void launch_packed(const PackedArgs &a, bool half, hipStream_t st) {
  constexpr int U = packed_unroll<NT, MT, WAVES>();
  const int n_tiles = (a.N + 15) / 16;
  const dim3 grid((n_tiles + NT - 1) / NT, (a.M + MT * 16 - 1) / (MT * 16));
  if constexpr (NT == 1) {
    if (half && !a.glu) {
      hipLaunchKernelGGL((linear_skinny_packed_kernel<NT, MT, WAVES, U, true, XT>), dim3(grid.x * 2, grid.y),
                         dim3(WAVES * 64), 0, st, a);
      return;
    }
  }
  hipLaunchKernelGGL((linear_skinny_packed_kernel<NT, MT, WAVES, U, false, XT>), grid, dim3(WAVES * 64), 0, st, a);
}

template <int NT, int MT, typename XT>
void dispatch_packed_waves(const PackedArgs &a, int waves, bool half, hipStream_t st) {
  if constexpr (NT * MT == 1) {
    if (waves >= 16) return launch_packed<NT, MT, 16, XT>(a, half, st);
  }
  if constexpr (NT < 4) {
    if (waves >= 8) return launch_packed<NT, MT, 8, XT>(a, half, st);
  }
  launch_packed<NT, MT, 4, XT>(a, half, st);
}

template <typename XT>
void dispatch_packed(const PackedArgs &a, const SkinnyPlan &p, hipStream_t st) {
  const bool half = p.half != 0;
  if (p.mt == 1) {
    if (p.nt == 4)
      dispatch_packed_waves<4, 1, XT>(a, p.waves, half, st);
    else if (p.nt == 3)
      dispatch_packed_waves<3, 1, XT>(a, p.waves, half, st);
    else if (p.nt == 2)
      dispatch_packed_waves<2, 1, XT>(a, p.waves, half, st);
    else
      dispatch_packed_waves<1, 1, XT>(a, p.waves, half, st);
  } else {
    if (p.nt == 4)
      dispatch_packed_waves<4, 2, XT>(a, p.waves, half, st);
    else if (p.nt == 3)
      dispatch_packed_waves<3, 2, XT>(a, p.waves, half, st);
    else if (p.nt == 2)
      dispatch_packed_waves<2, 2, XT>(a, p.waves, half, st);
    else
      dispatch_packed_waves<1, 2, XT>(a, p.waves, half, st);
  }
}

// ------------------------------------------------------------------------------------------------
// GEMM over packed weights (M > 32).  Workgroup tile: 256 rows of W (16 packed row tiles, 4 per
// wavefront; 2 or 1 per wavefront when the problem is too small to fill the chip with that) x 64 or
// 128 rows of x; K advances 128 per step.  The W fragments come straight from the
// packed buffer (1 KiB contiguous per load, no LDS); the x tile of a step (128 x 128 halves) is
// staged once per workgroup into LDS (XOR-swizzled, double-buffered) with coalesced loads and read
// back as MFMA "B" fragments by all four wavefronts.  Loads of step i+1 are issued before the 128
// MFMAs of step i.  Workgroup ids are mapped so that the m-blocks sharing a block of W rows run on
// the same XCD back to back: that XCD's L2 then serves W to all of them after one HBM read.
// ------------------------------------------------------------------------------------------------
constexpr int kGK = 128;  // workgroup tile: 64 TW weight rows (TW row tiles per wavefront) x GM rows of x, K in steps of kGK
int g_gemm_rows = 0;                 // measurement hook: 64 or 128 rows of x per workgroup (0 = default)
int g_gemm_tiles = 0;                // measurement hook: 1, 2 or 4 row tiles of W per wavefront (0 = by size)
int g_tile_order = -1;               // measurement hook: A * 256 + B rectangles of 256 x 128 tiles per XCD (0 = plain order, -1 = by size)
constexpr int kXcds = 8;

// FULL: K is a multiple of the 128-column step, so no load needs a predicate (rows and tiles past
// the edge are clamped to valid memory and their results never stored).  Predicated loads compile to
// branches, after which the compiler waits for every outstanding load before each MFMA group.
// GM: rows of x per workgroup (32 only for the smallest problems, with TW = 1).  128 gives the larger tile (one workgroup per CU, 87 flop per byte
// moved from L2); 64 halves the registers so that two workgroups share a CU and one's loads hide
// behind the other's MFMAs.
template <typename XT, bool FULL, int GM, int TW>
__global__ __launch_bounds__(256, GM == 128 ? 1 : (GM == 64 ? 2 : 4)) void linear_gemm_packed_kernel(PackedArgs a, int n_blocks, int m_blocks) {
  constexpr int MT = GM / 16;        // x row tiles per wavefront
  constexpr int XV = GM * 16 / 256;  // 16-byte x vectors staged per thread and step
  __shared__ __attribute__((aligned(16))) _Float16 xs[2][GM * kGK];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  // XCD-aware decode of the linear workgroup id (ids are dealt round-robin to the XCDs)
  const int id = blockIdx.x;
  const int xcd = id % kXcds, slot = id / kXcds;
  const int nb = (slot / m_blocks) * kXcds + xcd, mb = slot % m_blocks;
  if (nb >= n_blocks) return;
  const int n_tiles = (a.N + 15) / 16;
  const int tile0 = (nb * 4 + wave) * TW;  // first of this wavefront's TW row tiles
  const int m0 = mb * GM;
  const XT *x = static_cast<const XT *>(a.x);
  const int steps = (a.KC + 3) / 4;  // 4 chunks of 32 K per step

  const __half *wt[TW];
  bool wok[TW];
#pragma unroll
  for (int t = 0; t < TW; ++t) {
    wok[t] = tile0 + t < n_tiles;
    wt[t] = a.wp + (static_cast<int64_t>(wok[t] ? tile0 + t : 0) * a.KC) * 512 + lane * 8;
  }
  auto load_w = [&](int t, int cc) -> half8_t {
    if constexpr (FULL) return load_h8(wt[t] + static_cast<int64_t>(cc) * 512);
    return (wok[t] && cc < a.KC) ? load_h8(wt[t] + static_cast<int64_t>(cc) * 512) : zero_h8();
  };
  // x staging: GM rows x 16 units of 16 bytes per step, XV per thread
  auto load_x = [&](int step, half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) {
      const int v = p * 256 + tid;
      const int row = v >> 4, unit = v & 15;
      const int m = m0 + row, k = step * kGK + unit * 8;
      if constexpr (FULL)
        xv[p] = load_h8(x + static_cast<int64_t>(min(m, a.M - 1)) * a.K + k);
      else
        xv[p] = (m < a.M && k + 8 <= a.K) ? load_h8(x + static_cast<int64_t>(m) * a.K + k) : zero_h8();
    }
  };
  auto store_x = [&](int buf, const half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) {
      const int v = p * 256 + tid;
      const int row = v >> 4, unit = v & 15;
      *reinterpret_cast<half8_t *>(&xs[buf][row * kGK + ((unit ^ (row & 15)) * 8)]) = xv[p];
    }
  };

  float4_t acc[TW][MT];
#pragma unroll
  for (int t = 0; t < TW; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};

  half8_t wf[TW][4];  // [row tile][chunk within the step]
  half8_t xv[XV];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < TW; ++t) wf[t][j] = load_w(t, j);
  load_x(0, xv);
  store_x(0, xv);
  __syncthreads();

  for (int i = 0; i < steps; ++i) {
    const int buf = i & 1;
    // FULL: the loop body is branch-free - the last step fetches its own data once more instead of
    // skipping the prefetch, so the compiler can count outstanding loads exactly
    const bool more = FULL || i + 1 < steps;
    const int nxt = FULL ? min(i + 1, steps - 1) : i + 1;
    if (more) load_x(nxt, xv);
    // keep the prefetches where they are written: left alone, the scheduler sinks them to the end of
    // the step (shorter live ranges) and the step then waits out a full memory latency
    __builtin_amdgcn_sched_barrier(0);
    // x fragments are read from LDS one chunk ahead of their products: four reads per 4 TW products
    // keep the LDS half busy, and a wavefront that waits for its reads before every chunk leaves the
    // matrix pipe idle for as long
    half8_t bf[2][MT];
    auto load_bf = [&](int j, half8_t (&f)[MT]) {
#pragma unroll
      for (int u = 0; u < MT; ++u) {
        const int row = u * 16 + r, unit = j * 4 + g;
        f[u] = *reinterpret_cast<const half8_t *>(&xs[buf][row * kGK + ((unit ^ (row & 15)) * 8)]);
      }
    };
    load_bf(0, bf[0]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j + 1 < 4) load_bf(j + 1, bf[(j + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TW; ++t)
#pragma unroll
        for (int u = 0; u < MT; ++u)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[t][j], bf[j & 1][u], acc[t][u], 0, 0, 0);
      // the fragments of chunk j are consumed: fetch chunk j of the next step into the same registers
      if (more) {
#pragma unroll
        for (int t = 0; t < TW; ++t) wf[t][j] = load_w(t, nxt * 4 + j);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) store_x(buf ^ 1, xv);
    __syncthreads();
  }

  LinearArgs o;
  o.bias = a.bias;
  o.out = a.out;
  o.M = a.M;
  o.N = a.glu ? a.N / 2 : a.N;
  o.out_f16 = a.out_f16;
#pragma unroll
  for (int u = 0; u < MT; ++u) {
    const int m = m0 + u * 16 + r;
    if (a.glu) {
#pragma unroll
      for (int t = 0; t < TW; ++t) store_glu_tile(o, m, tile0 + t, g, acc[t][u]);
    } else {
#pragma unroll
      for (int t = 0; t < TW; ++t) {
        const float v[4] = {acc[t][u][0], acc[t][u][1], acc[t][u][2], acc[t][u][3]};
        store_out4(o, m, (tile0 + t) * 16 + 4 * g, v);
      }
    }
  }
}

// The smallest problems (one row tile of W per wavefront, 64 weight rows x GM rows of x per workgroup,
// at most two workgroups per CU): a step of 128 K is 4 * GM/16 products per wavefront, far less than a
// memory latency, so the loads run P steps ahead of the products (W fragments and the x vectors of a
// step wait in registers; x goes into the LDS double buffer one step before its use).  K is a multiple
// of P * 128; rows and tiles past the edge are clamped to valid memory and never stored.
template <typename XT, int GM, int P>
__global__ __launch_bounds__(256, GM == 64 ? 2 : 4) void linear_gemm_packed_deep_kernel(PackedArgs a, int n_blocks,
                                                                                      int m_blocks) {
  constexpr int MT = GM / 16;
  constexpr int XV = GM * 16 / 256;
  __shared__ __attribute__((aligned(16))) _Float16 xs[2][GM * kGK];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int id = blockIdx.x;
  const int xcd = id % kXcds, slot = id / kXcds;
  const int nb = (slot / m_blocks) * kXcds + xcd, mb = slot % m_blocks;
  if (nb >= n_blocks) return;
  const int n_tiles = (a.N + 15) / 16;
  const int tile = nb * 4 + wave;
  const int m0 = mb * GM;
  const XT *x = static_cast<const XT *>(a.x);
  const int steps = a.KC / 4;

  const __half *wt = a.wp + (static_cast<int64_t>(min(tile, n_tiles - 1)) * a.KC) * 512 + lane * 8;
  const XT *xp[XV];
#pragma unroll
  for (int p = 0; p < XV; ++p) {
    const int v = p * 256 + tid;
    xp[p] = x + static_cast<int64_t>(min(m0 + (v >> 4), a.M - 1)) * a.K + (v & 15) * 8;
  }
  auto load_step = [&](int step, half8_t (&w)[4], half8_t (&xv)[XV]) __attribute__((always_inline)) {
    const int sc = min(step, steps - 1);  // past the end: the last step again, never used
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = load_h8(wt + static_cast<int64_t>(sc * 4 + j) * 512);
#pragma unroll
    for (int p = 0; p < XV; ++p) xv[p] = load_h8(xp[p] + sc * kGK);
  };
  auto store_x = [&](int buf, const half8_t (&xv)[XV]) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < XV; ++p) {
      const int v = p * 256 + tid;
      const int row = v >> 4, unit = v & 15;
      *reinterpret_cast<half8_t *>(&xs[buf][row * kGK + ((unit ^ (row & 15)) * 8)]) = xv[p];
    }
  };

  float4_t acc[MT];
#pragma unroll
  for (int u = 0; u < MT; ++u) acc[u] = float4_t{0.f, 0.f, 0.f, 0.f};

  half8_t wf[P][4], xv[P][XV];
#pragma unroll
  for (int s = 0; s < P; ++s) load_step(s, wf[s], xv[s]);
  store_x(0, xv[0]);
  __syncthreads();

  for (int i0 = 0; i0 < steps; i0 += P) {
#pragma unroll
    for (int s = 0; s < P; ++s) {
      const int buf = (i0 + s) & 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half8_t bf[MT];
#pragma unroll
        for (int u = 0; u < MT; ++u) {
          const int row = u * 16 + r, unit = j * 4 + g;
          bf[u] = *reinterpret_cast<const half8_t *>(&xs[buf][row * kGK + ((unit ^ (row & 15)) * 8)]);
        }
#pragma unroll
        for (int u = 0; u < MT; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[s][j], bf[u], acc[u], 0, 0, 0);
      }
      // x of the next step (requested P - 1 steps ago) goes to the other LDS buffer; this step's
      // registers then take the loads of step i + P
      store_x(buf ^ 1, xv[(s + 1) % P]);
      load_step(i0 + s + P, wf[s], xv[s]);
      __syncthreads();
    }
  }

  LinearArgs o;
  o.bias = a.bias;
  o.out = a.out;
  o.M = a.M;
  o.N = a.N;
  o.out_f16 = a.out_f16;
  if (tile >= n_tiles) return;
#pragma unroll
  for (int u = 0; u < MT; ++u) {
    const float v[4] = {acc[u][0], acc[u][1], acc[u][2], acc[u][3]};
    store_out4(o, m0 + u * 16 + r, tile * 16 + 4 * g, v);
  }
}

// 256 weight rows x 128 rows of x with two workgroups per CU (fp16 x, K % 128 == 0).  Against the 256 x 64 tile
// this halves the W bytes that pass through the CU's vector memory path per product.  Measured facts that shape it:
// the matrix pipes of this part are clocked by power - the same launch runs 20-45 % faster on all-zero data - and the
// time of a launch is, to within a few percent, the sum of what its matrix instructions take alone (the loop with
// every load and store removed) and what each kind of data movement adds when it is put back: output stores, x
// loads, W loads, LDS reads, in that order of cost.  Hiding latency better buys nothing (a second set of x
// fragments read one half chunk ahead, W fragments three or four chunks ahead: same time); moving fewer bytes does.
// Hence:
//  * all global loads are buffer loads - one 32-bit lane offset for the eight x vectors of a step and one for the W
//    fragments, everything else in scalar registers; rows of x past M read as zeros by the buffer's bounds check;
//  * the x fragments of a half chunk (4 of the 8 row tiles) are read from LDS while the 16 products of the half
//    chunk before them issue (two register sets: the registers the scalar addressing freed);
//  * tiles are handed out in rectangles of A weight-row blocks x B blocks of x rows, one rectangle to one XCD at a
//    time (workgroup ids are dealt round-robin to the XCDs): the 64 workgroups an XCD runs together then share A W
//    tiles and B x tiles through its L2 instead of one W tile and 64 x tiles (2048 -> 151936 at M = 4096: 947 ->
//    1074 TFLOP/s; nothing where x fits the L2 anyway, as at M = 512).
// Every output element sums its products in K order: the same bits as the 64-row tile.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ half8_t buffer_load_h8(__amdgpu_buffer_rsrc_t rsrc, int voffset, int soffset) {
  return __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voffset, soffset, 0));
}

struct TileOrder {
  int A, B;  // rectangle of A n-blocks x B m-blocks per XCD at a time; A == 0: n-blocks dealt to XCDs, m fastest
};

__global__ __launch_bounds__(256, 2) void linear_gemm_packed_128_kernel(PackedArgs a, int n_blocks, int m_blocks, TileOrder ord) {
  constexpr int GM = 128, MT = 8, TW = 4, XV = 8;
  __shared__ __attribute__((aligned(16))) _Float16 xs[2][GM * kGK];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int id = blockIdx.x;
  const int xcd = id % kXcds, slot = id / kXcds;
  int nb, mb;
  if (ord.A > 0) {
    const int per = ord.A * ord.B, within = slot % per;
    const int rect = (slot / per) * kXcds + xcd;          // rectangles in the order they are handed out
    const int rect_m = (m_blocks + ord.B - 1) / ord.B;
    mb = (rect % rect_m) * ord.B + within % ord.B;
    nb = (rect / rect_m) * ord.A + within / ord.B;
    if (mb >= m_blocks) return;
  } else {
    nb = (slot / m_blocks) * kXcds + xcd;
    mb = slot % m_blocks;
  }
  if (nb >= n_blocks) return;
  const int n_tiles = (a.N + 15) / 16;
  const int tile0 = (nb * 4 + wave) * TW;
  const int m0 = mb * GM;
  const int chunks = a.K / 32, steps = chunks / 4;

  // W: a buffer per wavefront that starts at its first row tile (tiles past the last one: the last one again)
  const int t0c = min(tile0, n_tiles - 1);
  const int64_t wbytes = static_cast<int64_t>(n_tiles - t0c) * a.KC * 1024;
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<__half *>(a.wp + static_cast<int64_t>(t0c) * a.KC * 512), 0,
      static_cast<int>(wbytes < 0x7fffffff ? wbytes : 0x7fffffff), 0x00020000);
  int wso[TW];
#pragma unroll
  for (int t = 0; t < TW; ++t) wso[t] = (min(tile0 + t, n_tiles - 1) - t0c) * a.KC * 1024;
  const int wvo = lane * 16;
  auto load_w = [&](int chunk, half8_t (&f)[TW]) {
    const int co = min(chunk, chunks - 1) * 1024;  // past the end: the last chunk again
#pragma unroll
    for (int t = 0; t < TW; ++t) f[t] = buffer_load_h8(wrs, wvo, wso[t] + co);
  };
  // x: a buffer of this workgroup's rows; vector p of a thread is row (tid >> 4) + 16 p, 16-byte unit tid & 15
  const int rows_here = min(GM, a.M - m0);
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16 *>(static_cast<const _Float16 *>(a.x) + static_cast<int64_t>(m0) * a.K), 0,
      rows_here * a.K * 2, 0x00020000);
  const int xvo = ((tid >> 4) * a.K + (tid & 15) * 8) * 2;
  const int xrow16 = 16 * a.K * 2;
  auto load_x = [&](int step, half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) xv[p] = buffer_load_h8(xrs, xvo, p * xrow16 + step * (kGK * 2));
  };
  const int xrow = tid >> 4, xunit = tid & 15;
  _Float16 *xst = &xs[0][xrow * kGK + ((xunit ^ (xrow & 15)) * 8)];  // rows 16 apart keep row & 15
  auto store_x = [&](int buf, const half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) *reinterpret_cast<half8_t *>(xst + buf * (GM * kGK) + p * 16 * kGK) = xv[p];
  };
  // fragment reads: row tile u, chunk j of the step -> rows u*16 + r, unit j*4 + g
  const _Float16 *xrd = &xs[0][r * kGK];
  auto load_bf = [&](int buf, int j, int uh, half8_t (&f)[4]) {
    const int uo = ((j * 4 + g) ^ r) * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      f[u] = *reinterpret_cast<const half8_t *>(xrd + buf * (GM * kGK) + (uh + u) * 16 * kGK + uo);
  };

  float4_t acc[TW][MT];
#pragma unroll
  for (int t = 0; t < TW; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};

  half8_t wf[2][TW];  // chunk c waits in wf[c & 1]
  half8_t xv[XV];
  half8_t bfa[4], bfb[4];
  load_w(0, wf[0]);
  load_w(1, wf[1]);
  load_x(0, xv);
  store_x(0, xv);
  __syncthreads();

  for (int i = 0; i < steps; ++i) {
    const int buf = i & 1;
    load_x(min(i + 1, steps - 1), xv);
    load_bf(buf, 0, 0, bfa);
    // the scheduling barriers keep the requests where they are written: left alone, the scheduler sinks them to
    // their uses (shorter live ranges) and every group of products then waits out a full latency
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      load_bf(buf, j, 4, bfb);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TW; ++t)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[j & 1][t], bfa[u], acc[t][u], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (j + 1 < 4) load_bf(buf, j + 1, 0, bfa);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TW; ++t)
#pragma unroll
        for (int u = 0; u < 4; ++u)
          acc[t][4 + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[j & 1][t], bfb[u], acc[t][4 + u], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      load_w(i * 4 + j + 2, wf[j & 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    store_x(buf ^ 1, xv);
    __syncthreads();
  }

  LinearArgs o;
  o.bias = a.bias;
  o.out = a.out;
  o.M = a.M;
  o.N = a.glu ? a.N / 2 : a.N;
  o.out_f16 = a.out_f16;
  if (a.glu) {
#pragma unroll
    for (int u = 0; u < MT; ++u) {
#pragma unroll
      for (int t = 0; t < TW; ++t) store_glu_tile(o, m0 + u * 16 + r, tile0 + t, g, acc[t][u]);
    }
  } else {
#pragma unroll
    for (int u = 0; u < MT; ++u) {
#pragma unroll
      for (int t = 0; t < TW; ++t) {
        const float v[4] = {acc[t][u][0], acc[t][u][1], acc[t][u][2], acc[t][u][3]};
        store_out4(o, m0 + u * 16 + r, (tile0 + t) * 16 + 4 * g, v);
      }
    }
  }
}

// How the 256 x 128 tiles of a problem are handed to the XCDs.  An XCD runs 64 workgroups at a time (32 CUs, two
// each).  In the plain order they are a strip of up to 64 x blocks under one or two W blocks; a rectangle of A W
// blocks x B x blocks has the same workgroups share A W tiles and B x tiles through the XCD's L2.  The choice is
// the rectangle (A, B powers of two, 16 to 64 tiles) with the smallest estimate of
//   (workgroup slots launched / tiles) x (1 + 0.3 x operand bytes fetched per tile / bytes of a W tile):
// slots count the rectangles rounded up to whole rounds over the eight XCDs (few rectangles leave XCDs idle: 2048 ->
// 2048 at M = 4096 is 256 tiles = 8 rectangles of 8 x 4, not 4 of 8 x 8), and 0.3 fits the measured gains (M = 4096:
// 2048 -> 4096 861 -> 969 TFLOP/s, 2048 -> 151936 926 -> 992; M = 65536: 2048 -> 2048 849 -> 905).  Not worth it
// while x (M x K) fits one XCD's L2 next to the W stream, as at M = 512.
TileOrder gemm_tile_order(const PackedArgs &a, int n_blocks, int m_blocks) {
  TileOrder o{0, 0};
  if (g_tile_order >= 0) {  // measurement hook: A * 256 + B, 0 = the plain order
    o.A = g_tile_order >> 8;
    o.B = g_tile_order & 255;
    if (o.A <= 0 || o.B <= 0) o = TileOrder{0, 0};
    return o;
  }
  if (static_cast<int64_t>(a.M) * a.K * 2 <= (3 << 20)) return o;
  const double tiles = static_cast<double>(n_blocks) * m_blocks;
  auto estimate = [&](double slots, double A, double B) { return slots / tiles * (1.0 + 0.3 * (A + 0.5 * B) / (A * B)); };
  // plain order: n-blocks dealt to the XCDs, whole rounds; the 64 workgroups of an XCD are x blocks first
  const double nb_pad = (n_blocks + kXcds - 1) / kXcds * kXcds;
  const double Bp = m_blocks < 64 ? m_blocks : 64, Ap = m_blocks < 64 ? (64 + m_blocks - 1) / m_blocks : 1;
  double best = estimate(nb_pad * m_blocks, Ap, Bp);
  for (int A = 1; A <= 16; A *= 2)
    for (int B = 1; B <= 64; B *= 2) {
      const int per = A * B;
      if (per < 16 || per > 64 || A > 2 * n_blocks || B > 2 * m_blocks) continue;
      const int64_t rects = static_cast<int64_t>((n_blocks + A - 1) / A) * ((m_blocks + B - 1) / B);
      const double slots = static_cast<double>((rects + kXcds - 1) / kXcds * kXcds) * per;
      const double e = estimate(slots, A, B) * (per < 64 ? 1.02 : 1.0);  // ties go to full rectangles
      if (e < best) {
        best = e;
        o = TileOrder{A, B};
      }
    }
  return o;
}

// One workgroup per CU with eight wavefronts for the problems that give a CU only one tile of 64 TW weight
// rows x 64 rows of x (M = 512 with N = 2048 or 4096).  The bytes a CU pulls through its vector memory path per
// product fall with the tile's area, so the tile is the CU's whole share of the output; the second wavefront
// per SIMD that hides the latency of a step then has to come from inside the workgroup: wavefronts 0-3 sum the
// first half of K, wavefronts 4-7 the second half (each half with its own x double buffer in LDS and its own W
// fragments, so no byte is fetched twice), and the halves are added through LDS at the end: out = S(first
// half) + S(second half), each S accumulated in K order, the same for every launch.  fp16 x, K % 512 == 0.
template <int TW>
__global__ __launch_bounds__(512, 1) void linear_gemm_packed_khalves_kernel(PackedArgs a, int n_blocks, int m_blocks) {
  constexpr int GM = 64, MT = GM / 16;
  constexpr int XV = GM * 16 / 256;  // 16-byte x vectors per thread of a half and step
  __shared__ __attribute__((aligned(16))) _Float16 xs[2][2][GM * kGK];  // [K half][buffer]: 64 KiB
  const int tid = threadIdx.x, kh = tid >> 8, ht = tid & 255, wave = ht >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int id = blockIdx.x;
  const int xcd = id % kXcds, slot = id / kXcds;
  const int nb = (slot / m_blocks) * kXcds + xcd, mb = slot % m_blocks;
  if (nb >= n_blocks) return;
  const int n_tiles = (a.N + 15) / 16;
  const int tile0 = (nb * 4 + wave) * TW;
  const int m0 = mb * GM;
  const __half *x = static_cast<const __half *>(a.x);
  const int steps = a.KC / 8;    // steps of 128 K per half
  const int step0 = kh * steps;  // first step of this half

  const __half *wt[TW];
#pragma unroll
  for (int t = 0; t < TW; ++t)
    wt[t] = a.wp + (static_cast<int64_t>(min(tile0 + t, n_tiles - 1)) * a.KC + step0 * 4) * 512 + lane * 8;
  const __half *xp[XV];
#pragma unroll
  for (int p = 0; p < XV; ++p) {
    const int v = p * 256 + ht;
    xp[p] = x + static_cast<int64_t>(min(m0 + (v >> 4), a.M - 1)) * a.K + step0 * kGK + (v & 15) * 8;
  }
  auto load_x = [&](int step, half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) xv[p] = load_h8(xp[p] + step * kGK);
  };
  auto store_x = [&](int buf, const half8_t (&xv)[XV]) {
#pragma unroll
    for (int p = 0; p < XV; ++p) {
      const int v = p * 256 + ht;
      const int row = v >> 4, unit = v & 15;
      *reinterpret_cast<half8_t *>(&xs[kh][buf][row * kGK + ((unit ^ (row & 15)) * 8)]) = xv[p];
    }
  };

  float4_t acc[TW][MT];
#pragma unroll
  for (int t = 0; t < TW; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = float4_t{0.f, 0.f, 0.f, 0.f};

  // W fragments wait two steps ahead of their products (a weight line comes from HBM, and a step of this
  // tile is shorter than that trip); x, which every workgroup of a row block shares in L2, one step ahead.
  // (Running the halves in opposite phases - one multiplies while the other fills LDS, two barriers per
  // step - measured 3-5 % slower than letting them run side by side.)
  half8_t wf[2][TW][4];  // [step parity][row tile][chunk]
  half8_t xv[XV];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < TW; ++t) wf[s][t][j] = load_h8(wt[t] + (s * 4 + j) * 512);
  load_x(0, xv);
  store_x(0, xv);
  __syncthreads();

  for (int i0 = 0; i0 < steps; i0 += 2) {  // steps is even
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int i = i0 + s;  // LDS buffer and fragment set s
      // past the end the last step is fetched once more: no branch in the loop
      load_x(min(i + 1, steps - 1), xv);
      const int64_t w2 = static_cast<int64_t>(min(i + 2, steps - 1)) * 4 * 512;
      __builtin_amdgcn_sched_barrier(0);
      half8_t bf[2][MT];
      auto load_bf = [&](int j, half8_t (&f)[MT]) {
#pragma unroll
        for (int u = 0; u < MT; ++u) {
          const int row = u * 16 + r, unit = j * 4 + g;
          f[u] = *reinterpret_cast<const half8_t *>(&xs[kh][s][row * kGK + ((unit ^ (row & 15)) * 8)]);
        }
      };
      load_bf(0, bf[0]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j + 1 < 4) load_bf(j + 1, bf[(j + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < TW; ++t)
#pragma unroll
          for (int u = 0; u < MT; ++u)
            acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[s][t][j], bf[j & 1][u], acc[t][u], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < TW; ++t) wf[s][t][j] = load_h8(wt[t] + w2 + j * 512);
        __builtin_amdgcn_sched_barrier(0);
      }
      store_x(s ^ 1, xv);
      __syncthreads();
    }
  }

  // the second half hands its sums over through LDS (every x fragment has been read: the loop ends on a barrier)
  float4_t *red = reinterpret_cast<float4_t *>(&xs[0][0][0]);
  if (kh == 1) {
#pragma unroll
    for (int t = 0; t < TW; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u) red[((wave * TW + t) * MT + u) * 64 + lane] = acc[t][u];
  }
  __syncthreads();
  if (kh == 1) return;
  LinearArgs o;
  o.bias = a.bias;
  o.out = a.out;
  o.M = a.M;
  o.N = a.N;
  o.out_f16 = a.out_f16;
#pragma unroll
  for (int u = 0; u < MT; ++u)
#pragma unroll
    for (int t = 0; t < TW; ++t) {
      const float4_t s = acc[t][u] + red[((wave * TW + t) * MT + u) * 64 + lane];
      const float v[4] = {s[0], s[1], s[2], s[3]};
      if (tile0 + t < n_tiles) store_out4(o, m0 + u * 16 + r, (tile0 + t) * 16 + 4 * g, v);
    }
}

// Weight rows per workgroup: 256 (four row tiles per wavefront), or 128 / 64 when 256 would leave CUs
// without a workgroup (M = 512, N = 2048: 64 workgroups of 256 x 64, 256 of 64 x 64).
int gemm_tiles_per_wave(const PackedArgs &a, int gm) {
  if (g_gemm_tiles == 1 || g_gemm_tiles == 2 || g_gemm_tiles == 4) return g_gemm_tiles;
  const int64_t m_blocks = (a.M + gm - 1) / gm;
  int tw = 4;
  const int cus = device_cu_count();
  while (tw > 1 && ((a.N + 64 * tw - 1) / (64 * tw)) * m_blocks < cus) tw /= 2;
  return tw;
}

template <typename XT, int TW>
void launch_gemm_packed_tw(const PackedArgs &a, int gm, hipStream_t st) {
  const int gn = 64 * TW;
  const int n_blocks = (a.N + gn - 1) / gn, m_blocks = (a.M + gm - 1) / gm;
  const int nb_pad = (n_blocks + kXcds - 1) / kXcds * kXcds;  // whole rounds over the XCDs
  const dim3 grid(static_cast<unsigned>(nb_pad) * m_blocks);
  const bool full = a.K % kGK == 0;
#define AXHIP_GEMM_LAUNCH(F, G) \
  hipLaunchKernelGGL((linear_gemm_packed_kernel<XT, F, G, TW>), grid, dim3(256), 0, st, a, n_blocks, m_blocks)
  if (gm == 128) {
    if (full) AXHIP_GEMM_LAUNCH(true, 128); else AXHIP_GEMM_LAUNCH(false, 128);
  } else if (gm == 32 && TW == 1) {  // the 32-row tile exists for one row tile of W per wavefront only
    if constexpr (TW == 1) {
      if (full) AXHIP_GEMM_LAUNCH(true, 32); else AXHIP_GEMM_LAUNCH(false, 32);
    }
  } else {
    if (full) AXHIP_GEMM_LAUNCH(true, 64); else AXHIP_GEMM_LAUNCH(false, 64);
  }
#undef AXHIP_GEMM_LAUNCH
}

template <typename XT>
void launch_gemm_packed(const PackedArgs &a, hipStream_t st) {
  if constexpr (sizeof(XT) == 2) {  // fp32 x waits for its conversion in twice the registers: it keeps the 64-row tile
    // by default wherever it gives three quarters of the CUs a workgroup (M = 512, 2048 -> 12288, 192 tiles:
    // 41.2 us against 45.7 with the 64-row tile)
    const bool fits = a.K % kGK == 0 && static_cast<int64_t>(a.M) * a.K < (1ll << 32);
    const int64_t tiles128 = static_cast<int64_t>((a.N + 255) / 256) * ((a.M + 127) / 128);
    if (fits && (g_gemm_rows == 256 || (g_gemm_rows == 0 && g_gemm_tiles == 0 && tiles128 >= 3 * device_cu_count() / 4))) {
      const int n_blocks = (a.N + 255) / 256, m_blocks = (a.M + 127) / 128;
      const int nb_pad = (n_blocks + kXcds - 1) / kXcds * kXcds;
      const TileOrder ord = gemm_tile_order(a, n_blocks, m_blocks);
      unsigned grid128 = static_cast<unsigned>(nb_pad) * m_blocks;
      if (ord.A > 0) {
        const int64_t rects = static_cast<int64_t>((n_blocks + ord.A - 1) / ord.A) * ((m_blocks + ord.B - 1) / ord.B);
        grid128 = static_cast<unsigned>((rects + kXcds - 1) / kXcds * kXcds * ord.A * ord.B);
      }
      hipLaunchKernelGGL(linear_gemm_packed_128_kernel, dim3(grid128), dim3(256), 0, st, a, n_blocks, m_blocks, ord);
      return;
    }
  }
  if constexpr (sizeof(XT) == 2) {
    // the CU's whole share of the output as one tile, K in two halves inside the workgroup
    if (!a.glu && a.K % (4 * kGK) == 0 && (g_gemm_rows == 512 || (g_gemm_rows == 0 && g_gemm_tiles == 0))) {
      const int64_t mb64 = (a.M + 63) / 64;
      const int64_t t2 = static_cast<int64_t>((a.N + 127) / 128) * mb64, t1 = static_cast<int64_t>((a.N + 63) / 64) * mb64;
      const int cus = device_cu_count();
      int tw = 0;
      if (g_gemm_rows == 512) tw = g_gemm_tiles == 2 ? 2 : 1;
      else if (t2 <= cus && 2 * t2 > cus) tw = 2;
      else if (t1 <= cus && 2 * t1 > cus) tw = 1;
      if (tw) {
        const int n_blocks = (a.N + 64 * tw - 1) / (64 * tw), m_blocks = static_cast<int>(mb64);
        const int nb_pad = (n_blocks + kXcds - 1) / kXcds * kXcds;
        const dim3 grid(static_cast<unsigned>(nb_pad) * m_blocks);
        if (tw == 2)
          hipLaunchKernelGGL((linear_gemm_packed_khalves_kernel<2>), grid, dim3(512), 0, st, a, n_blocks, m_blocks);
        else
          hipLaunchKernelGGL((linear_gemm_packed_khalves_kernel<1>), grid, dim3(512), 0, st, a, n_blocks, m_blocks);
        return;
      }
    }
  }
  int gm = (g_gemm_rows == 32 || g_gemm_rows == 64 || g_gemm_rows == 128) ? g_gemm_rows : 64;
  const int tw = gemm_tiles_per_wave(a, gm == 32 ? 64 : gm);
  // a problem that gives no CU a second workgroup even with the smallest weight tile is bounded by the
  // latency of its K steps: 32 rows of x per workgroup double the workgroups that can overlap
  if (g_gemm_rows == 0 && tw == 1 && static_cast<int64_t>((a.N + 63) / 64) * ((a.M + 63) / 64) <= device_cu_count()) gm = 32;
  if (gm == 32 && tw != 1) gm = 64;
  constexpr int kDeep = 4;  // steps the loads of the smallest tile run ahead
  // (fp16 x only: fp32 x is converted as it arrives, which would put a wait behind every load)
  // only while no CU gets a second workgroup: with more of them the L2 bandwidth of these small tiles
  // is the bound, not the latency of a step
  if (sizeof(XT) == 2 && tw == 1 && !a.glu && (gm == 32 || gm == 64) && a.K % (kDeep * kGK) == 0 && g_gemm_tiles == 0 &&
      static_cast<int64_t>((a.N + 63) / 64) * ((a.M + gm - 1) / gm) <= device_cu_count()) {
    const int n_blocks = (a.N + 63) / 64, m_blocks = (a.M + gm - 1) / gm;
    const int nb_pad = (n_blocks + kXcds - 1) / kXcds * kXcds;
    const dim3 grid(static_cast<unsigned>(nb_pad) * m_blocks);
    if constexpr (sizeof(XT) == 2) {
      if (gm == 32)
        hipLaunchKernelGGL((linear_gemm_packed_deep_kernel<XT, 32, kDeep>), grid, dim3(256), 0, st, a, n_blocks, m_blocks);
      else
        hipLaunchKernelGGL((linear_gemm_packed_deep_kernel<XT, 64, kDeep>), grid, dim3(256), 0, st, a, n_blocks, m_blocks);
    }
    return;
  }
  switch (tw) {
    case 1: return launch_gemm_packed_tw<XT, 1>(a, gm, st);
    case 2: return launch_gemm_packed_tw<XT, 2>(a, gm, st);
    default: return launch_gemm_packed_tw<XT, 4>(a, gm, st);
  }
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

// Measurement hook for sweeps (0 restores a default).
AXHIP_API void axhip_linear_f16_tune(int target_waves, int force_nt, int force_waves, int gemm_rows) {
  // gemm_rows: 64 or 128 rows of x per GEMM workgroup, plus 1000 t to force t = 1, 2, 4 row tiles of W per wavefront
  g_gemm_tiles = gemm_rows >= 1000 ? gemm_rows / 1000 : 0;
  gemm_rows %= 1000;
  g_gemm_rows = (gemm_rows == 32 || gemm_rows == 64 || gemm_rows == 128 || gemm_rows == 256 || gemm_rows == 512) ? gemm_rows : 0;
  // target_waves >= 100000 carries a tile order for the 256 x 128 GEMM tile: 100000 + A * 256 + B (100000: plain order)
  g_tile_order = target_waves >= 100000 ? target_waves - 100000 : -1;
  if (target_waves >= 100000) target_waves = 0;
  g_lin.target_waves = target_waves > 0 ? target_waves : 0;
  g_lin.force_nt = (force_nt >= 1 && force_nt <= 4) ? force_nt : 0;
  g_lin.force_waves = (force_waves == 4 || force_waves == 8 || force_waves == 16) ? force_waves : 0;
}

// Every shape is finished by one launch; no workspace is needed (the argument stays in the ABI for
// callers that size buffers generically).
AXHIP_API size_t axhip_linear_f16_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  (void)M;
  (void)K;
  (void)N;
  return 0;
}

AXHIP_API int axhip_linear_f16(const void *x, int x_dtype, const void *w, const void *bias, void *out,
                               int out_dtype, int64_t M, int64_t K, int64_t N, void *workspace,
                               size_t workspace_bytes, axhip_stream stream) {
  (void)workspace;
  (void)workspace_bytes;
  if (!is_float_dtype(x_dtype) || !is_float_dtype(out_dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (M < 0 || K <= 0 || N <= 0 || K % 8 != 0) return AXHIP_INVALID_ARGUMENT;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
  if (M == 0) return AXHIP_OK;
  if (!x || !w || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) return AXHIP_INVALID_PTR;
  if (reinterpret_cast<uintptr_t>(out) & 15) return AXHIP_INVALID_PTR;
  hipStream_t st = as_stream(stream);
  LinearArgs a;
  a.x = x;
  a.w = static_cast<const __half *>(w);
  a.bias = static_cast<const __half *>(bias);
  a.out = out;
  a.M = static_cast<int>(M);
  a.K = static_cast<int>(K);
  a.N = static_cast<int>(N);
  a.out_f16 = out_dtype == AXHIP_FLOAT16;
  a.k_per_wave = 0;

  if (M <= kSkinnyMaxM) {
    const SkinnyPlan p = plan_skinny(M, K, N);
    a.k_per_wave = p.k_per_wave;
    if (x_dtype == AXHIP_FLOAT16)
      dispatch_skinny<__half>(a, p, st);
    else
      dispatch_skinny<float>(a, p, st);
    return launch_status();
  }
  const dim3 grid((a.N + kTN - 1) / kTN, (a.M + kTM - 1) / kTM);
  if (grid.y > 65535) return AXHIP_INVALID_ARGUMENT;
  if (x_dtype == AXHIP_FLOAT16)
    hipLaunchKernelGGL((linear_gemm_kernel<__half>), grid, dim3(kThreads), 0, st, a);
  else
    hipLaunchKernelGGL((linear_gemm_kernel<float>), grid, dim3(kThreads), 0, st, a);
  return launch_status();
}

AXHIP_API size_t axhip_linear_f16_packed_bytes(int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  const int64_t tiles = (N + 15) / 16, kc = (K + 31) / 32;
  return static_cast<size_t>(tiles) * kc * 1024;
}

AXHIP_API int axhip_linear_f16_pack(const void *w, void *packed, int64_t N, int64_t K, int glu,
                                    axhip_stream stream) {
  if (N <= 0 || K <= 0 || K % 8 != 0 || N > INT32_MAX || K > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
  if (glu && N % 32 != 0) return AXHIP_INVALID_ARGUMENT;  // both halves must be whole 16-row tiles
  if (!w || !packed) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(packed)) & 15) return AXHIP_INVALID_PTR;
  const int64_t tiles = (N + 15) / 16, kc = (K + 31) / 32;
  const int64_t frags = tiles * kc * 64;
  hipLaunchKernelGGL(pack_weight_kernel, dim3(static_cast<unsigned>((frags + 255) / 256)), dim3(256), 0,
                     as_stream(stream), static_cast<const __half *>(w), static_cast<__half *>(packed),
                     static_cast<int>(N), static_cast<int>(K), static_cast<int>(kc), frags, glu ? 1 : 0);
  return launch_status();
}

AXHIP_API int axhip_linear_f16_packed(const void *x, int x_dtype, const void *packed_w, const void *bias,
                                      void *out, int out_dtype, int64_t M, int64_t K, int64_t N, int glu,
                                      axhip_stream stream) {
  if (!is_float_dtype(x_dtype) || !is_float_dtype(out_dtype)) return AXHIP_UNSUPPORTED_TYPE;
  if (M < 0 || K <= 0 || N <= 0 || K % 8 != 0) return AXHIP_INVALID_ARGUMENT;
  if (glu && (N % 32 != 0 || bias)) return AXHIP_INVALID_ARGUMENT;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
  if (M == 0) return AXHIP_OK;
  if (!x || !packed_w || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(packed_w) | reinterpret_cast<uintptr_t>(out)) & 15)
    return AXHIP_INVALID_PTR;
  // Up to 64 rows a narrow matrix (N <= 2048) stays with the weight-streaming kernels, two blocks of 32
  // rows each: the tiled GEMM would have too few workgroups there (M = 64: 2048 -> 2048 6.3 us against
  // 11.2, 6144 -> 2048 12.9 against 27.4; wider matrices and more rows go the other way).
  const bool skinny = M <= kSkinnyMaxM || (M <= 2 * kSkinnyMaxM && N <= 2048);
  if (!skinny) {  // MFMA-bound regime: tiled GEMM over the same packed buffer
    PackedArgs ga;
    ga.x = x;
    ga.wp = static_cast<const __half *>(packed_w);
    ga.bias = static_cast<const __half *>(bias);
    ga.out = out;
    ga.M = static_cast<int>(M);
    ga.K = static_cast<int>(K);
    ga.N = static_cast<int>(N);
    ga.KC = static_cast<int>((K + 31) / 32);
    ga.chunks_per_wave = 0;
    ga.out_f16 = out_dtype == AXHIP_FLOAT16;
    ga.glu = glu ? 1 : 0;
    const int64_t wgs = ((N + 63) / 64 + kXcds - 1) / kXcds * kXcds * ((M + 63) / 64);  // the smallest tile
    if (wgs > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
    if (x_dtype == AXHIP_FLOAT16)
      launch_gemm_packed<__half>(ga, as_stream(stream));
    else
      launch_gemm_packed<float>(ga, as_stream(stream));
    return launch_status();
  }
  SkinnyPlan p = plan_skinny(M, K, N);
  // two row tiles per workgroup that would put a second workgroup on half of the CUs only (gate+up 2048 -> 12288:
  // 384 workgroups on 256 CUs): three tiles give every CU one (M = 16: 11.0 us against 12.0 us)
  if (g_lin.force_nt == 0 && p.nt == 2) {
    const int64_t tiles = (N + 15) / 16, cus = device_cu_count();
    if (tiles % 3 == 0 && tiles / 3 <= cus && (tiles + 1) / 2 > cus) {
      p.nt = 3;
      // 32 rows of x: eight wavefronts again (M = 32: 13.0 us against 14.1 us with two tiles and four wavefronts)
      if (p.mt == 2 && g_lin.force_waves == 0 && K / 8 >= 128) p.waves = 8;
    }
  }
  PackedArgs a;
  a.glu = glu ? 1 : 0;
  a.x = x;
  a.wp = static_cast<const __half *>(packed_w);
  a.bias = static_cast<const __half *>(bias);
  a.out = out;
  a.M = static_cast<int>(M);
  a.K = static_cast<int>(K);
  a.N = static_cast<int>(N);
  a.KC = static_cast<int>((K + 31) / 32);
  // any multiple of 4 works with every unroll the kernels use (a short last iteration is masked)
  int cpw = (a.KC + p.waves - 1) / p.waves;
  a.chunks_per_wave = (cpw + 3) / 4 * 4;
  a.out_f16 = out_dtype == AXHIP_FLOAT16;
  hipStream_t st = as_stream(stream);
  if (x_dtype == AXHIP_FLOAT16)
    dispatch_packed<__half>(a, p, st);
  else
    dispatch_packed<float>(a, p, st);
  return launch_status();
}

}  // extern "C"
