// Causal attention for prefill on the matrix cores: S query tokens per sequence attend to the keys
// already written to the static KV cache [B, Hkv, rows, D] (fp16), query i of sequence b sitting at
// absolute position start[b] + i and seeing keys 0 .. start[b] + i.
//
// Work decomposition.  One workgroup (4 or 8 wavefronts) owns 64 or 128 consecutive positions of one sequence
// and the G query heads of one kv-head group; a wavefront owns 16 of those positions for all G
// heads, i.e. G "query tiles" of 16 rows that share every K and V fragment it reads.  K and V
// travel through LDS in stages of 64 keys (double-buffered, 16-byte units XOR-swizzled by key so
// that fragment reads of 16 keys hit 16 different bank groups).
//
// Everything is computed transposed so that no operand ever has to change layout in registers:
//   S^T = K . Q^T   A = K rows (16 keys x 32 d), B = Q rows       -> C: lane owns query l%16,
//                                                                     keys 4*(l/16) + e
//   O^T = V^T . P^T A = V^T (16 d x 32 keys),    B = P^T           -> C: lane owns query l%16,
//                                                                     d = 4*(l/16) + e
// P^T in the B layout needs, per lane, 8 keys of its own query: exactly what the lane holds after
// two S^T tiles (keys 4g+e of each), if the 32 keys of a block are taken in the order
// k' = 8g + j <-> key 4g + j (j < 4), 16 + 4g + (j - 4) (j >= 4).  V^T fragments in that same key
// order come from row-major V in LDS through the transposing LDS read of gfx950
// (ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of 4 consecutive elements and
// receives element i of each of the 4 rows of 16 elements the group addressed).  The running
// maximum and the rescale factor of a query live in the lanes that own that query in both products.
//
// Softmax: online, log2 domain, fp32; P is rounded to fp16 for the second product (values in
// [0, 1]); the row sum is kept per lane and reduced once at the end.
#include "common.hpp"

#include <type_traits>

namespace axhip {
namespace {

constexpr int kStageKeys = 64;  // keys per LDS stage
constexpr int kXcdCount = 8;
int g_pairs_by_xcd = -1;  // measurement hook: 0 / 1 force the workgroup order, -1 = by pair count
constexpr float kMasked = -1.0e30f;

struct PrefillArgs {
  const __half *q;   // [B, S, Hq, D]
  const __half *k;   // [B, Hkv, rows, D]
  const __half *v;
  const int32_t *start;  // [B] absolute position of query 0 (null: 0)
  __half *out;       // [B, S, Hq, D]
  int S, Hq, Hkv, rows, group;
  float scale_log2e;
  // general form only (GEN): K/V strides in elements, and whether the causal rule applies
  int64_t kv_batch_stride, kv_head_stride, kv_row_stride;
  int causal;
  int pos_blocks, head_groups, n_pairs, pairs_by_xcd;  // launch geometry (filled by launch_prefill)
};

// Up to two query heads per workgroup the kernel is held to 256 registers, so that two workgroups share
// a CU (their 64 KB of LDS each fit): a wavefront's products wait on its own softmax arithmetic, and a
// second wavefront per SIMD fills those gaps (B=1, S=4096: 372 -> 219 us).  Left to itself the
// compiler takes 296 registers.  Sharing every K/V fragment among two tiles of 16 positions per
// wavefront instead (half the LDS reads per product, one workgroup per CU) measured slower.
//
// GEN = false is the cache form: K/V rows of a head are contiguous, the rule is causal and every query's
// position lies inside the cache.  GEN = true takes any row/head/batch stride (token-major K/V), an
// optional causal rule, and queries whose position is past the last key (they see every key).
// WAVES = 4: 64 positions per workgroup, two workgroups per CU (one's prologue and tail overlap the other's
// blocks: best when a launch runs many workgroups per CU one after the other).  WAVES = 8: 128 positions, one
// workgroup per CU, every K/V stage fetched and written to LDS once for eight wavefronts instead of four (best
// when every workgroup has a long row of stages, or the launch is a single round of workgroups).
//
// Measured and not kept: the blocks of a wavefront as a software pipeline - the scores of block n + 1 issued
// before the softmax of block n, K one stage ahead of V in a ring of three LDS stages, matrix and vector
// instructions interleaved by scheduling groups (one basic block per mask variant).  Same results, 2 % slower:
// what bounded this kernel was not the dependency chain inside a wavefront but the fabric - see the workgroup
// order below.
template <int D, int G, bool GEN, int WAVES>
__global__ __launch_bounds__(WAVES * 64, (WAVES == 4 && G <= 2) ? 2 : 1) void prefill_attn_kernel(PrefillArgs a) {
  constexpr int kPThreads = WAVES * 64;
  constexpr int kPosPerWg = WAVES * 16;  // query positions per workgroup (16 per wavefront)
  constexpr int KK = D / 32;   // MFMA steps over d for S^T
  constexpr int DT = D / 16;   // d tiles of O^T
  constexpr int UPR = D / 8;   // 16-byte units per K/V row
  constexpr int VEC = kStageKeys * UPR / kPThreads;  // staging vectors per thread, per tensor
  __shared__ __attribute__((aligned(16))) _Float16 ks[2][kStageKeys * D];
  __shared__ __attribute__((aligned(16))) _Float16 vs[2][kStageKeys * D];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c = lane & 15, g = lane >> 4;
  // Workgroup ids are dealt round-robin to the eight XCDs.  All position blocks of one (sequence, head group) go to
  // the same XCD, one pair after the other, so that the pair's keys and values (re-read by every position block)
  // stay in that XCD's L2 instead of coming over the fabric once per workgroup.
  // (With fewer pairs than would keep eight XCDs busy the position blocks of a pair are spread over all of them.)
  int pair, pb;
  if (a.pairs_by_xcd) {
    const int xcd = blockIdx.x % kXcdCount, slot = blockIdx.x / kXcdCount;
    pair = (slot / a.pos_blocks) * kXcdCount + xcd;
    pb = slot % a.pos_blocks;
  } else {
    pair = blockIdx.x / a.pos_blocks;
    pb = blockIdx.x % a.pos_blocks;
  }
  if (pair >= a.n_pairs) return;
  pb = a.pos_blocks - 1 - pb;  // long rows first
  const int hg = pair % a.head_groups, b = pair / a.head_groups;
  const int h0 = hg * G, hk = h0 / a.group;
  const int start = a.start ? max(a.start[b], 0) : 0;
  const int p0 = pb * kPosPerWg;
  const int pr = p0 + wave * 16 + c;           // this lane's query (as B column), relative position
  int pos = start + pr;                        // its absolute position = last visible key
  int wave_first = start + p0 + wave * 16;     // smallest and largest position of this wavefront
  int wave_last = wave_first + 15;
  int k_end = start + min(p0 + kPosPerWg, a.S);  // keys the workgroup needs: [0, k_end)
  k_end = min(k_end, a.rows);
  if constexpr (GEN) {
    if (!a.causal) {
      pos = wave_first = wave_last = a.rows - 1;
      k_end = a.rows;
    } else {
      pos = min(pos, a.rows - 1);
      wave_first = min(wave_first, a.rows - 1);
    }
  }

  // Q fragments stay in registers for the whole kernel
  half8_t qf[G][KK];
  {
    const int prc = min(pr, a.S - 1);
    const __half *qrow = a.q + ((static_cast<int64_t>(b) * a.S + prc) * a.Hq + h0) * D;
#pragma unroll
    for (int t = 0; t < G; ++t)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        qf[t][kk] = *reinterpret_cast<const half8_t *>(qrow + t * D + kk * 32 + g * 8);
  }

  const int64_t kv_off = GEN ? b * a.kv_batch_stride + hk * a.kv_head_stride
                             : (static_cast<int64_t>(b) * a.Hkv + hk) * a.rows * D;
  const int64_t row_stride = GEN ? a.kv_row_stride : D;
  const __half *kbase = a.k + kv_off;
  const __half *vbase = a.v + kv_off;
  half8_t kst[VEC], vst[VEC];
  // A thread's VEC vectors of a stage: row and 16-byte unit are the same in every stage, so their element
  // offsets and LDS positions are computed once; the stage's first row is the same for the whole workgroup and
  // goes into the scalar base address.  Only a stage that reaches past the cache clamps rows, only a stage
  // that reaches past the last visible key zeroes V rows (both tests are uniform).
  unsigned voff[VEC];
  int lds_o[VEC], vrow[VEC];
#pragma unroll
  for (int p = 0; p < VEC; ++p) {
    const int vi = p * kPThreads + tid;
    const int row = vi / UPR, unit = vi % UPR;
    vrow[p] = row;
    voff[p] = static_cast<unsigned>(row) * static_cast<unsigned>(row_stride) + unit * 8;
    lds_o[p] = row * D + ((unit ^ (row & (UPR - 1))) << 3);
  }
  auto load_stage = [&](int key0) {
    if (key0 + kStageKeys <= a.rows) {
      const __half *kb = kbase + static_cast<int64_t>(key0) * row_stride;
      const __half *vb = vbase + static_cast<int64_t>(key0) * row_stride;
#pragma unroll
      for (int p = 0; p < VEC; ++p) {
        kst[p] = *reinterpret_cast<const half8_t *>(kb + voff[p]);
        vst[p] = *reinterpret_cast<const half8_t *>(vb + voff[p]);
      }
    } else {
#pragma unroll
      for (int p = 0; p < VEC; ++p) {
        const int unit = (p * kPThreads + tid) % UPR;
        const int64_t off = static_cast<int64_t>(min(key0 + vrow[p], a.rows - 1)) * row_stride + unit * 8;
        kst[p] = *reinterpret_cast<const half8_t *>(kbase + off);
        vst[p] = *reinterpret_cast<const half8_t *>(vbase + off);
      }
    }
  };
  // V rows past the last key any query of this workgroup may see are stored as zeros: their
  // probabilities are zero, but 0 * (whatever bits the unwritten cache holds) must stay 0
  auto store_stage = [&](int buf, int key0) {
    if (key0 + kStageKeys <= k_end) {
#pragma unroll
      for (int p = 0; p < VEC; ++p) {
        *reinterpret_cast<half8_t *>(&ks[buf][lds_o[p]]) = kst[p];
        *reinterpret_cast<half8_t *>(&vs[buf][lds_o[p]]) = vst[p];
      }
    } else {
#pragma unroll
      for (int p = 0; p < VEC; ++p) {
        *reinterpret_cast<half8_t *>(&ks[buf][lds_o[p]]) = kst[p];
        half8_t vv = vst[p];
        if (key0 + vrow[p] >= k_end) vv = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        *reinterpret_cast<half8_t *>(&vs[buf][lds_o[p]]) = vv;
      }
    }
  };

  float4_t o[G][DT];
  // the row sums of the probabilities are a product too: a V^T fragment of ones gives, in every output row,
  // the sum over the block's keys of the (fp16-rounded) probabilities of the lane's query - one matrix
  // instruction per block and tile instead of eight additions, and no reduction across lanes at the end
  float m[G];
  float4_t lsum[G];
#pragma unroll
  for (int t = 0; t < G; ++t) {
    m[t] = kMasked;
    lsum[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[t][dt] = float4_t{0.f, 0.f, 0.f, 0.f};
  }

  const int n_stages = (k_end + kStageKeys - 1) / kStageKeys;
  const half8_t ones = {1, 1, 1, 1, 1, 1, 1, 1};

  // ---- the three parts of a block of 32 keys for this wavefront ---------------------------------------------
  // scores S^T = K . Q^T of the 32 keys at rows `row0` of the K stage `kst_l`
  auto scores = [&](const _Float16 *kst_l, float4_t (&sc)[G][2]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < G; ++t) sc[t][0] = sc[t][1] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tk = 0; tk < 2; ++tk)
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const int row = tk * 16 + c, unit = kk * 4 + g;  // row & 15 == c
        const half8_t kf = lds_h8(kst_l + row * D + ((unit ^ (c & (UPR - 1))) << 3));
#pragma unroll
        for (int t = 0; t < G; ++t)
          sc[t][tk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[t][kk], sc[t][tk], 0, 0, 0);
      }
  };
  // mask + online softmax of a block's scores -> probabilities in the B layout of the second product.
  // DIAG: some key of the block may lie behind a query of the wavefront (the block touches the diagonal, or the
  // end of the cache); every other block skips the masks, which are a third of the softmax instructions.  The
  // scale is folded into the exponent's argument: p = exp2(s * scale - m) with m the running maximum of s * scale.
  auto softmax = [&](const float4_t (&sc)[G][2], int kb, half8_t (&pf)[G], auto diag_c) __attribute__((always_inline)) {
    constexpr bool DIAG = decltype(diag_c)::value;
    bool moved[G];
    float mnew[G];
#pragma unroll
    for (int t = 0; t < G; ++t) {
      float x[8];
#pragma unroll
      for (int tk = 0; tk < 2; ++tk)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = sc[t][tk][e];
          if constexpr (DIAG) {
            const int key = kb + tk * 16 + 4 * g + e;
            if (key > pos) v = kMasked;
          }
          x[tk * 4 + e] = v;
        }
      float mx = x[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) mx = fmaxf(mx, x[j]);
      mx = max_xor32(max_xor16(mx));
      // masked scores are -1e30 before the (positive) scale: they stay far below every real score.
      // The running maximum moves only when a block exceeds it by more than 8 (a factor 256): until then
      // the exponents stay <= 8, p <= 256 keeps its 11 bits in fp16 whatever its magnitude, and the block
      // rescales nothing - with a maximum that follows every block, most blocks of a row's first few
      // hundred keys pay 4 DT multiplications per query tile.  (A maximum that lags makes every p larger, never
      // smaller: nothing that the exact maximum would keep is flushed.)
      const float mxs = mx * a.scale_log2e;
      moved[t] = __any(mxs > m[t] + 8.0f);
      const float mn = moved[t] ? fmaxf(m[t], mxs) : m[t];
      mnew[t] = mn;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(x[j], a.scale_log2e, -mn));
        if constexpr (DIAG) {
          // a fully masked row keeps m == kMasked * scale: exp2(0) would count
          if (x[j] <= kMasked) p = 0.f;
        }
        pf[t][j] = static_cast<_Float16>(p);
      }
    }
    // the rescaling, where the maximum moved (rare after a row's first blocks), after all the straight-line work
#pragma unroll
    for (int t = 0; t < G; ++t) {
      if (moved[t]) {
        const float corr = __builtin_amdgcn_exp2f(m[t] - mnew[t]);
        lsum[t] *= corr;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[t][dt] *= corr;
        m[t] = mnew[t];
      }
    }
  };
  // row sums (a product with ones) and O^T += V^T . P^T over the 32 keys at `vst_l`
  auto accumulate = [&](const _Float16 *vst_l, const half8_t (&pf)[G]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < G; ++t) lsum[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pf[t], lsum[t], 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const half4_t lo = lds_v_tr<D>(vst_l, 4 * g, dt * 16, c);
      const half4_t hi = lds_v_tr<D>(vst_l, 16 + 4 * g, dt * 16, c);
      const half8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int t = 0; t < G; ++t)
        o[t][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[t], o[t][dt], 0, 0, 0);
    }
  };

  load_stage(0);
  store_stage(0, 0);
  __syncthreads();

  auto block = [&](int buf, int sub, int kb, auto diag_c) __attribute__((always_inline)) {
    float4_t sc[G][2];
    half8_t pf[G];
    scores(&ks[buf][sub * 32 * D], sc);
    softmax(sc, kb, pf, diag_c);
    accumulate(&vs[buf][sub * 32 * D], pf);
  };

  for (int s = 0; s < n_stages; ++s) {
    const int buf = s & 1;
    const int nxt = min(s + 1, n_stages - 1);  // the last stage fetches itself again: no branch
    load_stage(nxt * kStageKeys);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sub = 0; sub < kStageKeys / 32; ++sub) {
      const int kb = s * kStageKeys + sub * 32;      // first key of this block of 32
      if (kb <= wave_last && kb < k_end) {           // wave-uniform: otherwise every key is masked
        if (kb + 31 > wave_first)                    // wave-uniform too
          block(buf, sub, kb, std::true_type{});
        else
          block(buf, sub, kb, std::false_type{});
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    store_stage(buf ^ 1, nxt * kStageKeys);
    __syncthreads();
  }

  if (pr >= a.S) return;
  __half *orow = a.out + ((static_cast<int64_t>(b) * a.S + pr) * a.Hq + h0) * D;
#pragma unroll
  for (int t = 0; t < G; ++t) {
    const float l = lsum[t][0];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      half4_t h;
#pragma unroll
      for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(o[t][dt][e] * inv);
      *reinterpret_cast<half4_t *>(reinterpret_cast<_Float16 *>(orow) + t * D + dt * 16 + 4 * g) = h;
    }
  }
}

template <int D, bool GEN>
int launch_prefill(const PrefillArgs &a_in, int B, int G, hipStream_t st) {
  const PrefillArgs &a0 = a_in;
  // eight wavefronts per workgroup where every workgroup has all keys to go through (no causal rule), or where
  // the launch is one round of workgroups anyway; G = 4 keeps four (its registers leave no room for eight)
  const int64_t wgs8 = static_cast<int64_t>((a0.S + 127) / 128) * (a0.Hq / G) * B;
  const bool eight = G <= 2 && ((GEN && !a0.causal) || wgs8 <= device_cu_count());
  const int pos = eight ? 128 : 64;
  PrefillArgs a = a_in;
  a.pos_blocks = (a.S + pos - 1) / pos;
  a.head_groups = a.Hq / G;
  a.n_pairs = a.head_groups * B;
  // a pair per XCD at a time needs enough pairs to go round: whole rounds of eight, or so many that a short last
  // round does not matter
  a.pairs_by_xcd = (a.n_pairs % kXcdCount == 0 || a.n_pairs >= 4 * kXcdCount) ? 1 : 0;
  if (g_pairs_by_xcd >= 0) a.pairs_by_xcd = g_pairs_by_xcd;  // measurement hook
  const int64_t wgs = a.pairs_by_xcd ? static_cast<int64_t>((a.n_pairs + kXcdCount - 1) / kXcdCount * kXcdCount) * a.pos_blocks
                                     : static_cast<int64_t>(a.n_pairs) * a.pos_blocks;
  if (wgs > INT32_MAX) return AXHIP_INVALID_ARGUMENT;
  const dim3 grid(static_cast<unsigned>(wgs));
  if (eight) {
    if (G == 2) hipLaunchKernelGGL((prefill_attn_kernel<D, 2, GEN, 8>), grid, dim3(512), 0, st, a);
    else hipLaunchKernelGGL((prefill_attn_kernel<D, 1, GEN, 8>), grid, dim3(512), 0, st, a);
    return launch_status();
  }
  switch (G) {
    case 4: hipLaunchKernelGGL((prefill_attn_kernel<D, 4, GEN, 4>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((prefill_attn_kernel<D, 2, GEN, 4>), grid, dim3(256), 0, st, a); break;
    default: hipLaunchKernelGGL((prefill_attn_kernel<D, 1, GEN, 4>), grid, dim3(256), 0, st, a); break;
  }
  return launch_status();
}

}  // namespace
}  // namespace axhip

using namespace axhip;

extern "C" {

// Measurement hook: the order in which workgroups are handed to the XCDs (see the kernel).
AXHIP_API void axhip_prefill_attention_tune(int pairs_by_xcd) { g_pairs_by_xcd = pairs_by_xcd < 0 ? -1 : (pairs_by_xcd ? 1 : 0); }

AXHIP_API int axhip_prefill_attention(const void *q, const void *k_cache, const void *v_cache,
                                      const int32_t *start, void *out, int dtype, int B, int S, int Hq,
                                      int Hkv, int D, int cache_rows, axhip_stream stream) {
  if (dtype != AXHIP_FLOAT16) return AXHIP_UNSUPPORTED_TYPE;
  if (B < 0 || S < 0 || Hq <= 0 || Hkv <= 0 || cache_rows <= 0) return AXHIP_INVALID_ARGUMENT;
  if (Hq % Hkv != 0) return AXHIP_SHAPE_MISMATCH;
  if (D != 64 && D != 128) return AXHIP_INVALID_ARGUMENT;
  if (B == 0 || S == 0) return AXHIP_OK;
  if (B > 65535 || Hq > 65535) return AXHIP_INVALID_ARGUMENT;
  if (!q || !k_cache || !v_cache || !out) return AXHIP_INVALID_PTR;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache) |
       reinterpret_cast<uintptr_t>(out)) & 15)
    return AXHIP_INVALID_PTR;
  const int group = Hq / Hkv;
  const int G = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
  PrefillArgs a;
  a.q = static_cast<const __half *>(q);
  a.k = static_cast<const __half *>(k_cache);
  a.v = static_cast<const __half *>(v_cache);
  a.start = start;
  a.out = static_cast<__half *>(out);
  a.S = S;
  a.Hq = Hq;
  a.Hkv = Hkv;
  a.rows = cache_rows;
  a.group = group;
  a.scale_log2e = 1.4426950408889634f / sqrtf(static_cast<float>(D));
  hipStream_t st = as_stream(stream);
  a.kv_batch_stride = a.kv_head_stride = a.kv_row_stride = 0;
  a.causal = 1;
  return D == 128 ? launch_prefill<128, false>(a, B, G, st) : launch_prefill<64, false>(a, B, G, st);
}

// Attention of q [Sq,Hq,D] over token-major k/v [Skv,Hkv,D] (fp16, D 64 or 128, 16-byte aligned) on
// the matrix cores; row t sees min(t+1, Skv) keys under the causal rule, all Skv otherwise.  The caller
// has checked shapes and pointers.
int axhip_internal_sdpa_f16_mfma(const void *q, const void *k, const void *v, void *out, int Sq, int Hq,
                                 int Hkv, int D, int Skv, int is_causal, hipStream_t st) {
  const int group = Hq / Hkv;
  const int G = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
  PrefillArgs a;
  a.q = static_cast<const __half *>(q);
  a.k = static_cast<const __half *>(k);
  a.v = static_cast<const __half *>(v);
  a.start = nullptr;
  a.out = static_cast<__half *>(out);
  a.S = Sq;
  a.Hq = Hq;
  a.Hkv = Hkv;
  a.rows = Skv;
  a.group = group;
  a.scale_log2e = 1.4426950408889634f / sqrtf(static_cast<float>(D));
  a.kv_batch_stride = 0;
  a.kv_head_stride = D;
  a.kv_row_stride = static_cast<int64_t>(Hkv) * D;
  a.causal = is_causal;
  return D == 128 ? launch_prefill<128, true>(a, 1, G, st) : launch_prefill<64, true>(a, 1, G, st);
}

}  // extern "C"
