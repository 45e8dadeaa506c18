/*
 * CPU oracle for the Axono LLM decode path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It restates, in plain C, the fp32 arithmetic of the
 * reference's CPU operators so that the HIP kernels can be checked against it.  Only the test
 * suite, the smoke check and the benchmark's CPU-baseline leg may load it; the shipped library
 * never links, imports or calls anything in this directory.
 *
 * Every function names the reference lines it follows.  Loop order and evaluation order are
 * kept where they decide the last bit: sequential fp32 accumulation, `acc * scale` after the
 * dot product, `1/sqrt(sum/H + eps)`, `(y * rms) * w`, `g / (1 + exp(-g)) * up`.
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   sdpa / gqa        NumPy closed forms the reference's own tests use (tests/core/test_gqa.py:11-25,
 *                     tests/core/test_sequence_ops.py:31-46) on their seeds, fp64 brute force,
 *                     L=1 => out=v, uniform K => mean(V); bit-compared with the compiled
 *                     reference (oracle/_ref) where that is built.
 *   add_rms_norm      tests/core/test_fused.py:43-78 seeds + chaining identity.
 *   silu_mul          tests/core/test_fused.py:19-39 seeds + edge vector.
 *   rope              tests/core/test_sequence_ops.py:62-79 closed form; pos=0 identity; pair norms.
 *   mrope_cos_sin     tests/core/test_sequence_ops.py:252-275 closed form (default_rng(7)).
 *   rope_thd, rope_with_cos_sin
 *                     no reference test exists; pinned by rope_thd == rope when T=H=W,
 *                     rope_thd == rope_with_cos_sin(mrope_cos_sin), and by oracle/_ref.
 *   rms_norm          closed form, equals add_rms_norm with zero residual.
 *   linear            x @ W^T + b against fp64 NumPy.
 *   concat/embedding/argmax  NumPy equivalents (byte equality).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define AXO_API __attribute__((visibility("default")))

/* Status values of the reference (include/axono/core/types.h:54-64). */
enum {
  AXO_OK = 0,
  AXO_INVALID_ARGUMENT = 1,
  AXO_OUT_OF_MEMORY = 2,
  AXO_UNSUPPORTED_TYPE = 3,
  AXO_SHAPE_MISMATCH = 4,
};

AXO_API int axo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------------------------------------
 * Attention.  Follows src/ops/cpu/sequence.cpp:236-301 (ScaledDotProductAttention), which is what
 * gqa_decode_attention is defined to equal (axono/python/axono/gqa.py:31).
 * q (sq,hq,d)  k,v (skv,hkv,d)  out (sq,hq,d); row strides are given explicitly so that the same
 * routine serves the reference layout [L,Hkv,D] (k_row_stride = hkv*d, k_head_stride = d) and the
 * batched cache layout [B,Hkv,Lmax,D] (k_row_stride = d, k_head_stride = Lmax*d) of one sequence.
 * ------------------------------------------------------------------------------------------- */
AXO_API int axo_sdpa_strided(const float *q, const float *k, const float *v, float *out,
                             int64_t sq, int64_t hq, int64_t hkv, int64_t d, int64_t skv,
                             int64_t k_row_stride, int64_t k_head_stride, int is_causal) {
  if (hkv <= 0 || hq % hkv != 0) return AXO_SHAPE_MISMATCH;
  if (skv <= 0) return AXO_INVALID_ARGUMENT;
  const int64_t group = hq / hkv;
  const float scale = 1.0f / sqrtf((float)d);
  int failed = 0;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t t = 0; t < sq; ++t) {
    for (int64_t h = 0; h < hq; ++h) {
      const float *qrow = q + (t * hq + h) * d;
      float *orow = out + (t * hq + h) * d;
      const int64_t hk = h / group;
      int64_t visible = skv;
      if (is_causal && skv >= t + 1) visible = t + 1;
      float *w = (float *)malloc((size_t)visible * sizeof(float));
      if (!w) {
        failed = 1;
        continue;
      }
      const float *kbase = k + hk * k_head_stride;
      const float *vbase = v + hk * k_head_stride;
      for (int64_t s = 0; s < visible; ++s) {
        const float *krow = kbase + s * k_row_stride;
        float dot = 0.0f;
        for (int64_t i = 0; i < d; ++i) dot += qrow[i] * krow[i];
        w[s] = dot * scale;
      }
      float top = w[0];
      for (int64_t s = 1; s < visible; ++s)
        if (w[s] > top) top = w[s];
      float denom = 0.0f;
      for (int64_t s = 0; s < visible; ++s) {
        w[s] = expf(w[s] - top);
        denom += w[s];
      }
      const float inv = 1.0f / denom;
      for (int64_t i = 0; i < d; ++i) orow[i] = 0.0f;
      for (int64_t s = 0; s < visible; ++s) {
        const float p = w[s] * inv;
        const float *vrow = vbase + s * k_row_stride;
        for (int64_t i = 0; i < d; ++i) orow[i] += p * vrow[i];
      }
      free(w);
    }
  }
  return failed ? AXO_OUT_OF_MEMORY : AXO_OK;
}

/* Reference layout entry: k,v (skv,hkv,d).  sequence.cpp:236-301. */
AXO_API int axo_sdpa(const float *q, const float *k, const float *v, float *out, int64_t sq,
                     int64_t hq, int64_t hkv, int64_t d, int64_t skv, int is_causal) {
  return axo_sdpa_strided(q, k, v, out, sq, hq, hkv, d, skv, hkv * d, d, is_causal);
}

/* Batched decode over a [B,Hkv,Lmax,D] cache: the reference op applied to each sequence b with
 * its own length seq_lens[b] (one query token).  A sequence of length 0 yields zeros: the
 * reference cannot express that case, the value is this build's convention. */
AXO_API int axo_gqa_decode_cache(const float *q, const float *kc, const float *vc,
                                 const int32_t *seq_lens, float *out, int64_t B, int64_t hq,
                                 int64_t hkv, int64_t d, int64_t lmax) {
  for (int64_t b = 0; b < B; ++b) {
    const int64_t L = seq_lens ? seq_lens[b] : lmax;
    float *ob = out + b * hq * d;
    if (L <= 0) {
      memset(ob, 0, (size_t)(hq * d) * sizeof(float));
      continue;
    }
    if (L > lmax) return AXO_INVALID_ARGUMENT;
    int st = axo_sdpa_strided(q + b * hq * d, kc + b * hkv * lmax * d, vc + b * hkv * lmax * d, ob,
                              1, hq, hkv, d, L, d, lmax * d, 0);
    if (st != AXO_OK) return st;
  }
  return AXO_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Fused ops.  src/ops/cpu/fused.cpp:16-35 (SiluMul) and :37-76 (AddRmsNorm).
 * ------------------------------------------------------------------------------------------- */
AXO_API int axo_silu_mul(const float *gate, const float *up, float *y, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const float g = gate[i];
    y[i] = g / (1.0f + expf(-g)) * up[i];
  }
  return AXO_OK;
}

AXO_API int axo_add_rms_norm(const float *x, const float *res, const float *w, float eps,
                             float *y, float *out, int64_t rows, int64_t hidden) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t o = r * hidden;
    float ss = 0.0f;
    for (int64_t i = 0; i < hidden; ++i) {
      const float s = x[o + i] + res[o + i];
      y[o + i] = s;
      ss += s * s;
    }
    const float rms = 1.0f / sqrtf(ss / (float)hidden + eps);
    for (int64_t i = 0; i < hidden; ++i) out[o + i] = y[o + i] * rms * w[i];
  }
  return AXO_OK;
}

/* RmsNorm.  src/ops/cpu/llm.cpp:58-73 (NormRows, rms branch) and :240-264.  w may be NULL. */
AXO_API int axo_rms_norm(const float *x, const float *w, float eps, float *out, int64_t rows,
                         int64_t cols) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float *orow = out + r * cols;
    float ss = 0.0f;
    for (int64_t c = 0; c < cols; ++c) ss += xr[c] * xr[c];
    const float inv = 1.0f / sqrtf(ss / (float)cols + eps);
    for (int64_t c = 0; c < cols; ++c) {
      const float nv = xr[c] * inv;
      orow[c] = w ? nv * w[c] : nv;
    }
  }
  return AXO_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Rotary embeddings.  x (rows,heads,dim), rotate-half pairing (i, i+dim/2).
 * ------------------------------------------------------------------------------------------- */

/* Rope: src/ops/cpu/sequence.cpp:54-93.  freq = powf(theta, -2*i/dim), angle = float(pos)*freq,
 * all in fp32. */
AXO_API int axo_rope(const float *x, const int64_t *pos, float theta, float *out, int64_t rows,
                     int64_t heads, int64_t dim) {
  if (dim % 2) return AXO_INVALID_ARGUMENT;
  const int64_t half = dim / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t h = 0; h < heads; ++h) {
      const float *src = x + (r * heads + h) * dim;
      float *dst = out + (r * heads + h) * dim;
      const float p = (float)pos[r];
      for (int64_t i = 0; i < half; ++i) {
        const float freq = powf(theta, -2.0f * (float)i / (float)dim);
        const float ang = p * freq;
        const float c = cosf(ang), s = sinf(ang);
        const float a = src[i], b = src[i + half];
        dst[i] = a * c - b * s;
        dst[i + half] = b * c + a * s;
      }
    }
  }
  return AXO_OK;
}

/* The frequency table Rope uses, exposed so the device entry point can be fed the very same
 * fp32 values (sequence.cpp:80-81). */
AXO_API void axo_rope_inv_freq(float theta, int64_t dim, float *freq_out) {
  for (int64_t i = 0; i < dim / 2; ++i) freq_out[i] = powf(theta, -2.0f * (float)i / (float)dim);
}

/* RopeWithCosSin: sequence.cpp:96-135.  cos,sin (rows,dim); the second half of the pair uses the
 * second half of the table. */
AXO_API int axo_rope_with_cos_sin(const float *x, const float *cs, const float *sn, float *out,
                                  int64_t rows, int64_t heads, int64_t dim) {
  if (dim % 2) return AXO_INVALID_ARGUMENT;
  const int64_t half = dim / 2;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t h = 0; h < heads; ++h) {
      const float *src = x + (r * heads + h) * dim;
      float *dst = out + (r * heads + h) * dim;
      const float *cr = cs + r * dim;
      const float *sr = sn + r * dim;
      for (int64_t i = 0; i < half; ++i) {
        const float a = src[i], b = src[i + half];
        dst[i] = a * cr[i] - b * sr[i];
        dst[i + half] = b * cr[i + half] + a * sr[i + half];
      }
    }
  }
  return AXO_OK;
}

/* Angle selection shared by MropeCosSin and RopeThd (sequence.cpp:166-171, 219-225): channel i
 * takes the T position unless i%3==1 and i<3*h_sec (H) or i%3==2 and i<3*w_sec (W). */
static inline float mrope_angle(float pt, float ph, float pw, float f, int64_t i, int64_t h_lim,
                                int64_t w_lim) {
  float angle = pt * f;
  if (i % 3 == 1 && i < h_lim)
    angle = ph * f;
  else if (i % 3 == 2 && i < w_lim)
    angle = pw * f;
  return angle;
}

/* MropeCosSin: sequence.cpp:140-182.  pos (3,rows) int64; tables (rows, 2*half), halves equal. */
AXO_API int axo_mrope_cos_sin(const int64_t *pos, const float *inv_freq, int h_sec, int w_sec,
                              float *cos_out, float *sin_out, int64_t rows, int64_t half) {
  if (half <= 0) return AXO_INVALID_ARGUMENT;
  const int64_t h_lim = (int64_t)h_sec * 3, w_lim = (int64_t)w_sec * 3;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float pt = (float)pos[r], ph = (float)pos[rows + r], pw = (float)pos[2 * rows + r];
    float *cr = cos_out + r * 2 * half;
    float *sr = sin_out + r * 2 * half;
    for (int64_t i = 0; i < half; ++i) {
      const float ang = mrope_angle(pt, ph, pw, inv_freq[i], i, h_lim, w_lim);
      const float c = cosf(ang), s = sinf(ang);
      cr[i] = c;
      cr[i + half] = c;
      sr[i] = s;
      sr[i + half] = s;
    }
  }
  return AXO_OK;
}

/* RopeThd: sequence.cpp:184-234.  t_sec is accepted and ignored, as there (:201). */
AXO_API int axo_rope_thd(const float *x, const int64_t *pos, const float *inv_freq, int t_sec,
                         int h_sec, int w_sec, float *out, int64_t rows, int64_t heads,
                         int64_t dim) {
  (void)t_sec;
  if (dim % 2) return AXO_INVALID_ARGUMENT;
  const int64_t half = dim / 2;
  const int64_t h_lim = (int64_t)h_sec * 3, w_lim = (int64_t)w_sec * 3;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t h = 0; h < heads; ++h) {
      const float *src = x + (r * heads + h) * dim;
      float *dst = out + (r * heads + h) * dim;
      const float pt = (float)pos[r], ph = (float)pos[rows + r], pw = (float)pos[2 * rows + r];
      for (int64_t i = 0; i < half; ++i) {
        const float ang = mrope_angle(pt, ph, pw, inv_freq[i], i, h_lim, w_lim);
        const float c = cosf(ang), s = sinf(ang);
        const float a = src[i], b = src[i + half];
        dst[i] = a * c - b * s;
        dst[i + half] = b * c + a * s;
      }
    }
  }
  return AXO_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Linear: out = x @ W^T (+ bias).  src/ops/cpu/linear.cpp:95-110 (the non-BLAS branch, which is
 * what a build without CBLAS runs).  x (rows,k)  w (out_f,k)  bias (out_f) or NULL.
 * ------------------------------------------------------------------------------------------- */
AXO_API int axo_linear(const float *x, const float *w, const float *bias, float *out,
                       int64_t rows, int64_t k, int64_t out_f) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t i = 0; i < rows; ++i) {
    for (int64_t j = 0; j < out_f; ++j) {
      float acc = 0.0f;
      for (int64_t p = 0; p < k; ++p) acc += x[i * k + p] * w[j * k + p];
      if (bias) acc += bias[j];
      out[i * out_f + j] = acc;
    }
  }
  return AXO_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Byte movers and index ops.
 * ------------------------------------------------------------------------------------------- */

/* Concat along an axis: sequence.cpp:303-338.  `outer` = product of dims before the axis;
 * a_bytes / b_bytes = bytes of one outer block of a and b.  KV append is axis 0 (outer = 1). */
AXO_API int axo_concat(const void *a, const void *b, void *out, int64_t outer, int64_t a_bytes,
                       int64_t b_bytes) {
  const char *ap = (const char *)a, *bp = (const char *)b;
  char *dst = (char *)out;
  for (int64_t o = 0; o < outer; ++o) {
    memcpy(dst, ap + o * a_bytes, (size_t)a_bytes);
    dst += a_bytes;
    memcpy(dst, bp + o * b_bytes, (size_t)b_bytes);
    dst += b_bytes;
  }
  return AXO_OK;
}

/* Scatter-append into a static [B,Hkv,Lmax,D] cache: cache[b,h,pos[b],:] = new[b,h,:].  Equals
 * the reference's concat-append (nn/kv_cache.py:96-102) when pos[b] is the current length. */
AXO_API int axo_kv_append(const void *k_new, const void *v_new, void *k_cache, void *v_cache,
                          const int64_t *pos, int64_t B, int64_t hkv, int64_t lmax,
                          int64_t row_bytes) {
  for (int64_t b = 0; b < B; ++b) {
    if (pos[b] < 0 || pos[b] >= lmax) return AXO_INVALID_ARGUMENT;
    for (int64_t h = 0; h < hkv; ++h) {
      const int64_t src = (b * hkv + h) * row_bytes;
      const int64_t dst = ((b * hkv + h) * lmax + pos[b]) * row_bytes;
      memcpy((char *)k_cache + dst, (const char *)k_new + src, (size_t)row_bytes);
      memcpy((char *)v_cache + dst, (const char *)v_new + src, (size_t)row_bytes);
    }
  }
  return AXO_OK;
}

/* Embedding gather: sequence.cpp:18-52. */
AXO_API int axo_embedding(const int64_t *ids, const float *table, float *out, int64_t n,
                          int64_t hidden) {
  for (int64_t i = 0; i < n; ++i)
    memcpy(out + i * hidden, table + ids[i] * hidden, (size_t)hidden * sizeof(float));
  return AXO_OK;
}

/* Argmax over the last dim, first maximum wins: sequence.cpp:372-384. */
AXO_API int axo_argmax(const float *x, int64_t *out, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *row = x + r * cols;
    int64_t best = 0;
    for (int64_t c = 1; c < cols; ++c)
      if (row[c] > row[best]) best = c;
    out[r] = best;
  }
  return AXO_OK;
}

/* Elementwise add (the final residual of a decoder layer, examples/vlm/qwen3vl/model.py:435). */
AXO_API int axo_add(const float *a, const float *b, float *out, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
  return AXO_OK;
}
