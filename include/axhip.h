/*
 * axhip.h — C ABI of libaxhip.so: the LLM decode path of Axono as hand-written gfx950 kernels,
 * plus the small device runtime (caching allocator, current stream, hipGraph capture) that path
 * needs.  Plain pointers and sizes only; every operator takes the HIP stream it must run on.
 *
 * Conventions (they mirror the reference's operator layer, whose functions have the form
 * `Status Op(const Context&, const Tensor&..., Tensor& result)`, include/axono/ops/cuda/ headers):
 *   - every function returns an `axhip_status`; its values are the reference's `core::Status`
 *     (include/axono/core/types.h:54-64), so a binding can forward the int unchanged;
 *   - `dtype` arguments use the reference's `core::DataType` numbering (types.h:18-27);
 *   - buffers are caller-owned device memory, contiguous row-major unless strides are passed;
 *   - nothing synchronises: work is enqueued on `stream` (NULL = the legacy default stream) and
 *     is safe to record into a hipGraph (no allocation, no host<->device copy, no memset node).
 */
#ifndef AXHIP_H_
#define AXHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXHIP_API __attribute__((visibility("default")))

/* core::Status, include/axono/core/types.h:54-64 */
typedef enum {
  AXHIP_OK = 0,
  AXHIP_INVALID_ARGUMENT = 1,
  AXHIP_OUT_OF_MEMORY = 2,
  AXHIP_UNSUPPORTED_TYPE = 3,
  AXHIP_SHAPE_MISMATCH = 4,
  AXHIP_INTERNAL_ERROR = 5,
  AXHIP_DEVICE_ERROR = 6,
  AXHIP_INVALID_PTR = 7,
  AXHIP_DEVICE_MISMATCH = 8
} axhip_status;

/* core::DataType, include/axono/core/types.h:18-27 */
typedef enum {
  AXHIP_INT8 = 0,
  AXHIP_INT16 = 1,
  AXHIP_INT32 = 2,
  AXHIP_INT64 = 3,
  AXHIP_FLOAT16 = 4,
  AXHIP_FLOAT32 = 5,
  AXHIP_FLOAT64 = 6,
  AXHIP_BOOLEAN = 7
} axhip_dtype;

typedef void *axhip_stream; /* a hipStream_t */

/* ============================================================================================
 * Device runtime
 * ========================================================================================== */

/* Library version string, "0.2.0-hip" (the reference module reports "0.2.0",
 * axono/python/src/nanobind_module.cpp:1327). */
AXHIP_API const char *axhip_version(void);

/* Number of HIP devices; the `hip:<id>` device of the Python surface maps to these ids.
 * Replaces cuda_available(), nanobind_module.cpp:1211-1217. */
AXHIP_API int axhip_device_count(int *count);
AXHIP_API int axhip_set_device(int device_id);
/* Device name and whether it is the gfx950 target the kernels are built for. */
AXHIP_API int axhip_device_info(int device_id, char *name, size_t name_len, int *is_gfx950,
                                size_t *total_bytes, int *compute_units);

/* Caching allocator.  Replaces cuda::detail::CudaAllocateStorage / ReturnToCache,
 * src/core/cuda/detail.cu:93-289.  Exact-size free lists; released blocks stay cached up to the
 * budget (default: half of the device's memory, where the reference used 2 GiB) and are evicted
 * oldest first.  `zero` != 0 zero-fills the block on the current stream, as the reference does
 * for every tensor it creates (detail.cu:221-222,246); kernels that overwrite their whole output
 * pass 0 and skip that write.  While a capture-pool recording or a graph capture is active the
 * call follows the capture pool instead (see axhip_capture_pool_*). */
AXHIP_API int axhip_alloc(size_t bytes, int zero, void **out);
AXHIP_API int axhip_free(void *ptr);
/* Whether a live block belongs to the capture pool or to a captured graph (then axhip_free on it
 * is a no-op and the block is released by axhip_capture_pool_reset / axhip_graph_destroy; a holder
 * must not free it after that).  The reference expresses the same with a no-op deleter,
 * detail.cu:196-199,262-264. */
AXHIP_API int axhip_block_is_capture_owned(const void *ptr, int *owned);
/* cached_bytes() / set_cache_budget(bytes), nanobind_module.cpp:398-400 */
AXHIP_API size_t axhip_cached_bytes(void);
AXHIP_API int axhip_set_cache_budget(size_t bytes);
AXHIP_API size_t axhip_cache_budget(void);
/* Frees every cached block (ClearDeviceCache, detail.cu:106-122). */
AXHIP_API int axhip_empty_cache(void);
/* Bytes currently handed out (diagnostic; no reference counterpart). */
AXHIP_API size_t axhip_allocated_bytes(void);

/* Copies.  Host<->device copies are synchronous with respect to the current stream, like the
 * reference's blocking cudaMemcpy (src/core/cuda/detail.cu:314-350, tensor.cpp:186-215), and are
 * refused with AXHIP_INVALID_ARGUMENT while the calling thread is capturing a graph.
 * Device-to-device copies and fills are kernels on the current stream (capturable). */
AXHIP_API int axhip_memcpy_h2d(void *dst, const void *src, size_t bytes);
AXHIP_API int axhip_memcpy_d2h(void *dst, const void *src, size_t bytes);
AXHIP_API int axhip_memcpy_d2d(void *dst, const void *src, size_t bytes);
AXHIP_API int axhip_fill_zero(void *dst, size_t bytes);

/* The stream operators should be given: the calling thread's capture stream while it captures,
 * else the legacy default stream.  Replaces cuda::AxonoCurrentStream, src/core/cuda/graph.cu:58-60. */
AXHIP_API axhip_stream axhip_current_stream(void);

/* Kernels that finish through static ticket counters (axhip_gqa_decode[_qkv] when it merges key
 * ranges in the kernel, axhip_argmax over wide rows) take the counters of the calling thread's
 * ticket lane, 0 .. AXHIP_TICKET_LANES-1 (default 0); a captured launch keeps the lane it was captured
 * under.  Launches of these kernels that overlap in time on one device must come from different lanes.
 * A lane holds 65536 (sequence, head group) slots for attention and 1024 rows for argmax.  No
 * reference counterpart (the reference merges in a second kernel, gqa.cu:95-129). */
#define AXHIP_TICKET_LANES 8
AXHIP_API int axhip_set_ticket_lane(int lane);
AXHIP_API int axhip_ticket_lane(void);
/* Puts every ticket counter of the current device back to zero.  The counters are self-resetting (the
 * workgroup that takes the last ticket clears it), so this is only needed for recovery: a launch that
 * ended abnormally (a device error reported by a later call) can leave counters non-zero, and every later
 * launch of the same slot would then merge early or never.  Synchronises the device; refused with
 * AXHIP_INVALID_ARGUMENT while the calling thread captures a graph; call it while no attention / argmax
 * launch is in flight on any thread (counters of a launch in flight would be zeroed under it).  No other
 * call resets the counters implicitly.  No reference counterpart. */
AXHIP_API int axhip_reset_tickets(void);
/* 1 while the calling thread is between axhip_graph_begin_capture and end/abort
 * (cuda::IsCapturing, include/axono/core/cuda/capture.h:19-33). */
AXHIP_API int axhip_is_capturing(void);
/* Waits for the current stream (no-op error while capturing). */
AXHIP_API int axhip_synchronize(void);

/* hipGraph capture.  Replaces BeginGraphCapture / EndGraphCapture / AbortGraphCapture and
 * CudaGraphExec::{Finalize,Replay,Sync,Reset}, src/core/cuda/graph.cu:79-215, and the binding's
 * CUDAGraph class, nanobind_module.cpp:1226-1324.
 *   begin    creates a non-blocking capture stream, starts a thread-local capture on it and
 *            makes it the thread's current stream;
 *   end      ends the capture, rejects an empty graph (AXHIP_INVALID_ARGUMENT), instantiates it
 *            and returns the executable graph and its node count;
 *   abort    ends and discards a capture after a failure inside the captured body;
 *   launch   enqueues one replay on the graph's stream (no wait); `sync` waits for it.
 *            The reference's replay() is launch + sync. */
typedef void *axhip_graph; /* opaque executable graph */
AXHIP_API int axhip_graph_begin_capture(axhip_stream *stream_out);
AXHIP_API int axhip_graph_end_capture(axhip_stream stream, axhip_graph *graph_out,
                                      size_t *num_nodes_out);
AXHIP_API int axhip_graph_abort_capture(axhip_stream stream);
AXHIP_API int axhip_graph_launch(axhip_graph graph);
/* One replay on the graph's own stream without any ordering against the default stream: replays of
 * different graphs then run side by side on the device (replays of one graph keep their order).
 * The caller orders them against other work with axhip_graph_sync.  Graphs that run side by side
 * must have been captured under different ticket lanes (axhip_set_ticket_lane) if they hold
 * attention or argmax launches.  No reference counterpart. */
AXHIP_API int axhip_graph_launch_async(axhip_graph graph);
/* One replay that has finished when the call returns, after all earlier default-stream work: the
 * reference's CudaGraphExec::Replay (launch + stream synchronise, src/core/cuda/graph.cu:123-139). */
AXHIP_API int axhip_graph_replay(axhip_graph graph);
AXHIP_API int axhip_graph_sync(axhip_graph graph);
AXHIP_API int axhip_graph_destroy(axhip_graph graph);

/* Capture pool: address stability between the warm-up run and the captured run of the same
 * body.  Replaces ResetCapturePool / SetCapturePoolRecording / the size->ptr FIFO,
 * src/core/cuda/capture_pool.cu:21-51 and detail.cu:193-199,259-264.  While recording, every
 * axhip_alloc is remembered (size -> pointer, in order); while capturing, an axhip_alloc of the
 * same size pops the remembered pointer instead of allocating, so the graph sees the warm-up's
 * addresses.  Blocks remembered by the pool are owned by it until axhip_capture_pool_reset. */
AXHIP_API int axhip_capture_pool_reset(void);
AXHIP_API int axhip_capture_pool_set_recording(int on);

/* Events on the current stream, for timing kernels (no reference counterpart; the reference
 * times with the host clock). */
typedef void *axhip_event;
AXHIP_API int axhip_event_create(axhip_event *out);
AXHIP_API int axhip_event_record(axhip_event ev, axhip_stream stream);
AXHIP_API int axhip_event_elapsed_ms(axhip_event start, axhip_event stop, float *ms_out);
AXHIP_API int axhip_event_destroy(axhip_event ev);

/* ============================================================================================
 * Decode attention
 * ========================================================================================== */

/* Split-K flash-decoding for one query token per sequence, grouped-query heads.
 * Replaces ops::cuda::GqaDecodeAttention (include/axono/ops/cuda/gqa.h:16-20,
 * src/ops/cuda/gqa.cu:139-182: GqaDecodeSplitKernel :31-92, GqaDecodeMergeKernel :95-129) and its
 * short-context fallback to ScaledDotProductAttention(is_causal=false) (gqa.cu:150-151).
 * Result per sequence b and head h:  softmax(q[b,h] . K[b, h/group, 0:len_b]^T / sqrt(D)) V[...].
 *
 *   q, out      [B, Hq, D], dtype `dtype` (FLOAT16 or FLOAT32), contiguous
 *   k, v        element (b, hk, s, :) at  base + b*stride_b + hk*stride_h + s*stride_s  (strides in
 *               elements, rows of D contiguous elements).  The batched cache [B,Hkv,Lmax,D] has
 *               stride_b = Hkv*Lmax*D, stride_h = Lmax*D, stride_s = D; the reference's per-call
 *               layout (L,Hkv,D) is B = 1, stride_h = D, stride_s = Hkv*D.
 *   seq_lens    device int32[B] with each sequence's current length, or NULL: every sequence has
 *               `max_len` keys.  Read by the kernels, so a captured graph follows lengths that
 *               change between replays.  A length of 0 yields zeros.
 *   max_len     upper bound of every length (sizes the split grid; lengths above it are clamped)
 *   workspace   device scratch of at least axhip_gqa_decode_workspace_bytes(...) bytes
 *   D in {64, 128, 256}; Hq % Hkv == 0.  fp32 accumulation throughout; fp16 data is widened
 *   exactly and only the final store rounds. */
AXHIP_API size_t axhip_gqa_decode_workspace_bytes(int B, int Hq, int Hkv, int D, int max_len);
AXHIP_API int axhip_gqa_decode(const void *q, const void *k, const void *v,
                               const int32_t *seq_lens, void *out, void *workspace,
                               size_t workspace_bytes, int dtype, int B, int Hq, int Hkv, int D,
                               int max_len, int64_t stride_b, int64_t stride_h, int64_t stride_s,
                               axhip_stream stream);

/* axhip_gqa_decode over a paged KV cache.  Keys and values live in pools
 *   k_pool, v_pool  [n_pages, Hkv, 128, D]   (pages of AXHIP_PAGE_KEYS = 128 consecutive keys of one sequence)
 * and key s of sequence b is row s % 128 of page  page_table[b * max_pages + s / 128]  (device int32
 * [B, max_pages]; entries behind a sequence's last page are never read, and an entry outside [0, n_pages) is
 * clamped into the pool: wrong values, never an access outside it).  Everything else - q, out, seq_lens,
 * max_len, workspace, the split plan, the in-kernel merge - is as in axhip_gqa_decode, and so is the
 * result, bit for bit, for the same keys in the same order: only the address of a key row differs (each
 * workgroup copies the page numbers of its key range from the table into LDS before its first tile).
 * max_pages * 128 >= max_len; max_len <= 131072; head groups of four and more query heads run on the vector
 * ALUs here (the matrix-core variant reads a dense cache).  A cache that grows by pages allocates
 * memory for the tokens that exist instead of B * Lmax rows; the reference's cache grows by re-copying
 * (axono/python/axono/nn/kv_cache.py:96-102) and has no paged form. */
#define AXHIP_PAGE_KEYS 128
AXHIP_API int axhip_gqa_decode_paged(const void *q, const void *k_pool, const void *v_pool,
                                     const int32_t *page_table, const int32_t *seq_lens, void *out,
                                     void *workspace, size_t workspace_bytes, int dtype, int B, int Hq,
                                     int Hkv, int D, int max_len, int max_pages, int n_pages,
                                     axhip_stream stream);

/* axhip_gqa_decode for callers that cannot allocate (code under hipGraph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and therefore have no workspace to pass: the split partials go to a
 * static device array inside the library, AXHIP_GQA_DECODE_STATIC_SCRATCH_BYTES per device, held until
 * the process ends.  Same arguments (without workspace), same kernels, same split plan and bit-identical
 * results; neither the call nor anything it runs allocates or frees memory.  It has no counterpart in the
 * reference (whose operator allocates three workspace tensors per call, src/ops/cuda/gqa.cu:166-168).
 *   - a problem whose split plan needs more scratch than the array holds is refused with
 *     AXHIP_OUT_OF_MEMORY before anything is launched (B * Hq * ranges-per-sequence * (D + 2) * 4 bytes
 *     are needed; with the default plan ranges-per-sequence <= max(256 / head groups, B), so e.g. every
 *     batch up to B = 64 at Hq = 16, D = 128 fits);
 *   - every call on a device shares that device's array, whatever its ticket lane: calls that overlap
 *     in time on one device race.  Calls on one stream, and replays of one captured graph, never overlap.
 *     Nothing in the array has to start at zero (a partial is always written before it is read), so the
 *     previous call's contents are simply overwritten;
 *   - the array's address is looked up on the first call on each device; make that first call outside a
 *     graph capture. */
#define AXHIP_GQA_DECODE_STATIC_SCRATCH_BYTES (48u << 20)
AXHIP_API int axhip_gqa_decode_static(const void *q, const void *k, const void *v,
                                      const int32_t *seq_lens, void *out, int dtype, int B, int Hq,
                                      int Hkv, int D, int max_len, int64_t stride_b, int64_t stride_h,
                                      int64_t stride_s, axhip_stream stream);

/* The split plan the launcher uses for these sizes (it depends on host-side sizes only, so a captured launch
 * stays valid while the device-side lengths change).  For batches of up to 64 sequences the launch holds a
 * fixed number of workgroups (one per compute unit) which are dealt to the sequences on the device in
 * proportion to their current lengths (n_splits = workgroup slots per sequence, chunk = keys per workgroup if
 * every sequence had max_len keys): whole workgroups per sequence when that is within an eighth of the even
 * share, otherwise equal runs of keys over the sequences laid end to end; the last workgroup of a sequence
 * merges its ranges.  Larger batches cut every sequence into n_splits ranges of chunk keys.  No reference
 * counterpart (the reference hard-codes min(256, ceil(L/64)), gqa.cu:158-160). */
AXHIP_API void axhip_gqa_decode_plan(int B, int Hq, int Hkv, int max_len, int *n_splits, int *chunk);

/* General attention for prefill and short contexts: q [Sq,Hq,D], k/v [Skv,Hkv,D] contiguous,
 * optional causal mask with the reference's rule (keys 0..t visible when Skv >= t+1).
 * Replaces ops::cuda::ScaledDotProductAttention, src/ops/cuda/sequence.cu:105-163,451-472.
 * fp16 with D 64 or 128, 32 or more query rows and 16-byte aligned pointers runs the tiled
 * matrix-core kernel of axhip_prefill_attention over the token-major K/V; other fp16/fp32 cases
 * with D 64/128/256 run the split-K decode kernel with one "sequence" per query row; any other
 * D takes a plain three-phase kernel. */
AXHIP_API int axhip_sdpa(const void *q, const void *k, const void *v, void *out, int dtype,
                         int Sq, int Hq, int Hkv, int D, int Skv, int is_causal,
                         axhip_stream stream);

/* ============================================================================================
 * KV-cache append
 * ========================================================================================== */

/* cache[b, hk, pos[b], :] = new[b, hk, :] for K and V in one launch; a byte copy (bit exact).
 * Replaces DynamicKVCache.update's concat-append (axono/python/axono/nn/kv_cache.py:96-102 ->
 * ops::cuda::Concat axis 0, src/ops/cuda/sequence.cu:474-521), which re-copies the whole cache
 * every step.  k_new, v_new [B,Hkv,D]; caches [B,Hkv,Lmax,D]; pos device int32[B] or int64[B]
 * (`pos_dtype`); a position outside [0,Lmax) is skipped.  `elem_bytes` is 2 or 4. */
AXHIP_API int axhip_kv_append(const void *k_new, const void *v_new, void *k_cache, void *v_cache,
                              const void *pos, int pos_dtype, int elem_bytes, int B, int Hkv,
                              int Lmax, int D, axhip_stream stream);

/* KV append into a paged cache (pools and page table as for axhip_gqa_decode_paged): token t of sequence
 * b, rows k_new / v_new [B, S, Hkv, D] (token-major: the (seq, n_kv_head, d_head) layout of the
 * reference's cache with a batch axis in front), goes to key position start[b] + t (start: device int32 or
 * int64 [B], or NULL for 0).  A byte copy (bit exact).  Positions behind the table and page numbers
 * outside [0, n_pages) are skipped.  Counterpart of DynamicKVCache.update
 * (axono/python/axono/nn/kv_cache.py:96-102). */
AXHIP_API int axhip_kv_append_paged(const void *k_new, const void *v_new, void *k_pool, void *v_pool,
                                    const int32_t *page_table, const void *start, int start_dtype,
                                    int elem_bytes, int B, int S, int Hkv, int D, int max_pages,
                                    int n_pages, axhip_stream stream);

/* Copies sequences from a dense cache into a paged one (after a prefill that filled dense rows): key positions
 * 0 .. lens[b]-1 (device int32 [B]; NULL: all `rows`) of k_dense / v_dense [B, Hkv, rows, D] go to row
 * (position % 128) of page page_table[b, position / 128].  A byte copy; positions behind the table and page
 * numbers outside [0, n_pages) are skipped.  No reference counterpart. */
AXHIP_API int axhip_kv_dense_to_paged(const void *k_dense, const void *v_dense, void *k_pool, void *v_pool,
                                      const int32_t *page_table, const int32_t *lens, int elem_bytes, int B,
                                      int Hkv, int rows, int D, int max_pages, int n_pages,
                                      axhip_stream stream);

/* out = [a ; b] along an axis: `outer` blocks of a_bytes then b_bytes each (axis 0: outer = 1).
 * Replaces ops::cuda::Concat, src/ops/cuda/sequence.cu:474-521. */
AXHIP_API int axhip_concat(const void *a, const void *b, void *out, int64_t outer, int64_t a_bytes,
                           int64_t b_bytes, axhip_stream stream);

/* ============================================================================================
 * Fused and row-wise operators (dtype FLOAT16 or FLOAT32; arithmetic in fp32)
 * ========================================================================================== */

/* y = x + residual ; out = y * rsqrt(mean(y^2) + eps) * weight.  Two results, like the reference.
 * Replaces ops::cuda::AddRmsNorm, src/ops/cuda/fused.cu:38-72,91-110.  weight dtype may differ
 * from the activation dtype (`w_dtype`). */
AXHIP_API int axhip_add_rms_norm(const void *x, const void *residual, const void *weight, float eps,
                                 void *y, void *out, int dtype, int w_dtype, int64_t rows,
                                 int64_t hidden, axhip_stream stream);

/* Same, with the normalised output stored as `out_dtype`: FLOAT16 while x / residual / y are
 * FLOAT32, for a result that only feeds an fp16 Linear (which would round it to fp16 itself, so the
 * values the Linear sees are identical).  No reference counterpart. */
AXHIP_API int axhip_add_rms_norm_ex(const void *x, const void *residual, const void *weight, float eps,
                                    void *y, void *out, int dtype, int w_dtype, int out_dtype,
                                    int64_t rows, int64_t hidden, axhip_stream stream);

/* y = gate / (1 + exp(-gate)) * up.  Replaces ops::cuda::SiluMul, src/ops/cuda/fused.cu:28-34,76-89. */
AXHIP_API int axhip_silu_mul(const void *gate, const void *up, void *y, int dtype, int64_t n,
                             axhip_stream stream);

/* out = x * rsqrt(mean(x^2) + eps) [* weight] over the last dim; weight may be NULL.
 * Replaces ops::cuda::RmsNorm, src/ops/cuda/llm.cu:140-158. */
AXHIP_API int axhip_rms_norm(const void *x, const void *weight, float eps, void *out, int dtype,
                             int w_dtype, int64_t rows, int64_t cols, axhip_stream stream);

AXHIP_API int axhip_rms_norm_ex(const void *x, const void *weight, float eps, void *out, int dtype,
                                int w_dtype, int out_dtype, int64_t rows, int64_t cols,
                                axhip_stream stream);

/* out = a + b.  Replaces ops::cuda::Add for equal shapes, src/ops/cuda/add.cu:17-24. */
AXHIP_API int axhip_add(const void *a, const void *b, void *out, int dtype, int64_t n,
                        axhip_stream stream);

/* dst = src with two dimensions exchanged (a copy; any element size of 1, 2, 4 or 8 bytes).  The
 * contiguous source is described as [outer, dim_a, mid, dim_b, inner] and the destination is
 * [outer, dim_b, mid, dim_a, inner]: for Tensor::Transpose(d0 < d1) outer / mid / inner are the products of
 * the extents before d0, between d0 and d1, and after d1.  Replaces cuda::tensor::TransposeKernel
 * (src/core/cuda/tensor/transpose.cu:17-143, called from src/core/tensor.cpp:386-424). */
AXHIP_API int axhip_transpose(const void *src, void *dst, int elem_bytes, int64_t outer, int64_t dim_a,
                              int64_t mid, int64_t dim_b, int64_t inner, axhip_stream stream);

/* fp16 <-> fp32 conversion, IEEE round-to-nearest-even.  Replaces Half2FloatKernel /
 * Float2HalfKernel, src/core/cuda/tensor/kernel.cu:175-223 (Tensor::CastTo on device). */
AXHIP_API int axhip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n,
                         axhip_stream stream);

/* ============================================================================================
 * Rotary position embeddings.  x, out [rows, heads, dim]; rotate-half pairing (i, i + dim/2).
 * ========================================================================================== */

/* freq_i = powf(theta, -2 i / dim) evaluated on the host in fp32 exactly as the reference's CPU
 * operator does, angle = float(pos) * freq_i in fp32, accurate sinf/cosf.  pos device int64[rows].
 * Replaces ops::cuda::Rope, src/ops/cuda/sequence.cu:84-101,318-342 (CPU: sequence.cpp:54-93).
 * dim <= 512. */
AXHIP_API int axhip_rope(const void *x, const int64_t *pos, float theta, void *out, int dtype,
                         int64_t rows, int64_t heads, int64_t dim, axhip_stream stream);

/* axhip_rope on the q and the k heads of the same rows in one launch (they share the positions, so each
 * row's angles are evaluated once): q [rows, q_heads, dim] -> q_out, k [rows, k_heads, dim] -> k_out.  Same
 * arithmetic as two axhip_rope calls, bit for bit.  The reference's operator takes one tensor per call
 * (src/ops/cuda/sequence.cu:318-342) and its model calls it twice per layer
 * (examples/vlm/qwen3vl/model.py:358-359). */
AXHIP_API int axhip_rope_qk(const void *q, const void *k, const int64_t *pos, float theta, void *q_out,
                            void *k_out, int dtype, int64_t rows, int64_t q_heads, int64_t k_heads,
                            int64_t dim, axhip_stream stream);

/* M-RoPE with interleaved T/H/W channels: pos device int64[3, rows], inv_freq device fp32[dim/2];
 * channel i uses H if i%3==1 && i<3*h_sec, W if i%3==2 && i<3*w_sec, else T (t_sec is unused, as
 * in the reference).  Replaces ops::cuda::RopeThd, src/ops/cuda/sequence.cu:186-212,421-449. */
AXHIP_API int axhip_rope_thd(const void *x, const int64_t *pos, const float *inv_freq, int t_sec,
                             int h_sec, int w_sec, void *out, int dtype, int64_t rows,
                             int64_t heads, int64_t dim, axhip_stream stream);

/* cos/sin tables [rows, 2*half] fp32 (both halves equal) for M-RoPE.
 * Replaces ops::cuda::MropeCosSin, src/ops/cuda/sequence.cu:372-419. */
AXHIP_API int axhip_mrope_cos_sin(const int64_t *pos, const float *inv_freq, int h_sec, int w_sec,
                                  float *cos_out, float *sin_out, int64_t rows, int64_t half,
                                  axhip_stream stream);

/* Rotation by given fp32 tables cos, sin [rows, dim]; the second element of a pair uses the
 * second half of the table.  Replaces ops::cuda::RopeWithCosSin, src/ops/cuda/sequence.cu:166-183,344-369. */
AXHIP_API int axhip_rope_with_cos_sin(const void *x, const float *cos_t, const float *sin_t,
                                      void *out, int dtype, int64_t rows, int64_t heads,
                                      int64_t dim, axhip_stream stream);

/* ============================================================================================
 * fp16 Linear (cast_linear_fp16)
 * ========================================================================================== */

/* out[M,N] = x[M,K] . W[N,K]^T (+ bias[N]); W and bias FLOAT16, fp32 accumulation on MFMA.
 * x is FLOAT32 (converted to fp16 round-to-nearest-even first, as the reference does,
 * src/ops/cuda/linear.cu:105-110) or FLOAT16; out is FLOAT32 (the reference's contract,
 * nanobind_module.cpp:760-762) or FLOAT16.  bias may be NULL.
 * Replaces the fp16 branch of ops::cuda::Linear, src/ops/cuda/linear.cu:105-176 (cast kernel +
 * bias/zero fill + cublasGemmEx).  K % 8 == 0.  `workspace` holds split-K partial sums for skinny
 * M: at least axhip_linear_f16_workspace_bytes(M,K,N) bytes (may be 0, then pass NULL). */
AXHIP_API size_t axhip_linear_f16_workspace_bytes(int64_t M, int64_t K, int64_t N);
AXHIP_API int axhip_linear_f16(const void *x, int x_dtype, const void *w, const void *bias,
                               void *out, int out_dtype, int64_t M, int64_t K, int64_t N,
                               void *workspace, size_t workspace_bytes, axhip_stream stream);

/* out[M,N] = x[M,K] . w[N,K]^T (+ bias[N]), every operand FLOAT32: the Linear of a module whose weights have
 * not been cast to fp16, ops::cuda::Linear's FLOAT32 branch (src/ops/cuda/linear.cu:178-251, cublasSgemm).
 * fp32 products and sums in K order on the fp32 matrix instruction; bias may be NULL.  The FLOAT64 branch of
 * the reference has no counterpart here.  Not on the decode path and not tuned. */
AXHIP_API int axhip_linear_f32(const float *x, const float *w, const float *bias, float *out, int64_t M,
                               int64_t K, int64_t N, axhip_stream stream);

/* Packed weights for skinny M.  axhip_linear_f16_pack re-orders a row-major FLOAT16 W [N,K] once
 * into MFMA fragment order (1 KiB blocks of 16 rows x 32 K, consecutive along K; rows and K
 * zero-padded to whole blocks) into a buffer of axhip_linear_f16_packed_bytes(N,K) bytes, so that
 * every wavefront streams consecutive memory.  axhip_linear_f16_packed computes the same result as
 * axhip_linear_f16 from it: the HBM-bound skinny kernels for M <= 32, a 256x128-tile MFMA GEMM above.  The packing is the build's counterpart of what
 * Module.cast_linear_fp16 does to a Linear's weights (axono/python/axono/nn/module.py:158-184): a
 * one-off conversion into the resident format the inference kernels read.
 * glu != 0 (both calls): W is a fused [gate ; up] projection (N = 2*I rows, N % 32 == 0); the rows
 * are packed as tiles of 8 gate rows and their 8 up rows and the kernel stores silu(gate) * up, an [M, N/2]
 * result, instead of the [M, N] projection (same arithmetic as axhip_silu_mul on the two halves;
 * no bias). */
AXHIP_API size_t axhip_linear_f16_packed_bytes(int64_t N, int64_t K);
AXHIP_API int axhip_linear_f16_pack(const void *w, void *packed, int64_t N, int64_t K, int glu,
                                    axhip_stream stream);
AXHIP_API int axhip_linear_f16_packed(const void *x, int x_dtype, const void *packed_w, const void *bias,
                                      void *out, int out_dtype, int64_t M, int64_t K, int64_t N, int glu,
                                      axhip_stream stream);

/* ============================================================================================
 * Index operators of the decode step
 * ========================================================================================== */

/* out[i, :] = table[ids[i], :]; ids device int64 (or int32 via `ids_dtype`); table/out `dtype`.
 * Replaces ops::cuda::Embedding, src/ops/cuda/sequence.cu:75-81,296-316. */
AXHIP_API int axhip_embedding(const void *ids, int ids_dtype, const void *table, void *out,
                              int dtype, int64_t n_ids, int64_t vocab, int64_t hidden,
                              axhip_stream stream);

/* out[r] = index of the first maximum of x[r, :]; out device int64[rows].
 * Replaces ops::cuda::ArgmaxLastDim, src/ops/cuda/sequence.cu:262-292. */
AXHIP_API int axhip_argmax(const void *x, int64_t *out, int dtype, int64_t rows, int64_t cols,
                           axhip_stream stream);

/* ============================================================================================
 * Glue kernels of the captured decode step (fusions of the operators above)
 * ========================================================================================== */

/* For every token r (B sequences of S consecutive tokens each, r = b*S + t; S = 1 in a decode
 * step, S = prompt length in prefill) and head: q heads -> rms_norm over D (weight q_weight) ->
 * M-RoPE -> stored as `cache_dtype` into q_out [B*S,Hq,D]; k heads -> rms_norm (k_weight) -> M-RoPE
 * -> written to k_cache[b, hk, seq_lens[b] + t, :]; v heads -> converted and written to
 * v_cache[b, hk, seq_lens[b] + t, :].  seq_lens may be NULL (append from position 0).
 * Equals rms_norm + rope_thd + cast + kv_append applied in that order (the reference's sequence,
 * examples/vlm/qwen3vl/model.py:353-364), with one rounding at the store.  q, k, v are fp32 rows of
 * the projection output with the given row strides (elements), so a fused QKV projection can be
 * passed as three offsets into one buffer.  pos int64 [3,B*S]; inv_freq fp32 [D/2]; seq_lens int32 [B]
 * (an append position outside [0,Lmax) is skipped).  Norm weights may be NULL. */
AXHIP_API int axhip_qkv_norm_rope_append(const float *q, int64_t q_stride, const float *k,
                                         int64_t k_stride, const float *v, int64_t v_stride,
                                         const void *q_weight, const void *k_weight, int w_dtype,
                                         float eps, const int64_t *pos, const float *inv_freq,
                                         int h_sec, int w_sec, const int32_t *seq_lens, void *q_out,
                                         void *k_cache, void *v_cache, int cache_dtype, int B, int S,
                                         int Hq, int Hkv, int D, int Lmax, axhip_stream stream);

/* Causal attention for prefill on the matrix cores: q [B,S,Hq,D] fp16, keys / values already in the
 * caches [B,Hkv,cache_rows,D] fp16; query i of sequence b sits at absolute position start[b] + i
 * (start NULL: 0) and attends to cache rows 0 .. start[b] + i.  out [B,S,Hq,D] fp16.  D = 64 or 128.
 * Same result as ops::cuda::ScaledDotProductAttention with is_causal (src/ops/cuda/sequence.cu:105-163,
 * 451-472) on each sequence, with fp32 softmax statistics and probabilities rounded to fp16 for the
 * second product. */
AXHIP_API int axhip_prefill_attention(const void *q, const void *k_cache, const void *v_cache,
                                      const int32_t *start, void *out, int dtype, int B, int S, int Hq,
                                      int Hkv, int D, int cache_rows, axhip_stream stream);

/* The attention block of one decode step in one launch (plus the split merge): equals
 * axhip_qkv_norm_rope_append with S = 1 followed by axhip_gqa_decode over seq_lens[b] + 1 keys of the
 * caches [B,Hkv,cache_rows,D], without materialising q and without a second read of the row just
 * appended.  q / k / v, their strides, the norm weights, pos [3,B], inv_freq, h_sec / w_sec as in
 * axhip_qkv_norm_rope_append; seq_lens int32 [B] holds the lengths BEFORE the append (required); the new
 * row is written at seq_lens[b] when that is < max_len, otherwise nothing is appended and max_len cached
 * keys are attended.  max_len <= cache_rows bounds the attended length (the split plan is made from it, so a
 * captured launch stays valid while seq_lens grows).  out [B,Hq,D] in the cache dtype.  Workspace as for
 * axhip_gqa_decode.  No reference counterpart (the reference's layer runs these as separate operators,
 * examples/vlm/qwen3vl/model.py:330-373). */
AXHIP_API int axhip_gqa_decode_qkv(const float *q, int64_t q_stride, const float *k, int64_t k_stride,
                                   const float *v, int64_t v_stride, const void *q_weight,
                                   const void *k_weight, int w_dtype, float eps, const int64_t *pos,
                                   const float *inv_freq, int h_sec, int w_sec, const int32_t *seq_lens,
                                   void *k_cache, void *v_cache, void *out, void *workspace,
                                   size_t workspace_bytes, int cache_dtype, int B, int Hq, int Hkv, int D,
                                   int cache_rows, int max_len, axhip_stream stream);

/* The attention launches of one decode step (one per layer) are given the same seq_lens, and each deals the key
 * ranges to its workgroups from them in the same way.  With mode 1 set on the calling thread, an
 * axhip_gqa_decode_qkv[_paged] launch also leaves what each workgroup slot found in a table on the device (per
 * ticket lane); with mode 2 a launch takes its ranges from that table instead of dealing again.  Mode 0
 * (default): every launch deals for itself.  A captured launch keeps the mode it was captured under.  The
 * caller promises, for a mode-2 launch: the mode-1 launch before it on the same stream had the same seq_lens
 * pointer and contents, B, heads, max_len and cache_rows.  A mode-2 launch whose shape or seq_lens pointer
 * differs from the table's deals for itself; same results either way.  No reference counterpart. */
AXHIP_API int axhip_set_plan_reuse(int mode);
AXHIP_API int axhip_plan_reuse(void);

/* axhip_gqa_decode_qkv over a paged cache (pools, page table, max_pages, n_pages as for
 * axhip_gqa_decode_paged; FLOAT16 caches): the new token's k / v row goes to row seq_lens[b] % 128 of page
 * page_table[b, seq_lens[b] / 128] - that page must already be in the table - when seq_lens[b] < max_len, and
 * the keys are read through the table.  A table entry outside [0, n_pages) for that page (a sequence whose pages
 * were given back and not reserved again) skips the store, as axhip_kv_append_paged does; reads clamp such
 * entries into the pool.  Same bits as axhip_gqa_decode_qkv on a dense cache holding the same rows.
 * No reference counterpart. */
AXHIP_API int axhip_gqa_decode_qkv_paged(const float *q, int64_t q_stride, const float *k, int64_t k_stride,
                                         const float *v, int64_t v_stride, const void *q_weight,
                                         const void *k_weight, int w_dtype, float eps, const int64_t *pos,
                                         const float *inv_freq, int h_sec, int w_sec, const int32_t *seq_lens,
                                         void *k_pool, void *v_pool, const int32_t *page_table, void *out,
                                         void *workspace, size_t workspace_bytes, int cache_dtype, int B, int Hq,
                                         int Hkv, int D, int max_len, int max_pages, int n_pages,
                                         axhip_stream stream);

/* y[r, c] = silu(gate_up[r, c]) * gate_up[r, cols + c] for a fused [gate | up] projection output
 * [rows, 2*cols] -> [rows, cols].  Same arithmetic as axhip_silu_mul.  cols % 8 == 0.  out_dtype
 * may be FLOAT16 for FLOAT32 input (see axhip_add_rms_norm_ex). */
AXHIP_API int axhip_silu_mul_fused(const void *gate_up, void *y, int dtype, int out_dtype, int64_t rows,
                                   int64_t cols, axhip_stream stream);

/* First launch of a decode step: h[i, :] = float(table[ids[i], :]) (FLOAT16 table, FLOAT32 h: the
 * residual stream) and xn[i, :] = FLOAT16 of rms_norm(h[i, :]) * weight - the arithmetic of
 * axhip_embedding, axhip_cast and axhip_rms_norm_ex in that order, bit for bit.  dim % 8 == 0,
 * dim <= 8192.  Replaces the sequence Embedding -> CastTo -> RmsNorm that opens
 * Qwen3VLTextModel.forward, examples/vlm/qwen3vl/model.py:470-476. */
AXHIP_API int axhip_embedding_rms_norm(const void *ids, int ids_dtype, const void *table, const void *weight,
                                       int w_dtype, float eps, void *h, void *xn, int64_t n_ids, int64_t vocab,
                                       int64_t dim, axhip_stream stream);

/* Everything of a decoder layer behind the attention, plus the next layer's fused q/k/v projection, for at most
 * 16 rows, in one persistent launch whose four phases are separated by barriers across the resident workgroups
 * (one per CU; the weights of a phase are requested before the barrier in front of it):
 *   h1 = attn . Wo^T + h_in;  act = silu(g) * u with [g | u] = rmsnorm(h1, w_post) . Wgu^T;
 *   h_out = act . Wd^T + h1;  y = rmsnorm(h_out, w_next) . Wn^T.
 * attn FLOAT16 [M, K1]; h_in, h_out FLOAT32 [M, H] (different buffers); w_post, w_next FLOAT32 [H]; w_o [H, K1],
 * w_gate_up [2 I, H] (packed with glu = 1), w_down [H, I], w_next_linear [N_next, H]: packed by
 * axhip_linear_f16_pack; y FLOAT32 [M, N_next]; workspace: axhip_decode_layer_tail_workspace_bytes(H, I) bytes,
 * 128-byte aligned.  Built for K1 = H = 2048, I = 6144 (and K1 = H = 512, I = 1024 for tests), N_next <= 16 per
 * workgroup: other widths return AXHIP_INVALID_ARGUMENT and the caller uses the single operators.  Must be the
 * only work on the device while it runs (all its workgroups have to be resident); a barrier wait that runs out
 * is counted, see axhip_decode_layer_tail_status, and the results of that launch are undefined.  Replaces
 * the operator sequence of Qwen3VLTextDecoderLayer.forward behind the attention and the q/k/v projections that open
 * the next layer (the reference runs them one launch each, examples/vlm/qwen3vl/model.py:408-436). */
/* 1 when axhip_decode_layer_tail is built for these widths on the current device (it needs a workgroup per unit of
 * every phase: 256 compute units for the 2B widths), else 0. */
AXHIP_API int axhip_decode_layer_tail_supported(int M, int H, int K1, int I, int N_next);
AXHIP_API size_t axhip_decode_layer_tail_workspace_bytes(int H, int I);
AXHIP_API int axhip_decode_layer_tail(const void *attn, const float *h_in, const void *w_o, const float *w_post,
                                      const void *w_gate_up, const void *w_down, const float *w_next,
                                      const void *w_next_linear, float *h_out, float *y, void *workspace,
                                      size_t workspace_bytes, int M, int H, int K1, int I, int N_next, float eps,
                                      axhip_stream stream);
/* The same launch for the last layer of a model: nothing follows the closing norm, and the launch ends with
 * xn_out = rmsnorm(h_out, w_final_norm) as FLOAT16 [M, H] (the rows the lm_head reads) instead of y.  Supported
 * where axhip_decode_layer_tail_supported(M, H, K1, I, 0) is 1.  Replaces the same operator sequence followed by the
 * model's final norm (examples/vlm/qwen3vl/model.py:408-436, 760-761). */
AXHIP_API int axhip_decode_layer_tail_last(const void *attn, const float *h_in, const void *w_o, const float *w_post,
                                           const void *w_gate_up, const void *w_down, const float *w_final_norm,
                                           float *h_out, void *xn_out, void *workspace, size_t workspace_bytes, int M,
                                           int H, int K1, int I, float eps, axhip_stream stream);
/* Barrier waits of axhip_decode_layer_tail that ran out since the last reset (0 in a healthy process); reset != 0
 * also puts the barrier counters back to zero (only while no such launch is in flight). */
AXHIP_API int axhip_decode_layer_tail_status(int reset, unsigned *failed_waits);
/* Last launch of a greedy decode step: ids[b] = next_ids[b]; pos[r, b] += 1 for r < pos_rows;
 * seq_lens[b] += 1; log[*counter, b] = next_ids[b] while *counter < log_rows; *counter += 1.  Any of
 * ids, pos (with pos_rows 0), seq_lens, log and counter may be NULL.  The reference does all of this
 * on the host between steps (examples/vlm/qwen3vl/model.py:739-748, 846-858); inside a captured step
 * it has to happen on the device. */
AXHIP_API int axhip_decode_advance(const int64_t *next_ids, int64_t *ids, int64_t *pos, int pos_rows,
                                   int32_t *seq_lens, int64_t *log, int64_t log_rows, uint64_t *counter, int B,
                                   axhip_stream stream);

/* x[i] += delta in place for INT32 / INT64 device arrays (sequence lengths and positions that a
 * captured decode step advances on the device; the reference rebuilds them on the host each step,
 * examples/vlm/qwen3vl/model.py:739-748). */
AXHIP_API int axhip_index_add(void *x, int dtype, int64_t n, int64_t delta, axhip_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* AXHIP_H_ */
