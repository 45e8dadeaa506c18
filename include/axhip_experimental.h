/*
 * axhip_experimental.h - measurement hooks of libaxhip.so.  NOT part of the drop-in boundary (axhip.h):
 * these entry points exist so that tests can force every kernel variant and benchmarks can sweep plans.
 * They set process-global, unsynchronised state: call them from one thread while no operator call is in
 * flight, and restore the defaults (all arguments 0) afterwards.  The library as a whole is a single-stream
 * drop-in in this respect: operator calls themselves are safe from several threads and streams (the merging
 * launches under distinct ticket lanes, axhip_set_ticket_lane in axhip.h), the hooks here are not.  No reference counterparts (the
 * reference hard-codes its split count, src/ops/cuda/gqa.cu:158-160, and leaves GEMM algorithm choice to
 * cuBLAS, src/ops/cuda/linear.cu:131-138).
 */
#ifndef AXHIP_EXPERIMENTAL_H_
#define AXHIP_EXPERIMENTAL_H_

#include "axhip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Decode attention split plan.  target_workgroups = workgroups to keep streaming (default: one per compute
 * unit; a negative value selects a second merge kernel for a forced split count instead of the in-kernel
 * merge), force_splits > 0 cuts every sequence into that many ranges (+ 1000: head groups of four and more
 * stay on the vector ALUs instead of the matrix cores, for comparison); 0 restores the defaults. */
AXHIP_API void axhip_gqa_decode_tune(int target_workgroups, int force_splits);

/* fp16 Linear plans (0 restores a default).  Skinny M: wavefronts to aim for, 16-row groups of W per
 * wavefront (1 to 4), wavefronts (K slices) per workgroup (4, 8, 16).  M > 32 GEMM, gemm_rows: 64 or 128
 * rows of x per workgroup (128: one workgroup per CU), 256 = the 256 x 128 tile at two workgroups per CU
 * (the default for large problems), 512 = the eight-wavefront workgroup that sums K in two halves (fp16 x,
 * K % 512 == 0, otherwise ignored; with 1000 t: t = 1 or 2 row tiles), plus 1000 t to force t = 1, 2 or 4 row
 * tiles of W per wavefront (64, 128 or 256 weight rows per workgroup; by default the largest that still
 * gives every CU a workgroup).  target_waves >= 100000 does not set the skinny plan but the order in which the
 * 256 x 128 tiles are handed to the XCDs: 100000 + 256 A + B = rectangles of A weight-row blocks x B blocks of
 * x rows per XCD at a time, 100000 = weight-row blocks dealt to the XCDs with the x blocks fastest (the default
 * picks by problem size). */
AXHIP_API void axhip_linear_f16_tune(int target_waves, int force_nt, int force_waves, int gemm_rows);

/* Prefill / general fp16 attention on the matrix cores: 1 = all position blocks of a (sequence, head group) run on
 * one XCD, pair after pair (their keys and values stay in that XCD's L2), 0 = position blocks dealt round-robin over
 * the XCDs, -1 = the default (by XCD when the pairs go round the eight XCDs evenly or there are at least 32). */
AXHIP_API void axhip_prefill_attention_tune(int pairs_by_xcd);

/* Measurement: bit p of skip_phases set = phase p + 1 computes nothing, 32 = no barriers (results are then
 * meaningless); 256 = every barrier gives up after one look at its flag, which is how the tests reach the path of
 * a wait that runs out (the launch still ends by itself). */
AXHIP_API void axhip_decode_layer_tail_tune(int skip_phases);
/* Measurement: launches made while `stamps` is not null leave 32 readings of the 100 MHz device clock per
 * workgroup there (device memory, workgroups x 32 x 8 bytes): slots 0-12 of wavefront 0 and 16-28 of wavefront 5 at
 * the start, after the matrix instructions of phase 1, before and after barrier 1, after the row sums of phase 2,
 * after its matrix instructions, before and after barrier 2, after the matrix instructions of phase 3, before and
 * after barrier 3, after the matrix instructions of phase 4, at the end. */
AXHIP_API void axhip_decode_layer_tail_trace(void *stamps);

#ifdef __cplusplus
}
#endif
#endif /* AXHIP_EXPERIMENTAL_H_ */
