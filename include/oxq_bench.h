/* Measurement aids of liboxq_hip.so: kernels with no counterpart in the reference and no part in
 * the matmul path.  bench.py times them beside the matmul kernels, in the same run and the same way,
 * so that a kernel's time can be set against what the machine does with the same bytes and the
 * same launch shape when there is no arithmetic at all.  Kept out of oxq.h: a binding of the
 * reference's interface does not need them. */
#ifndef OXQ_BENCH_H
#define OXQ_BENCH_H

#include "oxq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming read of `src` (U8, contiguous, 16-byte aligned; its size a multiple of
 * workgroups * 8 KiB) by `workgroups` workgroups of 512 threads, each reading one contiguous span
 * with 16-byte loads, eight in flight per lane, in passes of 64 KiB.  `checksums` (U32
 * [>= workgroups]) receives an xor of every span, which keeps the loads alive and lets a test check
 * the read. */
int oxq_calib_read(oxq_ctx *ctx, void *stream, const oxq_tensor *src, int workgroups, int nontemporal,
                   const oxq_tensor *checksums);

/* The same read as the fastest matmul kernels issue it: `waves` waves (8 or 16) per workgroup, every
 * lane requesting its whole share - span / (waves * 1 KiB) loads of 16 bytes, at most 32 - before it
 * waits for the first.  Size of `src`: a multiple of workgroups * waves * 1 KiB, at most 32 KiB per
 * wave.  What this takes for a byte count is the best a read-once kernel has been seen to do here. */
int oxq_bench_read_upfront(oxq_ctx *ctx, void *stream, const oxq_tensor *src, int workgroups, int waves,
                           int nontemporal, const oxq_tensor *checksums);

/* Two request streams from every compute unit.  Workgroups of 12 waves: waves 0 - 7 read the workgroup's
 * span of `w` (U8; workgroups x 64, 128 or 136 KiB; cold, so from HBM) with everything requested first, waves
 * 8 - 11 read all of `x` (U8, a multiple of 32 KiB; the same bytes in every workgroup, so L2 hits) straight
 * into LDS, as a tile kernel stages its activations.  which = 1: only w, 2: only x, 3: both at once.  On
 * this machine "both" takes about the sum of the two, not the larger (a compute unit serves its vector-memory
 * requests in issue order): that is the price of the activation rows a tile kernel re-reads per strip. */
int oxq_bench_two_streams(oxq_ctx *ctx, void *stream, const oxq_tensor *w, const oxq_tensor *x, int workgroups,
                          int which, const oxq_tensor *checksums);

/* An empty kernel with the given launch shape (threads a multiple of 64, up to 1024; lds_bytes of
 * dynamic LDS, up to 160 KiB): what one launch costs when it does nothing. */
int oxq_bench_empty_launch(oxq_ctx *ctx, void *stream, int workgroups, int threads, int lds_bytes);

/* A launch that does nothing but one grid barrier: thread 0 of every workgroup takes a ticket from the
 * device-scope counter state[0] and polls it until its round is complete; after spin_limit polls
 * (1 .. 4194304) it gives up, sets state[1] to 1 and leaves, so every wave exits.  `state`: two zeroed
 * 32-bit words on the device, never reset between launches.  workgroups must all be resident at once (at
 * most one per compute unit at more than 512 threads, two below).  Against oxq_bench_empty_launch: what a
 * persistent kernel would pay to make one layer's outputs visible to the next inside one launch. */
int oxq_bench_grid_barrier(oxq_ctx *ctx, void *stream, int workgroups, int threads, const oxq_tensor *state,
                           uint32_t spin_limit);

#ifdef __cplusplus
}
#endif
#endif
