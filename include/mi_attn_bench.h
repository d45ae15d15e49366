/*
 * mi_attn_bench.h - timing helper for benchmarks of the mi_attn.h entry points.
 *
 * Kept apart from mi_attn.h because, unlike everything declared there, this
 * call creates HIP events and blocks the calling thread.  It has no
 * counterpart in the reference (which times with triton.testing.do_bench,
 * e.g. tutorial/4.4.causal_attention.py:296-309).
 */
#ifndef MI_ATTN_BENCH_H
#define MI_ATTN_BENCH_H

#include "mi_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Average device time per launch, measured with HIP events on `stream` around
 * `iters` back-to-back launches of the given entry point (after `warmup`
 * untimed ones).
 * kind: 0 = mi_attn_fwd, 1 = mi_attn_fwd_blocksparse, 2 = mi_decode,
 *       3 = mi_decode_splitkv, 4 = mi_decode_merge, 5 = mi_attn_bwd,
 *       6 = mi_rmsnorm_fwd, 7 = mi_rmsnorm_bwd, 8 = mi_xent_fwd,
 *       9 = mi_xent_dlogits, 10 = mi_xent_bwd_dlogits, 11 = mi_decode_noalloc.
 * `args` points to `n_args` argument structs of that entry point laid out
 * `arg_stride` bytes apart; launch i uses struct i % n_args, so a benchmark can
 * rotate inputs that would otherwise stay in the last-level cache.
 * Returns MI_OK and writes milliseconds to *ms_per_launch. */
int mi_time_launches(int kind, const void *args, int n_args, size_t arg_stride,
                     void *stream, int warmup, int iters, float *ms_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* MI_ATTN_BENCH_H */
