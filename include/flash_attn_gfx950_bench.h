/*
 * flash_attn_gfx950_bench.h -- instrumentation entry point of libflash_attn_gfx950.so for benchmarks.  Not part of the
 * drop-in boundary (include/flash_attn_gfx950.h): no counterpart in the reference, nothing a binding needs.
 */
#ifndef FLASH_ATTN_GFX950_BENCH_H_
#define FLASH_ATTN_GFX950_BENCH_H_

#include "flash_attn_gfx950.h"

#ifdef __cplusplus
extern "C" {
#endif

/* fa_bwd with two timing events (hipEvent_t, either may be NULL) recorded on args->stream immediately before and after the
 * backward's longest kernel: the dK/dV kernel of the two-kernel backward (dQ + softmax_d kernel first, then dK/dV), or the
 * main kernel of the one-kernel backward.  For benchmarks that price that kernel against its roofline with events on the
 * stream it runs on.  Results are those of fa_bwd. */
int fa_bwd_profiled(const fa_bwd_args* args, void* ev_main_start, void* ev_main_stop);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_ATTN_GFX950_BENCH_H_ */
