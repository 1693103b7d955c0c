/*
 * pkh3_attn_bench.h -- measurement hook of libpkh3attn.so.  Not part of the product interface
 * (include/pkh3_attn.h): it is the one export that synchronises with the device, and only
 * benchmark harnesses call it.  It replaces nothing in the reference, which publishes no kernel
 * timings (it records wall-clock per pipeline stage, src/pika_h3/pipeline.py:91-93,168).
 */
#ifndef PKH3_ATTN_BENCH_H
#define PKH3_ATTN_BENCH_H

#include "pkh3_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Runs `iters` back-to-back launches of ONLY the attention kernel of the given call (the prologue
   that normalises/rotates/lays out K and V runs once before), brackets them with HIP events on
   `stream`, and returns the mean milliseconds per launch in *ms_out.  Synchronises. */
int pkh3_attn_time_kernel(const pkh3_attn_args* a, void* stream, int iters, float* ms_out);

#ifdef __cplusplus
}
#endif
#endif
