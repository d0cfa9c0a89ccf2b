/* Measurement aids of bench.py, exported by libtvmkv_bench.so (NOT part of the drop-in library
 * libtvmkv.so and without a counterpart in the reference).  Plain pointers and sizes; every function
 * returns 0 or a non-zero code (-1: bad argument, otherwise the hipError_t of the launch). */
#ifndef TVMKV_BENCH_H_
#define TVMKV_BENCH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming read (XOR-folded, the result is discarded) and a plain copy of `num_bytes` (a
 * multiple of 16) bytes: what the memory system of the box gives the simplest kernels, and dispatches of
 * known size to scale the FETCH_SIZE / WRITE_SIZE counters with.  `sink` is 4 writable bytes. */
int tvmkvb_stream_read(const void* src, int64_t num_bytes, void* sink, void* stream);
/* the same read with non-temporal loads, the kind the decode kernel issues */
int tvmkvb_stream_read_nt(const void* src, int64_t num_bytes, void* sink, void* stream);
int tvmkvb_stream_copy(const void* src, void* dst, int64_t num_bytes, void* stream);
/* `workgroups` workgroups of 4 waves run `iters` rounds of 8 v_mfma_f32_32x32x16_f16 each (4
 * accumulators, nothing else in the loop) on the A and B fragments read from `operands` (256 lanes x 16
 * halfs); `out` gets workgroups x 256 floats.  2 * 32 * 32 * 16 * 8 * iters * 4 * workgroups flop. */
int tvmkvb_mfma_loop(const void* operands, float* out, int32_t iters, int32_t workgroups, void* stream);
#ifdef __cplusplus
}
#endif
#endif /* TVMKV_BENCH_H_ */
