/* odmkv_bench.h - measurement entry points of libodmkv_bench.so (no counterpart in the reference).
 *
 * libodmkv_bench.so is libodmkv.so's object files plus this translation unit (csrc/bench_hooks.hip);
 * the product library exports none of these.  Nothing here keeps state between calls except the
 * timer object the caller creates, owns and destroys.
 */
#ifndef ODMKV_BENCH_H
#define ODMKV_BENCH_H

#include "odmkv.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A pool of HIP event pairs owned by the caller.  odmkv_bench_decode_attn attaches the next free
 * pair to its main kernel's dispatch (the kernel's own start and end timestamps);
 * odmkv_bench_timer_collect waits for the pairs used so far, returns their durations in
 * milliseconds and makes the pool empty again.  One thread at a time per timer. */
int odmkv_bench_timer_create(int max_records, void** timer);
int odmkv_bench_timer_collect(void* timer, float* ms, int capacity, int* n_out);
int odmkv_bench_timer_destroy(void* timer);

/* odmkv_decode_attn with the stages chosen per call: bit 0 the query preparation, bit 1 the main
 * (streaming) kernel, bit 2 the merge at its end.  7 is the product call; 2 times the streaming part
 * alone over buffers a full call has filled (its output is then not written).  timer: NULL, or a
 * timer whose next event pair is attached to the main kernel. */
int odmkv_bench_decode_attn(const void* q, int q_dtype, int B, int Hq, float scaling,
                            const odmkv_packed_t* store, const odmkv_worklist_t* work,
                            const uint16_t* pi_k_ops, const float* pi_v, const float* codebooks,
                            const float* codebooks_host, const float* inv_scales,
                            void* out, int out_dtype, float* lse, void* workspace, size_t workspace_bytes,
                            void* stream, int stage_mask, void* timer);

/* Yardstick for the roofline: a plain streaming read of `bytes` bytes at `buf` (device, 16-byte
 * aligned) by `grid` workgroups of 256 threads; `sink` is a device word that is practically never
 * written.  Timing it over buffers that rotate through more than the last-level cache shows what
 * one launch of that size can reach on the machine. */
int odmkv_bench_probe_read(const void* buf, size_t bytes, int grid, void* sink, void* stream);

/* After odmkv_quant_pack(B, Hkv, T, ..., workspace) with fp16 or bf16 tensors: how many key tiles (counts[0]) and
 * value tiles (counts[1]) of that call the matrix-core quantiser handed to the exact one (8-bit tiles,
 * tiles with a row whose norm is not finite, tiles with more values next to a decision threshold than
 * its list holds).  counts: host int32[2].  Waits for the stream. */
int odmkv_bench_pack_handed_over(const void* workspace, int B, int Hkv, int T, int32_t* counts, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ODMKV_BENCH_H */
