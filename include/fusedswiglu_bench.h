/*
 * libfusedswiglu_bench -- machine probes for the benchmark harness.  Not part of the drop-in boundary
 * (include/fusedswiglu.h) and not linked into libfusedswiglu.so: a separate library built from
 * fusedswiglu_amd/csrc/fsw_probe.hip.  Status codes are those of fusedswiglu.h.
 */
#ifndef FUSEDSWIGLU_BENCH_H_
#define FUSEDSWIGLU_BENCH_H_

#include <stdint.h>

/* Every entry point is exported with default visibility; the libraries hide everything else. */
#ifndef FSW_API
#define FSW_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

/*
 * No counterpart in the reference.  Each call enqueues one
 * kernel on `stream`; the caller times it with events.  sink4 is a 4-byte device scratch word.
 * fsw_probe_mfma: `workgroups` x 8 waves issue `iters` x 8 back-to-back 32x32x16 bf16 MFMAs from
 * registers (operands constant, or ~N(0,1) if random_operands != 0); *flop_out receives the flop count.
 * fsw_probe_stream_read: grid-stride non-temporal 16-byte reads of `bytes` bytes at buf (16-byte aligned), eight
 * in flight per lane: the rate of a plain streaming kernel, for orientation (not a bound - the product's own
 * streaming kernels may exceed it).
 * fsw_probe_dma_read: every byte of buf (a multiple of 1 KiB, < 2 GiB) once through direct global->LDS loads of
 * whole 128-byte lines, as the tiled and weight-streaming kernels read; non_temporal != 0 adds their hint for
 * read-once operands.  Known traffic for scaling the profiler's byte counters per request pattern.
 * fsw_probe_mfma_mix: `workgroups` x 8 waves issue `iters` x 32 16x16x32 bf16 MFMAs on ~N(0,1) operands
 * with, per 8 MFMAs, the data movement of mix 0: none, 1: three 16-byte LDS reads per lane + one 1 KiB
 * direct global->LDS load per wave (what the tiled kernels do), 2: two reads + one load, 3: three reads,
 * 4: one load, 5: mix 1 with the weight-side fragment of each 8 MFMAs FORMED from the three values read (taken as
 * dout, g, u): four gating gradients per lane and 8 MFMAs, the arithmetic a weight-gradient GEMM would carry in its
 * operand path if the gating-gradient kernel were folded into it.  The loads walk `bytes` bytes at buf (a multiple of
 * 256 KiB, >= 1 MiB, < 2 GiB).
 */
FSW_API int fsw_probe_mfma(int random_operands, int iters, int workgroups, void* sink4, void* stream,
                   double* flop_out);
FSW_API int fsw_probe_stream_read(const void* buf, int64_t bytes, void* sink4, void* stream);
FSW_API int fsw_probe_dma_read(const void* buf, int64_t bytes, int non_temporal, void* stream);
FSW_API int fsw_probe_mfma_mix(int mix, int iters, int workgroups, const void* buf, int64_t bytes, void* sink4,
                       void* stream, double* flop_out);

#ifdef __cplusplus
}
#endif
#endif /* FUSEDSWIGLU_BENCH_H_ */
