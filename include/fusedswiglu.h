/*
 * libfusedswiglu -- C ABI of the MI355X (gfx950) fused SwiGLU forward/backward.
 *
 * This is the drop-in boundary underneath the two autograd Functions of
 * fattorib/fusedswiglu (`FusedSwiGLU`, fused_swiglu/swiglu.py:16-58, and
 * `FastAccumFusedSwiGLU`, fused_swiglu/swiglu_f16.py:16-58).  The reference has no
 * FFI of its own: its seam is the three Python launchers in
 * fused_swiglu/kernels/kernels_bf16.py (and the fp16 twins in kernels_fp16.py), plus one
 * line of torch matmuls for the input gradient.  Each entry point below replaces one of
 * those and is what a ctypes / pybind / cgo binding for this path would bind.
 *
 * Conventions
 *   - T = number of tokens (all leading dimensions of x flattened), D = d_model,
 *     I = d_intermediate.  All matrices are row-major with unit inner stride; `ld*`
 *     arguments are leading dimensions (row pitches) in ELEMENTS.
 *   - Every pointer is a device pointer on the current HIP device.  The caller owns every
 *     buffer; the library never allocates, frees or keeps a pointer after returning.
 *   - `dtype` selects 16-bit storage: FSW_DTYPE_BF16 or FSW_DTYPE_FP16 (optionally | FSW_WEIGHTS_OUT_IN).  Products are
 *     accumulated in fp32 on the MFMA units for both (CDNA4 has no fp16-accumulate mode,
 *     so the reference's fp16 "fast accumulation" maps to fp32 accumulation).
 *   - `stream` is a hipStream_t (NULL = the default stream).  Calls only enqueue work; they
 *     never synchronize.  The library keeps no state between calls and is re-entrant (the one
 *     exception, the built-in scratch of fsw_input_grad_noalloc, is described there).
 *   - Return value: FSW_OK or an FSW_ERR_* code; arguments are validated before anything is
 *     enqueued.  fsw_last_error() gives a thread-local message for the last failure.
 *   - Operands whose dimensions and leading dimensions are multiples of 8 elements and whose
 *     pointers are 16-byte aligned run on the tiled direct-to-LDS MFMA kernels; anything else
 *     runs on a slower edge-shape kernel with identical arithmetic.
 */
#ifndef FUSEDSWIGLU_H_
#define FUSEDSWIGLU_H_

#include <stdint.h>

/* Every entry point is exported with default visibility; the libraries hide everything else. */
#ifndef FSW_API
#define FSW_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* major*10000 + minor*100 + patch.
 * 0.4.0: fsw_swiglu_backward (the three backward steps in one call).
 * 0.3.0: FSW_WEIGHTS_OUT_IN, the fsw_down_proj_* entry points, fsw_input_grad_noalloc and status 7,
 *        fsw_uses_tiled_kernel answers 2 for the weight-streaming kernels and knows steps 4 / 5 / 6,
 *        fsw_workspace_bytes may ask for up to 64 MiB for large gradient GEMMs (tail split).
 * 0.2.0: fsw_gating_grad_recompute. */
#define FSW_VERSION 400

enum { FSW_DTYPE_BF16 = 0, FSW_DTYPE_FP16 = 1 };
/* May be OR-ed into any `dtype` argument (and into the `step` of fsw_workspace_bytes): the weights of the
 * call - w_gate, w_up, w_down and their gradients - are stored "out x in" like torch.nn.Linear.weight, i.e.
 * w_gate, w_up [I, D] and w_down [D, I], instead of the reference's "in x out" ([D, I]; README.md:26-27,
 * fused_swiglu/test_swiglu.py:30-35).  `ldw` / `ld_dw` are then leading dimensions of those arrays.  Nothing is
 * transposed in memory: other variants of the tiled kernels and of the weight-streaming kernel (T <= 128) read
 * and write the layout in place. */
#define FSW_WEIGHTS_OUT_IN 0x100

enum {
  FSW_OK = 0,
  FSW_ERR_NULL_POINTER = 1,
  FSW_ERR_BAD_DTYPE = 2,
  FSW_ERR_BAD_SHAPE = 3,  /* a dimension is <= 0 or exceeds 2^31-1 */
  FSW_ERR_BAD_STRIDE = 4, /* a leading dimension is smaller than the row it describes */
  FSW_ERR_ALIGNMENT = 5,  /* a pointer is not 2-byte aligned */
  FSW_ERR_LAUNCH = 6,     /* the HIP runtime refused the launch; see fsw_last_error() */
  FSW_ERR_SCRATCH_LIMIT = 7 /* fsw_input_grad_noalloc: the problem needs more than FSW_NOALLOC_SCRATCH_BYTES */
};

/* Library version (FSW_VERSION it was built with). */
FSW_API int fsw_version(void);
/* Static description of a status code. */
FSW_API const char* fsw_status_string(int status);
/* Message of the calling thread's most recent failed call ("" if none). */
FSW_API const char* fsw_last_error(void);
/* Which kernel the arguments of the named step would run on: 1 the tiled MFMA kernels, 2 the
 * weight-streaming kernel (at most 128 tokens: the forward, and the down projection and its input gradient
 * when half their result columns are a multiple of 8 elements for a k-contiguous W_down - [D,I] in the
 * forward, [I,D] in the input gradient - and of 64 otherwise), 0 the edge-shape kernel.
 * step: 0 forward, 1 input_grad, 2 weight_grad, 3 gating_grad_recompute, 4 / 5 / 6 down projection forward /
 * input gradient / weight gradient, each optionally | FSW_WEIGHTS_OUT_IN.  ldx: the [T,D] arrays, ldw: the
 * weights, ldo: the [T,I] arrays, ld_grad: grad_x or the weight gradient.  Pure host logic. */
FSW_API int fsw_uses_tiled_kernel(int step, int64_t T, int64_t D, int64_t I, int64_t ldx, int64_t ldw,
                          int64_t ldo, int64_t ld_grad, unsigned pointer_alignment);

/*
 * Forward: g = x Wg, u = x Wu, out = silu(g) * u.
 * Replaces fused_swiglu_fwd + swiglu_kernel (fused_swiglu/kernels/kernels_bf16.py:162-206,
 * :41-160; fp16: kernels_fp16.py:171-216).
 *   x [T,D] (ldx)   w_gate, w_up [D,I] (ldw)   out, xw_gate, xw_up [T,I] (ldo)
 * xw_gate and xw_up (the pre-activations the backward needs) may both be NULL, in which
 * case they are not written (inference).
 */
FSW_API int fsw_swiglu_forward(const void* x, const void* w_gate, const void* w_up, void* out,
                       void* xw_gate, void* xw_up, int64_t T, int64_t D, int64_t I, int64_t ldx,
                       int64_t ldw, int64_t ldo, int dtype, void* stream);

/*
 * Gating gradient: grad_xw_up = grad_out * silu(xw_gate),
 *                  grad_xw_gate = grad_out * xw_up * silu'(xw_gate).
 * Replaces elementwise_backward + kernel (kernels_bf16.py:236-255, :210-234).  All five
 * arrays are dense with `numel` elements.
 */
FSW_API int fsw_elementwise_backward(const void* grad_out, const void* xw_gate, const void* xw_up,
                             void* grad_xw_up, void* grad_xw_gate, int64_t numel, int dtype,
                             void* stream);

/*
 * Gating gradient without saved pre-activations: recomputes g = x Wg and u = x Wu (fp32, never
 * stored) and writes grad_xw_up = grad_out * silu(g), grad_xw_gate = grad_out * u * silu'(g).
 * Stands in for the pair "save x@Wg, x@Wu in the forward (fused_swiglu/swiglu.py:28) + elementwise_backward
 * (kernels_bf16.py:236-255)" for callers that prefer 4*T*D*I extra flops to keeping 2*T*I saved
 * elements per layer; the reference has no such mode.
 *   x [T,D] (ldx)   w_gate, w_up [D,I] (ldw)   grad_out, grad_xw_up, grad_xw_gate [T,I] (ldo)
 */
FSW_API int fsw_gating_grad_recompute(const void* x, const void* w_gate, const void* w_up,
                              const void* grad_out, void* grad_xw_up, void* grad_xw_gate, int64_t T,
                              int64_t D, int64_t I, int64_t ldx, int64_t ldw, int64_t ldo, int dtype,
                              void* stream);

/*
 * Optional scratch for the two gradient GEMMs.  When a problem has too few output tiles to fill the
 * chip (small d_model), several workgroups split the reduction of one tile, write fp32 partial
 * tiles to `workspace` (device memory owned by the caller, 16-byte aligned, contents irrelevant) and
 * a second kernel adds them in a fixed order.  Large problems whose tiles leave a short last round of
 * workgroups use it the same way for the tiles of that round only (at most 64 MiB).  The few-token down
 * projection plans its split with the compute-unit count of the current device: query and call with the
 * same device current.  fsw_workspace_bytes gives a sufficient size for
 * step 1 (input_grad), 2 (weight_grad), 4 / 5 / 6 (down projection forward / input grad / weight grad),
 * each optionally | FSW_WEIGHTS_OUT_IN; with workspace == NULL or a smaller size the call still
 * works, just without the split.
 */
FSW_API int64_t fsw_workspace_bytes(int step, int64_t T, int64_t D, int64_t I);

/*
 * Input gradient: grad_x = grad_xw_gate Wg^T + grad_xw_up Wu^T, one kernel, one accumulator.
 * Replaces the two torch matmuls and the add at fused_swiglu/swiglu.py:45.
 *   grad_xw_gate, grad_xw_up [T,I] (ldo)   w_gate, w_up [D,I] (ldw)   grad_x [T,D] (ld_dx)
 */
FSW_API int fsw_input_grad(const void* grad_xw_gate, const void* grad_xw_up, const void* w_gate,
                   const void* w_up, void* grad_x, int64_t T, int64_t D, int64_t I, int64_t ldo,
                   int64_t ldw, int64_t ld_dx, void* workspace, int64_t workspace_bytes, int dtype,
                   void* stream);

/*
 * fsw_input_grad for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * arguments and results as fsw_input_grad, but the fp32 scratch of the split reduction is a buffer of
 * FSW_NOALLOC_SCRATCH_BYTES built into the library (one copy per GPU, held until the process ends)
 * instead of a caller workspace; the call itself allocates and frees nothing.  Small problems whose
 * split reduction needs more than that size are rejected with FSW_ERR_SCRATCH_LIMIT (large problems need no
 * scratch and always pass; the optional tail split of a large problem uses the buffer when it fits and is
 * skipped when it does not).  Results are bit-identical to fsw_input_grad called with a workspace of
 * FSW_NOALLOC_SCRATCH_BYTES; fsw_input_grad with a larger workspace may split a tail that this call does not,
 * and then sums in another order (the last bit of a few results in ten thousand differs, the error does not).
 * All calls on one GPU share that GPU's buffer:
 * calls that overlap in time on one GPU (different streams or threads) race on it.  The first call
 * on a device looks the buffer's address up; make that call outside graph capture.
 */
#define FSW_NOALLOC_SCRATCH_BYTES (32u << 20)
FSW_API int fsw_input_grad_noalloc(const void* grad_xw_gate, const void* grad_xw_up, const void* w_gate,
                           const void* w_up, void* grad_x, int64_t T, int64_t D, int64_t I, int64_t ldo,
                           int64_t ldw, int64_t ld_dx, int dtype, void* stream);

/*
 * Weight gradients: grad_w_gate = x^T grad_xw_gate, grad_w_up = x^T grad_xw_up, reduced over
 * all T tokens in fp32.  Replaces fused_bmm + bmm_kernel (kernels_bf16.py:385-412, :280-382)
 * together with the batch sum `unbroadcast` (fused_swiglu/swiglu.py:11-13, :56-57).
 *   x [T,D] (ldx)   grad_xw_up, grad_xw_gate [T,I] (ldo)   grad_w_up, grad_w_gate [D,I] (ld_dw)
 * Argument order (up before gate) follows fused_bmm.
 */
FSW_API int fsw_weight_grad(const void* x, const void* grad_xw_up, const void* grad_xw_gate,
                    void* grad_w_up, void* grad_w_gate, int64_t T, int64_t D, int64_t I,
                    int64_t ldx, int64_t ldo, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                    int dtype, void* stream);

/*
 * The whole backward of the path in one call: the body of FusedSwiGLU.backward (fused_swiglu/swiglu.py:34-58).
 * Exactly fsw_elementwise_backward, then fsw_weight_grad (if the two weight gradients are given), then fsw_input_grad
 * (if grad_x is given), enqueued on `stream` in that order - for hosts where three calls through a foreign-function
 * interface cost more than the small kernels they launch.
 *   grad_out, xw_gate, xw_up, grad_xw_gate, grad_xw_up [T,I] dense (leading dimension I)
 *   x [T,D] (ldx)   w_gate, w_up (ldw)   grad_x [T,D] (ld_dx)   grad_w_gate, grad_w_up (ld_dw)
 * grad_xw_gate and grad_xw_up are results too (the gating gradients), always written.  grad_x may be NULL, and
 * grad_w_gate / grad_w_up both NULL: that gradient is skipped (ctx.needs_input_grad).  `workspace` is used by the
 * two GEMMs one after the other: the larger of fsw_workspace_bytes(1, ...) and fsw_workspace_bytes(2, ...) serves both.
 */
FSW_API int fsw_swiglu_backward(const void* grad_out, const void* xw_gate, const void* xw_up, const void* x,
                        const void* w_gate, const void* w_up, void* grad_xw_gate, void* grad_xw_up, void* grad_x,
                        void* grad_w_gate, void* grad_w_up, int64_t T, int64_t D, int64_t I, int64_t ldx,
                        int64_t ldw, int64_t ld_dx, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                        int dtype, void* stream);

/*
 * The down projection that follows the SwiGLU in an MLP block, y = act W_down, and its two gradients, on the
 * same tiled kernels.  The reference stops at FusedSwiGLU.apply (README.md:25-38: the caller multiplies by
 * its own down weight); these three entry points are that next step for callers that want the whole block from
 * one library.  act = the SwiGLU output.
 *   act, grad_act [T,I] (ld_act)   w_down, grad_w_down [I,D] (ldw, ld_dw; [D,I] with FSW_WEIGHTS_OUT_IN)
 *   y, grad_y [T,D] (ldy)
 *   forward      y           = act W_down
 *   input_grad   grad_act    = grad_y W_down^T
 *   weight_grad  grad_w_down = act^T grad_y      (summed over all T tokens in fp32)
 * `workspace` as for fsw_input_grad (steps 4, 5, 6 of fsw_workspace_bytes).  Up to 128 tokens, forward and
 * input_grad stream the weight once from HBM on the kernel of the few-token SwiGLU forward; the result is then
 * short (D or I columns) and the reduction long, so the reduction is split over the CUs through `workspace`
 * (without it the call is correct but leaves most CUs idle).
 */
FSW_API int fsw_down_proj_forward(const void* act, const void* w_down, void* y, int64_t T, int64_t I, int64_t D,
                                  int64_t ld_act, int64_t ldw, int64_t ldy, void* workspace,
                                  int64_t workspace_bytes, int dtype, void* stream);
FSW_API int fsw_down_proj_input_grad(const void* grad_y, const void* w_down, void* grad_act, int64_t T, int64_t I,
                                     int64_t D, int64_t ldy, int64_t ldw, int64_t ld_act, void* workspace,
                                     int64_t workspace_bytes, int dtype, void* stream);
FSW_API int fsw_down_proj_weight_grad(const void* act, const void* grad_y, void* grad_w_down, int64_t T, int64_t I,
                                      int64_t D, int64_t ld_act, int64_t ldy, int64_t ld_dw, void* workspace,
                                      int64_t workspace_bytes, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FUSEDSWIGLU_H_ */
