// Host-side declarations shared by the translation units of libfusedswiglu.
#pragma once
#include "fsw_common.hpp"

namespace fsw {

// dtype codes used across the library (the C ABI's FSW_DTYPE_* values)
constexpr int kDtypeBF16 = 0;
constexpr int kDtypeFP16 = 1;

struct Problem {
  const void *x, *wg, *wu;       // x [T,D]; Wg, Wu [D,I]
  const void *dG, *dU;           // [T,I]
  void *out, *g, *u;             // [T,I]   (g, u may be null in the forward)
  const void* dout;              // [T,I]   non-null: the forward recomputes g, u and writes the gating
                                 //         gradients dG -> g, dU -> u instead (out is not written)
  void *dx;                      // [T,D]
  void *dWg, *dWu;               // [D,I]
  long long T, D, I;
  long long ldx, ldw, ldo;       // leading dimensions (elements) of x, the weights, the [T,I] arrays
  long long lddx, lddw;          // of dx and of dWg/dWu
  bool w_out_in;                 // weights and their gradients are [I,D] (nn.Linear's layout) instead of [D,I]
};

// A plain GEMM on the same kernels (the down projection that follows the SwiGLU and its two gradients).
// layout 0: C = A B (A [M,K], B [K,N]); 1: C = A B^T (B [N,K]); 2: C = A^T B (A [K,M], B [K,N]); all row-major.
struct GemmProblem {
  const void *a, *b;
  void* c;
  long long M, N, K, lda, ldb, ldc;
  int layout;
};
bool fast_path_ok_gemm(const GemmProblem& p);
hipError_t launch_gemm_fast(int dtype, const GemmProblem& p, hipStream_t s, void* ws, long long ws_bytes);
hipError_t launch_gemm_generic(int dtype, const GemmProblem& p, hipStream_t s);
long long gemm_workspace_bytes(int layout, long long M, long long N, long long K);

// Tiled direct-to-LDS MFMA kernels: need every dimension and leading dimension to be a multiple
// of 8 elements and every pointer 16-byte aligned.
bool fast_path_ok_forward(const Problem& p);
bool fast_path_ok_input_grad(const Problem& p);
bool fast_path_ok_weight_grad(const Problem& p);
hipError_t launch_forward_fast(int dtype, const Problem& p, hipStream_t s);
hipError_t launch_input_grad_fast(int dtype, const Problem& p, hipStream_t s, void* ws, long long ws_bytes);
hipError_t launch_weight_grad_fast(int dtype, const Problem& p, hipStream_t s, void* ws, long long ws_bytes);
// Bytes of fp32 scratch that let small input-grad (step 1; 4 for [I,D] weights) / weight-grad (step 2; 5)
// problems split their reduction and, with_tail, large ones share the tiles of a short last round (at most
// 64 MiB; without that scratch they run exactly as before).
long long splitk_workspace_bytes(int step, long long T, long long D, long long I, bool with_tail = true);

// Weight-streaming forward for T <= 128 tokens (same eligibility as the tiled forward otherwise).
bool skinny_forward_ok(const Problem& p);
hipError_t launch_forward_skinny(int dtype, const Problem& p, hipStream_t s);

// The same kernel as a plain GEMM for the down projection of few tokens (layouts 0 and 1, M <= 128, N even and
// its half aligned); splits the reduction into the caller's scratch when column blocks alone leave CUs idle.
bool skinny_gemm_ok(const GemmProblem& p);
long long skinny_gemm_workspace_bytes(int layout, long long M, long long N, long long K);
hipError_t launch_gemm_skinny(int dtype, const GemmProblem& p, hipStream_t s, void* ws, long long ws_bytes);

// Any shape, any stride, 2-byte alignment: guarded element loads, same MFMA arithmetic.
hipError_t launch_forward_generic(int dtype, const Problem& p, hipStream_t s);
hipError_t launch_input_grad_generic(int dtype, const Problem& p, hipStream_t s);
hipError_t launch_weight_grad_generic(int dtype, const Problem& p, hipStream_t s);

hipError_t launch_elementwise(int dtype, const void* dout, const void* g, const void* u, void* dU,
                              void* dG, size_t n, hipStream_t stream);

}  // namespace fsw
