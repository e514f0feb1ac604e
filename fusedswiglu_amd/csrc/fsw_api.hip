// extern "C" entry points of libfusedswiglu: argument validation, kernel selection, status codes.
#include "../../include/fusedswiglu.h"
#include "fsw_internal.hpp"
#include <cstdarg>
#include <cstdio>
#include <algorithm>
#include <mutex>

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// `dtype` arguments carry the element type in the low byte and optional FSW_* layout flags above it
bool dtype_ok(int d) {
  const int e = d & 0xff;
  return (e == FSW_DTYPE_BF16 || e == FSW_DTYPE_FP16) && (d & ~(0xff | FSW_WEIGHTS_OUT_IN)) == 0;
}
int elem_of(int d) { return d & 0xff; }
bool out_in_of(int d) { return (d & FSW_WEIGHTS_OUT_IN) != 0; }
bool al2(const void* p) { return ((uintptr_t)p & 1) == 0; }

int check_dims(const char* fn, int64_t T, int64_t D, int64_t I) {
  if (T <= 0 || D <= 0 || I <= 0)
    return fail(FSW_ERR_BAD_SHAPE, "%s: dimensions must be positive (T=%lld D=%lld I=%lld)", fn,
                (long long)T, (long long)D, (long long)I);
  if (T > 0x7fffffffLL || D > 0x7fffffffLL || I > 0x7fffffffLL)
    return fail(FSW_ERR_BAD_SHAPE, "%s: dimension exceeds 2^31-1 (T=%lld D=%lld I=%lld)", fn,
                (long long)T, (long long)D, (long long)I);
  return FSW_OK;
}

int check_ld(const char* fn, const char* name, int64_t ld, int64_t cols) {
  if (ld < cols)
    return fail(FSW_ERR_BAD_STRIDE, "%s: leading dimension %s=%lld is smaller than the row length %lld",
                fn, name, (long long)ld, (long long)cols);
  return FSW_OK;
}

int launched(const char* fn, hipError_t e) {
  if (e != hipSuccess) return fail(FSW_ERR_LAUNCH, "%s: %s", fn, hipGetErrorString(e));
  return FSW_OK;
}

}  // namespace

extern "C" {

int fsw_version(void) { return FSW_VERSION; }

const char* fsw_status_string(int status) {
  switch (status) {
    case FSW_OK: return "ok";
    case FSW_ERR_NULL_POINTER: return "null pointer";
    case FSW_ERR_BAD_DTYPE: return "unsupported dtype";
    case FSW_ERR_BAD_SHAPE: return "bad shape";
    case FSW_ERR_BAD_STRIDE: return "bad leading dimension";
    case FSW_ERR_ALIGNMENT: return "pointer not 2-byte aligned";
    case FSW_ERR_LAUNCH: return "kernel launch failed";
    case FSW_ERR_SCRATCH_LIMIT: return "problem needs more scratch than the built-in buffer holds";
    default: return "unknown status";
  }
}

const char* fsw_last_error(void) { return g_err; }

int fsw_uses_tiled_kernel(int step, int64_t T, int64_t D, int64_t I, int64_t ldx, int64_t ldw,
                          int64_t ldo, int64_t ld_grad, unsigned pointer_alignment) {
  // stand-in pointers that carry only the alignment
  const void* ptr = (const void*)(uintptr_t)(pointer_alignment ? pointer_alignment : 1);
  fsw::Problem p{};
  p.x = p.wg = p.wu = p.dG = p.dU = ptr;
  p.out = p.g = p.u = p.dx = p.dWg = p.dWu = (void*)ptr;
  p.T = T; p.D = D; p.I = I; p.ldx = ldx; p.ldw = ldw; p.ldo = ldo; p.lddx = ld_grad; p.lddw = ld_grad;
  p.w_out_in = (step & FSW_WEIGHTS_OUT_IN) != 0;
  switch (step & 0xff) {
    case 0: return fsw::skinny_forward_ok(p) ? 2 : (fsw::fast_path_ok_forward(p) ? 1 : 0);
    case 3: return fsw::fast_path_ok_forward(p) ? 1 : 0;
    case 1: return fsw::fast_path_ok_input_grad(p) ? 1 : 0;
    case 2: return fsw::fast_path_ok_weight_grad(p) ? 1 : 0;
    default: break;
  }
  // the down projection: y, grad_y [T,D] (ldx)   w_down (ldw)   act, grad_act [T,I] (ldo)   grad_w_down (ld_grad)
  const bool oi = p.w_out_in;
  fsw::GemmProblem q{ptr, ptr, (void*)ptr, 0, 0, 0, 0, 0, 0, 0};
  switch (step & 0xff) {
    case 4: q.M = T; q.N = D; q.K = I; q.lda = ldo; q.ldb = ldw; q.ldc = ldx; q.layout = oi ? 1 : 0; break;
    case 5: q.M = T; q.N = I; q.K = D; q.lda = ldx; q.ldb = ldw; q.ldc = ldo; q.layout = oi ? 0 : 1; break;
    case 6:
      q.layout = 2; q.K = T; q.ldc = ld_grad;
      if (oi) { q.M = D; q.N = I; q.lda = ldx; q.ldb = ldo; }
      else { q.M = I; q.N = D; q.lda = ldo; q.ldb = ldx; }
      break;
    default: return 0;
  }
  if (!fsw::fast_path_ok_gemm(q)) return 0;
  return fsw::skinny_gemm_ok(q) ? 2 : 1;
}

int64_t fsw_workspace_bytes(int step, int64_t T, int64_t D, int64_t I) {
  if (T <= 0 || D <= 0 || I <= 0) return 0;
  const bool oi = (step & FSW_WEIGHTS_OUT_IN) != 0;
  switch (step & 0xff) {
    case 1: return fsw::splitk_workspace_bytes(oi ? 4 : 1, T, D, I);
    case 2: return fsw::splitk_workspace_bytes(oi ? 5 : 2, T, D, I);
    // down projection: forward y [T,D] over I; input grad [T,I] over D; weight grad [I,D] ([D,I]) over T
    case 4: return std::max(fsw::gemm_workspace_bytes(oi ? 1 : 0, T, D, I), fsw::skinny_gemm_workspace_bytes(oi ? 1 : 0, T, D, I));
    case 5: return std::max(fsw::gemm_workspace_bytes(oi ? 0 : 1, T, I, D), fsw::skinny_gemm_workspace_bytes(oi ? 0 : 1, T, I, D));
    case 6: return oi ? fsw::gemm_workspace_bytes(2, D, I, T) : fsw::gemm_workspace_bytes(2, I, D, T);
    default: return 0;
  }
}

int fsw_swiglu_forward(const void* x, const void* w_gate, const void* w_up, void* out,
                       void* xw_gate, void* xw_up, int64_t T, int64_t D, int64_t I, int64_t ldx,
                       int64_t ldw, int64_t ldo, int dtype, void* stream) {
  const char* fn = "fsw_swiglu_forward";
  if (!x || !w_gate || !w_up || !out) return fail(FSW_ERR_NULL_POINTER, "%s: x, w_gate, w_up and out must be non-null", fn);
  if ((xw_gate == nullptr) != (xw_up == nullptr))
    return fail(FSW_ERR_NULL_POINTER, "%s: xw_gate and xw_up must both be given or both be null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  const bool oi = out_in_of(dtype);
  dtype = elem_of(dtype);
  if (int e = check_ld(fn, "ldx", ldx, D)) return e;
  if (int e = check_ld(fn, "ldw", ldw, oi ? D : I)) return e;
  if (int e = check_ld(fn, "ldo", ldo, I)) return e;
  if (!al2(x) || !al2(w_gate) || !al2(w_up) || !al2(out) || !al2(xw_gate) || !al2(xw_up))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  fsw::Problem p{};
  p.x = x; p.wg = w_gate; p.wu = w_up; p.out = out; p.g = xw_gate; p.u = xw_up;
  p.T = T; p.D = D; p.I = I; p.ldx = ldx; p.ldw = ldw; p.ldo = ldo; p.w_out_in = oi;
  hipStream_t s = (hipStream_t)stream;
  if (fsw::skinny_forward_ok(p)) return launched(fn, fsw::launch_forward_skinny(dtype, p, s));
  if (fsw::fast_path_ok_forward(p)) return launched(fn, fsw::launch_forward_fast(dtype, p, s));
  return launched(fn, fsw::launch_forward_generic(dtype, p, s));
}

int fsw_gating_grad_recompute(const void* x, const void* w_gate, const void* w_up,
                              const void* grad_out, void* grad_xw_up, void* grad_xw_gate, int64_t T,
                              int64_t D, int64_t I, int64_t ldx, int64_t ldw, int64_t ldo, int dtype,
                              void* stream) {
  const char* fn = "fsw_gating_grad_recompute";
  if (!x || !w_gate || !w_up || !grad_out || !grad_xw_up || !grad_xw_gate)
    return fail(FSW_ERR_NULL_POINTER, "%s: all six arrays must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  const bool oi = out_in_of(dtype);
  dtype = elem_of(dtype);
  if (int e = check_ld(fn, "ldx", ldx, D)) return e;
  if (int e = check_ld(fn, "ldw", ldw, oi ? D : I)) return e;
  if (int e = check_ld(fn, "ldo", ldo, I)) return e;
  if (!al2(x) || !al2(w_gate) || !al2(w_up) || !al2(grad_out) || !al2(grad_xw_up) || !al2(grad_xw_gate))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  fsw::Problem p{};
  p.x = x; p.wg = w_gate; p.wu = w_up; p.dout = grad_out; p.g = grad_xw_gate; p.u = grad_xw_up;
  p.T = T; p.D = D; p.I = I; p.ldx = ldx; p.ldw = ldw; p.ldo = ldo; p.w_out_in = oi;
  hipStream_t s = (hipStream_t)stream;
  if (fsw::fast_path_ok_forward(p)) return launched(fn, fsw::launch_forward_fast(dtype, p, s));
  return launched(fn, fsw::launch_forward_generic(dtype, p, s));
}

int fsw_elementwise_backward(const void* grad_out, const void* xw_gate, const void* xw_up,
                             void* grad_xw_up, void* grad_xw_gate, int64_t numel, int dtype,
                             void* stream) {
  const char* fn = "fsw_elementwise_backward";
  if (!grad_out || !xw_gate || !xw_up || !grad_xw_up || !grad_xw_gate)
    return fail(FSW_ERR_NULL_POINTER, "%s: all five arrays must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  dtype = elem_of(dtype);
  if (numel <= 0) return fail(FSW_ERR_BAD_SHAPE, "%s: numel must be positive (got %lld)", fn, (long long)numel);
  if (!al2(grad_out) || !al2(xw_gate) || !al2(xw_up) || !al2(grad_xw_up) || !al2(grad_xw_gate))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  return launched(fn, fsw::launch_elementwise(dtype, grad_out, xw_gate, xw_up, grad_xw_up, grad_xw_gate,
                                              (size_t)numel, (hipStream_t)stream));
}

static int check_input_grad_args(const char* fn, const void* grad_xw_gate, const void* grad_xw_up,
                                 const void* w_gate, const void* w_up, void* grad_x, int64_t T, int64_t D,
                                 int64_t I, int64_t ldo, int64_t ldw, int64_t ld_dx, int dtype) {
  if (!grad_xw_gate || !grad_xw_up || !w_gate || !w_up || !grad_x)
    return fail(FSW_ERR_NULL_POINTER, "%s: all five arrays must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  if (int e = check_ld(fn, "ldo", ldo, I)) return e;
  if (int e = check_ld(fn, "ldw", ldw, out_in_of(dtype) ? D : I)) return e;
  if (int e = check_ld(fn, "ld_dx", ld_dx, D)) return e;
  if (!al2(grad_xw_gate) || !al2(grad_xw_up) || !al2(w_gate) || !al2(w_up) || !al2(grad_x))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  return FSW_OK;
}

static int input_grad_checked(const char* fn, const void* grad_xw_gate, const void* grad_xw_up,
                              const void* w_gate, const void* w_up, void* grad_x, int64_t T, int64_t D,
                              int64_t I, int64_t ldo, int64_t ldw, int64_t ld_dx, void* workspace,
                              int64_t workspace_bytes, int dtype, void* stream) {
  fsw::Problem p{};
  p.dG = grad_xw_gate; p.dU = grad_xw_up; p.wg = w_gate; p.wu = w_up; p.dx = grad_x;
  p.T = T; p.D = D; p.I = I; p.ldo = ldo; p.ldw = ldw; p.lddx = ld_dx; p.w_out_in = out_in_of(dtype);
  dtype = elem_of(dtype);
  hipStream_t s = (hipStream_t)stream;
  if (fsw::fast_path_ok_input_grad(p)) {
    const bool ws_ok = workspace && workspace_bytes > 0 && ((uintptr_t)workspace & 15) == 0;
    return launched(fn, fsw::launch_input_grad_fast(dtype, p, s, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0));
  }
  return launched(fn, fsw::launch_input_grad_generic(dtype, p, s));
}

int fsw_input_grad(const void* grad_xw_gate, const void* grad_xw_up, const void* w_gate,
                   const void* w_up, void* grad_x, int64_t T, int64_t D, int64_t I, int64_t ldo,
                   int64_t ldw, int64_t ld_dx, void* workspace, int64_t workspace_bytes, int dtype,
                   void* stream) {
  const char* fn = "fsw_input_grad";
  if (int e = check_input_grad_args(fn, grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, ldo, ldw, ld_dx, dtype))
    return e;
  return input_grad_checked(fn, grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, ldo, ldw, ld_dx,
                            workspace, workspace_bytes, dtype, stream);
}

static int check_weight_grad_args(const char* fn, const void* x, const void* grad_xw_up, const void* grad_xw_gate,
                                  void* grad_w_up, void* grad_w_gate, int64_t T, int64_t D, int64_t I, int64_t ldx,
                                  int64_t ldo, int64_t ld_dw, int dtype) {
  if (!x || !grad_xw_up || !grad_xw_gate || !grad_w_up || !grad_w_gate)
    return fail(FSW_ERR_NULL_POINTER, "%s: all five arrays must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  if (int e = check_ld(fn, "ldx", ldx, D)) return e;
  if (int e = check_ld(fn, "ldo", ldo, I)) return e;
  if (int e = check_ld(fn, "ld_dw", ld_dw, out_in_of(dtype) ? D : I)) return e;
  if (!al2(x) || !al2(grad_xw_up) || !al2(grad_xw_gate) || !al2(grad_w_up) || !al2(grad_w_gate))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  return FSW_OK;
}

int fsw_weight_grad(const void* x, const void* grad_xw_up, const void* grad_xw_gate,
                    void* grad_w_up, void* grad_w_gate, int64_t T, int64_t D, int64_t I,
                    int64_t ldx, int64_t ldo, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                    int dtype, void* stream) {
  const char* fn = "fsw_weight_grad";
  if (int e = check_weight_grad_args(fn, x, grad_xw_up, grad_xw_gate, grad_w_up, grad_w_gate, T, D, I, ldx, ldo, ld_dw, dtype))
    return e;
  const bool oi = out_in_of(dtype);
  dtype = elem_of(dtype);
  fsw::Problem p{};
  p.x = x; p.dG = grad_xw_gate; p.dU = grad_xw_up; p.dWg = grad_w_gate; p.dWu = grad_w_up;
  p.T = T; p.D = D; p.I = I; p.ldx = ldx; p.ldo = ldo; p.lddw = ld_dw; p.w_out_in = oi;
  hipStream_t s = (hipStream_t)stream;
  if (fsw::fast_path_ok_weight_grad(p)) {
    const bool ws_ok = workspace && workspace_bytes > 0 && ((uintptr_t)workspace & 15) == 0;
    return launched(fn, fsw::launch_weight_grad_fast(dtype, p, s, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0));
  }
  return launched(fn, fsw::launch_weight_grad_generic(dtype, p, s));
}

int fsw_swiglu_backward(const void* grad_out, const void* xw_gate, const void* xw_up, const void* x,
                        const void* w_gate, const void* w_up, void* grad_xw_gate, void* grad_xw_up, void* grad_x,
                        void* grad_w_gate, void* grad_w_up, int64_t T, int64_t D, int64_t I, int64_t ldx,
                        int64_t ldw, int64_t ld_dx, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                        int dtype, void* stream) {
  const char* fn = "fsw_swiglu_backward";
  if ((grad_w_gate == nullptr) != (grad_w_up == nullptr))
    return fail(FSW_ERR_NULL_POINTER, "%s: grad_w_gate and grad_w_up must both be given or both be null", fn);
  if (grad_x && (!w_gate || !w_up)) return fail(FSW_ERR_NULL_POINTER, "%s: grad_x needs w_gate and w_up", fn);
  if (grad_w_gate && !x) return fail(FSW_ERR_NULL_POINTER, "%s: the weight gradients need x", fn);
  // everything is validated before the first launch: a call that fails has enqueued nothing
  if (!grad_out || !xw_gate || !xw_up || !grad_xw_gate || !grad_xw_up)
    return fail(FSW_ERR_NULL_POINTER, "%s: grad_out, xw_gate, xw_up, grad_xw_gate and grad_xw_up must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  if (!al2(grad_out) || !al2(xw_gate) || !al2(xw_up))
    return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  if (grad_x)
    if (int e = check_input_grad_args(fn, grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, I, ldw, ld_dx, dtype))
      return e;
  if (grad_w_gate)
    if (int e = check_weight_grad_args(fn, x, grad_xw_up, grad_xw_gate, grad_w_up, grad_w_gate, T, D, I, ldx, I, ld_dw, dtype))
      return e;
  if (int e = fsw_elementwise_backward(grad_out, xw_gate, xw_up, grad_xw_up, grad_xw_gate, T * I, elem_of(dtype), stream))
    return e;
  // the weight gradient first: measured at 8192 x 4096 x 12288, the input gradient runs 4 % faster behind it than
  // behind the gating-gradient kernel (its dG / dU operand is still in the memory-side cache), the step 0.3 % faster
  if (grad_w_gate)
    if (int e = fsw_weight_grad(x, grad_xw_up, grad_xw_gate, grad_w_up, grad_w_gate, T, D, I, ldx, I, ld_dw, workspace,
                                workspace_bytes, dtype, stream))
      return e;
  if (grad_x)
    if (int e = fsw_input_grad(grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, I, ldw, ld_dx, workspace,
                               workspace_bytes, dtype, stream))
      return e;
  return FSW_OK;
}

// ---- the down projection that follows the SwiGLU: three plain GEMMs on the same tiled kernels ----
static int run_gemm(const char* fn, int layout, const void* a, const void* b, void* c, int64_t M, int64_t N,
                    int64_t K, int64_t lda, int64_t ldb, int64_t ldc, void* workspace, int64_t workspace_bytes,
                    int dtype, void* stream) {
  fsw::GemmProblem p{a, b, c, M, N, K, lda, ldb, ldc, layout};
  hipStream_t s = (hipStream_t)stream;
  if (fsw::fast_path_ok_gemm(p)) {
    const bool ws_ok = workspace && workspace_bytes > 0 && ((uintptr_t)workspace & 15) == 0;
    if (fsw::skinny_gemm_ok(p))   // few rows: stream the weights
      return launched(fn, fsw::launch_gemm_skinny(dtype, p, s, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0));
    return launched(fn, fsw::launch_gemm_fast(dtype, p, s, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0));
  }
  return launched(fn, fsw::launch_gemm_generic(dtype, p, s));
}

static int check_down_proj(const char* fn, const void* p0, const void* p1, const void* p2, int64_t T, int64_t I,
                           int64_t D, int64_t ld_act, int64_t ldw, int64_t ldy, int dtype) {
  if (!p0 || !p1 || !p2) return fail(FSW_ERR_NULL_POINTER, "%s: all three arrays must be non-null", fn);
  if (!dtype_ok(dtype)) return fail(FSW_ERR_BAD_DTYPE, "%s: dtype %d is neither bf16 (0) nor fp16 (1)", fn, dtype);
  if (int e = check_dims(fn, T, D, I)) return e;
  if (int e = check_ld(fn, "ld_act", ld_act, I)) return e;
  if (int e = check_ld(fn, "ldw", ldw, out_in_of(dtype) ? I : D)) return e;
  if (int e = check_ld(fn, "ldy", ldy, D)) return e;
  if (!al2(p0) || !al2(p1) || !al2(p2)) return fail(FSW_ERR_ALIGNMENT, "%s: pointers must be 2-byte aligned", fn);
  return FSW_OK;
}

int fsw_down_proj_forward(const void* act, const void* w_down, void* y, int64_t T, int64_t I, int64_t D,
                          int64_t ld_act, int64_t ldw, int64_t ldy, void* workspace, int64_t workspace_bytes,
                          int dtype, void* stream) {
  const char* fn = "fsw_down_proj_forward";
  if (int e = check_down_proj(fn, act, w_down, y, T, I, D, ld_act, ldw, ldy, dtype)) return e;
  // y [T,D] = act [T,I] W_down [I,D]   (or act W_down^T for W_down [D,I])
  return run_gemm(fn, out_in_of(dtype) ? 1 : 0, act, w_down, y, T, D, I, ld_act, ldw, ldy, workspace, workspace_bytes,
                  elem_of(dtype), stream);
}

int fsw_down_proj_input_grad(const void* grad_y, const void* w_down, void* grad_act, int64_t T, int64_t I,
                             int64_t D, int64_t ldy, int64_t ldw, int64_t ld_act, void* workspace,
                             int64_t workspace_bytes, int dtype, void* stream) {
  const char* fn = "fsw_down_proj_input_grad";
  if (int e = check_down_proj(fn, grad_y, w_down, grad_act, T, I, D, ld_act, ldw, ldy, dtype)) return e;
  // grad_act [T,I] = grad_y [T,D] W_down^T   (or grad_y W_down for W_down [D,I])
  return run_gemm(fn, out_in_of(dtype) ? 0 : 1, grad_y, w_down, grad_act, T, I, D, ldy, ldw, ld_act, workspace,
                  workspace_bytes, elem_of(dtype), stream);
}

int fsw_down_proj_weight_grad(const void* act, const void* grad_y, void* grad_w_down, int64_t T, int64_t I,
                              int64_t D, int64_t ld_act, int64_t ldy, int64_t ld_dw, void* workspace,
                              int64_t workspace_bytes, int dtype, void* stream) {
  const char* fn = "fsw_down_proj_weight_grad";
  if (int e = check_down_proj(fn, act, grad_y, grad_w_down, T, I, D, ld_act, ld_dw, ldy, dtype)) return e;
  // grad_W_down [I,D] = act^T grad_y   (or [D,I] = grad_y^T act)
  if (out_in_of(dtype))
    return run_gemm(fn, 2, grad_y, act, grad_w_down, D, I, T, ldy, ld_act, ld_dw, workspace, workspace_bytes,
                    elem_of(dtype), stream);
  return run_gemm(fn, 2, act, grad_y, grad_w_down, I, D, T, ld_act, ldy, ld_dw, workspace, workspace_bytes,
                  elem_of(dtype), stream);
}

}  // extern "C"

// ---- the entry point that allocates nothing -------------------------------------------------
// Scratch for the split reduction of fsw_input_grad_noalloc: one copy per GPU, part of the library's
// code object, held until the process ends.  In host code `scratch` is only a handle; the device
// address is looked up once per device with hipGetSymbolAddress and kept in g_scratch_ptr.
static __device__ __align__(256) unsigned char scratch[FSW_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of this device's copy of `scratch` (nullptr + message on failure).
void* scratch_address(const char* fn) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(FSW_ERR_LAUNCH, "%s: hipGetDevice failed or device index %d is beyond %d", fn, dev, kMaxDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      fail(FSW_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

int fsw_input_grad_noalloc(const void* grad_xw_gate, const void* grad_xw_up, const void* w_gate,
                           const void* w_up, void* grad_x, int64_t T, int64_t D, int64_t I, int64_t ldo,
                           int64_t ldw, int64_t ld_dx, int dtype, void* stream) {
  const char* fn = "fsw_input_grad_noalloc";
  if (int e = check_input_grad_args(fn, grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, ldo, ldw, ld_dx, dtype))
    return e;
  // only the split reduction of small problems needs its scratch; a large problem whose optional tail split
  // would not fit the buffer simply runs without it
  const int64_t need = fsw::splitk_workspace_bytes(out_in_of(dtype) ? 4 : 1, T, D, I, /*with_tail=*/false);
  if (need > (int64_t)FSW_NOALLOC_SCRATCH_BYTES)
    return fail(FSW_ERR_SCRATCH_LIMIT,
                "%s: T=%lld D=%lld I=%lld needs %lld bytes of split-reduction scratch, the built-in buffer holds %lld; "
                "use fsw_input_grad with a caller workspace",
                fn, (long long)T, (long long)D, (long long)I, (long long)need, (long long)FSW_NOALLOC_SCRATCH_BYTES);
  void* ptr = scratch_address(fn);
  if (!ptr) return FSW_ERR_LAUNCH;
  // Every partial the reduction kernel reads is written by the GEMM kernel of the same call, so nothing in
  // the buffer has to start at zero.
  return input_grad_checked(fn, grad_xw_gate, grad_xw_up, w_gate, w_up, grad_x, T, D, I, ldo, ldw, ld_dx, ptr,
                            (int64_t)FSW_NOALLOC_SCRATCH_BYTES, dtype, stream);
}

}  // extern "C"
