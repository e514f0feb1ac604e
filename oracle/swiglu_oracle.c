/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of the fused SwiGLU
 * forward/backward of fattorib/fusedswiglu, in plain C with fp64 arithmetic and
 * naive loops.  Nothing in the product path may link or call this file; it is
 * the checker that tests, the smoke check and the CPU-baseline leg of the
 * benchmark compare the HIP kernels against.
 *
 * Parity status of every function below: PINNED, by brute force against an
 * independent numpy/BLAS evaluation, torch.autograd of the eager formula in
 * fp64, central finite differences and closed-form special cases (the tests in
 * tests/test_oracle.py).  The reference holds no golden vectors for this path
 * (its tests draw values from the CUDA generator at run time), so there is no
 * fixture to compare with; bit-exact Triton rounding order is out of reach
 * and not required (parity is tolerance based).
 *
 * Notation: T tokens (= batch*seq), D = d_model, I = d_intermediate.
 * All matrices row-major, densely packed.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

/* fused_swiglu/kernels/kernels_bf16.py:9-11  silu(z) = z * sigmoid(z) */
double osw_silu(double z) { return z / (1.0 + exp(-z)); }

/* fused_swiglu/kernels/kernels_bf16.py:14-16
 * silu'(z) = sigmoid(z) + z * sigmoid(z) * (1 - sigmoid(z)) */
double osw_silu_grad(double z) {
  double s = 1.0 / (1.0 + exp(-z));
  return s + z * s * (1.0 - s);
}

/* fused_swiglu/kernels/kernels_bf16.py:102-160 (swiglu_kernel) and
 * fused_swiglu/test_swiglu.py:47-55 (swiglu_ref_torch):
 *   g = x @ Wg, u = x @ Wu, out = silu(g) * u.
 * x [T,D], wg/wu [D,I]; g, u, out [T,I]. */
void osw_forward(const double* x, const double* wg, const double* wu, int64_t T, int64_t D,
                 int64_t I, double* g, double* u, double* out) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; t++) {
    for (int64_t i = 0; i < I; i++) {
      double sg = 0.0, su = 0.0;
      for (int64_t d = 0; d < D; d++) {
        double xv = x[t * D + d];
        sg += xv * wg[d * I + i];
        su += xv * wu[d * I + i];
      }
      g[t * I + i] = sg;
      u[t * I + i] = su;
      out[t * I + i] = osw_silu(sg) * su;
    }
  }
}

/* fused_swiglu/kernels/kernels_bf16.py:228-234 (elementwise_backward_kernel):
 *   dU = dout * silu(g);  dG = dout * u * silu'(g).  Flat arrays of n elements. */
void osw_elementwise_backward(const double* dout, const double* g, const double* u, int64_t n,
                              double* dU, double* dG) {
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < n; k++) {
    dU[k] = dout[k] * osw_silu(g[k]);
    dG[k] = dout[k] * u[k] * osw_silu_grad(g[k]);
  }
}

/* fused_swiglu/swiglu.py:45   dx = dG @ Wg^T + dU @ Wu^T   -> [T,D] */
void osw_input_grad(const double* dG, const double* dU, const double* wg, const double* wu,
                    int64_t T, int64_t D, int64_t I, double* dx) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; t++) {
    for (int64_t d = 0; d < D; d++) {
      double s = 0.0;
      for (int64_t i = 0; i < I; i++)
        s += dG[t * I + i] * wg[d * I + i] + dU[t * I + i] * wu[d * I + i];
      dx[t * D + d] = s;
    }
  }
}

/* fused_swiglu/swiglu.py:50-57 with kernels_bf16.py:343-348 (bmm_kernel) and the
 * batch sum of swiglu.py:11-13:  dWg = x^T @ dG, dWu = x^T @ dU, reduced over all
 * tokens -> [D,I].  The per-batch partials of the reference summed over the batch
 * are the same sum over t. */
void osw_weight_grad(const double* x, const double* dG, const double* dU, int64_t T, int64_t D,
                     int64_t I, double* dWg, double* dWu) {
#pragma omp parallel for schedule(static)
  for (int64_t d = 0; d < D; d++) {
    for (int64_t i = 0; i < I; i++) {
      double sg = 0.0, su = 0.0;
      for (int64_t t = 0; t < T; t++) {
        double xv = x[t * D + d];
        sg += xv * dG[t * I + i];
        su += xv * dU[t * I + i];
      }
      dWg[d * I + i] = sg;
      dWu[d * I + i] = su;
    }
  }
}

/* fused_swiglu/swiglu.py:34-58 (FusedSwiGLU.backward): composition and return
 * order (dx, dWg, dWu).  g and u are recomputed here in fp64 from x and the
 * weights (the reference reads back its 16-bit saved copies).  scratch must hold
 * 4*T*I doubles. */
void osw_backward(const double* x, const double* wg, const double* wu, const double* dout,
                  int64_t T, int64_t D, int64_t I, double* scratch, double* dx, double* dWg,
                  double* dWu) {
  double* g = scratch;
  double* u = scratch + T * I;
  double* dG = scratch + 2 * T * I;
  double* dU = scratch + 3 * T * I;
  /* out lands in dG, overwritten next */
  osw_forward(x, wg, wu, T, D, I, g, u, dG);
  osw_elementwise_backward(dout, g, u, T * I, dU, dG);
  osw_input_grad(dG, dU, wg, wu, T, D, I, dx);
  osw_weight_grad(x, dG, dU, T, D, I, dWg, dWu);
}

/* The step after the path: the down projection y = act @ W_down that the reference leaves to its caller
 * (README.md:25-38).  act [T,I], w [I,D] -> y [T,D]. */
void osw_down_proj_forward(const double* act, const double* w, int64_t T, int64_t I, int64_t D, double* y) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; t++)
    for (int64_t d = 0; d < D; d++) {
      double s = 0.0;
      for (int64_t i = 0; i < I; i++) s += act[t * I + i] * w[i * D + d];
      y[t * D + d] = s;
    }
}

/* Its gradients: d_act = dy @ W^T [T,I], dW = act^T @ dy [I,D] summed over all tokens. */
void osw_down_proj_backward(const double* act, const double* w, const double* dy, int64_t T, int64_t I,
                            int64_t D, double* d_act, double* dw) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < T; t++)
    for (int64_t i = 0; i < I; i++) {
      double s = 0.0;
      for (int64_t d = 0; d < D; d++) s += dy[t * D + d] * w[i * D + d];
      d_act[t * I + i] = s;
    }
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < I; i++)
    for (int64_t d = 0; d < D; d++) {
      double s = 0.0;
      for (int64_t t = 0; t < T; t++) s += act[t * I + i] * dy[t * D + d];
      dw[i * D + d] = s;
    }
}
