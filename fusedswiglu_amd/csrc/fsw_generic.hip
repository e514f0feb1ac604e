// Edge-shape path: the same three GEMM-shaped steps for operands the tiled kernels cannot take
// (dimensions or leading dimensions that are not multiples of 8 elements, pointers that are not
// 16-byte aligned).  Elements are fetched one by one with bounds checks and zero padding, staged
// k-contiguous in LDS, and multiplied on the same 32x32x16 MFMA with fp32 accumulation.
// One workgroup = 4 waves = a 64 x 64 tile of each of the two results.
#include "fsw_internal.hpp"

namespace fsw {

struct GenericParams {
  const unsigned short* a[2];   // pass 0 / pass 1 A operand
  const unsigned short* b[2][2];  // [pass][which]  (which = gate/up result; single-result modes use [.][0])
  unsigned short* c[3];
  long long a_sm, a_sk, b_sk, b_sn, ldc;
  int M, N, K;
  int passes;   // 1, or 2 for dx (second pass accumulates into the same tile)
  int dual;     // 1: two B matrices -> two results sharing A;  0: one result
  int swiglu;   // 1: c[0] = silu(acc0)*acc1, c[1] = acc0, c[2] = acc1 (c[1], c[2] may be null)
                // 2: gating gradients from the recomputed pre-activations: c[1] = dG, c[2] = dU
  const unsigned short* dout;  // swiglu == 2: upstream gradient, leading dimension ldc
};

constexpr int kGT = 64;      // tile edge
constexpr int kGPitch = 40;  // LDS row pitch in elements (80 bytes, keeps 16-byte alignment)

template <typename E>
__global__ __launch_bounds__(256) void generic_kernel(GenericParams p) {
  __shared__ __attribute__((aligned(16))) unsigned short As[kGT * kGPitch];
  __shared__ __attribute__((aligned(16))) unsigned short Bs[2][kGT * kGPitch];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + kGT - 1) / kGT;
  const int m0 = (int)(blockIdx.x / tiles_n) * kGT, n0 = (int)(blockIdx.x % tiles_n) * kGT;
  f32x16 acc[2];
#pragma unroll
  for (int r = 0; r < 16; r++) acc[0][r] = acc[1][r] = 0.f;

  for (int pass = 0; pass < p.passes; pass++) {
    const unsigned short* A = p.a[pass];
    for (int k0 = 0; k0 < p.K; k0 += kBK) {
      // A tile: 64 rows x 32 k
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int idx = tid + 256 * j;
        int m, k;
        if (p.a_sk == 1) { m = idx >> 5; k = idx & 31; } else { k = idx >> 6; m = idx & 63; }
        unsigned short v = 0;
        if (m0 + m < p.M && k0 + k < p.K) v = A[(long long)(m0 + m) * p.a_sm + (long long)(k0 + k) * p.a_sk];
        As[m * kGPitch + k] = v;
      }
      for (int w = 0; w <= p.dual; w++) {
        const unsigned short* B = p.b[pass][w];
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const int idx = tid + 256 * j;
          int n, k;
          if (p.b_sn == 1) { k = idx >> 6; n = idx & 63; } else { n = idx >> 5; k = idx & 31; }
          unsigned short v = 0;
          if (n0 + n < p.N && k0 + k < p.K) v = B[(long long)(k0 + k) * p.b_sk + (long long)(n0 + n) * p.b_sn];
          Bs[w][n * kGPitch + k] = v;
        }
      }
      __syncthreads();
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const int koff = ks * 16 + 8 * (lane >> 5);
        const i16x8 fa = *(const i16x8*)&As[(wm * 32 + (lane & 31)) * kGPitch + koff];
        const i16x8 fb0 = *(const i16x8*)&Bs[0][(wn * 32 + (lane & 31)) * kGPitch + koff];
        acc[0] = E::mfma(fb0, fa, acc[0]);
        if (p.dual) {
          const i16x8 fb1 = *(const i16x8*)&Bs[1][(wn * 32 + (lane & 31)) * kGPitch + koff];
          acc[1] = E::mfma(fb1, fa, acc[1]);
        }
      }
      __syncthreads();
    }
  }
  // acc[.][r] of lane l: row m0 + wm*32 + (l & 31), column n0 + wn*32 + 8*(r>>2) + 4*(l>>5) + (r&3)
  const int m = m0 + wm * 32 + (lane & 31);
  if (m >= p.M) return;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int n = n0 + wn * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
    if (n >= p.N) continue;
    const long long o = (long long)m * p.ldc + n;
    if (p.swiglu == 2) {
      float dU, dG;
      gating_grad(E::to_float(p.dout[o]), acc[0][r], acc[1][r], dU, dG);
      p.c[1][o] = E::from_float(dG);
      p.c[2][o] = E::from_float(dU);
    } else if (p.swiglu) {
      p.c[0][o] = E::from_float(silu_mul(acc[0][r], acc[1][r]));
      if (p.c[1]) { p.c[1][o] = E::from_float(acc[0][r]); p.c[2][o] = E::from_float(acc[1][r]); }
    } else {
      p.c[0][o] = E::from_float(acc[0][r]);
      if (p.dual) p.c[1][o] = E::from_float(acc[1][r]);
    }
  }
}

static hipError_t launch_generic(int dtype, const GenericParams& gp, hipStream_t s) {
  const long long tiles = (long long)((gp.N + kGT - 1) / kGT) * ((gp.M + kGT - 1) / kGT);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)tiles;
  if (dtype == kDtypeBF16) generic_kernel<BF16><<<grid, 256, 0, s>>>(gp);
  else generic_kernel<FP16><<<grid, 256, 0, s>>>(gp);
  return hipGetLastError();
}

typedef const unsigned short* cus;
typedef unsigned short* us;

hipError_t launch_forward_generic(int dtype, const Problem& p, hipStream_t s) {
  GenericParams g{};
  g.a[0] = (cus)p.x; g.b[0][0] = (cus)p.wg; g.b[0][1] = (cus)p.wu;
  g.c[0] = (us)p.out; g.c[1] = (us)p.g; g.c[2] = (us)p.u;
  g.a_sm = p.ldx; g.a_sk = 1; g.ldc = p.ldo;
  if (p.w_out_in) { g.b_sk = 1; g.b_sn = p.ldw; } else { g.b_sk = p.ldw; g.b_sn = 1; }
  g.M = (int)p.T; g.N = (int)p.I; g.K = (int)p.D; g.passes = 1; g.dual = 1; g.swiglu = 1;
  if (p.dout) { g.swiglu = 2; g.dout = (cus)p.dout; }
  return launch_generic(dtype, g, s);
}

hipError_t launch_input_grad_generic(int dtype, const Problem& p, hipStream_t s) {
  GenericParams g{};
  g.a[0] = (cus)p.dG; g.a[1] = (cus)p.dU; g.b[0][0] = (cus)p.wg; g.b[1][0] = (cus)p.wu;
  g.c[0] = (us)p.dx;
  g.a_sm = p.ldo; g.a_sk = 1; g.ldc = p.lddx;
  if (p.w_out_in) { g.b_sk = p.ldw; g.b_sn = 1; } else { g.b_sk = 1; g.b_sn = p.ldw; }
  g.M = (int)p.T; g.N = (int)p.D; g.K = (int)p.I; g.passes = 2; g.dual = 0; g.swiglu = 0;
  return launch_generic(dtype, g, s);
}

hipError_t launch_weight_grad_generic(int dtype, const Problem& p, hipStream_t s) {
  GenericParams g{};
  if (p.w_out_in) {  // results [I,D]: dW = dG^T x, one launch per result (this kernel shares A, not B)
    g.b[0][0] = (cus)p.x; g.a_sm = 1; g.a_sk = p.ldo; g.b_sk = p.ldx; g.b_sn = 1; g.ldc = p.lddw;
    g.M = (int)p.I; g.N = (int)p.D; g.K = (int)p.T; g.passes = 1; g.dual = 0; g.swiglu = 0;
    g.a[0] = (cus)p.dG; g.c[0] = (us)p.dWg;
    hipError_t e = launch_generic(dtype, g, s);
    if (e != hipSuccess) return e;
    g.a[0] = (cus)p.dU; g.c[0] = (us)p.dWu;
    return launch_generic(dtype, g, s);
  }
  g.a[0] = (cus)p.x; g.b[0][0] = (cus)p.dG; g.b[0][1] = (cus)p.dU;
  g.c[0] = (us)p.dWg; g.c[1] = (us)p.dWu;
  g.a_sm = 1; g.a_sk = p.ldx; g.b_sk = p.ldo; g.b_sn = 1; g.ldc = p.lddw;
  g.M = (int)p.D; g.N = (int)p.I; g.K = (int)p.T; g.passes = 1; g.dual = 1; g.swiglu = 0;
  return launch_generic(dtype, g, s);
}

hipError_t launch_gemm_generic(int dtype, const GemmProblem& p, hipStream_t s) {
  GenericParams g{};
  g.a[0] = (cus)p.a; g.b[0][0] = (cus)p.b; g.c[0] = (us)p.c; g.ldc = p.ldc;
  if (p.layout == 2) { g.a_sm = 1; g.a_sk = p.lda; } else { g.a_sm = p.lda; g.a_sk = 1; }
  if (p.layout == 1) { g.b_sk = 1; g.b_sn = p.ldb; } else { g.b_sk = p.ldb; g.b_sn = 1; }
  g.M = (int)p.M; g.N = (int)p.N; g.K = (int)p.K; g.passes = 1; g.dual = 0; g.swiglu = 0;
  return launch_generic(dtype, g, s);
}

}  // namespace fsw
