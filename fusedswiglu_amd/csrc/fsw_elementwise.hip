// Fused gating-gradient kernel of the SwiGLU backward:
//   dU = dout * silu(g)            dG = dout * u * silu'(g),   silu'(z) = s + z*s*(1-s), s = sigmoid(z)
// Replaces fused_swiglu/kernels/kernels_bf16.py:210-255 (and the fp16 twin).  HBM bound: reads three
// and writes two 16-bit arrays, 10 bytes per element.  All math in fp32, one rounding per output.
// The grid covers ceil(n / elements-per-block): the reference's floor-division grid
// (kernels_bf16.py:246) leaves a tail unwritten when n % 128 != 0; that is not reproduced.
#include "fsw_internal.hpp"

namespace fsw {

template <typename E>
FSW_DEV void gate_grad(unsigned short dout, unsigned short g, unsigned short u, unsigned short& dU,
                       unsigned short& dG) {
  float fu, fg;
  gating_grad(E::to_float(dout), E::to_float(g), E::to_float(u), fu, fg);
  dU = E::from_float(fu);
  dG = E::from_float(fg);
}

template <typename E>
__global__ __launch_bounds__(256) void elementwise_backward_kernel(
    const unsigned short* __restrict__ dout, const unsigned short* __restrict__ g,
    const unsigned short* __restrict__ u, unsigned short* __restrict__ dU,
    unsigned short* __restrict__ dG, size_t n, int vec_ok) {
  const size_t nvec = vec_ok ? n / 8 : 0;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (size_t v = tid; v < nvec; v += stride) {
    const u32x4 a = __builtin_nontemporal_load((const u32x4*)dout + v);
    const u32x4 b = __builtin_nontemporal_load((const u32x4*)g + v);
    const u32x4 c = __builtin_nontemporal_load((const u32x4*)u + v);
    u32x4 ru, rg;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      float u0, g0, u1, g1;
      gating_grad(E::to_float(a[w] & 0xffff), E::to_float(b[w] & 0xffff), E::to_float(c[w] & 0xffff), u0, g0);
      gating_grad(E::to_float(a[w] >> 16), E::to_float(b[w] >> 16), E::to_float(c[w] >> 16), u1, g1);
      ru[w] = E::pack2(u0, u1);
      rg[w] = E::pack2(g0, g1);
    }
    __builtin_nontemporal_store(ru, (u32x4*)dU + v);
    __builtin_nontemporal_store(rg, (u32x4*)dG + v);
  }
  // scalar tail (everything, when the pointers are not 16-byte aligned)
  for (size_t i = nvec * 8 + tid; i < n; i += stride) gate_grad<E>(dout[i], g[i], u[i], dU[i], dG[i]);
}

template <typename E>
static hipError_t launch_elementwise_t(const void* dout, const void* g, const void* u, void* dU,
                                       void* dG, size_t n, hipStream_t stream) {
  const uintptr_t all = (uintptr_t)dout | (uintptr_t)g | (uintptr_t)u | (uintptr_t)dU | (uintptr_t)dG;
  const int vec_ok = (all & 15) == 0;
  size_t work = vec_ok ? (n + 7) / 8 : n;
  size_t blocks = (work + 255) / 256;
  // two passes of the grid-stride loop per thread keep enough loads in flight per CU
  if (blocks > 65536) blocks = (blocks + 1) / 2;
  if (blocks > 0x7fffffffu) blocks = 0x7fffffffu;
  if (blocks == 0) return hipSuccess;
  elementwise_backward_kernel<E><<<(unsigned)blocks, 256, 0, stream>>>(
      (const unsigned short*)dout, (const unsigned short*)g, (const unsigned short*)u,
      (unsigned short*)dU, (unsigned short*)dG, n, vec_ok);
  return hipGetLastError();
}

hipError_t launch_elementwise(int dtype, const void* dout, const void* g, const void* u, void* dU,
                              void* dG, size_t n, hipStream_t stream) {
  return dtype == 0 ? launch_elementwise_t<BF16>(dout, g, u, dU, dG, n, stream)
                    : launch_elementwise_t<FP16>(dout, g, u, dU, dG, n, stream);
}

}  // namespace fsw
