// Two machine probes used by the benchmark to state practical ceilings next to the nominal peaks:
// a register-only MFMA loop (no memory traffic at all) and a streaming read.  They only enqueue a
// kernel; the caller times them with events on the same stream.
#include "../../include/fusedswiglu.h"
#include "../../include/fusedswiglu_bench.h"
#include "fsw_common.hpp"

namespace fsw {

__device__ float probe_normal(unsigned i, unsigned seed) {
  unsigned h = (i * 2654435761u) ^ seed;
  h ^= h >> 15; h *= 0x2c1b3c6du; h ^= h >> 12; h *= 0x297a2d39u; h ^= h >> 15;
  unsigned h2 = h * 0x9e3779b9u + 0x7f4a7c15u;
  h2 ^= h2 >> 13; h2 *= 0x85ebca6bu; h2 ^= h2 >> 16;
  const float u1 = ((h >> 8) + 1) * (1.0f / 16777217.0f), u2 = (h2 >> 8) * (1.0f / 16777216.0f);
  return sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);
}

// 8 waves per workgroup, each issuing 8 independent 32x32x16 bf16 MFMAs per iteration.
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* sink, int iters, int random_operands) {
  bf16x8 a[4], b[2];
  for (int f = 0; f < 4; f++)
    for (int j = 0; j < 8; j++)
      a[f][j] = random_operands ? (__bf16)probe_normal(threadIdx.x * 64 + f * 8 + j + blockIdx.x * 77777, 1) : (__bf16)1.0f;
  for (int f = 0; f < 2; f++)
    for (int j = 0; j < 8; j++)
      b[f][j] = random_operands ? (__bf16)(probe_normal(threadIdx.x * 64 + f * 8 + j + blockIdx.x * 33333, 2) * 0.015625f)
                                : (__bf16)0.015625f;
  f32x16 acc[2][4];
  for (int x = 0; x < 2; x++)
    for (int q = 0; q < 4; q++)
      for (int r = 0; r < 16; r++) acc[x][q][r] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int x = 0; x < 2; x++) acc[x][q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[x], a[q], acc[x][q], 0, 0, 0);
  }
  float s = 0;
  for (int x = 0; x < 2; x++)
    for (int q = 0; q < 4; q++)
      for (int r = 0; r < 16; r++) s += acc[x][q][r];
  if (s == 12345.678f) sink[0] = s;  // keeps the loop alive; practically never true
}

// The tiled kernels' instruction mix without any of their dependencies: per 8 MFMAs (16x16x32, N(0,1)
// operands held in registers) NR 16-byte LDS reads per lane and ND direct global->LDS loads of 1 KiB
// per wave, the loads hitting L2 (the 32 CUs of an XCD walk one 8 MiB window).  LDS values are consumed
// one iteration after they were read, so nothing ever waits for fresh data: what this loop sustains is
// what the matrix cores deliver while that much data moves beside them.
// GATING (needs NR == 3): the weight-side fragment of the NEXT 8 MFMAs is not held in registers but formed from
// the three values just read from LDS, taken as dout, g, u (bf16 ~N(0,1)): four gating gradients dG, dU per lane
// and 8 MFMAs, which is what a 128x128 wave tile of the weight-gradient GEMM would have to compute if the
// gating-gradient kernel were folded into its operand path (8 fragments of 8 values per 64 MFMAs).
template <int NR, int ND, bool GATING = false>
__global__ __launch_bounds__(512) void probe_mfma_mix_kernel(const char* src, unsigned src_bytes, float* sink, int iters) {
  static_assert(!GATING || NR == 3, "the gating mix takes dout, g, u from the three reads");
  __shared__ __attribute__((aligned(1024))) char smem[64 * 1024];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  for (int i = tid; i < 64 * 1024 / 16; i += 512) {
    u32x4 v;
    for (int e = 0; e < 4; e++) v[e] = BF16::pack2(probe_normal(i * 8 + 2 * e, 7), probe_normal(i * 8 + 2 * e + 1, 7));
    ((FSW_LDS u32x4*)smem)[i] = v;
  }
  __syncthreads();
  bf16x8 a[8], b[4];
  for (int f = 0; f < 8; f++)
    for (int j = 0; j < 8; j++) a[f][j] = (__bf16)probe_normal(tid * 64 + f * 8 + j + blockIdx.x * 77777, 1);
  for (int f = 0; f < 4; f++)
    for (int j = 0; j < 8; j++) b[f][j] = (__bf16)(probe_normal(tid * 64 + f * 8 + j + blockIdx.x * 33333, 2) * 0.015625f);
  f32x4 acc[4][8];
  for (int x = 0; x < 4; x++)
    for (int q = 0; q < 8; q++) acc[x][q] = f32x4{0.f, 0.f, 0.f, 0.f};
  const i32x4 rs = make_rsrc(src, src_bytes);
  const unsigned lds_base = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const unsigned goff = ((blockIdx.x & 31) * 8 + wave) * 1024 + lane * 16;
  u32x4 x0 = {0, 0, 0, 0};
  u32x4 pending[4][NR > 0 ? NR : 1];
  for (int x = 0; x < 4; x++)
    for (int r = 0; r < (NR > 0 ? NR : 1); r++) pending[x][r] = x0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int x = 0; x < 4; x++) {
#pragma unroll
      for (int q = 0; q < 8; q++) acc[x][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[x], a[q], acc[x][q], 0, 0, 0);
      if constexpr (GATING) {
        // in the same scheduling region as the 8 MFMAs above, so the compiler may put it into their shadow
        const int nx = (x + 1) & 3;
        u32x4 w;
#pragma unroll
        for (int e = 0; e < 2; e++) {
          const unsigned d = pending[nx][0][e], g = pending[nx][1][e], u = pending[nx][2][e];
          float dU0, dG0, dU1, dG1;
          gating_grad(__uint_as_float(d << 16), __uint_as_float(g << 16), __uint_as_float(u << 16), dU0, dG0);
          gating_grad(__uint_as_float(d & 0xffff0000u), __uint_as_float(g & 0xffff0000u),
                      __uint_as_float(u & 0xffff0000u), dU1, dG1);
          w[e] = BF16::pack2(dG0 * 0.015625f, dG1 * 0.015625f);
          w[2 + e] = BF16::pack2(dU0 * 0.015625f, dU1 * 0.015625f);
        }
        b[nx] = __builtin_bit_cast(bf16x8, w);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < NR; r++) {
        x0 ^= pending[x][r];
        pending[x][r] = *(const FSW_LDS u32x4*)(smem + ((wave * 4 + x) * 4096 + r * 1024 + lane * 16) % 65536);
      }
#pragma unroll
      for (int d = 0; d < ND; d++) {
        const unsigned voff = (goff + (unsigned)(it * 4 + x) * 262144u) % src_bytes;  // 16-byte aligned, < src_bytes
        load16_to_lds(rs, voff, lds_base + ((wave * 4 + x) * 4096 + d * 1024) % 65536);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  for (int x = 0; x < 4; x++)
    for (int r = 0; r < (NR > 0 ? NR : 1); r++) x0 ^= pending[x][r];
  float s = __uint_as_float(x0[0] ^ x0[1] ^ x0[2] ^ x0[3]);
  for (int x = 0; x < 4; x++)
    for (int q = 0; q < 8; q++)
      for (int r = 0; r < 4; r++) s += acc[x][q][r];
  if (s == 12345.678f) sink[0] = s;
}

__global__ __launch_bounds__(256) void probe_read_kernel(const u32x4* __restrict__ p, size_t n16, unsigned* sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  unsigned s = 0;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    u32x4 v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = __builtin_nontemporal_load(p + i + k * stride);
#pragma unroll
    for (int k = 0; k < 8; k++) s += v[k][0] ^ v[k][1] ^ v[k][2] ^ v[k][3];
  }
  for (; i < n16; i += stride) { const u32x4 a = p[i]; s += a[0] ^ a[1] ^ a[2] ^ a[3]; }
  if (s == 0x12345678u) sink[0] = s;
}

// The tiled and the weight-streaming kernels' way of reading: direct global->LDS loads of 1 KiB per wave (eight
// rows of one 128-byte line), every byte of the buffer exactly once, optionally with the non-temporal hint.  The
// descriptor carries the exact size, so no lane can read outside the buffer.  Known traffic for calibrating the
// profiler's byte counters against this request pattern.
template <bool NT>
__global__ __launch_bounds__(256) void probe_dma_read_kernel(const char* buf, unsigned bytes) {
  __shared__ __attribute__((aligned(1024))) char smem[32 * 1024];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const i32x4 rs = make_rsrc(buf, bytes);
  const unsigned lds = (unsigned)(uintptr_t)(FSW_LDS char*)smem + wave * 8192;
  const unsigned chunks = bytes >> 10, waves = gridDim.x * 4;
  int k = 0;
  for (unsigned c = blockIdx.x * 4 + wave; c < chunks; c += waves, k++) {
    const unsigned off = c * 1024u + lane * 16u;
    if (NT) load16_to_lds_stream(rs, off, lds + (k & 7) * 1024);
    else load16_to_lds(rs, off, lds + (k & 7) * 1024);
    if ((k & 7) == 7) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace fsw

extern "C" {

int fsw_probe_mfma(int random_operands, int iters, int workgroups, void* sink4, void* stream, double* flop_out) {
  if (!sink4 || iters <= 0 || workgroups <= 0) return FSW_ERR_BAD_SHAPE;
  fsw::probe_mfma_kernel<<<workgroups, 512, 0, (hipStream_t)stream>>>((float*)sink4, iters, random_operands);
  if (flop_out) *flop_out = (double)workgroups * 8.0 * iters * 8.0 * 32768.0;
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_ERR_LAUNCH;
}

int fsw_probe_mfma_mix(int mix, int iters, int workgroups, const void* buf, int64_t bytes, void* sink4,
                       void* stream, double* flop_out) {
  // the window must hold whole 256 KiB strides and stay below the 2 GiB reach of the descriptor
  if (!buf || !sink4 || iters <= 0 || workgroups <= 0 || bytes < (1 << 20) || bytes >= (1LL << 31) ||
      (bytes & 0x3ffff) || ((uintptr_t)buf & 15))
    return FSW_ERR_BAD_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  const char* src = (const char*)buf;
  const unsigned n = (unsigned)bytes;
  switch (mix) {
    case 0: fsw::probe_mfma_mix_kernel<0, 0><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    case 1: fsw::probe_mfma_mix_kernel<3, 1><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    case 2: fsw::probe_mfma_mix_kernel<2, 1><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    case 3: fsw::probe_mfma_mix_kernel<3, 0><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    case 4: fsw::probe_mfma_mix_kernel<0, 1><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    case 5: fsw::probe_mfma_mix_kernel<3, 1, true><<<workgroups, 512, 0, s>>>(src, n, (float*)sink4, iters); break;
    default: return FSW_ERR_BAD_SHAPE;
  }
  if (flop_out) *flop_out = (double)workgroups * 8.0 * iters * 32.0 * 16384.0;
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_ERR_LAUNCH;
}

int fsw_probe_stream_read(const void* buf, int64_t bytes, void* sink4, void* stream) {
  if (!buf || !sink4 || bytes < 16 || ((uintptr_t)buf & 15)) return FSW_ERR_BAD_SHAPE;
  fsw::probe_read_kernel<<<4096, 256, 0, (hipStream_t)stream>>>((const fsw::u32x4*)buf, (size_t)bytes / 16, (unsigned*)sink4);
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_ERR_LAUNCH;
}

int fsw_probe_dma_read(const void* buf, int64_t bytes, int non_temporal, void* stream) {
  if (!buf || bytes < 1024 || bytes > 0x7fffffffLL || (bytes & 1023) || ((uintptr_t)buf & 15)) return FSW_ERR_BAD_SHAPE;
  if (non_temporal) fsw::probe_dma_read_kernel<true><<<2048, 256, 0, (hipStream_t)stream>>>((const char*)buf, (unsigned)bytes);
  else fsw::probe_dma_read_kernel<false><<<2048, 256, 0, (hipStream_t)stream>>>((const char*)buf, (unsigned)bytes);
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_ERR_LAUNCH;
}

}  // extern "C"
