// Shared device-side building blocks for the gfx950 (CDNA4) fused SwiGLU kernels:
// element types, MFMA wrappers, raw buffer descriptors, direct global->LDS loads,
// LDS swizzles and the XCD-aware tile order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fsw {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef short i16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define FSW_LDS __attribute__((address_space(3)))
#define FSW_DEV __device__ __forceinline__

// ---- element traits -------------------------------------------------------
struct BF16 {
  using vec8 = bf16x8;
  static FSW_DEV f32x16 mfma(i16x8 a, i16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // 16x16x32: half the accumulator traffic per flop of the 32x32x16 form (measurably less power)
  static FSW_DEV f32x4 mfma16(i16x8 a, i16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static FSW_DEV float to_float(unsigned short v) { return __uint_as_float((unsigned)v << 16); }
  // round-to-nearest-even; NaN stays NaN
  static FSW_DEV unsigned short from_float(float f) {
    return __builtin_bit_cast(unsigned short, (__bf16)f);
  }
  // two values in one v_cvt_pk_bf16_f32 (same rounding): `lo` in bits 0..15.  Through the compiler and not as
  // inline assembly: it knows the wait state this instruction needs before an LDS or memory instruction reads
  // its result (without it, some lanes store the unconverted input).
  static FSW_DEV unsigned pack2(float lo, float hi) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  }
};
struct FP16 {
  using vec8 = f16x8;
  static FSW_DEV f32x16 mfma(i16x8 a, i16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static FSW_DEV f32x4 mfma16(i16x8 a, i16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static FSW_DEV float to_float(unsigned short v) {
    return (float)__builtin_bit_cast(_Float16, v);
  }
  static FSW_DEV unsigned short from_float(float f) {
    return __builtin_bit_cast(unsigned short, (_Float16)f);
  }
  // two values in one v_cvt_pk_f16_f32 (same rounding): `lo` in bits 0..15
  static FSW_DEV unsigned pack2(float lo, float hi) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{lo, hi}, f16x2));
  }
};

// silu(g) * u and the gating gradients, fp32 throughout, one rounding at the store.
// v_rcp_f32 (1 ulp) instead of a correctly rounded division: ten instructions fewer per value in epilogues
// that are VALU bound, and far inside the rounding of the 16-bit results
FSW_DEV float sigmoidf_fast(float z) { return __builtin_amdgcn_rcpf(1.0f + __expf(-z)); }
FSW_DEV float silu_mul(float g, float u) { return g * sigmoidf_fast(g) * u; }
// dU = dout * silu(g), dG = dout * u * silu'(g), silu'(z) = s + z*s*(1 - s), s = sigmoid(z)
FSW_DEV void gating_grad(float dout, float g, float u, float& dU, float& dG) {
  const float s = sigmoidf_fast(g);
  const float zs = g * s;
  dU = dout * zs;
  dG = dout * u * (s + zs * (1.0f - s));
}

// ---- raw buffer descriptors and direct-to-LDS loads -------------------------
// Word 3 for gfx90a/gfx94x/gfx950 raw buffers (32-bit data format, no swizzle).
constexpr int kRsrcWord3 = 0x00020000;
// A byte offset that is out of range for every descriptor built here (num_records <= 2^31-1):
// the load then returns zeros, which is how all tile edges are padded.
constexpr unsigned kOobOffset = 0x80000000u;

FSW_DEV i32x4 make_rsrc(const void* base, unsigned num_records = 0x7fffffffu) {
  uint64_t a = (uint64_t)base;
  i32x4 r;
  r.x = (int)(unsigned)a;
  r.y = (int)((unsigned)(a >> 32) & 0xffffu);
  r.z = (int)num_records;
  r.w = kRsrcWord3;
  // the descriptor must live in SGPRs
  r.x = __builtin_amdgcn_readfirstlane(r.x);
  r.y = __builtin_amdgcn_readfirstlane(r.y);
  r.z = __builtin_amdgcn_readfirstlane(r.z);
  return r;
}

// 16 bytes per lane from `rsrc + voffset` straight into LDS at `lds_addr + lane*16`
// (the LDS destination of a wave is contiguous by lane; lds_addr is wave-uniform).
// Counted by vmcnt like any vector load; the compiler does not track it, so every consumer
// must be fenced with wait_vmcnt<N>() + a workgroup barrier.
FSW_DEV void load16_to_lds(i32x4 rsrc, unsigned voffset, unsigned lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 3\n\t"  // M0 write -> LDS-DMA use, and any VALU-written descriptor SGPR -> VMEM read
      "buffer_load_dwordx4 %1, %2, 0 offen lds"
      :
      : "s"(lds_addr), "v"(voffset), "s"(rsrc)
      : "memory");
}

// The same load with the non-temporal hint, for operands that are read exactly once per launch (the weights
// of a forward with a single row of tiles): the lines are not kept in L2 or the memory-side cache, which
// leaves those to the operand that is re-read and measurably raises the streaming rate from HBM.
FSW_DEV void load16_to_lds_stream(i32x4 rsrc, unsigned voffset, unsigned lds_addr) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 3\n\t"
      "buffer_load_dwordx4 %1, %2, 0 offen nt lds"
      :
      : "s"(lds_addr), "v"(voffset), "s"(rsrc)
      : "memory");
}

template <int N>
FSW_DEV void wait_vmcnt_and_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is 6 bits");
  // LDS reads issued before the barrier may still be in flight: their consumers carry their own
  // lgkmcnt waits, and no LDS slot is overwritten until a full step after it was last read
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(N) : "memory");
}

// ---- LDS tile formats -------------------------------------------------------
// The reduction advances kBK = 32 elements of a 16-bit type per step.
// MC ("m/n-contiguous") panel: the operand is row-major with the reduction index OUTERMOST.  A panel
//   is 32 k-rows x 256 bytes (128 columns); the four 64-byte blocks of a row are stored at block
//   position b ^ (k & 3), so the four k-rows gathered by one ds_read_b64_tr_b16 hit disjoint banks
//   (the tiled kernel additionally swaps the 32-byte halves of every block on k-rows 8..15 and
//   24..31, see read_frag_mc16).
// The k-contiguous formats (rows of 128 or 64 bytes with XOR-swizzled 16-byte chunks) are described
// where they are read: read_frag_kc16 in fsw_gemm.hpp, read_frag_kc32 in fsw_skinny.hip.
constexpr int kBK = 32;
constexpr int kMcRowBytes = 256;
constexpr int kMcPanelBytes = kBK * kMcRowBytes;  // 8 KiB

// ---- XCD-aware tile order -----------------------------------------------------
// Workgroups are dealt to the 8 XCDs round-robin by launch index.  Re-number them so that each
// XCD works through one contiguous range of logical tiles, and inside that range walk bands of
// `group_m` tile-rows column by column: the ~32 tiles an XCD runs at once then share few A and B
// panels in that XCD's private L2.
struct TileCoord {
  int tm, tn;
};
FSW_DEV TileCoord xcd_tile_order(int bid, int tiles_m, int tiles_n, int group_m) {
  const int nt = tiles_m * tiles_n;
  const int q = nt >> 3, r = nt & 7;
  const int xcd = bid & 7, i = bid >> 3;
  const int lin = (xcd < r) ? xcd * (q + 1) + i : r * (q + 1) + (xcd - r) * q + i;
  const int per_band = group_m * tiles_n;
  const int band = lin / per_band;
  const int first_m = band * group_m;
  const int rows = min(tiles_m - first_m, group_m);
  const int in_band = lin - band * per_band;
  TileCoord t;
  t.tm = first_m + in_band % rows;
  t.tn = in_band / rows;
  return t;
}

}  // namespace fsw
