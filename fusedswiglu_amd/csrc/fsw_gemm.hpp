// The tiled MFMA kernel behind the three GEMM-shaped steps of the SwiGLU path.
//
//   kFwd  out = silu(x Wg) * (x Wu)      A = x [T,D] (k-contiguous), B = Wg | Wu [D,I] (n-contiguous)
//   kDx   dx  = dG Wg^T + dU Wu^T        A = dG | dU [T,I] (k-contiguous), B = Wg | Wu [D,I] rows (k-contiguous)
//   kDw   dWg = x^T dG, dWu = x^T dU     A = x [T,D] (m-contiguous), B = dG | dU [T,I] (n-contiguous)
//
// One workgroup = 8 wavefronts (2 along M x 4 along N) = one 256 x 256 fp32 accumulator tile
// (kFwd / kDw: 256 rows x 128 columns of EACH of the two results, sharing the A tile).
// The reduction advances 32 elements per step through a 4-deep ring of 32 KiB LDS stages that
// is filled by direct global->LDS loads three steps ahead of the MFMAs.
#pragma once
#include "fsw_common.hpp"

namespace fsw {

enum Mode { kFwd = 0, kDx = 1, kDw = 2 };

struct GemmParams {
  const void* a0;  // kFwd: x      kDx: dG     kDw: x
  const void* a1;  //              kDx: dU
  const void* b0;  // kFwd: Wg     kDx: Wg     kDw: dG
  const void* b1;  // kFwd: Wu     kDx: Wu     kDw: dU
  void* c0;        // kFwd: out    kDx: dx     kDw: dWg
  void* c1;        // kFwd: g (may be null)    kDw: dWu
  void* c2;        // kFwd: u (may be null)
  int M, N, K;     // GEMM view: kFwd (T,I,D)  kDx (T,D,I)  kDw (D,I,T)
  int lda, ldb, ldc;  // leading dimensions in elements
  int tiles_m, tiles_n, group_m;
};

constexpr int kThreads = 512;
#ifndef FSW_STAGES
#define FSW_STAGES 4
#endif
constexpr int kStages = FSW_STAGES;
constexpr int kRegionBytes = 16384;           // one operand tile of one stage
constexpr int kStageBytes = 2 * kRegionBytes;  // A region then B region
constexpr int kTileM = 256;
template <int MODE>
constexpr int tile_n() {
  return MODE == kDx ? 256 : 128;
}

// ---- fragment reads -----------------------------------------------------------
// K-contiguous tile: lane l gets row (l & 31), k = ks*16 + 8*(l >> 5) .. +8 in one ds_read_b128.
FSW_DEV i16x8 read_frag_kc(const FSW_LDS char* region, int row_base, int ks, int lane) {
  const int row = row_base + (lane & 31);
  const int chunk = (ks * 2 + (lane >> 5)) ^ ((lane >> 2) & 3);
  return *(const FSW_LDS i16x8*)(region + row * kKcRowBytes + chunk * 16);
}

// M/N-contiguous panel: two transposing reads.  Within each group of 16 lanes, lane j supplies the
// address of 4 consecutive columns (j & 3)*4.. of k-row (j >> 2); the hardware hands lane i the
// column i of those four k-rows.  Lane groups 0/1 cover columns 0-15 / 16-31 of the 32-column
// fragment, groups 2/3 the same columns 8 k-rows further on -- the MFMA operand layout.
FSW_DEV i16x8 read_frag_mc(const FSW_LDS char* panel, int block64, int ks, int lane) {
  const int grp = lane >> 4, j = lane & 15;
  const int krow = ks * 16 + 8 * (grp >> 1) + (j >> 2);
  const int byte = krow * kMcRowBytes + ((block64 ^ (j >> 2)) * 64) + ((grp & 1) * 16 + (j & 3) * 4) * 2;
  i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)(panel + byte));
  i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)(panel + byte + 4 * kMcRowBytes));
  i16x8 r;
  r.s0 = lo.x; r.s1 = lo.y; r.s2 = lo.z; r.s3 = lo.w;
  r.s4 = hi.x; r.s5 = hi.y; r.s6 = hi.z; r.s7 = hi.w;
  return r;
}

// ---- per-thread description of one direct-to-LDS load -----------------------------
struct DmaSlot {
  unsigned lane_off;  // byte offset of this lane's 16 bytes relative to the moving base
  int klim;           // the load is in range while k0 < klim
};

template <typename E, int MODE>
__global__ __launch_bounds__(kThreads) void fsw_gemm_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(1024))) char smem[kStages * kStageBytes];
  constexpr bool A_KC = (MODE != kDw);
  constexpr bool B_KC = (MODE == kDx);
  constexpr int TN = tile_n<MODE>();

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;

  const TileCoord tc = xcd_tile_order(blockIdx.x, p.tiles_m, p.tiles_n, p.group_m);
  const int m0 = tc.tm * kTileM;
  const int n0 = tc.tn * TN;

  const int kt1 = (p.K + kBK - 1) / kBK;
  const int kt_total = (MODE == kDx) ? 2 * kt1 : kt1;

  const unsigned smem_addr = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const FSW_LDS char* smem_l = (const FSW_LDS char*)smem;

  // ---- DMA set-up: every wave issues instructions {wave, wave + 8} of each 16-instruction region
  DmaSlot sa[2], sb[2];
  const char* a_base[2];  // per instruction: pointer of the tile origin at k0 = 0 (uniform)
  const char* b_base[2];
  const char* a_base2[2];  // kDx second pass
  const char* b_base2[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int j = wave + 8 * i;
    if constexpr (A_KC) {
#ifdef FSW_DBG_KC128
      const int row = 8 * j + (lane >> 3);
      const int c = (lane & 7);
#else
      const int row = 16 * j + (lane >> 2);
      const int c = (lane & 3) ^ ((lane >> 4) & 3);
#endif
      sa[i].lane_off = (unsigned)row * (unsigned)p.lda * 2u + c * 16u;
      sa[i].klim = (m0 + row < p.M) ? p.K - c * 8 : -0x40000000;
      a_base[i] = (const char*)p.a0 + (size_t)m0 * p.lda * 2;
      a_base2[i] = (const char*)p.a1 + (size_t)m0 * p.lda * 2;
    } else {
      // kDw: panel (j >> 3) holds x columns m0 + 128*(j >> 3) ..
      const int row = 4 * (j & 7) + (lane >> 4);
      const int col = (((lane >> 2) & 3) ^ ((lane >> 4) & 3)) * 32 + (lane & 3) * 8;
      const int col0 = m0 + 128 * (j >> 3);
      sa[i].lane_off = (unsigned)row * (unsigned)p.lda * 2u + col * 2u;
      sa[i].klim = (col0 + col < p.M) ? p.K - row : -0x40000000;
      a_base[i] = (const char*)p.a0 + (size_t)col0 * 2;
      a_base2[i] = a_base[i];
    }
    if constexpr (B_KC) {
#ifdef FSW_DBG_KC128
      const int row = 8 * j + (lane >> 3);
      const int c = (lane & 7);
#else
      const int row = 16 * j + (lane >> 2);
      const int c = (lane & 3) ^ ((lane >> 4) & 3);
#endif
      sb[i].lane_off = (unsigned)row * (unsigned)p.ldb * 2u + c * 16u;
      sb[i].klim = (n0 + row < p.N) ? p.K - c * 8 : -0x40000000;
      b_base[i] = (const char*)p.b0 + (size_t)n0 * p.ldb * 2;
      b_base2[i] = (const char*)p.b1 + (size_t)n0 * p.ldb * 2;
    } else {
      // panel 0 = first B matrix, panel 1 = second, same 128 columns n0..
      const int row = 4 * (j & 7) + (lane >> 4);
      const int col = (((lane >> 2) & 3) ^ ((lane >> 4) & 3)) * 32 + (lane & 3) * 8;
      sb[i].lane_off = (unsigned)row * (unsigned)p.ldb * 2u + col * 2u;
      sb[i].klim = (n0 + col < p.N) ? p.K - row : -0x40000000;
      b_base[i] = (const char*)((j >> 3) ? p.b1 : p.b0) + (size_t)n0 * 2;
      b_base2[i] = b_base[i];
    }
  }
  const size_t a_kstep = A_KC ? (size_t)kBK * 2 : (size_t)kBK * p.lda * 2;
  const size_t b_kstep = B_KC ? (size_t)kBK * 2 : (size_t)kBK * p.ldb * 2;

  auto issue = [&](int kt) {
    const int pass = (MODE == kDx && kt >= kt1) ? 1 : 0;
    const int ktl = kt - pass * kt1;
    const int k0 = ktl * kBK;
    const unsigned stage_addr = smem_addr + (unsigned)(kt % kStages) * kStageBytes;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int j = wave + 8 * i;
      const char* ab = (pass ? a_base2[i] : a_base[i]) + (size_t)ktl * a_kstep;
      const unsigned off = (k0 < sa[i].klim) ? sa[i].lane_off : kOobOffset;
      load16_to_lds(make_rsrc(ab), off, stage_addr + j * 1024);
    }
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int j = wave + 8 * i;
      const char* bb = (pass ? b_base2[i] : b_base[i]) + (size_t)ktl * b_kstep;
      const unsigned off = (k0 < sb[i].klim) ? sb[i].lane_off : kOobOffset;
      load16_to_lds(make_rsrc(bb), off, stage_addr + kRegionBytes + j * 1024);
    }
  };

  f32x16 acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][q][r] = 0.f;

  // ---- main loop: two groups of four waves (one per SIMD each) run half a step out of phase.
  // While one group reads its fragments of a stage from LDS (and issues its share of the loads
  // for the stage three ahead), the other group issues the 16 MFMAs of the stage it read one
  // phase earlier, so the matrix cores of every SIMD always have a wave to serve.  Phases are
  // separated by workgroup barriers; group 1 enters one barrier late and leaves one early.
  const int grp = wave >> 2;
  auto phase_barrier = [&](int kt) {
    // stage kt+1 must have landed (for every wave's share) before the next phase reads it;
    // stages kt+2 and kt+3, if they exist, may stay in flight
    const int ahead = min(kt_total - 2 - kt, kStages - 2);
    if (ahead >= 3) wait_vmcnt_and_barrier<12>();
    else if (ahead == 2) wait_vmcnt_and_barrier<8>();
    else if (ahead == 1) wait_vmcnt_and_barrier<4>();
    else wait_vmcnt_and_barrier<0>();
  };
#pragma unroll
  for (int s = 0; s < kStages - 1; s++)
    if (s < kt_total) issue(s);
  phase_barrier(-1);
  if (grp == 1) wait_vmcnt_and_barrier<63>();

  for (int kt = 0; kt < kt_total; kt++) {
    const FSW_LDS char* ra = smem_l + (kt % kStages) * kStageBytes;
    const FSW_LDS char* rb = ra + kRegionBytes;
    i16x8 fq[2][4], fp[2][2];
#ifdef FSW_DBG_NO_LDSREAD
    for (int ks = 0; ks < 2; ks++) { for (int q = 0; q < 4; q++) fq[ks][q] = (i16x8)(short)(kt + q); for (int a = 0; a < 2; a++) fp[ks][a] = (i16x8)(short)(kt + a); }
    if (p.M < 0)
#endif
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int q = 0; q < 4; q++) {
        if constexpr (A_KC) fq[ks][q] = read_frag_kc(ra, wm * 128 + q * 32, ks, lane);
        else fq[ks][q] = read_frag_mc(ra + wm * kMcPanelBytes, q, ks, lane);
      }
#pragma unroll
      for (int a = 0; a < 2; a++) {
        if constexpr (B_KC) fp[ks][a] = read_frag_kc(rb, wn * 64 + a * 32, ks, lane);
        else fp[ks][a] = read_frag_mc(rb + a * kMcPanelBytes, wn, ks, lane);
      }
    }
#ifndef FSW_DBG_NO_DMA
    if (kt + kStages - 1 < kt_total) issue(kt + kStages - 1);
#endif
    phase_barrier(kt);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int a = 0; a < 2; a++) acc[a][q] = E::mfma(fp[ks][a], fq[ks][q], acc[a][q]);
    __builtin_amdgcn_sched_barrier(0);
    if (!(grp == 1 && kt == kt_total - 1)) phase_barrier(kt);
  }

  // ---- epilogue.  acc[a][q][r] of lane l is row  m0 + wm*128 + q*32 + (l & 31)  and column
  //      cbase(a) + 8*(r >> 2) + 4*(l >> 5) + (r & 3): four consecutive columns per 8-byte store.
#ifdef FSW_DBG_NO_STORE
  if (p.M > 0 && acc[0][0][0] != 123.456f) return;
#endif
  const int mrow = m0 + wm * 128 + (lane & 31);
  const int ncol_l = 4 * (lane >> 5);
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int m = mrow + q * 32;
    if (m >= p.M) continue;
#pragma unroll
    for (int r4 = 0; r4 < 4; r4++) {
      if constexpr (MODE == kFwd) {
        const int n = n0 + wn * 32 + 8 * r4 + ncol_l;
        if (n >= p.N) continue;
        const size_t o = (size_t)m * p.ldc + n;
        u32x2 vo, vg, vu;
        unsigned short ho[4], hg[4], hu[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float g = acc[0][q][r4 * 4 + e], u = acc[1][q][r4 * 4 + e];
          ho[e] = E::from_float(silu_mul(g, u));
          hg[e] = E::from_float(g);
          hu[e] = E::from_float(u);
        }
        vo.x = ho[0] | ((unsigned)ho[1] << 16); vo.y = ho[2] | ((unsigned)ho[3] << 16);
        *(u32x2*)((unsigned short*)p.c0 + o) = vo;
        if (p.c1) {
          vg.x = hg[0] | ((unsigned)hg[1] << 16); vg.y = hg[2] | ((unsigned)hg[3] << 16);
          vu.x = hu[0] | ((unsigned)hu[1] << 16); vu.y = hu[2] | ((unsigned)hu[3] << 16);
          *(u32x2*)((unsigned short*)p.c1 + o) = vg;
          *(u32x2*)((unsigned short*)p.c2 + o) = vu;
        }
      } else {
#pragma unroll
        for (int a = 0; a < 2; a++) {
          const int n = (MODE == kDx) ? n0 + wn * 64 + a * 32 + 8 * r4 + ncol_l
                                      : n0 + wn * 32 + 8 * r4 + ncol_l;
          if (n >= p.N) continue;
          const size_t o = (size_t)m * p.ldc + n;
          unsigned short h[4];
#pragma unroll
          for (int e = 0; e < 4; e++) h[e] = E::from_float(acc[a][q][r4 * 4 + e]);
          u32x2 v;
          v.x = h[0] | ((unsigned)h[1] << 16); v.y = h[2] | ((unsigned)h[3] << 16);
          unsigned short* dst = (MODE == kDx || a == 0) ? (unsigned short*)p.c0 : (unsigned short*)p.c1;
          *(u32x2*)(dst + o) = v;
        }
      }
    }
  }
}

}  // namespace fsw
