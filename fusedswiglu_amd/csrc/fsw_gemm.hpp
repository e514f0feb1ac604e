// The tiled MFMA kernel behind every GEMM-shaped step of the SwiGLU path.  Weights are [D, I] ("in x out",
// the reference's layout) in the first three modes and [I, D] (nn.Linear's layout) in the *T modes; the
// three plain modes serve the down projection y = out W_down that follows the SwiGLU in an MLP.
//
//   kFwd   out = silu(x Wg) * (x Wu)    A = x [T,D] (k-contiguous), B = Wg | Wu [D,I] (n-contiguous)
//   kDx    dx  = dG Wg^T + dU Wu^T      A = dG | dU [T,I] (k-contiguous), B = Wg | Wu [D,I] rows (k-contiguous)
//   kDw    dWg = x^T dG, dWu = x^T dU   A = x [T,D] (m-contiguous), B = dG | dU [T,I] (n-contiguous)
//   kNN    C = A B                      A [M,K] k-contiguous, B [K,N] n-contiguous
//   kNT    C = A B^T                    A [M,K] k-contiguous, B [N,K] k-contiguous
//   kTN    C = A^T B                    A [K,M] m-contiguous, B [K,N] n-contiguous
//   kFwdT  out = silu(x Wg^T) * (x Wu^T)   B = Wg | Wu [I,D] rows (k-contiguous)
//   kDxT   dx  = dG Wg + dU Wu             B = Wg | Wu [I,D] (n-contiguous), two passes
//   kDwT   dWg = dG^T x, dWu = dU^T x      A = dG | dU [T,I] (m-contiguous), B = x [T,D] (n-contiguous)
//
// One workgroup = 8 wavefronts (4 along M x 2 along N) = one 256 x 256 fp32 accumulator tile (in the dual
// modes 256 rows x 128 columns of EACH of the two results sharing the A tile; kDwT: 128 rows of each result
// sharing the B tile).
// The reduction advances 32 elements per step and is organised in PAIRS of steps.  Operand tiles are
// brought in by direct global->LDS loads one to two pairs ahead of the MFMAs and kept in LDS rings
// (A: three pairs, B: two pairs, 160 KiB in all):
//   * an m/n-contiguous ("MC") operand uses 16 KiB slots, one per step;
//   * a k-contiguous ("KC") operand is fetched 64 k-elements (one full 128-byte line per row) at a
//     time into 32 KiB areas, each serving the two steps of a pair.  Fetching half lines
//     (64 bytes per row per step) halves the throughput of the texture-address path.
// Every wave runs the same free-running loop: it holds the fragments of BOTH steps of the current pair
// in registers, so a pair's LDS space is released (and refilled) at the single barrier in the middle of
// the pair, and the fragment reads of a step are always one step ahead of the MFMAs that consume them.
#pragma once
#include <type_traits>
#include <utility>

#include "fsw_common.hpp"

namespace fsw {

enum Mode { kFwd = 0, kDx = 1, kDw = 2, kNN = 3, kNT = 4, kTN = 5, kFwdT = 6, kDxT = 7, kDwT = 8 };

struct GemmParams {
  const void* a0;  // kFwd*: x     kDx*: dG    kDw: x     kDwT: dG    plain: A
  const void* a1;  //              kDx*: dU               kDwT: dU
  const void* b0;  // kFwd*: Wg    kDx*: Wg    kDw: dG    kDwT: x     plain: B
  const void* b1;  // kFwd*: Wu    kDx*: Wu    kDw: dU
  void* c0;        // kFwd*: out   kDx*: dx    kDw*: dWg              plain: C
  void* c1;        // kFwd*: g (may be null)   kDw*: dWu
  void* c2;        // kFwd*: u (may be null)
  // kFwd* only, gating-gradient mode (d0 != null): nothing is written to c0; c1 = dG, c2 = dU with
  // dU = d0 * silu(g), dG = d0 * u * silu'(g) computed from the fp32 accumulators (d0 has ldc too)
  const void* d0;
  int M, N, K;     // result rows x columns (per result) and reduction length (per pass)
  int lda, ldb, ldc;  // leading dimensions in elements
  int tiles_m, tiles_n, group_m;
  // split-K (every mode but the forwards, on small problems): `splits` workgroups per tile each reduce
  // `steps_per_split` steps (even) and store an fp32 partial tile to ws[split][M][N] (second result:
  // + splits*M*N); fsw_splitk_reduce_kernel adds the partials in a fixed order.  splits == 1: results go
  // to c0/c1.
  float* ws;
  int splits, steps_per_split;
  // tail split (four-wave kernel, every mode but the forwards, splits == 1): the tiles of the last, partial round
  // of 256 workgroups - launch indices tail_first .. tail_first + tail_count - 1 - are each given to tail_parts
  // workgroups that reduce tail_steps steps (even) and leave an fp32 partial tile in ws[tile][part][kTileFloats];
  // fsw_tail_reduce_kernel adds the parts in a fixed order.  tail_count == 0: off.
  int tail_first, tail_count, tail_parts, tail_steps;
};
constexpr int kTileFloats = 256 * 256;  // accumulators of one workgroup

constexpr int kThreads = 512;
constexpr int kMcSlotBytes = 2 * kMcPanelBytes;  // two 128-column panels: 16 KiB
constexpr int kKcAreaBytes = 256 * 128;          // 256 rows x 64 k-elements: 32 KiB

template <int MODE>
struct Cfg {
  static constexpr bool kAKc = !(MODE == kDw || MODE == kTN || MODE == kDwT);
  static constexpr bool kBKc = (MODE == kDx || MODE == kNT || MODE == kFwdT);
  static constexpr bool kForward = (MODE == kFwd || MODE == kFwdT);
  static constexpr int kPasses = (MODE == kDx || MODE == kDxT) ? 2 : 1;
  // two results that share the A tile (128 columns of each per tile) / the B tile (128 rows of each)
  static constexpr bool kDualN = (MODE == kFwd || MODE == kDw || MODE == kFwdT);
  static constexpr bool kDualM = (MODE == kDwT);
  static constexpr int kResults = (MODE == kDw || MODE == kDwT) ? 2 : 1;
  static constexpr int kTileM = kDualM ? 128 : 256;  // result rows / columns one tile covers
  static constexpr int kTileN = kDualN ? 128 : 256;
  // rings in pairs of steps: 96 KiB for A, 64 KiB for B in either layout
  static constexpr int kPairsA = 3;
  static constexpr int kPairsB = 2;
  static constexpr int kBytesA = kPairsA * kKcAreaBytes;
  static constexpr int kBytesB = kPairsB * kKcAreaBytes;
};
static_assert(kKcAreaBytes == 2 * kMcSlotBytes, "a pair of steps takes 32 KiB in either layout");

// ---- fragment reads -----------------------------------------------------------
// KC area: 256 rows x 128 bytes; the 16-byte chunk c of row r sits at chunk position
// c ^ ((r >> 1) & 7), so that 16 consecutive rows cover all 64 banks for a fixed c.
// 16x16x32 operand: lane l gets row (l & 15), k = half*32 + 8*(l >> 4) .. +8 in one ds_read_b128.
FSW_DEV i16x8 read_frag_kc16(const FSW_LDS char* area, int row_base, int half, int lane) {
  const int row = row_base + (lane & 15);
  const int chunk = (half * 4 + (lane >> 4)) ^ ((lane >> 1) & 7);
  return *(const FSW_LDS i16x8*)(area + row * 128 + chunk * 16);
}

// MC panel of the weight-streaming kernel: 32 k-rows x 256 bytes; the 64-byte block b of k-row k sits
// at block position b ^ (k & 3).  32x32x16 operand by two transposing reads.  Within each group of 16
// lanes, lane j supplies the address of 4 consecutive columns (j & 3)*4.. of k-row (j >> 2); the
// hardware hands lane i the column i of those four k-rows.  Lane groups 0/1 cover columns 0-15 /
// 16-31 of the 32-column fragment, groups 2/3 the same columns 8 k-rows further on.
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

// MC panel of the tiled kernel: as above, and in k-rows with (k >> 3) odd the two 32-byte halves of
// every 64-byte block are swapped.  16x16x32 operand (16 columns x 32 k-rows) by two transposing
// reads: lane group g covers k-rows 8g .. 8g+7 (first read 8g..+3, second 8g+4..+7) of the same 16
// columns, lane j of a group supplying columns (j & 3)*8 bytes.. of k-row (j >> 2).  Groups 0 and 1 (and 2
// and 3) then sit in different 32-byte halves, so each half-wave touches every bank once.
// The byte address of fragment f (16-column block f of the panel) is
//   krow*256 + (((f >> 1) ^ (j >> 2)) * 64) + (((f ^ grp) & 1) * 32) + (j & 3)*8  =  mc_lane_offset ^ (f << 5):
// one per-lane offset serves every fragment, the fragment index only flips address bits 5..7.
FSW_DEV unsigned mc_lane_offset(int lane) {
  const int grp = lane >> 4, j = lane & 15;
  return (unsigned)((8 * grp + (j >> 2)) * kMcRowBytes + (j >> 2) * 64 + (grp & 1) * 32 + (j & 3) * 8);
}
// `lane_ptr` = start of the panel (1 KiB aligned) + mc_lane_offset(lane)
FSW_DEV i16x8 read_frag_mc16(const FSW_LDS char* lane_ptr, int frag16) {
  const FSW_LDS char* q = (const FSW_LDS char*)(uintptr_t)((unsigned)(uintptr_t)lane_ptr ^ (unsigned)(frag16 << 5));
  i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)q);
  i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)(q + 4 * kMcRowBytes));
  i16x8 r;
  r.s0 = lo.x; r.s1 = lo.y; r.s2 = lo.z; r.s3 = lo.w;
  r.s4 = hi.x; r.s5 = hi.y; r.s6 = hi.z; r.s7 = hi.w;
  return r;
}

// ---- per-wave description of an operand's direct-to-LDS loads -----------------------
// KC operand: a wave issues 4 instructions per area (tile rows 8*(wave + 8i) .. +8, 128 bytes each).
struct KcLoader {
  unsigned lane_off;   // byte offset of this lane's 16 bytes for i = 0, relative to the moving base
  unsigned row_step;   // bytes between the rows of consecutive i
  int klim[4];         // instruction i is in range while k0 < klim[i]
  const char* base0;   // tile origin at k = 0: first pass / first matrix
  const char* base1;   // second pass (kDx) or second matrix (kFwdT), else the same
};
// MC operand: 2 instructions per slot (wave, wave + 8): 4 k-rows x 256 bytes of panel (j >> 3).
struct McLoader {
  unsigned lane_off[2];
  int klim[2];
  const char* base[2];   // per panel
  const char* base2[2];  // per panel, second pass (kDxT), else the same
  size_t kstep;  // bytes per 32 k-rows
};

FSW_DEV void kc_setup(KcLoader& L, const void* p0, const void* p1, int row0, int rows_total, int K,
                      int ld, int wave, int lane) {
  const int row = 8 * wave + (lane >> 3);
  const int c = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
  L.lane_off = (unsigned)row * (unsigned)ld * 2u + c * 16u;
  L.row_step = 64u * (unsigned)ld * 2u;
#pragma unroll
  for (int i = 0; i < 4; i++) L.klim[i] = (row0 + row + 64 * i < rows_total) ? K - c * 8 : -0x40000000;
  L.base0 = (const char*)p0 + (size_t)row0 * ld * 2;
  L.base1 = (const char*)p1 + (size_t)row0 * ld * 2;
}

// kFwdT: the 256 tile rows interleave the two weight matrices in blocks of 64 - instruction i fetches rows
// row0 + 64*(i >> 1) + 8*wave.. of matrix (i & 1) - so that each wave's 128 B rows are 64 gate and 64 up
// rows of the same output columns.
FSW_DEV void kc_setup_interleaved(KcLoader& L, const void* p0, const void* p1, int row0, int rows_total,
                                  int K, int ld, int wave, int lane) {
  const int row = 8 * wave + (lane >> 3);
  const int c = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
  L.lane_off = (unsigned)row * (unsigned)ld * 2u + c * 16u;
  L.row_step = 64u * (unsigned)ld * 2u;
#pragma unroll
  for (int i = 0; i < 4; i++) L.klim[i] = (row0 + row + 64 * (i >> 1) < rows_total) ? K - c * 8 : -0x40000000;
  L.base0 = (const char*)p0 + (size_t)row0 * ld * 2;
  L.base1 = (const char*)p1 + (size_t)row0 * ld * 2;
}

FSW_DEV void mc_setup(McLoader& L, const void* p_panel0, const void* p_panel1, const void* q_panel0,
                      const void* q_panel1, int col0_panel0, int col0_panel1, int cols_total, int K, int ld,
                      int wave, int lane) {
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int j = wave + 8 * i;
    const int row = 4 * (j & 7) + (lane >> 4);
    // physical 16-byte chunk (lane & 15) of k-row `row` holds logical columns `col`.. (see read_frag_mc16)
    const int col = (((lane >> 2) & 3) ^ (row & 3)) * 32 + ((((lane >> 1) ^ (row >> 3)) & 1) * 16) + (lane & 1) * 8;
    const int col0 = (j >> 3) ? col0_panel1 : col0_panel0;
    L.lane_off[i] = (unsigned)row * (unsigned)ld * 2u + col * 2u;
    L.klim[i] = (col0 + col < cols_total) ? K - row : -0x40000000;
    L.base[i] = (const char*)((j >> 3) ? p_panel1 : p_panel0) + (size_t)col0 * 2;
    L.base2[i] = (const char*)((j >> 3) ? q_panel1 : q_panel0) + (size_t)col0 * 2;
  }
  L.kstep = (size_t)kBK * ld * 2;
}

// STREAM_B: the B operand is read once by the whole launch (a single row of tiles): load it non-temporally
template <int... I, typename F>
FSW_DEV void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
FSW_DEV void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// ---- the epilogue of both forms of the tiled kernel: rounding, silu(g) * u or the gating gradients, and whole
// 128-byte lines to memory.
//
// A wave holds 32*NQ rows x 128 columns of accumulators: acc[nb][mb][r] of lane l is the wave's row
// mb*16 + (l & 15) and, within the wave's half h = nb >> 2, column (nb & 3)*16 + 4*(l >> 4) + r of 64 consecutive
// result columns (128 bytes).  Half h goes to result res_half[h] (0: c0, 1: c1) at columns col_half[h]..; in the
// forwards the two halves are gate and up of the same 64 columns col_half[0].
//
// The work is a sequence of "parts" (32 rows x 64 columns of one result each) in a software pipeline: while the
// values of part k are computed and written into LDS patch k & 1 (32 rows x 128 bytes; 16-byte chunk c of row r
// sits at position c ^ ((r >> 1) & 7), so neither the 8-byte accumulator writes nor the 16-byte row reads
// conflict), the lines of part k-1 are on their way from the other patch to memory.  Everything is branch free -
// edges are masked through the offsets of buffer stores and loads, which the descriptors' range check drops - so
// the whole epilogue is one basic block that the compiler schedules across parts.  The results are written once
// and read by a later kernel at the earliest: non-temporal stores keep them out of the way of the operands.
//
// ACC_ASM: the accumulators live in the accumulation registers behind inline-asm MFMAs (four-wave form); they are
// then moved out by explicit instructions at their turn and not earlier (left to the compiler, they are moved out
// wholesale after the main loop and spill).
template <typename E, int MODE, int NQ, bool ACC_ASM>
FSW_DEV void store_tile(const GemmParams& p, f32x4 (&acc)[8][2 * NQ], FSW_LDS char* patch, int lane, int row_base,
                        int col_half0, int col_half1, int res_half0, int res_half1) {
  using C = Cfg<MODE>;
  constexpr int kPatchPitch = 128, kPatchBytes = 32 * kPatchPitch;
  const int wr_row = (lane & 15) * kPatchPitch, wr_swz = (lane >> 1) & 7, wr_grp = lane >> 4;
  // 8 bytes of column group wr_grp of 16-column block c:  chunk 2c + (wr_grp >> 1), half wr_grp & 1
  auto wr_off = [&](int mbl, int c) {
    return mbl * 16 * kPatchPitch + wr_row + (((2 * c + (wr_grp >> 1)) ^ wr_swz) << 4) + (wr_grp & 1) * 8;
  };
  // row 8i + (lane >> 3), chunk lane & 7
  auto rd_off = [&](int i) {
    const int row = 8 * i + (lane >> 3);
    return row * kPatchPitch + (((lane & 7) ^ ((row >> 1) & 7)) << 4);
  };
  const int rows_left = p.M - row_base;             // rows of this wave that exist (may be <= 0 or >= 32*NQ)
  const unsigned ldc_bytes = (unsigned)p.ldc * 2u;  // the host keeps 128 rows of a result below 2^31 bytes
  // a result seen from the wave's first row and column `col_base`
  auto result_rsrc = [&](const void* base, int col_base) {
    return __builtin_amdgcn_make_buffer_rsrc((char*)base + ((size_t)row_base * p.ldc + col_base) * 2, 0, 0x7fffffff,
                                             kRsrcWord3);
  };
  // line store i of a part: lane l holds chunk l & 7 of row 8*i + (l >> 3) of the part's 32 rows
  const unsigned st_lane = (unsigned)(lane >> 3) * ldc_bytes + (unsigned)(lane & 7) * 16u;
  u32x4 in_flight[4];
  auto read_part = [&](int k) {
#pragma unroll
    for (int i = 0; i < 4; i++) in_flight[i] = *(const FSW_LDS u32x4*)(patch + (k & 1) * kPatchBytes + rd_off(i));
  };
  // st_cols: st_lane, or the out-of-range offset in lanes whose columns do not exist
  auto store_part = [&](__amdgpu_buffer_rsrc_t rs, unsigned st_cols, int q) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int r0 = q * 32 + 8 * i;
      // The row offset goes through the vector offset, not the scalar one: behind a 16-byte store with a scalar
      // offset REGISTER the compiler leaves out the wait state before the next instruction that overwrites the
      // store's data registers, and on this hardware the store then picks up the new value in some lanes.
      const unsigned off = ((lane >> 3) < rows_left - r0 ? st_cols : kOobOffset) + (unsigned)r0 * ldc_bytes;
      __builtin_amdgcn_raw_buffer_store_b128(in_flight[i], rs, off, 0, 2 /* nt */);
    }
  };
  auto write_part = [&](int k, int mbl, int c, float a, float b, float cc, float d) {
    u32x2 v;
    v.x = E::pack2(a, b);
    v.y = E::pack2(cc, d);
    *(FSW_LDS u32x2*)(patch + (k & 1) * kPatchBytes + wr_off(mbl, c)) = v;
  };
  auto acc_read = [&](float a) {
    if constexpr (ACC_ASM) {
      float v;
      asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
      return v;
    } else {
      return a;
    }
  };
  auto acc_read4 = [&](const f32x4& a) { return f32x4{acc_read(a.x), acc_read(a.y), acc_read(a.z), acc_read(a.w)}; };
  if constexpr (C::kForward) {
    const int colw = col_half0;
    const unsigned st_cols = colw + (lane & 7) * 8 < p.N ? st_lane : kOobOffset;
    // first: 0 = out, g, u (or out alone when the caller passes no buffers for g and u); 1 = dG, dU from dout
    // (gating-gradient mode, d0 given).  Compile-time parameters, so that the parts carry no branch on them.
    auto forward_tile = [&](auto first_tag, auto count_tag) {
      constexpr int first = decltype(first_tag)::value, count = decltype(count_tag)::value;
      constexpr bool gating = first == 1;
      __amdgpu_buffer_rsrc_t rs[3] = {result_rsrc(p.c0, colw), result_rsrc(count > 1 ? p.c1 : p.c0, colw),
                                      result_rsrc(count > 1 ? p.c2 : p.c0, colw)};
      __amdgpu_buffer_rsrc_t rs_d = result_rsrc(gating ? p.d0 : p.c0, colw);
      // dout in the accumulator layout: 4 consecutive columns of row (l & 15) per lane and 16x16 block
      const unsigned ld_lane = (unsigned)(lane & 15) * ldc_bytes + (unsigned)(lane >> 4) * 8u;
      unsigned ld_cols[4];
#pragma unroll
      for (int c = 0; c < 4; c++) ld_cols[c] = colw + c * 16 + 4 * (lane >> 4) < p.N ? ld_lane + c * 32u : kOobOffset;
      u32x2 dv[2][4];
      f32x4 gq[2][4], uq[2][4];  // the gate and up values of the 32 rows in hand
      static_for<NQ * count>([&](auto kc) {
        constexpr int k = decltype(kc)::value, q = k / count, which = first + k % count;
        if constexpr (k % count == 0) {
#pragma unroll
          for (int mbl = 0; mbl < 2; mbl++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
              gq[mbl][c] = acc_read4(acc[c][2 * q + mbl]);
              uq[mbl][c] = acc_read4(acc[4 + c][2 * q + mbl]);
            }
          if constexpr (gating) {
#pragma unroll
            for (int mbl = 0; mbl < 2; mbl++)
#pragma unroll
              for (int c = 0; c < 4; c++) {
                const int r0 = (2 * q + mbl) * 16;
                const unsigned off = (lane & 15) < rows_left - r0 ? ld_cols[c] : kOobOffset;
                dv[mbl][c] = __builtin_amdgcn_raw_buffer_load_b64(rs_d, off, (unsigned)r0 * ldc_bytes, 0);
              }
          }
        }
        if constexpr (k > 0) read_part(k - 1);
#pragma unroll
        for (int mbl = 0; mbl < 2; mbl++)
#pragma unroll
          for (int c = 0; c < 4; c++) {
            const f32x4 g = gq[mbl][c], u = uq[mbl][c];
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
              if constexpr (gating) {
                const unsigned w = e < 2 ? dv[mbl][c].x : dv[mbl][c].y;
                float dU, dG;
                gating_grad(E::to_float((unsigned short)((e & 1) ? (w >> 16) : (w & 0xffffu))), g[e], u[e], dU, dG);
                v[e] = which == 1 ? dG : dU;
              } else {
                v[e] = which == 0 ? silu_mul(g[e], u[e]) : (which == 1 ? g[e] : u[e]);
              }
            }
            write_part(k, mbl, c, v[0], v[1], v[2], v[3]);
          }
        if constexpr (k > 0) store_part(rs[first + (k - 1) % count], st_cols, (k - 1) / count);
      });
      read_part(NQ * count - 1);
      store_part(rs[first + count - 1], st_cols, NQ - 1);
    };
    if (p.d0 != nullptr) forward_tile(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
    else if (p.c1 != nullptr) forward_tile(std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{});
    else forward_tile(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
  } else {
    __amdgpu_buffer_rsrc_t rs[2] = {result_rsrc(res_half0 == 0 ? p.c0 : p.c1, col_half0),
                                    result_rsrc(res_half1 == 0 ? p.c0 : p.c1, col_half1)};
    const unsigned st_cols[2] = {col_half0 + (lane & 7) * 8 < p.N ? st_lane : kOobOffset,
                                 col_half1 + (lane & 7) * 8 < p.N ? st_lane : kOobOffset};
    static_for<2 * NQ>([&](auto kc) {
      constexpr int k = decltype(kc)::value, q = k >> 1, h = k & 1;
      if constexpr (ACC_ASM) {
        // (one result per half: pinning the registers costs a copy, which two or three tiles per launch do not feel)
#pragma unroll
        for (int c = 0; c < 4; c++) asm volatile("" : "+a"(acc[4 * h + c][2 * q]), "+a"(acc[4 * h + c][2 * q + 1]));
      }
      if constexpr (k > 0) read_part(k - 1);
#pragma unroll
      for (int mbl = 0; mbl < 2; mbl++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const f32x4 t = acc[4 * h + c][2 * q + mbl];
          write_part(k, mbl, c, t[0], t[1], t[2], t[3]);
        }
      if constexpr (k > 0) store_part(rs[(k - 1) & 1], st_cols[(k - 1) & 1], (k - 1) >> 1);
    });
    read_part(2 * NQ - 1);
    store_part(rs[1], st_cols[1], NQ - 1);
  }
}

template <typename E, int MODE, bool STREAM_B = false>
__global__ __launch_bounds__(kThreads) void fsw_gemm_kernel(GemmParams p) {
  using C = Cfg<MODE>;
  __shared__ __attribute__((aligned(1024))) char smem[C::kBytesA + C::kBytesB];
  constexpr bool A_KC = C::kAKc, B_KC = C::kBKc;
  constexpr int TM = C::kTileM, TN = C::kTileN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;  // 4 waves along M x 2 along N

  const int ntiles = p.tiles_m * p.tiles_n;
  const int split = C::kForward ? 0 : (int)(blockIdx.x / ntiles);
  const TileCoord tc = xcd_tile_order((int)(blockIdx.x - split * ntiles), p.tiles_m, p.tiles_n, p.group_m);
  const int m0 = tc.tm * TM;
  const int n0 = tc.tn * TN;

  // steps per pass; the two-pass modes (dG.W then dU.W) keep pairs of steps inside a pass
  const int kt1 = (C::kPasses == 2) ? (((p.K + kBK - 1) / kBK + 1) & ~1) : (p.K + kBK - 1) / kBK;
  const int kt_all = C::kPasses * kt1;
  // this workgroup reduces steps kbase .. kbase + kt_total - 1 (everything unless split-K is on)
  const int kbase = split * p.steps_per_split;
  const int kt_total = C::kForward ? kt_all : min(p.steps_per_split, kt_all - kbase);

  const unsigned smem_a = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const unsigned smem_b = smem_a + C::kBytesA;
  const FSW_LDS char* lds_a = (const FSW_LDS char*)smem;
  const FSW_LDS char* lds_b = lds_a + C::kBytesA;

  KcLoader ka, kb;
  McLoader ma, mb;
  if constexpr (A_KC) kc_setup(ka, p.a0, C::kPasses == 2 ? p.a1 : p.a0, m0, p.M, p.K, p.lda, wave, lane);
  else if constexpr (C::kDualM) mc_setup(ma, p.a0, p.a1, p.a0, p.a1, m0, m0, p.M, p.K, p.lda, wave, lane);
  else mc_setup(ma, p.a0, p.a0, p.a0, p.a0, m0, m0 + 128, p.M, p.K, p.lda, wave, lane);
  if constexpr (MODE == kFwdT) kc_setup_interleaved(kb, p.b0, p.b1, n0, p.N, p.K, p.ldb, wave, lane);
  else if constexpr (B_KC) kc_setup(kb, p.b0, C::kPasses == 2 ? p.b1 : p.b0, n0, p.N, p.K, p.ldb, wave, lane);
  else if constexpr (C::kDualN) mc_setup(mb, p.b0, p.b1, p.b0, p.b1, n0, n0, p.N, p.K, p.ldb, wave, lane);
  else mc_setup(mb, p.b0, p.b0, C::kPasses == 2 ? p.b1 : p.b0, C::kPasses == 2 ? p.b1 : p.b0, n0, n0 + 128, p.N, p.K,
                p.ldb, wave, lane);

  // Loads of the pair of steps (st, st+1), st even: four 1 KiB instructions per wave in either layout.
  // They are issued for EVERY pair index the loop asks for, also beyond the end of the reduction, where
  // every lane is out of range and zero-fills: the loop below is branch-free and its vmcnt arithmetic
  // never changes (and a last, odd step is multiplied by zeros).
  auto kc_pair = [&](const KcLoader& L, int st, int pairs, unsigned lds_base, bool interleaved, auto stream) {
    constexpr bool kStream = decltype(stream)::value;
    const int apr = kbase + st;  // absolute step
    const int pass = (C::kPasses == 2 && apr >= kt1) ? 1 : 0;
    const int k0 = (apr - pass * kt1) * kBK;
    const unsigned dst = lds_base + (unsigned)((st >> 1) % pairs) * kKcAreaBytes + wave * 1024;
    if (interleaved) {
      const i32x4 rs0 = make_rsrc(L.base0 + (size_t)k0 * 2), rs1 = make_rsrc(L.base1 + (size_t)k0 * 2);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const unsigned off = (k0 < L.klim[i]) ? L.lane_off + (i >> 1) * L.row_step : kOobOffset;
        if constexpr (kStream) load16_to_lds_stream((i & 1) ? rs1 : rs0, off, dst + i * 8192);
        else load16_to_lds((i & 1) ? rs1 : rs0, off, dst + i * 8192);
      }
    } else {
      const i32x4 rs = make_rsrc((pass ? L.base1 : L.base0) + (size_t)k0 * 2);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const unsigned off = (k0 < L.klim[i]) ? L.lane_off + i * L.row_step : kOobOffset;
        if constexpr (kStream) load16_to_lds_stream(rs, off, dst + i * 8192);
        else load16_to_lds(rs, off, dst + i * 8192);
      }
    }
  };
  auto mc_step = [&](const McLoader& L, int st, int pairs, unsigned lds_base, auto stream) {
    constexpr bool kStream = decltype(stream)::value;
    const int apr = kbase + st;
    const int pass = (C::kPasses == 2 && apr >= kt1) ? 1 : 0;
    const int ks = apr - pass * kt1;  // step inside the pass
    const int k0 = ks * kBK;
    const unsigned dst = lds_base + (unsigned)(st % (2 * pairs)) * kMcSlotBytes + wave * 1024;
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const unsigned off = (k0 < L.klim[i]) ? L.lane_off[i] : kOobOffset;
      const i32x4 rs = make_rsrc((pass ? L.base2[i] : L.base[i]) + (size_t)ks * L.kstep);
      if constexpr (kStream) load16_to_lds_stream(rs, off, dst + i * 8192);
      else load16_to_lds(rs, off, dst + i * 8192);
    }
  };
  auto issue_a = [&](int st) {
    constexpr std::false_type keep{};
    if constexpr (A_KC) kc_pair(ka, st, C::kPairsA, smem_a, false, keep);
    else { mc_step(ma, st, C::kPairsA, smem_a, keep); mc_step(ma, st + 1, C::kPairsA, smem_a, keep); }
  };
  auto issue_b = [&](int st) {
    constexpr std::bool_constant<STREAM_B> hint{};
    if constexpr (B_KC) kc_pair(kb, st, C::kPairsB, smem_b, MODE == kFwdT, hint);
    else { mc_step(mb, st, C::kPairsB, smem_b, hint); mc_step(mb, st + 1, C::kPairsB, smem_b, hint); }
  };
  // the 4 + 8 fragments of step kt (reading beyond the last step returns stale LDS bytes nobody uses)
  const unsigned mc_off = mc_lane_offset(lane);
  auto read_frags = [&](int kt, i16x8 (&fq)[4], i16x8 (&fp)[8]) {
    const FSW_LDS char* ra;
    const FSW_LDS char* rb;
    // MC: the per-lane offset is added to the (step-dependent) slot address here, so that the fragment
    // addresses are recomputed with one XOR each instead of living in eight registers
    if constexpr (A_KC) ra = lds_a + ((kt >> 1) % C::kPairsA) * kKcAreaBytes;
    else ra = lds_a + (kt % (2 * C::kPairsA)) * kMcSlotBytes + (wm >> 1) * kMcPanelBytes + mc_off;
    if constexpr (B_KC) rb = lds_b + ((kt >> 1) % C::kPairsB) * kKcAreaBytes;
    else rb = lds_b + (kt % (2 * C::kPairsB)) * kMcSlotBytes + mc_off;
    const int half = kt & 1;
#pragma unroll
    for (int mb = 0; mb < 4; mb++) {
      if constexpr (A_KC) fq[mb] = read_frag_kc16(ra, wm * 64 + mb * 16, half, lane);
      else fq[mb] = read_frag_mc16(ra, (wm & 1) * 4 + mb);
    }
#pragma unroll
    for (int nb = 0; nb < 8; nb++) {
      if constexpr (B_KC) fp[nb] = read_frag_kc16(rb, wn * 128 + nb * 16, half, lane);
      else fp[nb] = read_frag_mc16(rb + (nb >> 2) * kMcPanelBytes, wn * 4 + (nb & 3));
    }
  };

  // acc[nb][mb]: 16x16 block of rows wm*64 + mb*16.. and 16-column block nb of this wave:
  //   kFwd/kDw  nb = 4*a + c: matrix a (gate | up), columns wn*64 + c*16..
  //   kDx       columns wn*128 + nb*16..
  f32x4 acc[8][4];
#pragma unroll
  for (int nb = 0; nb < 8; nb++)
#pragma unroll
    for (int mb = 0; mb < 4; mb++) acc[nb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // 16 of a step's 32 MFMAs; consecutive MFMAs share one operand (the m index snakes back and forth)
  auto mfma_half = [&](const i16x8 (&fq)[4], const i16x8 (&fp)[8], int h) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int nb = 4 * h; nb < 4 * h + 4; nb++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int mb = (nb & 1) ? 3 - i : i;
        acc[nb][mb] = E::mfma16(fp[nb], fq[mb], acc[nb][mb]);
      }
    __builtin_amdgcn_sched_barrier(0);
  };
  // The barrier in the middle of pair p.  Before it a wave waits until everything it loaded except the
  // four instructions of A(p+2), issued in this pair's first half, has landed - that includes its share of
  // pair p+1 - and until its own fragment reads of pair p have returned; after it every wave may read pair
  // p+1 and overwrite pair p's LDS space.
  auto mid_barrier = [&]() { asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // ---- main loop, per pair p of steps (kt = 2p, fragments of step kt already on their way to registers):
  //   first half   issue A(p+2) (its ring space, pair p-1, was released at the last barrier);
  //                read the fragments of step kt+1;  32 MFMAs of step kt
  //   barrier      (see mid_barrier)
  //   second half  issue B(p+2) into pair p's space;  read the fragments of step kt+2;  32 MFMAs of kt+1
  // The two waves of a SIMD (wave and wave + 4) meet that barrier half an MFMA block apart, so they never
  // issue their loads and fragment reads at the same moment and the matrix core always has work queued.
  const int grp = wave >> 2;
  issue_a(0); issue_b(0); issue_a(2); issue_b(2);
  wait_vmcnt_and_barrier<8>();
  i16x8 fq0[4], fp0[8], fq1[4], fp1[8];
  read_frags(0, fq0, fp0);
  for (int kt = 0; kt < kt_total; kt += 2) {
    issue_a(kt + 4);
    read_frags(kt + 1, fq1, fp1);
    mfma_half(fq0, fp0, 0);
    if (grp == 1) mid_barrier();
    mfma_half(fq0, fp0, 1);
    if (grp == 0) mid_barrier();
    issue_b(kt + 4);
    read_frags(kt + 2, fq0, fp0);
    mfma_half(fq1, fp1, 0);
    mfma_half(fq1, fp1, 1);
  }
  // the zero-filling loads beyond the end must have landed before the epilogue reuses LDS
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- epilogue.  acc[nb][mb][r] of lane l is tile row  wm*64 + mb*16 + (l & 15)  and, within the wave's
  // half h = nb >> 2, column (nb & 3)*16 + 4*(l >> 4) + r of 64 consecutive result columns (128 bytes).
  // Where those 64 columns go (col_of_half) and which result a wave writes (result_of_half, row_base)
  // depends on the mode.  Each wave transposes 32 rows x 64 columns at a time through a private LDS patch
  // and writes whole 128-byte lines: 8 rows x 128 bytes per store instruction.
  //   B k-contiguous (kDx, kNT): the wave's B rows wn*128 + h*64.. are result columns n0 + wn*128 + h*64..
  //   dual-N (kFwd*, kDw): half h is result h (gate | up), columns n0 + wn*64..
  //   one result from two B panels (kNN, kTN, kDxT, kDwT): columns n0 + h*128 + wn*64..
  //   kDwT: waves with wm < 2 hold rows of the first result, the others of the second; 128 rows per tile
  auto col_of_half = [&](int h) {
    if constexpr (B_KC && MODE != kFwdT) return n0 + wn * 128 + h * 64;
    else if constexpr (C::kDualN) return n0 + wn * 64;
    else return n0 + h * 128 + wn * 64;
  };
  const int row_base = C::kDualM ? m0 + (wm & 1) * 64 : m0 + wm * 64;
  auto result_of_half = [&](int h) -> int {
    if constexpr (MODE == kDw) return h;
    else if constexpr (C::kDualM) return wm >> 1;
    else return 0;
  };
  if (!C::kForward && p.splits > 1) {
    // fp32 partial tile, 16 bytes (4 consecutive columns) per lane and store
    const size_t plane = (size_t)p.M * p.N;
#pragma unroll
    for (int mb = 0; mb < 4; mb++) {
      const int m = row_base + mb * 16 + (lane & 15);
      if (m >= p.M) continue;
#pragma unroll
      for (int nb = 0; nb < 8; nb++) {
        const int n = col_of_half(nb >> 2) + (nb & 3) * 16 + 4 * (lane >> 4);
        if (n >= p.N) continue;
        const size_t which = (size_t)result_of_half(nb >> 2);
        float* dst = p.ws + (which * p.splits + split) * plane + (size_t)m * p.N + n;
        *(f32x4*)dst = acc[nb][mb];
      }
    }
    return;
  }
  store_tile<E, MODE, 2, false>(p, acc, (FSW_LDS char*)smem + wave * (2 * 32 * 128), lane, row_base, col_of_half(0),
                                col_of_half(1), result_of_half(0), result_of_half(1));
}

// out_r[i] = round(sum over s of ws[r][s][i]), i < n, fixed order: deterministic.  n is a multiple of 4.
// blockIdx.y = result r (the weight gradients come in pairs): one launch for both.
template <typename E>
__global__ __launch_bounds__(256) void fsw_splitk_reduce_kernel(const float* __restrict__ ws, unsigned short* __restrict__ out0,
                                                                unsigned short* __restrict__ out1, size_t n, int splits,
                                                                int N, int ldc) {
  const size_t i4 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i4 >= n) return;
  ws += (size_t)blockIdx.y * splits * n;
  unsigned short* out = blockIdx.y ? out1 : out0;
  f32x4 a = *(const f32x4*)(ws + i4);
  for (int s = 1; s < splits; s++) {
    const f32x4 b = *(const f32x4*)(ws + (size_t)s * n + i4);
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
  }
  const size_t m = i4 / (size_t)N, c = i4 - m * (size_t)N;
  u32x2 v;
  v.x = E::pack2(a.x, a.y);
  v.y = E::pack2(a.z, a.w);
  *(u32x2*)(out + m * (size_t)ldc + c) = v;
}

}  // namespace fsw
