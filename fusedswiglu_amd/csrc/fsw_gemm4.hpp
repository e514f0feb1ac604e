// Four-wave form of the tiled MFMA kernel (same modes, operands, LDS formats and rings as fsw_gemm.hpp).
//
// One workgroup = 4 wavefronts, ONE per SIMD (2 along M x 2 along N), each owning a 128 x 128 block of the
// 256 x 256 fp32 accumulator tile: 256 accumulator registers per lane, 8 + 8 operand fragments per 32-element
// step for 64 MFMAs.  Against the eight-wave form (64 x 128 per wave, 4 + 8 fragments for 32 MFMAs) a step
// reads 64 instead of 96 KiB of LDS per workgroup - the matrix cores are power limited with real data, and
// LDS traffic is the largest part of what a GEMM adds to the MFMAs themselves.
//
// With a single wave per SIMD nothing hides a bubble in that wave's instruction stream, so the main loop is
// written out MFMA by MFMA: after each of the 128 MFMAs of a pair of steps there is one "gap" that holds at
// most a few other instructions, and nothing is allowed to move between gaps.  What a gap can hold for free was
// measured with one wave per SIMD issuing 16x16x32 MFMAs back to back (16 cycles each): one scalar instruction
// (every further one costs 8 cycles), two vector ALU instructions, one LDS read (two behind the same MFMA cost
// 17 cycles), or one direct-to-LDS load (about 12 cycles in any case).  Per pair p (steps 2p and 2p+1, fragment
// register sets 0 and 1):
//   gaps   0.. 14   the A stream moves on to pair p+2, one or two scalar instructions per gap
//   gaps  15.. 58   the 8 loads of A(p+2) (ring slot of pair p-1, released at the last barrier), one per 6 gaps
//   gaps  16.. 47   fragment reads of step 2p+1 into set 1, one LDS instruction per gap
//   gaps  46.. 60   the B stream moves on to pair p+2
//   gap   64        s_waitcnt vmcnt(8) lgkmcnt(0); s_barrier: pair p+1 has landed for every wave, and every
//                   wave has finished reading pair p out of LDS
//   gaps  66..109   the 8 loads of B(p+2) into pair p's B space
//   gaps  80..111   fragment reads of step 2p+2 into set 0
#pragma once
#include <utility>

#include "fsw_gemm.hpp"

namespace fsw {

constexpr int kThreads4 = 256;
// index i (0 <= i < count) with start + stride*i == g, or -1
constexpr int gap_index(int g, int start, int stride, int count) {
  return (g >= start && (g - start) % stride == 0 && (g - start) / stride < count) ? (g - start) / stride : -1;
}

// c += a b with the accumulator pinned to the accumulation registers and the operands to ordinary vector
// registers.  Left to itself the register allocator mixes the two files for a 128 x 128 wave tile and shuffles
// accumulators back and forth around every MFMA.
template <typename E>
FSW_DEV void mfma16_acc(f32x4& c, i16x8 a, i16x8 b) {
  if constexpr (std::is_same<E, BF16>::value)
    asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else
    asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// LDS destination of the next direct-to-LDS load of this wave (M0), and the load itself.  Between the two
// there must be at least one other instruction (M0 write -> LDS-DMA use): in the main loop an MFMA.

template <bool NT>
FSW_DEV void dma_load16(i32x4 rsrc, unsigned voffset) {
  if constexpr (NT) asm volatile("buffer_load_dwordx4 %0, %1, 0 offen nt lds" : : "v"(voffset), "s"(rsrc) : "memory");
  else asm volatile("buffer_load_dwordx4 %0, %1, 0 offen lds" : : "v"(voffset), "s"(rsrc) : "memory");
}

// Per-wave description of an operand's loads: 8 instructions of 1 KiB per pair of steps in either layout.
//   KC: instruction i fetches tile rows 8*(wave + 4i) .. +8, one 128-byte line each (64 k-elements)
//   MC: instruction i = 4*s + j fetches, for step s of the pair, k-rows 4*((wave + 4j) & 7) .. +4 of panel
//       (j >> 1), 256 bytes each
struct Loader4 {
  unsigned voff[8];      // KC: per instruction; MC: [0..3] per j (both steps use the same)
  int klim[2];           // KC: [0]: this lane's chunk is inside its row while the pair's byte offset < klim;
                         // MC: per (j & 1): this lane's k-row exists while the step's first k < klim
  const char* base[2];   // KC: first / second pass (or matrix, kFwdT);  MC: per panel
  const char* base2[2];  // MC: per panel, second pass (kDxT)
  unsigned kstep;        // MC: bytes per 32 k-rows
  unsigned records[2];   // bytes of the matrix from base[] on (the same from base2[]): the descriptors' range
};
// Bytes from a tile's origin to the end of the matrix data, for the descriptor's range check; 0 when the origin is
// outside the matrix.  The host only picks this kernel for operands below 2^31 bytes.
FSW_DEV unsigned records_of(long long bytes) { return bytes <= 0 ? 0u : (bytes > 0x7fffffffLL ? 0x7fffffffu : (unsigned)bytes); }

FSW_DEV void kc4_setup(Loader4& L, const void* p0, const void* p1, int row0, int rows_total, int K, int ld,
                       int wave, int lane, bool interleaved) {
  const int row = 8 * wave + (lane >> 3);
  const int c = (lane & 7) ^ ((((wave & 1) << 2) + (lane >> 4)) & 7);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    // LDS rows 32i + row; interleaved (kFwdT): LDS 64-row block b = i >> 1 holds rows 64*(b >> 1).. of matrix b & 1
    const int grow = interleaved ? 64 * (i >> 2) + 32 * (i & 1) + row : 32 * i + row;
    L.voff[i] = (row0 + grow < rows_total) ? (unsigned)grow * (unsigned)ld * 2u + c * 16u : kOobOffset;
  }
  L.klim[0] = (K - c * 8) * 2;  // in bytes, compared with the pair's byte offset
  L.klim[1] = L.klim[0];
  L.base[0] = (const char*)p0 + (size_t)row0 * ld * 2;
  L.base[1] = (const char*)p1 + (size_t)row0 * ld * 2;
  L.base2[0] = L.base[0];
  L.base2[1] = L.base[1];
  L.kstep = 0;
  // rows row0 .. rows_total-1, the last one up to its K-th element
  L.records[0] = L.records[1] = records_of(((long long)rows_total - row0 - 1) * ld * 2 + (long long)K * 2);
}

FSW_DEV void mc4_setup(Loader4& L, const void* p_panel0, const void* p_panel1, const void* q_panel0,
                       const void* q_panel1, int col0_panel0, int col0_panel1, int cols_total, int K, int ld,
                       int wave, int lane) {
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int row = 4 * wave + 16 * (j & 1) + (lane >> 4);
    // physical 16-byte chunk (lane & 15) of k-row `row` holds logical columns `col`.. (see read_frag_mc16)
    const int col = (((lane >> 2) & 3) ^ (row & 3)) * 32 + ((((lane >> 1) ^ (row >> 3)) & 1) * 16) + (lane & 1) * 8;
    const int col0 = (j >> 1) ? col0_panel1 : col0_panel0;
    L.voff[j] = (col0 + col < cols_total) ? (unsigned)row * (unsigned)ld * 2u + col * 2u : kOobOffset;
    L.voff[4 + j] = L.voff[j];
    if (j < 2) L.klim[j] = K - row;
  }
  L.base[0] = (const char*)p_panel0 + (size_t)col0_panel0 * 2;
  L.base[1] = (const char*)p_panel1 + (size_t)col0_panel1 * 2;
  L.base2[0] = (const char*)q_panel0 + (size_t)col0_panel0 * 2;
  L.base2[1] = (const char*)q_panel1 + (size_t)col0_panel1 * 2;
  L.kstep = (unsigned)kBK * (unsigned)ld * 2u;
  // k-rows 0 .. K-1 from the panel's first column on, the last one up to the matrix's last column
  L.records[0] = records_of(((long long)K - 1) * ld * 2 + ((long long)cols_total - col0_panel0) * 2);
  L.records[1] = records_of(((long long)K - 1) * ld * 2 + ((long long)cols_total - col0_panel1) * 2);
  if (col0_panel0 >= cols_total) L.records[0] = 0;
  if (col0_panel1 >= cols_total) L.records[1] = 0;
}

template <typename E, int MODE, bool STREAM_B = false>
__global__ __launch_bounds__(kThreads4) void fsw_gemm4_kernel(GemmParams p) {
  using C = Cfg<MODE>;
  __shared__ __attribute__((aligned(1024))) char smem[C::kBytesA + C::kBytesB];
  constexpr bool A_KC = C::kAKc, B_KC = C::kBKc;
  constexpr bool B_INTER = (MODE == kFwdT);
  constexpr int TM = C::kTileM, TN = C::kTileN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;  // 2 waves along M x 2 along N

  const int ntiles = p.tiles_m * p.tiles_n;
  // a workgroup of the tail split: part `tail_part` of the tile with launch index tail_first + tail_tile
  const bool in_tail = !C::kForward && p.tail_count > 0 && (int)blockIdx.x >= p.tail_first;
  const int tail_part = in_tail ? ((int)blockIdx.x - p.tail_first) / p.tail_count : 0;
  const int tail_tile = in_tail ? ((int)blockIdx.x - p.tail_first) % p.tail_count : 0;
  const int split = (C::kForward || in_tail) ? 0 : (int)(blockIdx.x / ntiles);
  const int tile_index = in_tail ? p.tail_first + tail_tile : (int)(blockIdx.x - split * ntiles);
  const TileCoord tc = xcd_tile_order(tile_index, p.tiles_m, p.tiles_n, p.group_m);
  const int m0 = tc.tm * TM;
  const int n0 = tc.tn * TN;

  // steps per pass; the two-pass modes (dG.W then dU.W) keep pairs of steps inside a pass
  const int kt1 = (C::kPasses == 2) ? (((p.K + kBK - 1) / kBK + 1) & ~1) : (p.K + kBK - 1) / kBK;
  const int kt_all = C::kPasses * kt1;
  const int kbase = in_tail ? tail_part * p.tail_steps : split * p.steps_per_split;
  const int kt_total = C::kForward ? kt_all : min(in_tail ? p.tail_steps : p.steps_per_split, kt_all - kbase);

  const unsigned smem_a = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const unsigned smem_b = smem_a + C::kBytesA;

  Loader4 la, lb;
  if constexpr (A_KC) kc4_setup(la, p.a0, C::kPasses == 2 ? p.a1 : p.a0, m0, p.M, p.K, p.lda, wave, lane, false);
  else if constexpr (C::kDualM) mc4_setup(la, p.a0, p.a1, p.a0, p.a1, m0, m0, p.M, p.K, p.lda, wave, lane);
  else mc4_setup(la, p.a0, p.a0, p.a0, p.a0, m0, m0 + 128, p.M, p.K, p.lda, wave, lane);
  if constexpr (B_INTER) kc4_setup(lb, p.b0, p.b1, n0, p.N, p.K, p.ldb, wave, lane, true);
  else if constexpr (B_KC) kc4_setup(lb, p.b0, C::kPasses == 2 ? p.b1 : p.b0, n0, p.N, p.K, p.ldb, wave, lane, false);
  else if constexpr (C::kDualN) mc4_setup(lb, p.b0, p.b1, p.b0, p.b1, n0, n0, p.N, p.K, p.ldb, wave, lane);
  else mc4_setup(lb, p.b0, p.b0, C::kPasses == 2 ? p.b1 : p.b0, C::kPasses == 2 ? p.b1 : p.b0, n0, n0 + 128, p.N,
                 p.K, p.ldb, wave, lane);

  // ---- loads.  Each operand keeps a running description of "the pair being loaded": buffer descriptors (one, or
  // two for the two panels of an MC operand / the two matrices of kFwdT), how far the pair is into its pass, and
  // where it goes in LDS.  A single wave per SIMD issues at most one scalar instruction per MFMA for free (every
  // further one costs 8 cycles of MFMA time), so moving the description on by one pair is cut into micro-steps of
  // one or two scalar instructions that the main loop places in different gaps.
  struct Stream4 {
    i32x4 rs[2];
    unsigned koff;  // KC: byte offset of the pair's first k in its row; MC: first k-row
    unsigned soff[2];  // MC: byte offset of the two steps' first k-rows
    unsigned dst;   // LDS address of this wave's first KiB in the pair's ring slot
    unsigned wrap_at;  // two-pass modes: koff at which the second pass starts; all ones once it has (or never will)
    bool ok[4];     // k-edge: KC [0]: this lane's chunk is inside the row; MC [2s + parity]: its k-row exists
  };
  const unsigned wrap_k = (unsigned)kt1 * kBK;  // two-pass modes: k at which the second pass starts
  auto stream_edge = [&](Stream4& S, const Loader4& L, bool kc) {
    if (kc) {
      S.ok[0] = (int)S.koff < L.klim[0];
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) S.ok[e] = (int)S.koff + (e >> 1) * kBK < L.klim[e & 1];
    }
  };
  auto stream_init = [&](Stream4& S, const Loader4& L, bool kc, unsigned lds_base) {
    const int pass = (C::kPasses == 2 && kbase >= kt1) ? 1 : 0;
    const int ks = kbase - pass * kt1;
    // The descriptors stay at the tile's (panel's) origin with the exact extent of the matrix from there on, and
    // the reduction advances through the offsets of the loads: whatever offset a load ends up with, the hardware's
    // range check keeps it inside the matrix.
    if (kc) {
      S.rs[0] = make_rsrc(pass ? L.base[1] : L.base[0], L.records[0]);
      S.rs[1] = make_rsrc(L.base[1], L.records[1]);  // kFwdT only
      S.koff = (unsigned)ks * kBK * 2u;
      S.soff[0] = S.soff[1] = 0;
    } else {
      S.rs[0] = make_rsrc(pass ? L.base2[0] : L.base[0], L.records[0]);
      S.rs[1] = make_rsrc(pass ? L.base2[1] : L.base[1], L.records[1]);
      S.koff = (unsigned)ks * kBK;
      S.soff[0] = (unsigned)ks * L.kstep;
      S.soff[1] = S.soff[0] + L.kstep;
    }
    S.dst = lds_base + wave * 1024;
    S.wrap_at = (C::kPasses == 2 && pass == 0) ? (kc ? wrap_k * 2 : wrap_k) : 0xffffffffu;
    stream_edge(S, L, kc);
  };
  // Two-pass modes: at the pair where the first pass ends the descriptors jump to the second pair of matrices.
  // Written without a branch or select on the descriptors (either costs the loop a dozen scalar instructions
  // per pair): an all-ones / zero mask, one 64-bit add of the masked distance.
  auto wrap_delta = [&](const Loader4& L, bool kc, int panel) -> uint64_t {
    if (kc) return (uint64_t)(L.base[1] - L.base[0]);
    return (uint64_t)(L.base2[panel] - L.base[panel]);
  };
  const uint64_t wrap_a0 = (C::kPasses == 2) ? wrap_delta(la, A_KC, 0) : 0, wrap_a1 = (C::kPasses == 2) ? wrap_delta(la, A_KC, 1) : 0;
  const uint64_t wrap_b0 = (C::kPasses == 2) ? wrap_delta(lb, B_KC, 0) : 0, wrap_b1 = (C::kPasses == 2) ? wrap_delta(lb, B_KC, 1) : 0;
  auto rsrc_advance64 = [&](i32x4& r, unsigned lo, unsigned hi) {
    const uint64_t a = (((uint64_t)(unsigned)r.y << 32) | (unsigned)r.x) + (((uint64_t)hi << 32) | lo);
    r.x = (int)(unsigned)a;
    r.y = (int)(unsigned)(a >> 32);
  };
  // Micro-step n (0..14) of "next pair".  The empty asm statements before and after pin the scalar arithmetic of
  // a step to the place in the instruction stream where it is written (plain integer code would otherwise be
  // gathered at the top of the loop).
#define FSW_PIN_S(x) asm volatile("" : "+s"(x))
  unsigned wrap_mask = 0, wrap_lo = 0, wrap_hi = 0;
  auto stream_micro = [&](Stream4& S, const Loader4& L, bool kc, unsigned lds_base, int pairs, uint64_t wrap0,
                          uint64_t wrap1, int n) {
    const bool two = C::kPasses == 2;
    if (n == 0) { FSW_PIN_S(S.koff); S.koff += kc ? 2 * kBK * 2 : 2 * kBK; FSW_PIN_S(S.koff); }
    if (n == 1 && !kc) { FSW_PIN_S(S.soff[0]); S.soff[0] += 2u * L.kstep; FSW_PIN_S(S.soff[0]); }
    if (n == 2 && !kc) { FSW_PIN_S(S.soff[1]); S.soff[1] += 2u * L.kstep; FSW_PIN_S(S.soff[1]); }
    if (n == 3 && two)
      asm volatile("s_cmp_eq_u32 %1, %2\n\ts_cselect_b32 %0, -1, 0" : "=s"(wrap_mask) : "s"(S.koff), "s"(S.wrap_at) : "scc");
    // the jump happens once: the distance below is relative, and the pairs loaded beyond the end of the second
    // pass (all lanes out of range) reach the same koff again
    if (n == 4 && two) { FSW_PIN_S(wrap_mask); S.koff &= ~wrap_mask; S.wrap_at |= wrap_mask; FSW_PIN_S(S.koff); FSW_PIN_S(S.wrap_at); }
    if (n == 8 && two && !kc) { FSW_PIN_S(wrap_mask); S.soff[0] &= ~wrap_mask; FSW_PIN_S(S.soff[0]); }
    if (n == 9 && two && !kc) { FSW_PIN_S(wrap_mask); S.soff[1] = (S.soff[1] & ~wrap_mask) | (L.kstep & wrap_mask); FSW_PIN_S(S.soff[1]); }
    if (n == 5 && two) { FSW_PIN_S(wrap_mask); wrap_lo = (unsigned)wrap0 & wrap_mask; FSW_PIN_S(wrap_lo); }
    if (n == 6 && two) { FSW_PIN_S(wrap_mask); wrap_hi = (unsigned)(wrap0 >> 32) & wrap_mask; FSW_PIN_S(wrap_hi); }
    if (n == 7 && two) { FSW_PIN_S(S.rs[0]); rsrc_advance64(S.rs[0], wrap_lo, wrap_hi); FSW_PIN_S(S.rs[0]); }
    if (n == 10 && two && !kc) { FSW_PIN_S(wrap_mask); wrap_lo = (unsigned)wrap1 & wrap_mask; wrap_hi = (unsigned)(wrap1 >> 32) & wrap_mask; FSW_PIN_S(wrap_lo); FSW_PIN_S(wrap_hi); }
    if (n == 11 && two && !kc) { FSW_PIN_S(S.rs[1]); rsrc_advance64(S.rs[1], wrap_lo, wrap_hi); FSW_PIN_S(S.rs[1]); }
    if (n == 12) { FSW_PIN_S(S.dst); S.dst += kKcAreaBytes; FSW_PIN_S(S.dst); }
    if (n == 13) {
      FSW_PIN_S(S.dst);
      S.dst = (S.dst == lds_base + wave * 1024 + pairs * kKcAreaBytes) ? lds_base + wave * 1024 : S.dst;
      FSW_PIN_S(S.dst);
    }
    if (n == 14) { FSW_PIN_S(S.koff); stream_edge(S, L, kc); }
  };
  auto stream_next = [&](Stream4& S, const Loader4& L, bool kc, unsigned lds_base, int pairs, uint64_t wrap0,
                         uint64_t wrap1) {
#pragma unroll
    for (int n = 0; n < 15; n++) stream_micro(S, L, kc, lds_base, pairs, wrap0, wrap1, n);
  };
  // Load i (0..7) of the pair: it goes to LDS at dst + i * 4 KiB (KC: LDS rows 8*(wave + 4i); MC: step i >> 2,
  // KiB wave + 4*(i & 3) of its 16 KiB slot).  load_prep sets the destination (M0) and selects the lane's
  // offset; the load itself comes at least one instruction later (M0 write -> LDS-DMA use).
  auto load_prep = [&](const Stream4& S, const Loader4& L, bool kc, int i) -> unsigned {
    asm volatile("s_add_u32 m0, %0, %1" : : "s"(S.dst), "n"(i * 4096) : "scc", "memory");
    // the whole offset goes through the vector operand, which the descriptor's range check covers for certain
    if (kc) return S.ok[0] ? L.voff[i] + S.koff : kOobOffset;
    return S.ok[(i >> 2) * 2 + (i & 1)] ? L.voff[i & 3] + S.soff[i >> 2] : kOobOffset;
  };
  auto load_go = [&](const Stream4& S, const Loader4& L, bool kc, bool inter, int i, unsigned off, auto nt) {
    constexpr bool kNt = decltype(nt)::value;
    if (kc) dma_load16<kNt>(inter ? S.rs[(i >> 1) & 1] : S.rs[0], off);
    else dma_load16<kNt>(S.rs[(i & 3) >> 1], off);
  };
  constexpr std::false_type keep{};
  constexpr std::bool_constant<STREAM_B> hint_b{};
  // all 8 loads of a pair back to back (prologue only)
  auto pair_all = [&](const Stream4& S, const Loader4& L, bool kc, bool inter, auto nt) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const unsigned off = load_prep(S, L, kc, i);
      asm volatile("s_nop 3" ::: "memory");
      load_go(S, L, kc, inter, i, off, nt);
    }
  };

  // ---- fragment reads: per-lane byte offsets inside a pair's 32 KiB of ring space
  //   KC: [half] row (wm|wn)*128 + (lane & 15), chunk (half*4 + (lane >> 4)) ^ ((lane >> 1) & 7); fragment f adds
  //       f * 16 rows = f * 2048 bytes
  //   MC: mc_lane_offset(lane); step s adds 16 KiB, the panel 8 KiB, fragment f flips address bits 5..7
  unsigned rd_a[2], rd_b[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const unsigned kc_lane = (unsigned)(lane & 15) * 128u + (unsigned)(((h * 4 + (lane >> 4)) ^ ((lane >> 1) & 7)) * 16);
    const unsigned mc_lane = mc_lane_offset(lane) + h * kMcSlotBytes;
    rd_a[h] = A_KC ? kc_lane + wm * 128 * 128 : mc_lane + wm * kMcPanelBytes;
    rd_b[h] = B_KC ? kc_lane + wn * 128 * 128 : mc_lane;
  }
  const FSW_LDS char* lds0 = (const FSW_LDS char*)smem;
  // Read slot r (0..31) of a step: fragment r >> 1 (0..7 of A, then 0..7 of B).  A KC fragment is one
  // ds_read_b128 in the even slot; an MC fragment is two transposing reads, one per slot (two LDS reads behind
  // the same MFMA cost four times what they cost one MFMA apart).
  i16x8 fq[2][8], fp[2][8];
  i16x4 half_lo;
  auto read_slot = [&](int set, int r, const FSW_LDS char* ra, const FSW_LDS char* rb) {
    const int f = r >> 1, second = r & 1;
    const bool is_a = f < 8;
    const int fi = is_a ? f : f - 8;
    i16x8& dst = is_a ? fq[set][fi] : fp[set][fi];
    if (is_a ? A_KC : B_KC) {
      if (!second) dst = *(const FSW_LDS i16x8*)((is_a ? ra : rb) + fi * 2048);
    } else {
      const FSW_LDS char* base = is_a ? ra : rb + (fi >> 2) * kMcPanelBytes;
      const int f16 = is_a ? fi : wn * 4 + (fi & 3);
      const FSW_LDS char* q = (const FSW_LDS char*)(uintptr_t)((unsigned)(uintptr_t)base ^ (unsigned)(f16 << 5));
      if (!second) {
        half_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)q);
      } else {
        const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FSW_LDS i16x4*)(q + 4 * kMcRowBytes));
        dst = __builtin_shufflevector(half_lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
    }
  };

  // acc[nb][mb]: 16x16 block of rows wm*128 + mb*16.. and 16-column block nb of this wave:
  //   dual-N modes  nb = 4*a + c: matrix a (gate | up), columns wn*64 + c*16..
  //   else          B rows / columns wn*128 + nb*16.. (KC) or panel nb >> 2, columns wn*64 + (nb & 3)*16.. (MC)
  f32x4 acc[8][8];
#pragma unroll
  for (int nb = 0; nb < 8; nb++)
#pragma unroll
    for (int mb = 0; mb < 8; mb++) acc[nb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- prologue: pairs 0 and 1 of both operands, then the fragments of step 0
  Stream4 sa, sb;
  stream_init(sa, la, A_KC, smem_a);
  stream_init(sb, lb, B_KC, smem_b);
  pair_all(sa, la, A_KC, false, keep);
  pair_all(sb, lb, B_KC, B_INTER, hint_b);
  stream_next(sa, la, A_KC, smem_a, C::kPairsA, wrap_a0, wrap_a1);
  stream_next(sb, lb, B_KC, smem_b, C::kPairsB, wrap_b0, wrap_b1);
  pair_all(sa, la, A_KC, false, keep);
  pair_all(sb, lb, B_KC, B_INTER, hint_b);
  wait_vmcnt_and_barrier<16>();
  // LDS byte offsets of the pair being multiplied inside the A and B rings
  unsigned rd_pair_a = 0, rd_pair_b = 0;
  {
    const FSW_LDS char* ra = lds0 + rd_a[0];
    const FSW_LDS char* rb = lds0 + C::kBytesA + rd_b[0];
#pragma unroll
    for (int r = 0; r < 32; r++) read_slot(0, r, ra, rb);
  }

  // The schedule of one pair: which gap (after MFMA g of 128) holds what.
  //   kAMicro0 + n                 micro-step n of moving the A stream on to pair p+2
  //   kALd0 + kLdStrideA*i, +1     preparation and issue of load i of A(p+2)
  //   kRd1_0 + r                   read slot r of step 2p+1 (set 1)
  //   kBMicro0 + n, kBarrier       the B stream moves on to pair p+2; the barrier of pair p
  //   kBLd0 + kLdStrideB*i, +1     loads of B(p+2), after the barrier
  //   kRdNext .. +3                the ring offsets of pair p+1
  //   kRd0_0 + r                   read slot r of step 2p+2 (set 0), after the barrier
  constexpr int kLdStrideA = 6, kLdStrideB = 6;
  constexpr int kAMicro0 = 0, kALd0 = 15, kRd1_0 = 16;
  constexpr int kBMicro0 = 46, kBarrier = 64, kBLd0 = 66, kRdNext = 74, kRd0_0 = 80;
  static_assert(kALd0 + 1 + 7 * kLdStrideA < kBarrier && kBLd0 > kBarrier && kBLd0 + 1 + 7 * kLdStrideB < 128, "load gaps");
  static_assert(kRd1_0 + 31 < kBarrier && kRd0_0 > kBarrier && kRd0_0 + 31 < 128, "read gaps");

  for (int kt = 0; kt < kt_total; kt += 2) {
    unsigned off_a = 0, off_b = 0;
    const FSW_LDS char* ra;
    const FSW_LDS char* rb;
    static_for<128>([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      constexpr int h = g >> 6, idx = g & 63, nb = idx >> 3, ii = idx & 7, mb = (nb & 1) ? 7 - ii : ii;
      mfma16_acc<E>(acc[nb][mb], fp[h][nb], fq[h][mb]);
      __builtin_amdgcn_sched_barrier(0);
      // --- the A stream moves on to pair p+2 (ring slot of pair p-1, released at the last barrier); its loads
      if constexpr (g >= kAMicro0 && g < kAMicro0 + 15)
        stream_micro(sa, la, A_KC, smem_a, C::kPairsA, wrap_a0, wrap_a1, g - kAMicro0);
      constexpr int ia_prep = gap_index(g, kALd0, kLdStrideA, 8), ia_go = gap_index(g, kALd0 + 1, kLdStrideA, 8);
      if constexpr (ia_prep >= 0) off_a = load_prep(sa, la, A_KC, ia_prep);
      if constexpr (ia_go >= 0) load_go(sa, la, A_KC, false, ia_go, off_a, keep);
      // --- fragments of step kt+1 (second half of the same pair) into set 1
      if constexpr (g == kRd1_0 - 1) {
        ra = lds0 + rd_pair_a + rd_a[1];
        rb = lds0 + C::kBytesA + rd_pair_b + rd_b[1];
      }
      if constexpr (g >= kRd1_0 && g < kRd1_0 + 32) read_slot(1, g - kRd1_0, ra, rb);
      // --- the B stream moves on to pair p+2; the barrier of pair p; the loads of B(p+2) into pair p's space
      if constexpr (g >= kBMicro0 && g < kBMicro0 + 15)
        stream_micro(sb, lb, B_KC, smem_b, C::kPairsB, wrap_b0, wrap_b1, g - kBMicro0);
      if constexpr (g == kBarrier) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      constexpr int ib_prep = gap_index(g, kBLd0, kLdStrideB, 8), ib_go = gap_index(g, kBLd0 + 1, kLdStrideB, 8);
      if constexpr (ib_prep >= 0) off_b = load_prep(sb, lb, B_KC, ib_prep);
      if constexpr (ib_go >= 0) load_go(sb, lb, B_KC, B_INTER, ib_go, off_b, hint_b);
      // --- fragments of step kt+2 (pair p+1) into set 0
      if constexpr (g == kRdNext) { FSW_PIN_S(rd_pair_a); rd_pair_a += kKcAreaBytes; FSW_PIN_S(rd_pair_a); }
      if constexpr (g == kRdNext + 1) { FSW_PIN_S(rd_pair_a); rd_pair_a = rd_pair_a == C::kPairsA * kKcAreaBytes ? 0u : rd_pair_a; FSW_PIN_S(rd_pair_a); }
      if constexpr (g == kRdNext + 2) { FSW_PIN_S(rd_pair_b); rd_pair_b ^= kKcAreaBytes; FSW_PIN_S(rd_pair_b); }
      if constexpr (g == kRdNext + 3) {
        ra = lds0 + rd_pair_a + rd_a[0];
        rb = lds0 + C::kBytesA + rd_pair_b + rd_b[0];
      }
      if constexpr (g >= kRd0_0 && g < kRd0_0 + 32) read_slot(0, g - kRd0_0, ra, rb);
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  // the zero-filling loads beyond the end must have landed before the epilogue reuses LDS (the nops let the last
  // MFMAs, which the compiler cannot see inside the asm statements, retire before the accumulators are read)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier\n\ts_nop 15\n\ts_nop 15" ::: "memory");

  // ---- epilogue.  acc[nb][mb][r] of lane l is tile row  wm*128 + mb*16 + (l & 15)  and, within the wave's
  // half h = nb >> 2, column (nb & 3)*16 + 4*(l >> 4) + r of 64 consecutive result columns (128 bytes).
  // Each wave transposes 32 rows x 64 columns at a time through a private LDS patch and writes whole
  // 128-byte lines: 8 rows x 128 bytes per store instruction.
  //   B k-contiguous (kDx, kNT): the wave's B rows wn*128 + h*64.. are result columns n0 + wn*128 + h*64..
  //   dual-N (kFwd*, kDw): half h is result h (gate | up), columns n0 + wn*64..
  //   one result from two B panels (kNN, kTN, kDxT, kDwT): columns n0 + h*128 + wn*64..
  //   kDwT: wave row wm holds the 128 rows of result wm
  auto col_of_half = [&](int h) {
    if constexpr (B_KC && MODE != kFwdT) return n0 + wn * 128 + h * 64;
    else if constexpr (C::kDualN) return n0 + wn * 64;
    else return n0 + h * 128 + wn * 64;
  };
  const int row_base = C::kDualM ? m0 : m0 + wm * 128;
  auto result_of_half = [&](int h) -> int {
    if constexpr (MODE == kDw) return h;
    else if constexpr (C::kDualM) return wm;
    else return 0;
  };
  if (in_tail) {
    // fp32 partial tile in tile-local coordinates [result][row][column], 16 bytes per lane and store
    float* part = p.ws + ((size_t)tail_tile * p.tail_parts + tail_part) * kTileFloats;
#pragma unroll
    for (int mb = 0; mb < 8; mb++) {
      const int r = row_base - m0 + mb * 16 + (lane & 15);
#pragma unroll
      for (int nb = 0; nb < 8; nb++) {
        const int c = col_of_half(nb >> 2) - n0 + (nb & 3) * 16 + 4 * (lane >> 4);
        *(f32x4*)(part + ((size_t)result_of_half(nb >> 2) * TM + r) * TN + c) = acc[nb][mb];
      }
    }
    return;
  }
  if (!C::kForward && p.splits > 1) {
    const size_t plane = (size_t)p.M * p.N;
#pragma unroll
    for (int mb = 0; mb < 8; mb++) {
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
  store_tile<E, MODE, 4, true>(p, acc, (FSW_LDS char*)smem + wave * (2 * 32 * 128), lane, row_base, col_of_half(0),
                               col_of_half(1), result_of_half(0), result_of_half(1));
}

// Results of the tail tiles: out[tile] = round(sum over parts of ws[tile][part]), fixed order.  One workgroup of
// 256 threads per 32 rows x 256 floats of a tile (blockIdx.y = tail tile, blockIdx.x = slice of its 2*TM*TN / 8192).
template <typename E, int MODE>
__global__ __launch_bounds__(256) void fsw_tail_reduce_kernel(GemmParams p) {
  using C = Cfg<MODE>;
  constexpr int TM = C::kTileM, TN = C::kTileN;
  const TileCoord tc = xcd_tile_order(p.tail_first + (int)blockIdx.y, p.tiles_m, p.tiles_n, p.group_m);
  const float* ws = p.ws + (size_t)blockIdx.y * p.tail_parts * kTileFloats;
#pragma unroll
  for (int it = 0; it < 8; it++) {
    const int i4 = ((int)blockIdx.x * 2048 + it * 256 + (int)threadIdx.x) * 4;  // float index in the tile
    f32x4 a = *(const f32x4*)(ws + i4);
    for (int s = 1; s < p.tail_parts; s++) {
      const f32x4 b = *(const f32x4*)(ws + (size_t)s * kTileFloats + i4);
      a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    const int which = i4 / (TM * TN), rem = i4 - which * (TM * TN);
    const int m = tc.tm * TM + rem / TN, n = tc.tn * TN + rem % TN;
    if (m >= p.M || n >= p.N) continue;
    u32x2 v;
    v.x = E::pack2(a.x, a.y);
    v.y = E::pack2(a.z, a.w);
    unsigned short* out = (unsigned short*)(which == 0 ? p.c0 : p.c1);
    *(u32x2*)(out + (size_t)m * p.ldc + n) = v;
  }
}

}  // namespace fsw
