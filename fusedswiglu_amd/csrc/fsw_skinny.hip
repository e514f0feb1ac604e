// Weight-streaming forward for few tokens (T <= 128): out = silu(x Wg) * (x Wu).
// With so few rows the step is bound by reading Wg and Wu once from HBM, not by the MFMAs, so this
// kernel is built around keeping many weight bytes in flight per CU: one workgroup of 4 waves (one
// per SIMD) owns 128 columns of both weight matrices, walks the whole reduction in steps of 32, and
// keeps a ring of LDS stages (8 stages of 20 KiB for up to 64 rows, 6 of 24 KiB for 128)
// filled by direct global->LDS loads.  x (a few MiB at most, L2 resident) rides along in the same
// stages.  Each wave computes all BM rows x 32 columns of the gate and the up product and applies
// silu(g)*u in registers.  Fragment reads of the next step overlap the MFMAs of the current one, and a
// slot goes back to the loader as soon as its fragments are in registers.
#include "fsw_gemm.hpp"
#include "fsw_internal.hpp"

namespace fsw {

constexpr int kSkThreads = 256;

// Every stage holds an x tile of max(BM, 64) rows x 64 bytes (1 KiB loads of 16 rows, one or more
// per wave; rows beyond T zero-filled) and a 16 KiB weight slot.
template <int BM>
struct SkCfg {
  static constexpr int kRowsX = BM < 64 ? 64 : BM;
  static constexpr int kXBytes = kRowsX * 64;
  static constexpr int kXLoads = kRowsX / 64;            // per wave and stage
  static constexpr int kStage = kXBytes + kMcSlotBytes;  // 20 / 24 KiB
  static constexpr int kStages = (160 * 1024) / kStage;  // 8 / 6
  static constexpr int kPerStage = kXLoads + 4;          // loads a wave issues per stage
};

// x tile: BM rows x 64 bytes; chunk c of row r at position c ^ ((r >> 2) & 3) (see the MC/KC notes
// in fsw_gemm.hpp; with 64-byte rows sixteen rows span the 64 banks when XOR-ed by (r >> 2)).
FSW_DEV i16x8 read_frag_x(const FSW_LDS char* a, int row_base, int ks, int lane) {
  const int row = row_base + (lane & 31);
  const int chunk = (ks * 2 + (lane >> 5)) ^ ((lane >> 2) & 3);
  return *(const FSW_LDS i16x8*)(a + row * 64 + chunk * 16);
}

template <typename E, int BM>
__global__ __launch_bounds__(kSkThreads) void fsw_skinny_forward_kernel(GemmParams p) {
  using C = SkCfg<BM>;
  constexpr int NQ = BM / 32;
  constexpr int kSkStages = C::kStages, kSkStage = C::kStage, kSkABytes = C::kXBytes;
  __shared__ __attribute__((aligned(1024))) char smem[kSkStages * kSkStage];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * 128;
  const int kt_total = (p.K + kBK - 1) / kBK;
  const unsigned smem_addr = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const FSW_LDS char* smem_l = (const FSW_LDS char*)smem;

  // x: load j of wave w covers rows 64j + 16w .. +15 (4 lanes x 16 bytes per row)
  unsigned xa_off[C::kXLoads];
  int xa_klim[C::kXLoads];
#pragma unroll
  for (int j = 0; j < C::kXLoads; j++) {
    const int row = 64 * j + 16 * wave + (lane >> 2);
    const int c = (lane & 3) ^ ((lane >> 4) & 3);
    xa_off[j] = (unsigned)row * (unsigned)p.lda * 2u + c * 16u;
    xa_klim[j] = (row < p.M) ? p.K - c * 8 : -0x40000000;
  }
  // weights: 16 instructions per stage, 4 k-rows x 256 bytes each; instruction j -> panel j >> 3
  unsigned w_off[4];
  int w_klim[4];
  const char* w_base[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int j = wave + 4 * i;
    const int row = 4 * (j & 7) + (lane >> 4);
    const int col = (((lane >> 2) & 3) ^ ((lane >> 4) & 3)) * 32 + (lane & 3) * 8;
    w_off[i] = (unsigned)row * (unsigned)p.ldb * 2u + col * 2u;
    w_klim[i] = (n0 + col < p.N) ? p.K - row : -0x40000000;
    w_base[i] = (const char*)((j >> 3) ? p.b1 : p.b0) + (size_t)n0 * 2;
  }
  const size_t w_kstep = (size_t)kBK * p.ldb * 2;
  // Loads are issued for every slot index, also beyond the reduction (all lanes out of range -> zero fill, no
  // memory traffic), so the number of loads in flight at each wait is one compile-time constant.
  auto issue = [&](int s) {
    const int k0 = s * kBK;
    const unsigned st = smem_addr + (unsigned)(s % kSkStages) * kSkStage;
#pragma unroll
    for (int j = 0; j < C::kXLoads; j++) {
      const unsigned off = (k0 < xa_klim[j]) ? xa_off[j] : kOobOffset;
      load16_to_lds(make_rsrc((const char*)p.a0 + (size_t)k0 * 2), off, st + j * 4096 + wave * 1024);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int j = wave + 4 * i;
      const unsigned off = (k0 < w_klim[i]) ? w_off[i] : kOobOffset;
      load16_to_lds_stream(make_rsrc(w_base[i] + (size_t)s * w_kstep), off, st + kSkABytes + j * 1024);
    }
  };
  auto read_frags = [&](int s, i16x8 (&fq)[2][NQ], i16x8 (&fp)[2][2]) {
    const FSW_LDS char* sa = smem_l + (s % kSkStages) * kSkStage;
    const FSW_LDS char* sb = sa + kSkABytes;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int q = 0; q < NQ; q++) fq[ks][q] = read_frag_x(sa, q * 32, ks, lane);
#pragma unroll
      for (int a = 0; a < 2; a++) fp[ks][a] = read_frag_mc(sb + a * kMcPanelBytes, wave, ks, lane);
    }
  };

  f32x16 acc[2][NQ];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int q = 0; q < NQ; q++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][q][r] = 0.f;
  auto mfmas = [&](const i16x8 (&fq)[2][NQ], const i16x8 (&fp)[2][2]) {
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
      for (int q = 0; q < NQ; q++)
#pragma unroll
        for (int a = 0; a < 2; a++) acc[a][q] = E::mfma(fp[ks][a], fq[ks][q], acc[a][q]);
  };

  // Software pipeline over two register sets: the fragments of step kt+1 are read from LDS while the matrix
  // cores work on step kt.  hand_over() waits until (a) this wave's loads of the next step have landed (all
  // but the youngest kSkStages-2 stages) and (b) its own fragment reads of the current step have returned;
  // the barrier extends both to the workgroup, so the current step's slot can be refilled at once, before
  // the current step's products are even issued.  kSkStages-1 stages of weights stay in flight throughout.
  constexpr int kInFlight = (kSkStages - 2) * C::kPerStage;
  static_assert(kInFlight < 64, "vmcnt is 6 bits");
  auto hand_over = [&]() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(kInFlight) : "memory");
  };
#pragma unroll
  for (int s = 0; s < kSkStages - 1; s++) issue(s);
  i16x8 fq0[2][NQ], fp0[2][2], fq1[2][NQ], fp1[2][2];
  wait_vmcnt_and_barrier<kInFlight>();  // step 0 has landed
  read_frags(0, fq0, fp0);
  issue(kSkStages - 1);
  // an odd number of steps runs one more on zero-filled slots, which adds nothing
  for (int kt = 0; kt < kt_total; kt += 2) {
    hand_over();
    issue(kt + kSkStages);
    read_frags(kt + 1, fq1, fp1);
    mfmas(fq0, fp0);
    hand_over();
    issue(kt + 1 + kSkStages);
    read_frags(kt + 2, fq0, fp0);
    mfmas(fq1, fp1);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the zero-filling loads past the end
  // acc[a][q][r] of lane l: row q*32 + (l & 31), column n0 + wave*32 + 8*(r >> 2) + 4*(l >> 5) + (r & 3)
#pragma unroll
  for (int q = 0; q < NQ; q++) {
    const int m = q * 32 + (lane & 31);
    if (m >= p.M) continue;
#pragma unroll
    for (int r4 = 0; r4 < 4; r4++) {
      const int n = n0 + wave * 32 + 8 * r4 + 4 * (lane >> 5);
      if (n >= p.N) continue;
      const size_t o = (size_t)m * p.ldc + n;
      unsigned short ho[4], hg[4], hu[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float g = acc[0][q][r4 * 4 + e], u = acc[1][q][r4 * 4 + e];
        ho[e] = E::from_float(silu_mul(g, u));
        hg[e] = E::from_float(g);
        hu[e] = E::from_float(u);
      }
      u32x2 v;
      v.x = ho[0] | ((unsigned)ho[1] << 16); v.y = ho[2] | ((unsigned)ho[3] << 16);
      *(u32x2*)((unsigned short*)p.c0 + o) = v;
      if (p.c1) {
        v.x = hg[0] | ((unsigned)hg[1] << 16); v.y = hg[2] | ((unsigned)hg[3] << 16);
        *(u32x2*)((unsigned short*)p.c1 + o) = v;
        v.x = hu[0] | ((unsigned)hu[1] << 16); v.y = hu[2] | ((unsigned)hu[3] << 16);
        *(u32x2*)((unsigned short*)p.c2 + o) = v;
      }
    }
  }
}

// Beyond 128 rows the 64-byte x rows of this kernel (as many bytes per step as the weights by then)
// cost more than the deeper ring gains: the tiled kernel takes over (measured at 256 rows: 300 vs 258 us).
constexpr int kSkMaxRows = 128;

template <typename E>
static hipError_t launch_skinny_t(const GemmParams& g, hipStream_t s) {
  const unsigned tiles = (unsigned)((g.N + 127) / 128);
  if (g.M <= 32) fsw_skinny_forward_kernel<E, 32><<<tiles, kSkThreads, 0, s>>>(g);
  else if (g.M <= 64) fsw_skinny_forward_kernel<E, 64><<<tiles, kSkThreads, 0, s>>>(g);
  else fsw_skinny_forward_kernel<E, 128><<<tiles, kSkThreads, 0, s>>>(g);
  return hipGetLastError();
}

bool skinny_forward_ok(const Problem& p) { return !p.w_out_in && p.T <= kSkMaxRows && fast_path_ok_forward(p); }

hipError_t launch_forward_skinny(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.x; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.out; g.c1 = p.g; g.c2 = p.u;
  g.M = (int)p.T; g.N = (int)p.I; g.K = (int)p.D;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldw; g.ldc = (int)p.ldo;
  return dtype == kDtypeBF16 ? launch_skinny_t<BF16>(g, s) : launch_skinny_t<FP16>(g, s);
}

}  // namespace fsw
