// Weight-streaming forward for few tokens (T <= 128): out = silu(x Wg) * (x Wu).
// With so few rows the step is bound by reading Wg and Wu once from HBM, not by the MFMAs, so this
// kernel is built around keeping many weight bytes in flight per CU: one workgroup of 4 waves (one
// per SIMD) owns 128 columns of both weight matrices, walks the whole reduction in stages of 64 and
// keeps a ring of LDS stages filled by direct global->LDS loads (4 stages of 36 / 40 KiB up to 64 rows,
// 3 of 48 KiB for 65-128 rows).  x (a few MiB at most, L2 resident) rides along in the same stages as
// full 128-byte lines.  Each wave computes all BM rows x 32 columns of the gate and the up product and
// applies silu(g)*u in registers.  The weight loads carry the non-temporal hint: bytes that are read once
// then leave L2 and the memory-side cache to x.  Fragment reads of the next half stage overlap the MFMAs
// of the current one, and a slot goes back to the loader as soon as its fragments are in registers.
#include "fsw_gemm.hpp"
#include "fsw_internal.hpp"
#include <atomic>

namespace fsw {

constexpr int kSkThreads = 256;

// A stage holds 64 k-elements: BM rows of x, one full 128-byte line each, in the k-contiguous LDS format of the
// tiled kernels (16-byte chunk c of row r at position c ^ ((r >> 1) & 7), read with ds_read_b128), and 32 KiB of
// weights:
//   weights [I, D] (W_KC; reduction index contiguous, the nn.Linear layout): 128 gate rows and 128 up rows of
//     the workgroup's 128 output columns, one line each, same format as x;
//   weights [D, I]: 64 k-rows x 256 bytes of both matrices in two of the tiled kernels' 16 KiB slots (two
//     128-column panels of 32 k-rows each), read with the transposing ds_read_b64_tr_b16.
template <int BM>
struct SkCfg {
  static constexpr int kXBytes = BM * 128;
  static constexpr int kXLoads = BM / 32;               // per wave and stage (8 rows x 128 bytes each)
  static constexpr int kWBytes = 256 * 128;
  static constexpr int kStage = kXBytes + kWBytes;
  static constexpr int kStages = (160 * 1024) / kStage;
  static constexpr int kPerStage = kXLoads + 8;
};

// rows row_base .. +31 (lane & 31), k = 16*ks + 8*(lane >> 5) .. +7 of the stage's 64
FSW_DEV i16x8 read_frag_kc32(const FSW_LDS char* area, int row_base, int ks, int lane) {
  const int row = row_base + (lane & 31);
  const int chunk = (ks * 2 + (lane >> 5)) ^ ((row >> 1) & 7);
  return *(const FSW_LDS i16x8*)(area + row * 128 + chunk * 16);
}

// How a launch is cut up.  plain == 0: the SwiGLU forward (b0 = Wg, b1 = Wu, N = I).  plain == 1: one plain GEMM
// C = A B whose B is given as its two column halves (b0 = columns 0.., b1 = columns N.. of a matrix 2N wide;
// c1 = C, ws = fp32 partial planes [splits][M][2N] or null): the down projection for few tokens.  blockIdx.y
// = k-split: this workgroup reduces stages split*stages_per_split .. of the reduction.
struct SkArgs {
  int bn;                 // output columns per workgroup (of each half), <= 128
  int plain;
  int splits, stages_per_split;
};

template <typename E, int BM, bool W_KC>
__global__ __launch_bounds__(kSkThreads) void fsw_skinny_forward_kernel(GemmParams p, SkArgs a) {
  using C = SkCfg<BM>;
  constexpr int NQ = BM / 32;
  constexpr int kStages = C::kStages, kStage = C::kStage, kXBytes = C::kXBytes;
  __shared__ __attribute__((aligned(1024))) char smem[kStages * kStage];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // this workgroup's output columns n0 .. n0 + bn - 1 (bn <= 128: the rest of the 128-column slot stays
  // out of range, costs no memory traffic and multiplies zeros)
  const int bn = a.bn;
  const int n0 = blockIdx.x * bn;
  const int split = blockIdx.y;
  const int s_base = split * a.stages_per_split;                   // first stage of this workgroup
  const int st_total = min(a.stages_per_split, (p.K + 63) / 64 - s_base);
  const int k_end = min(p.K, (s_base + a.stages_per_split) * 64);  // loads beyond it zero-fill
  const unsigned smem_addr = (unsigned)(uintptr_t)(FSW_LDS char*)smem;
  const FSW_LDS char* smem_l = (const FSW_LDS char*)smem;

  // instruction idx covers area rows 8*idx .. +7; this wave issues idx = wave + 4*j
  unsigned x_off[C::kXLoads];
  int x_klim[C::kXLoads];
#pragma unroll
  for (int j = 0; j < C::kXLoads; j++) {
    const int row = 8 * (wave + 4 * j) + (lane >> 3);
    const int c = (lane & 7) ^ ((row >> 1) & 7);
    x_off[j] = (unsigned)row * (unsigned)p.lda * 2u + c * 16u;
    x_klim[j] = (row < p.M) ? k_end - c * 8 : -0x40000000;
  }
  unsigned w_off[8];
  int w_klim[8];        // W_KC: in range while k0 < klim;  else: while k0 < klim as well (k-row bound)
  const char* w_base[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    if constexpr (W_KC) {
      const int row = 8 * (wave + 4 * j) + (lane >> 3);  // 0..255: gate rows, then up rows (j >= 4)
      const int c = (lane & 7) ^ ((row >> 1) & 7);
      const int n = row & 127;
      w_off[j] = (unsigned)n * (unsigned)p.ldb * 2u + c * 16u;
      w_klim[j] = (n < bn && n0 + n < p.N) ? k_end - c * 8 : -0x40000000;
      w_base[j] = (const char*)(j < 4 ? p.b0 : p.b1) + (size_t)n0 * p.ldb * 2;
    } else {
      // slot j >> 2 (k-rows 32*(j >> 2)..), instruction i = wave + 4*(j & 3) of its 16: panel i >> 3, 4 k-rows
      const int i = wave + 4 * (j & 3);
      const int row = 32 * (j >> 2) + 4 * (i & 7) + (lane >> 4);
      const int col = (((lane >> 2) & 3) ^ ((lane >> 4) & 3)) * 32 + (lane & 3) * 8;
      w_off[j] = (unsigned)row * (unsigned)p.ldb * 2u + col * 2u;
      w_klim[j] = (col < bn && n0 + col < p.N) ? k_end - row : -0x40000000;
      w_base[j] = (const char*)((i >> 3) ? p.b1 : p.b0) + (size_t)n0 * 2;
    }
  }
  const size_t w_kstep = W_KC ? 128 : (size_t)64 * p.ldb * 2;  // bytes per stage along the reduction
  // issued for every stage index; beyond the reduction every lane is out of range and zero-fills
  auto issue = [&](int s) {
    const int k0 = (s_base + s) * 64;
    const unsigned st = smem_addr + (unsigned)(s % kStages) * kStage;
    const i32x4 rx = make_rsrc((const char*)p.a0 + (size_t)k0 * 2);
#pragma unroll
    for (int j = 0; j < C::kXLoads; j++)
      load16_to_lds(rx, (k0 < x_klim[j]) ? x_off[j] : kOobOffset, st + (wave + 4 * j) * 1024);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      // W_KC: area row block wave + 4*j;  else slot j >> 2, instruction wave + 4*(j & 3)
      const unsigned dst = W_KC ? (unsigned)(wave + 4 * j) * 1024u
                                : (unsigned)(j >> 2) * kMcSlotBytes + (unsigned)(wave + 4 * (j & 3)) * 1024u;
      load16_to_lds_stream(make_rsrc(w_base[j] + (size_t)(s_base + s) * w_kstep), (k0 < w_klim[j]) ? w_off[j] : kOobOffset,
                           st + kXBytes + dst);
    }
  };
  // half h of stage s: k = 32h .. 32h+31
  auto read_frags = [&](int s, int h, i16x8 (&fq)[2][NQ], i16x8 (&fp)[2][2]) {
    const FSW_LDS char* sx = smem_l + (s % kStages) * kStage;
    const FSW_LDS char* sw = sx + kXBytes;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int q = 0; q < NQ; q++) fq[ks][q] = read_frag_kc32(sx, q * 32, 2 * h + ks, lane);
#pragma unroll
      for (int a = 0; a < 2; a++) {
        if constexpr (W_KC) fp[ks][a] = read_frag_kc32(sw, a * 128 + wave * 32, 2 * h + ks, lane);
        else fp[ks][a] = read_frag_mc(sw + h * kMcSlotBytes + a * kMcPanelBytes, wave, ks, lane);
      }
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

  // Per stage: read its second half while the first is multiplied; then one barrier, before which a wave
  // waits for its loads of the next stage and for its own fragment reads of this one (both halves are in
  // registers by then), so the slot can be refilled at once; read the next stage's first half while the
  // second half is multiplied.
  constexpr int kInFlight = (kStages - 2) * C::kPerStage;
  static_assert(kInFlight < 64, "vmcnt is 6 bits");
#pragma unroll
  for (int s = 0; s < kStages; s++) issue(s);
  i16x8 fq0[2][NQ], fp0[2][2], fq1[2][NQ], fp1[2][2];
  wait_vmcnt_and_barrier<(kStages - 1) * C::kPerStage>();  // stage 0 has landed
  read_frags(0, 0, fq0, fp0);
  for (int s = 0; s < st_total; s++) {
    read_frags(s, 1, fq1, fp1);
    mfmas(fq0, fp0);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(kInFlight) : "memory");
    issue(s + kStages);
    read_frags(s + 1, 0, fq0, fp0);
    mfmas(fq1, fp1);
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the zero-filling loads past the end

  // acc[h][q][r] of lane l: row q*32 + (l & 31), column n0 + wave*32 + 8*(r >> 2) + 4*(l >> 5) + (r & 3)
#pragma unroll
  for (int q = 0; q < NQ; q++) {
    const int m = q * 32 + (lane & 31);
    if (m >= p.M) continue;
#pragma unroll
    for (int r4 = 0; r4 < 4; r4++) {
      const int nc = wave * 32 + 8 * r4 + 4 * (lane >> 5), n = n0 + nc;
      if (nc >= bn || n >= p.N) continue;
      if (a.plain) {
        // the two halves are columns n and N + n of one result, 2N wide
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const float v[4] = {acc[h][q][r4 * 4], acc[h][q][r4 * 4 + 1], acc[h][q][r4 * 4 + 2], acc[h][q][r4 * 4 + 3]};
          if (p.ws) {
            float* dst = p.ws + ((size_t)split * p.M + m) * (2 * (size_t)p.N) + (size_t)h * p.N + n;
            *(f32x4*)dst = f32x4{v[0], v[1], v[2], v[3]};
          } else {
            u32x2 w;
            w.x = E::pack2(v[0], v[1]);
            w.y = E::pack2(v[2], v[3]);
            *(u32x2*)((unsigned short*)p.c1 + (size_t)m * p.ldc + (size_t)h * p.N + n) = w;
          }
        }
        continue;
      }
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

// Beyond 128 rows a stage (x as many bytes as the weights by then) leaves room for two slots only: the tiled
// kernel takes over.
constexpr int kSkMaxRows = 128;

// Width of a workgroup's column block.  128 columns fill the LDS slot, but a launch is one workgroup per block
// and every block takes the same time, so what counts is rounds x width: the width that covers N with the
// fewest rounds of `cus` workgroups wins (I = 28672 on 256 CUs: 256 blocks of 112 instead of 224 of 128;
// I = 12288 and 16 rows: 256 blocks of 48 instead of 96 of 128).  Two limits, both measured:
//  * weights stored [D, I] are read in row segments that must start on 128-byte lines (partial lines are
//    fetched whole, by two workgroups): widths of 64 and 128 only; rows of [I, D] weights are lines of
//    their own: any multiple of 8;
//  * a narrower block leaves part of every 32 KiB weight slot empty while the x rows stay, so the useful
//    bytes in flight per CU shrink: not below 48 / 64 / 96 columns for up to 32 / 64 / 128 rows.
static int block_width(int N, int cus, bool w_kc, int bm) {
  const int step = w_kc ? 8 : 64;
  const int narrowest = w_kc ? (bm <= 32 ? 48 : (bm <= 64 ? 64 : 96)) : 64;
  int best = 128;
  long long best_cost = (long long)(((N + 127) / 128 + cus - 1) / cus) * 128;
  for (int bn = 128 - step; bn >= narrowest; bn -= step) {
    const long long cost = (long long)(((N + bn - 1) / bn + cus - 1) / cus) * bn;
    if (cost < best_cost) { best = bn; best_cost = cost; }
  }
  return best;
}

// Compute units of the current device, looked up once per device (these launches are 75-150 us kernels on the
// latency-critical decode path).  The plan of a launch depends on it, so a workspace query and the launch it
// sizes must run with the same device current.
static int cu_count() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus > 0) return cus;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
  cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

template <typename E, bool W_KC>
static hipError_t launch_skinny_t(const GemmParams& g, const SkArgs& a, hipStream_t s) {
  const dim3 grid((unsigned)((g.N + a.bn - 1) / a.bn), (unsigned)a.splits);
  if (g.M <= 32) fsw_skinny_forward_kernel<E, 32, W_KC><<<grid, kSkThreads, 0, s>>>(g, a);
  else if (g.M <= 64) fsw_skinny_forward_kernel<E, 64, W_KC><<<grid, kSkThreads, 0, s>>>(g, a);
  else fsw_skinny_forward_kernel<E, 128, W_KC><<<grid, kSkThreads, 0, s>>>(g, a);
  return hipGetLastError();
}

bool skinny_forward_ok(const Problem& p) { return p.T <= kSkMaxRows && fast_path_ok_forward(p); }

hipError_t launch_forward_skinny(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.x; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.out; g.c1 = p.g; g.c2 = p.u;
  g.M = (int)p.T; g.N = (int)p.I; g.K = (int)p.D;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldw; g.ldc = (int)p.ldo;
  const int stages = (int)((p.D + 63) / 64);
  const SkArgs a{block_width(g.N, cu_count(), p.w_out_in, g.M), 0, 1, stages};
  if (p.w_out_in) return dtype == kDtypeBF16 ? launch_skinny_t<BF16, true>(g, a, s) : launch_skinny_t<FP16, true>(g, a, s);
  return dtype == kDtypeBF16 ? launch_skinny_t<BF16, false>(g, a, s) : launch_skinny_t<FP16, false>(g, a, s);
}

// ---- the down projection for few tokens: y [M, N] = a [M, K] W, W stored [K, N] (layout 0) or [N, K] (layout 1)
// The same kernel with W's two column halves in the places of Wg and Wu.  N is short and K long here (D and I
// of the SwiGLU), so column blocks alone do not fill the chip: the reduction is split as well, the fp32 partial
// planes go to the caller's scratch and fsw_splitk_reduce_kernel adds them in a fixed order.
struct SkPlan { int bn, splits, stages_per_split; };

// Full 128-column blocks and as many k-splits as fit into one round of workgroups (measured at N = 8192,
// K = 28672: 32 blocks x 8 splits beat every narrower block with fewer splits, although the partial planes
// then cost 2 x 8 x M x N x 4 bytes of traffic: narrow blocks leave the 32 KiB weight slots half empty).
// Enough column blocks for a round on their own: no split, and the width rule of the forward.
static SkPlan plan_plain(long long M, long long Nh, long long K, int cus, bool w_kc, long long max_splits) {
  const int stages = (int)((K + 63) / 64);
  const long long tiles = (Nh + 127) / 128;
  long long splits = cus / tiles;
  if (splits > 16) splits = 16;
  if (splits > max_splits) splits = max_splits;
  if (splits > stages / 8) splits = stages / 8;   // a split shorter than 8 stages does not fill the ring
  if (splits <= 1) return SkPlan{block_width((int)Nh, cus, w_kc, (int)M), 1, stages};
  const int sps = (int)((stages + splits - 1) / splits);
  return SkPlan{128, (stages + sps - 1) / sps, sps};
}

bool skinny_gemm_ok(const GemmProblem& p) {
  if (p.layout > 1 || p.M > kSkMaxRows || (p.N & 1) || !fast_path_ok_gemm(p)) return false;
  const long long nh = p.N / 2;
  return p.layout == 1 ? (nh % 8 == 0) : (nh % 64 == 0);   // the second half starts on a line / a 16-byte boundary
}

long long skinny_gemm_workspace_bytes(int layout, long long M, long long N, long long K) {
  if (layout > 1 || M > kSkMaxRows || M <= 0 || (N & 1) || (N / 2) % (layout == 1 ? 8 : 64)) return 0;
  const SkPlan pl = plan_plain(M, N / 2, K, cu_count(), layout == 1, 16);
  return pl.splits > 1 ? (long long)pl.splits * M * N * 4 : 0;
}

hipError_t launch_gemm_skinny(int dtype, const GemmProblem& p, hipStream_t s, void* ws, long long ws_bytes) {
  const bool w_kc = p.layout == 1;
  const long long nh = p.N / 2;
  const long long fit = ws ? ws_bytes / (p.M * p.N * 4) : 1;
  const SkPlan pl = plan_plain(p.M, nh, p.K, cu_count(), w_kc, fit < 1 ? 1 : fit);
  GemmParams g{};
  g.a0 = p.a; g.b0 = p.b;
  g.b1 = (const char*)p.b + (w_kc ? (size_t)nh * p.ldb * 2 : (size_t)nh * 2);
  g.c1 = p.c;
  g.M = (int)p.M; g.N = (int)nh; g.K = (int)p.K;
  g.lda = (int)p.lda; g.ldb = (int)p.ldb; g.ldc = (int)p.ldc;
  g.ws = pl.splits > 1 ? (float*)ws : nullptr;
  const SkArgs a{pl.bn, 1, pl.splits, pl.stages_per_split};
  hipError_t e;
  if (w_kc) e = dtype == kDtypeBF16 ? launch_skinny_t<BF16, true>(g, a, s) : launch_skinny_t<FP16, true>(g, a, s);
  else e = dtype == kDtypeBF16 ? launch_skinny_t<BF16, false>(g, a, s) : launch_skinny_t<FP16, false>(g, a, s);
  if (e != hipSuccess || pl.splits == 1) return e;
  const size_t n = (size_t)p.M * p.N;
  const dim3 blocks((unsigned)((n / 4 + 255) / 256), 1);
  if (dtype == kDtypeBF16)
    fsw_splitk_reduce_kernel<BF16><<<blocks, 256, 0, s>>>((const float*)ws, (unsigned short*)p.c, nullptr, n, pl.splits,
                                                         (int)p.N, (int)p.ldc);
  else
    fsw_splitk_reduce_kernel<FP16><<<blocks, 256, 0, s>>>((const float*)ws, (unsigned short*)p.c, nullptr, n, pl.splits,
                                                         (int)p.N, (int)p.ldc);
  return hipGetLastError();
}

}  // namespace fsw
