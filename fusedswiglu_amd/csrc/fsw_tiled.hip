// Host side of the tiled MFMA kernels: eligibility checks and launches.
#include "fsw_gemm.hpp"
#include "fsw_gemm4.hpp"
#include "fsw_internal.hpp"

namespace fsw {

static bool mult8(long long v) { return v > 0 && (v & 7) == 0; }
static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }
// a per-lane byte offset inside one tile (up to 256 rows) must stay below 2^31
static bool ld_ok(long long ld) { return mult8(ld) && ld < (1LL << 21); }
// leading dimension of a result: a wave addresses its up to 128 rows through 32-bit byte offsets from the first
static bool ld_out_ok(long long ld) { return mult8(ld) && ld < (1LL << 23); }
static bool dims_ok(const Problem& p) {
  return mult8(p.D) && mult8(p.I) && p.T > 0 && p.T < (1LL << 31) && p.D < (1LL << 31) &&
         p.I < (1LL << 31);
}

// With [I,D] weights the roles of D and I as contiguous index swap for the weight operands, but both must be
// multiples of 8 either way (x, dx are D-contiguous, the [T,I] arrays I-contiguous).
bool fast_path_ok_forward(const Problem& p) {
  return dims_ok(p) && ld_ok(p.ldx) && ld_ok(p.ldw) && ld_out_ok(p.ldo) && al16(p.x) && al16(p.wg) &&
         al16(p.wu) && al16(p.out) && al16(p.g) && al16(p.u) && al16(p.dout);
}
bool fast_path_ok_input_grad(const Problem& p) {
  return dims_ok(p) && ld_ok(p.ldo) && ld_ok(p.ldw) && ld_out_ok(p.lddx) && al16(p.dG) && al16(p.dU) &&
         al16(p.wg) && al16(p.wu) && al16(p.dx);
}
bool fast_path_ok_weight_grad(const Problem& p) {
  // x and dG/dU are read with the token index outermost: T itself may be any positive count
  return dims_ok(p) && ld_ok(p.ldx) && ld_ok(p.ldo) && ld_out_ok(p.lddw) && al16(p.x) && al16(p.dG) &&
         al16(p.dU) && al16(p.dWg) && al16(p.dWu);
}

// Split-K plan for a GEMM with `tiles` output tiles and `steps` reduction steps: few tiles and a long
// reduction leave most of the 256 CUs idle, so several workgroups share a tile.  Returns 1 (no split)
// when the tiles already fill the chip or the workspace is missing/too small.
struct SplitPlan { int splits, steps_per_split; };
// Estimated time (microseconds) of running `tiles * s` workgroups, each reducing 1/s of `steps` steps,
// on 256 CUs: whole rounds of 256 workgroups at ~1 us per step, plus writing and re-reading the fp32
// partial tiles at ~4 TB/s when s > 1.
static double split_cost_us(long long tiles, int steps, int s, double result_elems) {
  const long long wgs = tiles * s;
  const double rounds = (double)((wgs + 255) / 256);
  const double compute = rounds * ((double)steps / s + 6.0) * 0.96;  // + pipeline fill/epilogue per workgroup
  const double partials = s > 1 ? 2.0 * s * result_elems * 4.0 / 4.0e6 : 0.0;
  return compute + partials;
}
static SplitPlan plan_split_unbounded(long long tiles, int steps, long long M, long long N, int results) {
  SplitPlan pl{1, steps};
  if (tiles >= 1024 || steps < 32) return pl;
  const double elems = (double)M * (double)N * results;
  int best = 1;
  double best_cost = split_cost_us(tiles, steps, 1, elems);
  const int max_s = steps / 16 < 64 ? steps / 16 : 64;  // at least 16 steps per workgroup
  for (int s = 2; s <= max_s; s++) {
    const double c = split_cost_us(tiles, steps, s, elems);
    if (c < best_cost * 0.95) { best_cost = c; best = s; }
  }
  if (best == 1) return pl;
  int sps = (steps + best - 1) / best;
  sps = (sps + 1) & ~1;                                  // pairs of steps stay together
  pl.steps_per_split = sps;
  pl.splits = (steps + sps - 1) / sps;
  return pl;
}
static SplitPlan plan_split(long long tiles, int steps, long long M, long long N, int results,
                            const void* ws, long long ws_bytes) {
  SplitPlan pl = plan_split_unbounded(tiles, steps, M, N, results);
  if (pl.splits > 1 && (!ws || (long long)pl.splits * M * N * 4 * results > ws_bytes)) return SplitPlan{1, steps};
  return pl;
}
// Tail split: when the tiles do not fill the last round of 256 workgroups, each tile of that round goes to
// `parts` workgroups that reduce a slice each (fsw_gemm.hpp, GemmParams).  Only for long reductions and at
// least one full round before; the partial tiles take count * parts * 256 KiB of scratch.
struct TailPlan { int first, count, parts, steps; };
static TailPlan plan_tail(long long tiles, int steps) {
  TailPlan t{0, 0, 1, steps};
  const int count = (int)(tiles % 256);
  if (tiles < 256 || count == 0 || count > 128 || steps < 128) return t;
  int parts = 256 / count;
  if (parts > 8) parts = 8;
  if (parts > steps / 32) parts = steps / 32;
  if (parts < 2) return t;
  int sp = (steps + parts - 1) / parts;
  sp = (sp + 1) & ~1;  // pairs of steps stay together
  t.first = (int)(tiles - count);
  t.count = count;
  t.steps = sp;
  t.parts = (steps + sp - 1) / sp;
  return t;
}
static long long tail_bytes(const TailPlan& t) { return (long long)t.count * t.parts * kTileFloats * 4; }

static int steps_of(int mode, long long K) {
  int steps = (int)((K + kBK - 1) / kBK);
  return (mode == kDx || mode == kDxT) ? 2 * ((steps + 1) & ~1) : steps;
}

// Scratch for a GEMM of the given mode with results `results` x [M, N] and a reduction of K per pass.
template <int MODE>
static long long workspace_of(long long M, long long N, long long K, bool with_tail = true) {
  using C = Cfg<MODE>;
  const long long tiles = ((M + C::kTileM - 1) / C::kTileM) * ((N + C::kTileN - 1) / C::kTileN);
  const SplitPlan pl = plan_split_unbounded(tiles, steps_of(MODE, K), M, N, C::kResults);
  if (pl.splits > 1) return (long long)pl.splits * M * N * 4 * C::kResults;
  return with_tail ? tail_bytes(plan_tail(tiles, steps_of(MODE, K))) : 0;
}

long long splitk_workspace_bytes(int step, long long T, long long D, long long I, bool with_tail) {
  switch (step) {
    case 1: return workspace_of<kDx>(T, D, I, with_tail);    // input_grad: result [T, D], reduction over 2*I
    case 2: return workspace_of<kDw>(D, I, T, with_tail);    // weight_grad: results 2 x [D, I], reduction over T
    case 4: return workspace_of<kDxT>(T, D, I, with_tail);   // the same two for [I, D] weights
    case 5: return workspace_of<kDwT>(I, D, T, with_tail);
    default: return 0;
  }
}

long long gemm_workspace_bytes(int layout, long long M, long long N, long long K) {
  switch (layout) {
    case 0: return workspace_of<kNN>(M, N, K);
    case 1: return workspace_of<kNT>(M, N, K);
    case 2: return workspace_of<kTN>(M, N, K);
    default: return 0;
  }
}

template <int MODE>
static hipError_t launch(int dtype, GemmParams g, hipStream_t s, void* ws = nullptr, long long ws_bytes = 0) {
  constexpr int TM = Cfg<MODE>::kTileM, TN = Cfg<MODE>::kTileN;
  g.tiles_m = (g.M + TM - 1) / TM;
  g.tiles_n = (g.N + TN - 1) / TN;
  // Height of the bands of tile-rows an XCD walks (xcd_tile_order).  The A panels of the 8 bands in
  // flight (8 XCDs x group_m panels of 256 rows x K) should stay in the 256 MB memory-side cache while
  // the B panels stream past: 8 tile-rows up to K = 4096, 4 beyond (measured at K = 8192: 4 % faster).
  g.group_m = g.K > 4096 ? 4 : 8;
  const long long tiles = (long long)g.tiles_m * g.tiles_n;
  const int steps = steps_of(MODE, g.K);
  const int results = Cfg<MODE>::kResults;
  const SplitPlan pl = Cfg<MODE>::kForward ? SplitPlan{1, steps}
                                      : plan_split(tiles, steps, g.M, g.N, results, ws, ws_bytes);
  g.ws = (float*)ws; g.splits = pl.splits; g.steps_per_split = pl.steps_per_split;
  const long long grid = tiles * pl.splits;
  if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
  // Which form of the kernel: four waves with 128 x 128 wave tiles read a third less from LDS per MFMA and run
  // the long reductions 3-8 % faster; their prologue and epilogue are slower (half the waves), so short reductions
  // stay on the eight-wave form (measured cross-over: about 64 steps, 96 for the forwards with their three
  // results).  The four-wave form walks an m/n-contiguous operand through 32-bit offsets from its first k-row.
  const bool w4_fits = (Cfg<MODE>::kAKc || (long long)g.K * g.lda * 2 < (1LL << 31)) &&
                       (Cfg<MODE>::kBKc || (long long)g.K * g.ldb * 2 < (1LL << 31));
  const int steps_per_workgroup = pl.splits > 1 ? pl.steps_per_split : steps;
  const bool four_waves = w4_fits && steps_per_workgroup >= (Cfg<MODE>::kForward ? 96 : 64);
  long long grid4 = grid;
  if constexpr (!Cfg<MODE>::kForward) {
    const TailPlan tp = plan_tail(tiles, steps);
    if (four_waves && pl.splits == 1 && tp.count > 0 && ws && tail_bytes(tp) <= ws_bytes) {
      g.tail_first = tp.first; g.tail_count = tp.count; g.tail_parts = tp.parts; g.tail_steps = tp.steps;
      grid4 = tp.first + (long long)tp.count * tp.parts;
    }
  }
  if (four_waves) {
    const long long grid = grid4;
    if (Cfg<MODE>::kForward && g.tiles_m == 1) {
      if constexpr (Cfg<MODE>::kForward) {
        if (dtype == kDtypeBF16) fsw_gemm4_kernel<BF16, MODE, true><<<(unsigned)grid, kThreads4, 0, s>>>(g);
        else fsw_gemm4_kernel<FP16, MODE, true><<<(unsigned)grid, kThreads4, 0, s>>>(g);
      }
    } else if (dtype == kDtypeBF16) fsw_gemm4_kernel<BF16, MODE><<<(unsigned)grid, kThreads4, 0, s>>>(g);
    else fsw_gemm4_kernel<FP16, MODE><<<(unsigned)grid, kThreads4, 0, s>>>(g);
  } else
  // a forward with a single row of tiles reads every weight byte exactly once: stream them past the caches
  if (Cfg<MODE>::kForward && g.tiles_m == 1) {
    if constexpr (Cfg<MODE>::kForward) {
      if (dtype == kDtypeBF16) fsw_gemm_kernel<BF16, MODE, true><<<(unsigned)grid, kThreads, 0, s>>>(g);
      else fsw_gemm_kernel<FP16, MODE, true><<<(unsigned)grid, kThreads, 0, s>>>(g);
    }
  } else if (dtype == kDtypeBF16) fsw_gemm_kernel<BF16, MODE><<<(unsigned)grid, kThreads, 0, s>>>(g);
  else fsw_gemm_kernel<FP16, MODE><<<(unsigned)grid, kThreads, 0, s>>>(g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if constexpr (!Cfg<MODE>::kForward) {
    if (g.tail_count > 0) {
      const dim3 blocks((unsigned)(kTileFloats / 8192), (unsigned)g.tail_count);
      if (dtype == kDtypeBF16) fsw_tail_reduce_kernel<BF16, MODE><<<blocks, 256, 0, s>>>(g);
      else fsw_tail_reduce_kernel<FP16, MODE><<<blocks, 256, 0, s>>>(g);
      return hipGetLastError();
    }
  }
  if (pl.splits == 1) return e;
  const size_t n = (size_t)g.M * g.N;
  const dim3 blocks((unsigned)((n / 4 + 255) / 256), (unsigned)results);
  if (dtype == kDtypeBF16)
    fsw_splitk_reduce_kernel<BF16><<<blocks, 256, 0, s>>>((const float*)ws, (unsigned short*)g.c0, (unsigned short*)g.c1, n,
                                                         pl.splits, g.N, g.ldc);
  else
    fsw_splitk_reduce_kernel<FP16><<<blocks, 256, 0, s>>>((const float*)ws, (unsigned short*)g.c0, (unsigned short*)g.c1, n,
                                                         pl.splits, g.N, g.ldc);
  return hipGetLastError();
}

hipError_t launch_forward_fast(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.x; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.out; g.c1 = p.g; g.c2 = p.u; g.d0 = p.dout;
  g.M = (int)p.T; g.N = (int)p.I; g.K = (int)p.D;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldw; g.ldc = (int)p.ldo;
  return p.w_out_in ? launch<kFwdT>(dtype, g, s) : launch<kFwd>(dtype, g, s);
}

hipError_t launch_input_grad_fast(int dtype, const Problem& p, hipStream_t s, void* ws, long long ws_bytes) {
  GemmParams g{};
  g.a0 = p.dG; g.a1 = p.dU; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.dx;
  g.M = (int)p.T; g.N = (int)p.D; g.K = (int)p.I;
  g.lda = (int)p.ldo; g.ldb = (int)p.ldw; g.ldc = (int)p.lddx;
  return p.w_out_in ? launch<kDxT>(dtype, g, s, ws, ws_bytes) : launch<kDx>(dtype, g, s, ws, ws_bytes);
}

hipError_t launch_weight_grad_fast(int dtype, const Problem& p, hipStream_t s, void* ws, long long ws_bytes) {
  GemmParams g{};
  if (p.w_out_in) {  // dWg [I,D] = dG^T x: the two results share the B tile (x)
    g.a0 = p.dG; g.a1 = p.dU; g.b0 = p.x; g.c0 = p.dWg; g.c1 = p.dWu;
    g.M = (int)p.I; g.N = (int)p.D; g.K = (int)p.T;
    g.lda = (int)p.ldo; g.ldb = (int)p.ldx; g.ldc = (int)p.lddw;
    return launch<kDwT>(dtype, g, s, ws, ws_bytes);
  }
  g.a0 = p.x; g.b0 = p.dG; g.b1 = p.dU; g.c0 = p.dWg; g.c1 = p.dWu;
  g.M = (int)p.D; g.N = (int)p.I; g.K = (int)p.T;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldo; g.ldc = (int)p.lddw;
  return launch<kDw>(dtype, g, s, ws, ws_bytes);
}

bool fast_path_ok_gemm(const GemmProblem& p) {
  return p.M > 0 && p.N > 0 && p.K > 0 && p.M < (1LL << 31) && p.N < (1LL << 31) && p.K < (1LL << 31) &&
         // the contiguous index of each operand must be a multiple of 8 elements
         mult8(p.layout == 2 ? p.M : p.K) && mult8(p.layout == 1 ? p.K : p.N) && mult8(p.N) &&
         ld_ok(p.lda) && ld_ok(p.ldb) && ld_out_ok(p.ldc) && al16(p.a) && al16(p.b) && al16(p.c);
}

hipError_t launch_gemm_fast(int dtype, const GemmProblem& p, hipStream_t s, void* ws, long long ws_bytes) {
  GemmParams g{};
  g.a0 = p.a; g.b0 = p.b; g.c0 = p.c;
  g.M = (int)p.M; g.N = (int)p.N; g.K = (int)p.K;
  g.lda = (int)p.lda; g.ldb = (int)p.ldb; g.ldc = (int)p.ldc;
  switch (p.layout) {
    case 0: return launch<kNN>(dtype, g, s, ws, ws_bytes);
    case 1: return launch<kNT>(dtype, g, s, ws, ws_bytes);
    default: return launch<kTN>(dtype, g, s, ws, ws_bytes);
  }
}

}  // namespace fsw
