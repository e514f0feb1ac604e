// Host side of the tiled MFMA kernels: eligibility checks and launches.
#include "fsw_gemm.hpp"
#include "fsw_internal.hpp"

namespace fsw {

static bool mult8(long long v) { return v > 0 && (v & 7) == 0; }
static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }
// a per-lane byte offset inside one tile (up to 256 rows) must stay below 2^31
static bool ld_ok(long long ld) { return mult8(ld) && ld < (1LL << 21); }
static bool dims_ok(const Problem& p) {
  return mult8(p.D) && mult8(p.I) && p.T > 0 && p.T < (1LL << 31) && p.D < (1LL << 31) &&
         p.I < (1LL << 31);
}

bool fast_path_ok_forward(const Problem& p) {
  return dims_ok(p) && ld_ok(p.ldx) && ld_ok(p.ldw) && mult8(p.ldo) && al16(p.x) && al16(p.wg) &&
         al16(p.wu) && al16(p.out) && al16(p.g) && al16(p.u);
}
bool fast_path_ok_input_grad(const Problem& p) {
  return dims_ok(p) && ld_ok(p.ldo) && ld_ok(p.ldw) && mult8(p.lddx) && al16(p.dG) && al16(p.dU) &&
         al16(p.wg) && al16(p.wu) && al16(p.dx);
}
bool fast_path_ok_weight_grad(const Problem& p) {
  // x and dG/dU are read with the token index outermost: T itself may be any positive count
  return dims_ok(p) && ld_ok(p.ldx) && ld_ok(p.ldo) && mult8(p.lddw) && al16(p.x) && al16(p.dG) &&
         al16(p.dU) && al16(p.dWg) && al16(p.dWu);
}

template <int MODE>
static hipError_t launch(int dtype, GemmParams g, hipStream_t s) {
  constexpr int TN = Cfg<MODE>::kTileN;
  g.tiles_m = (g.M + kTileM - 1) / kTileM;
  g.tiles_n = (g.N + TN - 1) / TN;
  g.group_m = 8;
  const long long tiles = (long long)g.tiles_m * g.tiles_n;
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  if (dtype == kDtypeBF16) fsw_gemm_kernel<BF16, MODE><<<(unsigned)tiles, kThreads, 0, s>>>(g);
  else fsw_gemm_kernel<FP16, MODE><<<(unsigned)tiles, kThreads, 0, s>>>(g);
  return hipGetLastError();
}

hipError_t launch_forward_fast(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.x; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.out; g.c1 = p.g; g.c2 = p.u;
  g.M = (int)p.T; g.N = (int)p.I; g.K = (int)p.D;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldw; g.ldc = (int)p.ldo;
  return launch<kFwd>(dtype, g, s);
}

hipError_t launch_input_grad_fast(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.dG; g.a1 = p.dU; g.b0 = p.wg; g.b1 = p.wu; g.c0 = p.dx;
  g.M = (int)p.T; g.N = (int)p.D; g.K = (int)p.I;
  g.lda = (int)p.ldo; g.ldb = (int)p.ldw; g.ldc = (int)p.lddx;
  return launch<kDx>(dtype, g, s);
}

hipError_t launch_weight_grad_fast(int dtype, const Problem& p, hipStream_t s) {
  GemmParams g{};
  g.a0 = p.x; g.b0 = p.dG; g.b1 = p.dU; g.c0 = p.dWg; g.c1 = p.dWu;
  g.M = (int)p.D; g.N = (int)p.I; g.K = (int)p.T;
  g.lda = (int)p.ldx; g.ldb = (int)p.ldo; g.ldc = (int)p.lddw;
  return launch<kDw>(dtype, g, s);
}

}  // namespace fsw
