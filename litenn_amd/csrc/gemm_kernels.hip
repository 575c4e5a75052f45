// Plain fp32 GEMM on the MFMA tile engine: NN, NT and TN operand layouts, so
// that matmul's gradients dA = dC.B^T and dB = A^T.dC never materialise a
// transposed operand.
#include <type_traits>

#include "common.hpp"

#ifndef LNN_GEMM_XCD_BLOCKS
#define LNN_GEMM_XCD_BLOCKS 1
#endif
#ifndef LNN_STAGES_GEMM
#define LNN_STAGES_GEMM 3
#endif

namespace lnn {

struct GemmArgs {
  const float* A;
  const float* B;
  float* C;
  int M, N, K, lda, ldb, ldc;
  long long sA, sB, sC;           // batch strides in elements
  uint32_t bytesA, bytesB, bytesC;  // extent of one batch item
  int beta;
  int n_units, total_units;       // schedule: units of 32*WN columns per M tile
  // Workgroup -> share of the output.  The hardware deals consecutive workgroups round-robin to the 8 XCDs (each
  // with its own L2), so by default an XCD's workgroups sit in every row of tiles and share only the B operand.
  // With xcd_bc > 0 the workgroups of one XCD own a block of xcd_br tile rows x xcd_bc shares per row instead,
  // so that xcd_bc of them read the same A tiles and xcd_br the same B tiles out of their L2 (wg_per_row shares
  // make up a row of tiles).
  int xcd_br, xcd_bc, wg_per_row;
};

// MODE: how operands travel.  0: 32-bit loads through registers (any alignment,
// any K); 1: 128-bit loads through registers; 2: 128-bit transfers straight
// into LDS (as 1, and K a multiple of BK).
template <int WM, int NTMAX, bool TA, bool TB, int MODE>
struct GemmCfg {
  static constexpr int WN = 4 / WM, BM = 32 * WM, BNMAX = 32 * WN * 2 * NTMAX;
  // direct transfers fill unpadded tiles and run three stages deep
  static constexpr int SA = MODE == 2 ? BM * BK : LdsSize<!TA, BM>::value;
  static constexpr int SB = MODE == 2 ? BNMAX * BK : LdsSize<TB, BNMAX>::value;
  static constexpr int STAGES = MODE == 2 ? LNN_STAGES_GEMM : 2;
};

// A operand: !TA -> A[M][K] row-major, K-contiguous; TA -> stored [K][M].
// B operand: !TB -> B[K][N], row(n)-contiguous;      TB -> stored [N][K].
template <bool TA, bool TB, int MODE, int ST>
struct GemmProblem {
  static constexpr int STAGES = ST;
  static constexpr bool STREAM_UNROLL = !TB;   // measured: A * B^T is slower with constant stages
  static constexpr bool STREAM_REGIONS = false;   // measured: A * B^T 0.948 -> 0.96 ms with one region per group
  static constexpr bool VEC = MODE >= 1, DIR = MODE == 2;
  template <int R> using KCL = typename std::conditional<DIR, DirectKC<R>, PlainKC<R, VEC>>::type;
  template <int R> using MCL = typename std::conditional<DIR, DirectMC<R>, PlainMC<R, VEC>>::type;
  template <int R> using LA = typename std::conditional<TA, MCL<R>, KCL<R>>::type;
  template <int R> using LB = typename std::conditional<TB, KCL<R>, MCL<R>>::type;
  rsrc_t ra, rb, rc;
  int lda, ldb, M, Ncols, K, kbeg, kend, beta;
  OutMap om;
  PostOp post;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(ra, lda, row0, M, K); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rb, ldb, col0, Ncols, K); }
};

template <int WM, int NTMAX, bool TA, bool TB, int MODE>
__global__ __launch_bounds__(512, 2) void gemm_kernel(GemmArgs a) {
  using Cfg = GemmCfg<WM, NTMAX, TA, TB, MODE>;
  __shared__ __attribute__((aligned(16))) float lds[Cfg::STAGES * (Cfg::SA + Cfg::SB)];
  const long long b = blockIdx.y;
  GemmProblem<TA, TB, MODE, Cfg::STAGES> p;
  p.ra = make_rsrc(a.A + b * a.sA, a.bytesA);
  p.rb = make_rsrc(a.B + b * a.sB, a.bytesB);
  p.rc = make_rsrc(a.C + b * a.sC, a.bytesC);
  p.lda = a.lda; p.ldb = a.ldb; p.M = a.M; p.Ncols = a.N; p.K = a.K;
  p.kbeg = 0; p.kend = a.K; p.beta = a.beta;
  p.post.bias = nullptr; p.post.act = 0; p.post.slope = 0.0f;
  p.om.nchw = 0; p.om.ld = a.ldc; p.om.mtot = 0; p.om.dHW = FastDiv{0, 0, 1};
  int wg = (int)blockIdx.x;
  if (a.xcd_bc > 0) {
    const int xcd = wg & 7, j = wg >> 3, blocks_per_row = a.wg_per_row / a.xcd_bc;
    const int r = (xcd / blocks_per_row) * a.xcd_br + j / a.xcd_bc, c = (xcd % blocks_per_row) * a.xcd_bc + j % a.xcd_bc;
    wg = r * a.wg_per_row + c;
  }
  walk_units<WM, NTMAX>(p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, a.n_units, a.total_units, wg, (int)gridDim.x);
}

template <int WM, int NTMAX, bool TA, bool TB>
static int launch_cfg(DeviceCtx* ctx, GemmArgs& a, int batch, int mode) {
  constexpr int WN = 4 / WM, BM = 32 * WM;
  const int m_tiles = (a.M + BM - 1) / BM;
  a.n_units = (a.N + 32 * WN - 1) / (32 * WN);
  const long long total = (long long)m_tiles * a.n_units;
  if (total > 0x7fffffffll) return set_error(LNN_ERR_UNSUPPORTED, "gemm: too many tiles");
  a.total_units = (int)total;
  long long slots = (long long)ctx->cus / (batch > 1 ? (batch > 8 ? 8 : batch) : 1);
  if (slots < 1) slots = 1;
  const int grid = (int)(total < slots ? total : slots);
  // XCD-local blocks of shares: when the shares tile the output exactly (every share the same run of units inside
  // one row of tiles) and 8 blocks of 8 tile rows x 4 shares cover it
  a.xcd_br = a.xcd_bc = a.wg_per_row = 0;
  if (LNN_GEMM_XCD_BLOCKS && batch == 1 && grid % 8 == 0 && total % grid == 0 && a.n_units % (total / grid) == 0) {
    const int per_row = (int)(a.n_units / (total / grid));
    if (per_row % 4 == 0 && m_tiles % 8 == 0 && (per_row / 4) * (m_tiles / 8) == 8 && per_row * m_tiles == grid) {
      a.xcd_br = 8; a.xcd_bc = 4; a.wg_per_row = per_row;
    }
  }
  dim3 g(grid, batch, 1), b(512, 1, 1);
  if (mode == 2)
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 2>), g, b, 0, ctx->stream, a);
  else if (mode == 1)
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 1>), g, b, 0, ctx->stream, a);
  else
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 0>), g, b, 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

template <bool TA, bool TB>
static int launch_layout(DeviceCtx* ctx, GemmArgs& a, int batch, int mode) {
  if (a.M > 64) return launch_cfg<4, 4, TA, TB>(ctx, a, batch, mode);
  if (a.M > 32) return launch_cfg<2, 2, TA, TB>(ctx, a, batch, mode);
  return launch_cfg<1, 1, TA, TB>(ctx, a, batch, mode);
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int launch_gemm(DeviceCtx* ctx, int ta, int tb, int batch, int M, int N, int K, const float* A, int lda,
                long long sA, const float* B, int ldb, long long sB, float* C, int ldc, long long sC, int beta) {
  if (M <= 0 || N <= 0 || K <= 0 || batch <= 0) return set_error(LNN_ERR_INVALID, "gemm: non-positive dimension");
  if (!A || !B || !C) return set_error(LNN_ERR_INVALID, "gemm: null pointer");
  if (batch > 65535) return set_error(LNN_ERR_UNSUPPORTED, "gemm: batch > 65535");
  const int a_rows = ta ? K : M, a_cols = ta ? M : K;
  const int b_rows = tb ? N : K, b_cols = tb ? K : N;
  if (lda < a_cols || ldb < b_cols || ldc < N) return set_error(LNN_ERR_INVALID, "gemm: leading dimension too small");
  const uint64_t bytesA = ((uint64_t)(a_rows - 1) * lda + a_cols) * 4;
  const uint64_t bytesB = ((uint64_t)(b_rows - 1) * ldb + b_cols) * 4;
  const uint64_t bytesC = ((uint64_t)(M - 1) * ldc + N) * 4;
  if (bytesA > kMaxTensorBytes || bytesB > kMaxTensorBytes || bytesC > kMaxTensorBytes)
    return set_error(LNN_ERR_UNSUPPORTED, "gemm: a matrix of 2 GiB or more");
  GemmArgs a;
  a.A = A; a.B = B; a.C = C;
  a.M = M; a.N = N; a.K = K;
  a.lda = lda; a.ldb = ldb; a.ldc = ldc;
  a.sA = sA; a.sB = sB; a.sC = sC;
  a.bytesA = (uint32_t)bytesA; a.bytesB = (uint32_t)bytesB; a.bytesC = (uint32_t)bytesC;
  a.beta = beta ? 1 : 0;
  // 128-bit loads run along K for a K-contiguous operand and along the rows
  // for a row-contiguous one; both the extent and every row start must be
  // multiples of four floats.
  const bool va = aligned16(A) && lda % 4 == 0 && sA % 4 == 0 && a_cols % 4 == 0;
  const bool vb = aligned16(B) && ldb % 4 == 0 && sB % 4 == 0 && b_cols % 4 == 0;
  const int mode = (va && vb) ? (K % BK == 0 ? 2 : 1) : 0;
  if (!ta && !tb) return launch_layout<false, false>(ctx, a, batch, mode);
  if (!ta && tb) return launch_layout<false, true>(ctx, a, batch, mode);
  if (ta && !tb) return launch_layout<true, false>(ctx, a, batch, mode);
  return set_error(LNN_ERR_UNSUPPORTED, "gemm: trans_a and trans_b together are not provided");
}

}  // namespace lnn
