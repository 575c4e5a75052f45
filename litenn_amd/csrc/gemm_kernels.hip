// Plain fp32 GEMM on the MFMA tile engine: NN, NT and TN operand layouts, so
// that matmul's gradients dA = dC.B^T and dB = A^T.dC never materialise a
// transposed operand.
#include <type_traits>

#include "common.hpp"

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
};

template <int WM, int NTMAX, bool TA, bool TB, bool VEC>
struct GemmCfg {
  static constexpr int WN = 4 / WM, BM = 32 * WM, BNMAX = 32 * WN * NTMAX;
  static constexpr int SA = LdsSize<!TA, BM>::value;
  static constexpr int SB = LdsSize<TB, BNMAX>::value;
};

template <class Cfg, int WM, int NT, bool TA, bool TB, bool VEC>
__device__ __forceinline__ void gemm_tile(const GemmArgs& p, rsrc_t ra, rsrc_t rb, rsrc_t rc, float* lds,
                                          int mt, int un) {
  constexpr int WN = 4 / WM, BM = 32 * WM, BN = 32 * WN * NT;
  using LA = typename std::conditional<TA, PlainMC<BM, VEC>, PlainKC<BM, VEC>>::type;
  using LB = typename std::conditional<TB, PlainKC<BN, VEC>, PlainMC<BN, VEC>>::type;
  const int m0 = mt * BM, n0 = un * 32 * WN;
  LA la;
  LB lb;
  la.init(ra, p.lda, m0, p.M, p.K);
  lb.init(rb, p.ldb, n0, p.N, p.K);
  OutMap om;
  om.nchw = 0;
  om.ld = p.ldc;
  om.mtot = 0;
  om.dHW = FastDiv{0, 0, 1};
  run_tile<WM, NT>(la, lb, lds, lds + 2 * Cfg::SA, Cfg::SA, Cfg::SB, 0, p.K, rc, om, m0, n0, p.M, p.N, p.beta);
}

template <int WM, int NTMAX, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(256, 2) void gemm_kernel(GemmArgs p) {
  using Cfg = GemmCfg<WM, NTMAX, TA, TB, VEC>;
  // at least 56 KB so that exactly two workgroups share a compute unit's 160 KB of LDS
  __shared__ __attribute__((aligned(16))) float lds[(2 * (Cfg::SA + Cfg::SB) > 14336) ? 2 * (Cfg::SA + Cfg::SB) : 14336];
  const long long b = blockIdx.y;
  const rsrc_t ra = make_rsrc(p.A + b * p.sA, p.bytesA);
  const rsrc_t rb = make_rsrc(p.B + b * p.sB, p.bytesB);
  const rsrc_t rc = make_rsrc(p.C + b * p.sC, p.bytesC);
  long long u0 = (long long)p.total_units * blockIdx.x / gridDim.x;
  const long long u1 = (long long)p.total_units * (blockIdx.x + 1) / gridDim.x;
  while (u0 < u1) {
    const int mt = (int)(u0 / p.n_units), un = (int)(u0 - (long long)mt * p.n_units);
    long long cnt = u1 - u0;
    if (cnt > p.n_units - un) cnt = p.n_units - un;
    const int nt = pick_units<NTMAX>((int)cnt);
    switch (nt) {
      case 1: gemm_tile<Cfg, WM, 1, TA, TB, VEC>(p, ra, rb, rc, lds, mt, un); break;
      case 2: gemm_tile<Cfg, WM, (NTMAX >= 2 ? 2 : 1), TA, TB, VEC>(p, ra, rb, rc, lds, mt, un); break;
      case 3: gemm_tile<Cfg, WM, (NTMAX >= 3 ? 3 : 1), TA, TB, VEC>(p, ra, rb, rc, lds, mt, un); break;
      default: gemm_tile<Cfg, WM, (NTMAX >= 4 ? 4 : 1), TA, TB, VEC>(p, ra, rb, rc, lds, mt, un); break;
    }
    u0 += nt;
  }
}

template <int WM, int NTMAX, bool TA, bool TB>
static int launch_cfg(DeviceCtx* ctx, GemmArgs& a, int batch, bool vec) {
  constexpr int WN = 4 / WM, BM = 32 * WM;
  const int m_tiles = (a.M + BM - 1) / BM;
  a.n_units = (a.N + 32 * WN - 1) / (32 * WN);
  const long long total = (long long)m_tiles * a.n_units;
  if (total > 0x7fffffffll) return set_error(LNN_ERR_UNSUPPORTED, "gemm: too many tiles");
  a.total_units = (int)total;
  long long slots = 2ll * ctx->cus / (batch > 1 ? (batch > 8 ? 8 : batch) : 1);
  if (slots < 1) slots = 1;
  const int grid = (int)(total < slots ? total : slots);
  dim3 g(grid, batch, 1), b(256, 1, 1);
  if (vec)
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, true>), g, b, 0, ctx->stream, a);
  else
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, false>), g, b, 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

template <bool TA, bool TB>
static int launch_layout(DeviceCtx* ctx, GemmArgs& a, int batch, bool vec) {
  if (a.M > 64) return launch_cfg<4, 4, TA, TB>(ctx, a, batch, vec);
  if (a.M > 32) return launch_cfg<2, 4, TA, TB>(ctx, a, batch, vec);
  return launch_cfg<1, 2, TA, TB>(ctx, a, batch, vec);
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
  const bool vec = va && vb;
  if (!ta && !tb) return launch_layout<false, false>(ctx, a, batch, vec);
  if (!ta && tb) return launch_layout<false, true>(ctx, a, batch, vec);
  if (ta && !tb) return launch_layout<true, false>(ctx, a, batch, vec);
  return set_error(LNN_ERR_UNSUPPORTED, "gemm: trans_a and trans_b together are not provided");
}

}  // namespace lnn
