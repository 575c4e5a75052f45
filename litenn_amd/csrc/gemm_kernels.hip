// Plain fp32 GEMM: NN, NT and TN operand layouts, so that matmul's gradients dA = dC.B^T and dB = A^T.dC never
// materialise a transposed operand.  Three kernel families:
//   gemm_kernel       the MFMA tile engine (LDS-staged operands), for problems with operand reuse; few output tiles
//                     and a long K are cut along K over the idle compute units (partial sums + slice reduction)
//   wave_gemm_kernel  one 32 x 128 output tile per wavefront with both operands read straight from memory into MFMA
//                     fragments: the bandwidth-bound shapes of a dense layer at small batch (few rows, the weight
//                     matrix streamed once) and of its weight gradient (short K, the result streamed once)
//   small_kn_kernel   K and N of a handful (the rank-3 products of a spatial transform): one output row per thread
#include <type_traits>

#include "common.hpp"
#include "slice_reduce.hpp"

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
  // K split (batch == 1 only): blockIdx.y = slice; slice s writes its partial sums, in GEMM order with pitch N,
  // to part + s*M*N; the slice reduction applies ldc, '+=' and the epilogue
  int ksplit;
  float* part;
  PostOp post;                    // bias per column / activation of the stored result ('=' only)
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
  static constexpr int STAGES = MODE == 2 ? 3 : 2;
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
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(ra, lda, row0, M, kend); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rb, ldb, col0, Ncols, kend); }
};

template <int WM, int NTMAX, bool TA, bool TB, int MODE>
__global__ __launch_bounds__(512, 2) void gemm_kernel(GemmArgs a) {
  using Cfg = GemmCfg<WM, NTMAX, TA, TB, MODE>;
  __shared__ __attribute__((aligned(16))) float lds[Cfg::STAGES * (Cfg::SA + Cfg::SB)];
  GemmProblem<TA, TB, MODE, Cfg::STAGES> p;
  p.lda = a.lda; p.ldb = a.ldb; p.M = a.M; p.Ncols = a.N; p.K = a.K;
  p.om.nchw = 0; p.om.mtot = 0; p.om.dHW = FastDiv{0, 0, 1};
  if (a.ksplit > 1) {
    const int slice = (int)blockIdx.y, nkt = (a.K + BK - 1) / BK;
    const int t0 = (int)((long long)nkt * slice / a.ksplit), t1 = (int)((long long)nkt * (slice + 1) / a.ksplit);
    p.kbeg = t0 * BK;
    p.kend = t1 * BK < a.K ? t1 * BK : a.K;
    p.ra = make_rsrc(a.A, a.bytesA);
    p.rb = make_rsrc(a.B, a.bytesB);
    p.rc = make_rsrc(a.part + (size_t)slice * a.M * a.N, (uint32_t)a.M * (uint32_t)a.N * 4u);
    p.om.ld = a.N;
    p.beta = 0;
    p.post = PostOp{nullptr, 0, 0.0f, 0};
  } else {
    const long long b = blockIdx.y;
    p.kbeg = 0;
    p.kend = a.K;
    p.ra = make_rsrc(a.A + b * a.sA, a.bytesA);
    p.rb = make_rsrc(a.B + b * a.sB, a.bytesB);
    p.rc = make_rsrc(a.C + b * a.sC, a.bytesC);
    p.om.ld = a.ldc;
    p.beta = a.beta;
    p.post = a.post;
  }
  int wg = (int)blockIdx.x;
  if (a.xcd_bc > 0) {
    const int xcd = wg & 7, j = wg >> 3, blocks_per_row = a.wg_per_row / a.xcd_bc;
    const int r = (xcd / blocks_per_row) * a.xcd_br + j / a.xcd_bc, c = (xcd % blocks_per_row) * a.xcd_bc + j % a.xcd_bc;
    wg = r * a.wg_per_row + c;
  }
  walk_units<WM, NTMAX>(p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, a.n_units, a.total_units, wg, (int)gridDim.x);
}

// Sum of the K slices of a split GEMM into C (pitch ldc), with '+=' and the epilogue.
static int launch_gemm_reduce(DeviceCtx* ctx, const float* part, int slices, int M, int N, float* C, int ldc, int beta,
                              const PostOp& post) {
  ReduceArgs r = {};
  r.n = M * N; r.slices = slices; r.slices_last = slices; r.beta = beta; r.ncols = N;
  r.bm_log = 5; r.uw_log = 5; r.per_mt = 0; r.last_unit0 = 0x7fffffff; r.kk = 0;
  r.dN = make_fastdiv((uint32_t)N);
  r.om.nchw = 0; r.om.ld = ldc; r.om.mtot = 0; r.om.dHW = FastDiv{0, 0, 1};
  r.om.dCW = FastDiv{0, 0, 1}; r.om.s = 0; r.om.iw = 0; r.om.org = 0;
  r.post = post;
  if (N % 4 == 0)   // the partial buffer starts 256-byte aligned
    hipLaunchKernelGGL(reduce_partials4, dim3((r.n + reduce4_block(r) - 1) / reduce4_block(r)), dim3(256), 0, ctx->stream, C, part, r);
  else
    hipLaunchKernelGGL(reduce_partials, dim3((r.n + 31) / 32), dim3(256), 0, ctx->stream, C, part, r);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
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
  int grid = (int)(total < slots ? total : slots), grid_y = batch;
  a.ksplit = 1;
  a.part = nullptr;
  // Few output tiles and a long K (a dense layer at small batch and its data gradient): a workgroup per sub-tile
  // would leave most compute units idle, each walking the whole K alone.  Cut the output into sub-tiles of half
  // the full width and K into as many slices as fill the chip; the slices' partial sums are added by a reduction
  // that also applies '+=' and the epilogue, as the convolution passes do.
  if (batch == 1) {
    const int chunk = NTMAX > 1 ? NTMAX : 2;
    const long long chunks = (total + chunk - 1) / chunk;
    const int nkt = (a.K + BK - 1) / BK;
    if (total < slots && chunks * 2 <= slots && nkt >= 16) {
      long long s = slots / chunks;
      if (s > nkt / 8) s = nkt / 8;
      if (s > 1) {
        a.ksplit = (int)s;
        grid = (int)chunks;
        grid_y = a.ksplit;
        const int st = ensure_workspace(ctx, (size_t)a.ksplit * a.M * a.N * sizeof(float));
        if (st != LNN_OK) return st;
        a.part = static_cast<float*>(ctx->ws);
      }
    }
  }
  // XCD-local blocks of shares: when the shares tile the output exactly (every share the same run of units inside
  // one row of tiles) and 8 blocks of 8 tile rows x 4 shares cover it
  a.xcd_br = a.xcd_bc = a.wg_per_row = 0;
  if (batch == 1 && a.ksplit == 1 && grid % 8 == 0 && total % grid == 0 && a.n_units % (total / grid) == 0) {
    const int per_row = (int)(a.n_units / (total / grid));
    if (per_row % 4 == 0 && m_tiles % 8 == 0 && (per_row / 4) * (m_tiles / 8) == 8 && per_row * m_tiles == grid) {
      a.xcd_br = 8; a.xcd_bc = 4; a.wg_per_row = per_row;
    }
  }
  dim3 g(grid, grid_y, 1), b(512, 1, 1);
  if (mode == 2)
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 2>), g, b, 0, ctx->stream, a);
  else if (mode == 1)
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 1>), g, b, 0, ctx->stream, a);
  else
    hipLaunchKernelGGL((gemm_kernel<WM, NTMAX, TA, TB, 0>), g, b, 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  if (a.ksplit > 1) return launch_gemm_reduce(ctx, a.part, a.ksplit, a.M, a.N, a.C, a.ldc, a.beta, a.post);
  return LNN_OK;
}

template <bool TA, bool TB>
static int launch_layout(DeviceCtx* ctx, GemmArgs& a, int batch, int mode) {
  if (a.M > 64) return launch_cfg<4, 4, TA, TB>(ctx, a, batch, mode);
  if (a.M > 32) return launch_cfg<2, 2, TA, TB>(ctx, a, batch, mode);
  return launch_cfg<1, 1, TA, TB>(ctx, a, batch, mode);
}

// ---------------------------------------------------------------------------
// One output tile per wavefront, operands straight from memory.
//
// A wavefront owns 32*MT rows x 128 columns of C: 4*MT accumulators of v_mfma_f32_32x32x2_f32.  Its B fragments are
// 128-bit loads along a row of B[K][N] (lanes 0-31: the 512 contiguous bytes of row k under the tile, lanes 32-63:
// row k + 4): the four floats of a lane are the same k for four columns, one per accumulator, so accumulator j holds
// columns n0 + 4*i + j (i = lane % 32) and a lane's four results for an output row are again four consecutive
// floats.  Its A fragments come from A[M][K] as one 128-bit load along k per 8 k (lane half h: k0 + 4h .. + 3) or
// from A[K][M] as four 32-bit loads.  No operand passes through LDS and wavefronts never wait for each other in the
// K loop; each keeps a ring of D groups of 8 k in flight (D * 5 loads).  Nothing is reused between wavefronts except
// through the caches, which is right exactly where there is nothing to reuse: few rows (a dense layer at batch <= 64
// streams its weight matrix once) or a short K (its weight gradient streams the result once).
//
// Work: tile = (row group, column strip); the KW wavefronts of a workgroup of four split a tile's K range and add
// their accumulators through LDS in a fixed order; ksplit workgroups split K further, through partial sums in memory.
// Rows of B (and of a K-major A) past a wavefront's K range read as zeros: its buffer descriptors end at its last row.
//
// The ring is shallow on purpose.  A compute unit accepts about one 1 KB load per 25 ns, whatever the number of
// wavefronts that offer them, and a wavefront cannot compute while it waits to issue: with everything requested up
// front (8 wavefronts x 40 loads) the younger wavefront of each SIMD got its first load in after 4 us and its data in
// a burst at the end, and the MFMAs ran behind the stream instead of beside it (dense forward at batch 32, 4096 x
// 4096: 20.0 us with eight groups in flight, 18.1 with four; loads alone 14.7, both including a 4 us slice reduction).
// ---------------------------------------------------------------------------
struct WaveGemmArgs {
  const float* A;
  const float* B;
  float* C;              // the result, or with ksplit > 1 the partial sums [slice][M][N]
  int M, N, K, lda, ldb, ldc;
  long long sA, sB, sC;
  uint32_t bytesA, bytesC;
  int beta;
  int n_strips, tiles;   // tiles = row groups * strips of 128 columns
  int kchunk;            // K range of one wavefront, a multiple of 8
  int ksplit;
  PostOp post;
};

__device__ __forceinline__ void buf_store4(rsrc_t r, uint32_t off, f32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, (int)off, 0, 0);
}

template <bool TA, int MT, int KW, int D, bool PRE>
__global__ __launch_bounds__(256) void wave_gemm_kernel(WaveGemmArgs a) {
  constexpr int WAVES = 4;
  constexpr int TPW = WAVES / KW;   // tiles per workgroup
  __shared__ __attribute__((aligned(16))) float red[KW > 1 ? WAVES * 4096 : 4];
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int tl = wave / KW, kwi = wave - tl * KW;
  const int tile = (int)blockIdx.x * TPW + tl;
  const bool live = tile < a.tiles;
  const int mg = live ? tile / a.n_strips : 0, strip = live ? tile - mg * a.n_strips : 0;
  const int m0 = mg * (32 * MT), n0 = strip * 128;
  const long long bz = blockIdx.z;
  const int slice = (int)blockIdx.y;
  int kbeg = (slice * KW + kwi) * a.kchunk;
  int kend = kbeg + a.kchunk < a.K ? kbeg + a.kchunk : a.K;
  if (!live || kbeg >= a.K) { kbeg = 0; kend = 0; }
  const int ng = (kend - kbeg + 7) >> 3;

  const float* Ab = a.A + bz * a.sA;
  const float* Bb = a.B + bz * a.sB;
  // descriptors that end with the wavefront's last K row
  const rsrc_t rb = make_rsrc(Bb, kend > 0 ? ((uint32_t)(kend - 1) * (uint32_t)a.ldb + (uint32_t)a.N) * 4u : 0u);
  const rsrc_t ra = make_rsrc(Ab, !TA ? a.bytesA : (kend > 0 ? ((uint32_t)(kend - 1) * (uint32_t)a.lda + (uint32_t)a.M) * 4u : 0u));
  const bool col_ok = n0 + 4 * i < a.N;   // N % 4 == 0: a lane's four columns are in or out together
  uint32_t vb[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) vb[p] = col_ok ? (uint32_t)((4 * h + p) * a.ldb + n0 + 4 * i) * 4u : OOB;
  uint32_t va[MT][TA ? 4 : 1];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + 32 * mt + i;
    if (TA) {
#pragma unroll
      for (int p = 0; p < 4; ++p) va[mt][TA ? p : 0] = m < a.M ? (uint32_t)((4 * h + p) * a.lda + m) * 4u : OOB;
    } else {
      va[mt][0] = m < a.M ? (uint32_t)(m * a.lda + 4 * h) * 4u : OOB;
    }
  }

  f32x16 acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][j][r] = 0.0f;

  // '+=' straight into C: the old values are requested before the K loop and arrive during it
  const rsrc_t rc = make_rsrc(a.C + bz * a.sC + (a.ksplit > 1 ? (long long)slice * a.M * a.N : 0ll), a.bytesC);
  const int ldc = a.ksplit > 1 ? a.N : a.ldc;
  auto c_off = [&](int mt, int r) -> uint32_t {
    const int m = m0 + 32 * mt + 8 * (r >> 2) + 4 * h + (r & 3);
    return (m < a.M && col_ok && live) ? (uint32_t)(m * ldc + n0 + 4 * i) * 4u : OOB;
  };
  f32x4 old[PRE ? MT : 1][PRE ? 16 : 1];
  if (PRE) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) old[PRE ? mt : 0][PRE ? r : 0] = buf_load4(rc, c_off(mt, r));
  }

  f32x4 bq[D][4];
  f32x4 aq[D][MT];
  auto load = [&](auto dc, int k0) {
    constexpr int d = decltype(dc)::value;
    const uint32_t sb = (uint32_t)(k0 * a.ldb) * 4u;
#pragma unroll
    for (int p = 0; p < 4; ++p) bq[d][p] = buf_load4_s(rb, vb[p], sb);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (TA) {
        const uint32_t sa = (uint32_t)(k0 * a.lda) * 4u;
#pragma unroll
        for (int p = 0; p < 4; ++p) aq[d][mt][p] = buf_load_s(ra, va[mt][TA ? p : 0], sa);
      } else {
        aq[d][mt] = buf_load4_s(ra, va[mt][0], (uint32_t)k0 * 4u);
      }
    }
  };
  auto compute = [&](auto dc) {
    constexpr int d = decltype(dc)::value;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[mt][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[d][mt][p], bq[d][p][j], acc[mt][j], 0, 0, 0);
  };
  auto for_ring = [&](auto f) {
    f(ic<0>());
    if constexpr (D > 1) f(ic<1>());
    if constexpr (D > 2) f(ic<2>());
    if constexpr (D > 3) f(ic<3>());
    if constexpr (D > 4) f(ic<4>());
    if constexpr (D > 5) f(ic<5>());
    if constexpr (D > 6) f(ic<6>());
    if constexpr (D > 7) f(ic<7>());
    static_assert(D <= 8, "ring depth");
  };
  if (ng > 0) {
    // groups past the K range are requested like the others (B rows past it are zeros, A values there are never
    // used) so that every ring slot always has the same number of loads in flight
    for_ring([&](auto dc) { load(dc, kbeg + 8 * decltype(dc)::value); });
    int g = 0;
    for (; g + D <= ng; g += D)
      for_ring([&](auto dc) {
        compute(dc);
        load(dc, kbeg + 8 * (g + D + decltype(dc)::value));
      });
    for_ring([&](auto dc) {
      if (g + decltype(dc)::value < ng) compute(dc);
    });
  }

  if constexpr (KW == 1) {
    f32x4 bias = {0.0f, 0.0f, 0.0f, 0.0f};
    const bool post = a.ksplit == 1 && a.post.any();
    if (post && a.post.bias != nullptr && col_ok) bias = *reinterpret_cast<const f32x4*>(a.post.bias + n0 + 4 * i);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        f32x4 v = {acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]};
        const uint32_t off = c_off(mt, r);
        if (PRE) {
          v += old[PRE ? mt : 0][PRE ? r : 0];
        } else if (a.beta && a.ksplit == 1) {
          v += buf_load4(rc, off);
        } else if (post) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = a.post.apply(v[q], bias[q]);
        }
        buf_store4(rc, off, v);
      }
  } else {
    // the KW wavefronts of a tile park their accumulators in LDS, tile row by tile row, and all threads of the
    // workgroup add them up in wavefront order and store: one group of 32 rows per round
    const int t = (int)threadIdx.x;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (mt > 0) __syncthreads();
      float* mine = red + wave * 4096;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * h + (r & 3);
        const f32x4 v = {acc[mt][0][r], acc[mt][1][r], acc[mt][2][r], acc[mt][3][r]};
        *reinterpret_cast<f32x4*>(&mine[row * 128 + 4 * i]) = v;
      }
      __syncthreads();
#pragma unroll
      for (int q = 0; q < 1024 * TPW / (WAVES * 64); ++q) {
        const int e = t + WAVES * 64 * q, tq = e >> 10, rem = e & 1023, row = rem >> 5, c4 = rem & 31;
        f32x4 s = *reinterpret_cast<const f32x4*>(&red[(tq * KW) * 4096 + row * 128 + 4 * c4]);
#pragma unroll
        for (int k = 1; k < KW; ++k) s += *reinterpret_cast<const f32x4*>(&red[(tq * KW + k) * 4096 + row * 128 + 4 * c4]);
        const int tile_q = (int)blockIdx.x * TPW + tq;
        const int mgq = tile_q / a.n_strips, sq = tile_q - mgq * a.n_strips;
        const int m = mgq * (32 * MT) + 32 * mt + row, n = sq * 128 + 4 * c4;
        const uint32_t off = (tile_q < a.tiles && m < a.M && n < a.N) ? (uint32_t)(m * ldc + n) * 4u : OOB;
        if (a.ksplit == 1) {
          if (a.beta) {
            s += buf_load4(rc, off);
          } else if (a.post.any()) {
            f32x4 bias = {0.0f, 0.0f, 0.0f, 0.0f};
            if (a.post.bias != nullptr && n < a.N) bias = *reinterpret_cast<const f32x4*>(a.post.bias + n);
#pragma unroll
            for (int c = 0; c < 4; ++c) s[c] = a.post.apply(s[c], bias[c]);
          }
        }
        buf_store4(rc, off, s);
      }
    }
  }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Whether the wavefront-tile kernel serves this product, and with which split.
struct WavePlan {
  bool use;
  int mt, kw, ksplit, kchunk, tiles, n_strips;
};
static WavePlan plan_wave(const DeviceCtx* ctx, int ta, int tb, int batch, int M, int N, int K, const float* A, int lda,
                          long long sA, const float* B, int ldb, long long sB, const float* C, int ldc, long long sC,
                          const PostOp& post) {
  WavePlan w{false, 1, 1, 1, 8, 0, 0};
  if (tb) return w;
  // 128-bit accesses of B rows and C rows (and of the bias), and of A along k when A is K-contiguous
  if (!aligned16(B) || ldb % 4 || sB % 4 || N % 4 || !aligned16(C) || ldc % 4 || sC % 4) return w;
  if (post.bias != nullptr && !aligned16(post.bias)) return w;
  if (!ta && (!aligned16(A) || lda % 4 || sA % 4 || K % 8)) return w;
  // the K advance travels in 32-bit byte offsets, up to a ring of groups of 8 rows past the end
  const uint64_t ld_max = (uint64_t)(lda > ldb ? lda : ldb);
  if (((uint64_t)K + 8 * 9) * ld_max * 4 >= 0x7fffffffull) return w;
  const bool few_rows = !ta && M <= 64 && (long long)N * K >= 1 << 16;   // dense layer, small batch
  const bool short_k = ta && K <= 64 && (long long)M * N >= 1 << 16;     // its weight gradient
  if (!few_rows && !short_k) return w;
  w.mt = (!ta && M > 32) ? 2 : 1;
  w.n_strips = (N + 127) / 128;
  const long long tiles = (long long)((M + 32 * w.mt - 1) / (32 * w.mt)) * w.n_strips;
  if (tiles * batch > 0x3fffffffll || batch > 65535) return w;
  w.tiles = (int)tiles;
  // enough wavefronts for four per compute unit (few rows) or eight (short K: two workgroups per compute unit, one
  // storing while the other computes), each with at least 16 k
  const long long want = (few_rows ? 4ll : 8ll) * ctx->cus;
  long long kws = tiles * batch >= want ? 1 : want / (tiles * batch);
  if (kws > K / 16) kws = K / 16;
  if (kws < 1) kws = 1;
  w.kw = kws >= 4 ? 4 : (kws >= 2 ? 2 : 1);
  long long ks = batch == 1 ? kws / w.kw : 1;   // slices through memory only without a batch
  if (ks < 1) ks = 1;
  const long long parts = ks * w.kw;
  long long chunk = ((K + parts - 1) / parts + 7) & ~7ll;
  w.kchunk = (int)chunk;
  w.ksplit = (int)((K + chunk * w.kw - 1) / (chunk * w.kw));
  w.use = true;
  return w;
}

template <bool TA, int MT>
static void launch_wave_kw(DeviceCtx* ctx, const WaveGemmArgs& a, const WavePlan& w, int batch, bool pre) {
  const int tpw = 4 / w.kw;
  dim3 g((w.tiles + tpw - 1) / tpw, w.ksplit, batch), b(256, 1, 1);
  constexpr int D = 4;
  if constexpr (TA) {
    // short K: the old values of a '+=' are requested ahead of the K loop
    if (w.kw == 4) hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 4, D, false>), g, b, 0, ctx->stream, a);
    else if (w.kw == 2) hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 2, D, false>), g, b, 0, ctx->stream, a);
    else if (pre) hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 1, D, true>), g, b, 0, ctx->stream, a);
    else hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 1, D, false>), g, b, 0, ctx->stream, a);
  } else {
    if (w.kw == 4) hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 4, D, false>), g, b, 0, ctx->stream, a);
    else if (w.kw == 2) hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 2, D, false>), g, b, 0, ctx->stream, a);
    else hipLaunchKernelGGL((wave_gemm_kernel<TA, MT, 1, D, false>), g, b, 0, ctx->stream, a);
  }
}

static int launch_wave(DeviceCtx* ctx, const WavePlan& w, int ta, int batch, int M, int N, int K, const float* A, int lda,
                       long long sA, const float* B, int ldb, long long sB, float* C, int ldc, long long sC, int beta,
                       uint32_t bytesA, uint32_t bytesC, const PostOp& post) {
  WaveGemmArgs a;
  a.A = A; a.B = B; a.C = C;
  a.M = M; a.N = N; a.K = K; a.lda = lda; a.ldb = ldb; a.ldc = ldc;
  a.sA = sA; a.sB = sB; a.sC = sC;
  a.bytesA = bytesA; a.bytesC = bytesC;
  a.beta = beta;
  a.n_strips = w.n_strips; a.tiles = w.tiles; a.kchunk = w.kchunk; a.ksplit = w.ksplit;
  a.post = post;
  if (w.ksplit > 1) {
    const int st = ensure_workspace(ctx, (size_t)w.ksplit * M * N * sizeof(float));
    if (st != LNN_OK) return st;
    a.C = static_cast<float*>(ctx->ws);
    a.bytesC = (uint32_t)M * (uint32_t)N * 4u;
    a.sC = 0;
  }
  const bool pre = beta && w.kw == 1 && w.ksplit == 1;
  if (ta) {
    launch_wave_kw<true, 1>(ctx, a, w, batch, pre);
  } else if (w.mt == 2) {
    launch_wave_kw<false, 2>(ctx, a, w, batch, false);
  } else {
    launch_wave_kw<false, 1>(ctx, a, w, batch, pre);
  }
  LNN_HIP(hipGetLastError());
  if (w.ksplit > 1) return launch_gemm_reduce(ctx, a.C, w.ksplit, M, N, C, ldc, beta, post);
  return LNN_OK;
}

// ---------------------------------------------------------------------------
// K and N of a handful: C[b][m][0..N) (+)= A[b][m][0..K) . op(B[b]), one output row per thread.  The rank-3 products
// of a spatial transform ([N, H*W, 3] . [N, 3, 2] and its data gradient) are pure streaming of A and C; an MFMA
// tile would spend 32 k and 32 columns on 3 and 2.  B is the same for the whole block: it travels in scalar registers.
// ---------------------------------------------------------------------------
constexpr int kSmallMax = 8;
struct SmallArgs {
  const float* A;
  const float* B;
  float* C;
  int M, N, K, lda, ldb, ldc, tb, beta;
  long long sA, sB, sC;
  PostOp post;
};
__global__ __launch_bounds__(256) void small_kn_kernel(SmallArgs a) {
  const long long bz = blockIdx.y;
  const float* __restrict__ A = a.A + bz * a.sA;
  const float* __restrict__ B = a.B + bz * a.sB;
  float* __restrict__ C = a.C + bz * a.sC;
  const int m = (int)blockIdx.x * 256 + (int)threadIdx.x;
  if (m >= a.M) return;
  float x[kSmallMax], acc[kSmallMax];
#pragma unroll
  for (int k = 0; k < kSmallMax; ++k) x[k] = k < a.K ? A[(size_t)m * a.lda + k] : 0.0f;
#pragma unroll
  for (int n = 0; n < kSmallMax; ++n) acc[n] = 0.0f;
#pragma unroll
  for (int k = 0; k < kSmallMax; ++k)
    if (k < a.K) {
#pragma unroll
      for (int n = 0; n < kSmallMax; ++n)
        if (n < a.N) acc[n] = fmaf(x[k], a.tb ? B[n * a.ldb + k] : B[k * a.ldb + n], acc[n]);
    }
#pragma unroll
  for (int n = 0; n < kSmallMax; ++n)
    if (n < a.N) {
      float* dst = C + (size_t)m * a.ldc + n;
      float v = acc[n];
      if (a.beta) v += *dst;
      else if (a.post.any()) v = a.post.apply(v, a.post.bias != nullptr ? a.post.bias[n] : 0.0f);
      *dst = v;
    }
}

int launch_gemm(DeviceCtx* ctx, int ta, int tb, int batch, int M, int N, int K, const float* A, int lda,
                long long sA, const float* B, int ldb, long long sB, float* C, int ldc, long long sC, int beta,
                const float* bias, int act, float slope) {
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
  const PostOp post{bias, act, slope, 1};
  if (beta && post.any()) return set_error(LNN_ERR_INVALID, "gemm: bias / activation cannot be combined with accumulation");
  if (ta && tb) return set_error(LNN_ERR_UNSUPPORTED, "gemm: trans_a and trans_b together are not provided");

  if (!ta && K <= kSmallMax && N <= kSmallMax && M >= 256) {
    SmallArgs s;
    s.A = A; s.B = B; s.C = C; s.M = M; s.N = N; s.K = K; s.lda = lda; s.ldb = ldb; s.ldc = ldc; s.tb = tb ? 1 : 0;
    s.beta = beta ? 1 : 0; s.sA = sA; s.sB = sB; s.sC = sC; s.post = post;
    hipLaunchKernelGGL(small_kn_kernel, dim3((M + 255) / 256, batch), dim3(256), 0, ctx->stream, s);
    LNN_HIP(hipGetLastError());
    return LNN_OK;
  }

  const WavePlan w = plan_wave(ctx, ta, tb, batch, M, N, K, A, lda, sA, B, ldb, sB, C, ldc, sC, post);
  if (w.use)
    return launch_wave(ctx, w, ta, batch, M, N, K, A, lda, sA, B, ldb, sB, C, ldc, sC, beta ? 1 : 0, (uint32_t)bytesA,
                       (uint32_t)bytesC, post);

  GemmArgs a;
  a.A = A; a.B = B; a.C = C;
  a.M = M; a.N = N; a.K = K;
  a.lda = lda; a.ldb = ldb; a.ldc = ldc;
  a.sA = sA; a.sB = sB; a.sC = sC;
  a.bytesA = (uint32_t)bytesA; a.bytesB = (uint32_t)bytesB; a.bytesC = (uint32_t)bytesC;
  a.beta = beta ? 1 : 0;
  a.post = post;
  // 128-bit loads run along K for a K-contiguous operand and along the rows
  // for a row-contiguous one; both the extent and every row start must be
  // multiples of four floats.
  const bool va = aligned16(A) && lda % 4 == 0 && sA % 4 == 0 && a_cols % 4 == 0;
  const bool vb = aligned16(B) && ldb % 4 == 0 && sB % 4 == 0 && b_cols % 4 == 0;
  const int mode = (va && vb) ? (K % BK == 0 ? 2 : 1) : 0;
  if (!ta && !tb) return launch_layout<false, false>(ctx, a, batch, mode);
  if (!ta && tb) return launch_layout<false, true>(ctx, a, batch, mode);
  return launch_layout<true, false>(ctx, a, batch, mode);
}

}  // namespace lnn
