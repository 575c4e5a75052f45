// Implicit-GEMM convolution passes on the MFMA tile engine: what the three passes share (argument block, gather
// tables, weight permutation, split-K slice reduction, the kernel template and its host-side planning).  Nothing is
// unfolded to memory: the loaders compute im2col addresses on the fly and the epilogue writes NCHW directly.
//
//   forward  Y [O  x P ] = W[O x CKK]        . im2col(X)[CKK x P]     P = N*OH*OW
//   dgrad    dX[C  x Q ] = Wt[C x O*KK]      . im2rowT(dY)[O*KK x Q]  Q = N*IH*IW
//   wgrad    dW[O  x CKK] = dY[O x P]        . im2row(X)[P x CKK]     (split over P)
//
// Included by conv_fwd.hip, conv_dgrad.hip and conv_wgrad.hip, one translation unit per pass so that they compile
// side by side; everything here has internal linkage (each unit carries its own copy of the small helper kernels).
#pragma once
#include <algorithm>
#include <vector>

#include "common.hpp"
#include "slice_reduce.hpp"


namespace lnn {
namespace {

struct ConvArgs {
  ConvGeom g;
  const float* X;    // fwd: X, dgrad: dY, wgrad: X
  const float* W;    // fwd: W, dgrad: W,  wgrad: dY
  float* Out;        // fwd: Y, dgrad: dX, wgrad: dW or the partial-sum buffer
  const KEntry* tab;
  uint32_t bytesX, bytesW, bytesOut;
  int M, Ncols, K;   // GEMM extents
  int beta;
  int n_units, total_units;
  int grid_x;        // workgroups along x that belong to this problem (a batched launch may have more)
  int ksplit;        // wgrad: number of K slices (tap-major: of every chunk but the last)
  PostOp post;       // forward only: bias / activation of the stored result
  size_t ws_used;    // bytes at the front of the scratch buffer that hold this call's permuted weights
  int n_chunks, ks_last;   // tap-major wgrad: chunks of chunk_units units; K slices of the last, possibly shorter one
  FastDiv dC;        // tap-major wgrad: divide a column index by the channel count
  int chunk_units;   // tap-major wgrad: units per workgroup
  // dgrad: g describes one pixel class (g.IH, g.IW = class grid); the plane it is cut from:
  int full_IW, full_IHW, cls_org, cls_s;
  int w_iohw;        // wgrad: dW is stored [C][O][KH][KW]
  // tap-major wgrad: the columns of an M tile form segs_per_mt segments of seg_units units; a group's columns stay
  // inside one segment (one tap, for the loaders that assume it; the whole row for the one that does not)
  int seg_units, segs_per_mt;
  // tap-major wgrad with equal K shares (eq_wgs > 0): the K steps of all chunks laid end to end are cut into eq_wgs
  // equal runs, one per workgroup, each shorter than a chunk's K: a run ends in the middle of a chunk and may go on
  // at the beginning of the next.  Workgroup w stores the sums of its first piece as a [BM][chunk width] block at
  // Out[2w] and of its second at Out[2w + 1]; the slice reduction adds up the blocks of the workgroups that touch
  // a chunk, in workgroup order.  (ksplit = 2 then only says "partial sums".)
  int eq_wgs;
  // ... and the order in which the chunks are laid end to end: place q holds chunk (q % eq_d) * eq_g + q / eq_d
  // (eq_d = 0: chunk q).  See plan_equal_shares.
  int eq_d, eq_g;
  // forward / dgrad without a K split: units that do not divide evenly among the workgroups.  The first main_units
  // units (a whole number per workgroup) are computed as usual; each of the tail_units left over is cut into
  // tail_split K slices, one per workgroup, whose partial sums go to tail_part[slice][unit][BM][unit width] and are
  // added up by reduce_tail.  tail_units = 0: no tail.
  int main_units, tail_units, tail_split;
  float* tail_part;
};

// One class of input pixels of a strided dgrad: pixels (h0 + S*i, w0 + S*j),
// fed by the taps with kh*D = rh (mod S) and kw*D = rw (mod S).
struct PixelClass {
  int rh, rw, h0, w0, nkh, nkw;
};
// the j-th k in [0, n) with k*D = r (mod S)
__host__ __device__ inline int nth_tap(int n, int D, int S, int r, int j) {
  for (int k = 0; k < n; ++k)
    if (k * D % S == r && j-- == 0) return k;
  return -1;
}

// mode 0: k = (c, kh, kw) for forward / wgrad.
// mode 1: dgrad, k = (o, tap of the class); mode 2: dgrad, one entry per tap of the class (tap-major K).
__global__ void build_ktable(KEntry* tab, int K, int Kpad, int mode, ConvGeom g, PixelClass pc) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k >= Kpad) return;
  KEntry e;
  e.x = 0;
  e.y = BIG;
  e.z = 0;
  e.w = 0x20000000;
  if (k < K) {
    if (mode == 0) {
      const int ch = k / g.KK, tap = k - ch * g.KK, kh = tap / g.KW, kw = tap - kh * g.KW;
      e.y = kh * g.D;
      e.z = kw * g.D;
      e.x = ch * g.IHW + kh * g.D * g.IW + kw * g.D;
      e.w = 0;
    } else {
      const int nt = pc.nkh * pc.nkw;
      const int ch = mode == 1 ? k / nt : 0, t = mode == 1 ? k - ch * nt : k;
      const int jh = t / pc.nkw, jw = t - jh * pc.nkw;
      const int kh = nth_tap(g.KH, g.D, g.S, pc.rh, jh), kw = nth_tap(g.KW, g.D, g.S, pc.rw, jw);
      e.y = (kh * g.D - g.PADT - pc.h0) / g.S;   // exact by the definition of the class
      e.z = (kw * g.D - g.PADL - pc.w0) / g.S;
      e.x = ch * g.OHW;
      e.w = ch * g.C * g.KK + kh * g.KW + kw;
    }
  }
  tab[k] = e;
}

// *_TAP: tap-major K order over channel-permuted weights (channels % BK == 0)
// PASS_WGRAD_TAP4: PASS_WGRAD_TAP with 128-bit transfers of the pixel gather too (stride 1, OW % 4 == 0, no padded columns)
// PASS_FWD_ANYC: forward for any channel count (gather table), both operands straight into LDS, three stages
// PASS_WGRAD_ANYC: wgrad for any channel count with transfers straight into LDS; a group's columns may span taps
// PASS_DGRAD_TAPW: tap-major dgrad that reads the weights in the forward pass's permuted layout (C % 4 == 0)
enum { PASS_DGRAD = 1, PASS_WGRAD = 2, PASS_FWD_TAP = 3, PASS_DGRAD_TAP = 4, PASS_WGRAD_TAP = 5, PASS_WGRAD_TAP4 = 6,
       PASS_DGRAD_TAPW = 7, PASS_WGRAD_ANYC = 8, PASS_FWD_ANYC = 9 };
// the weight-gradient passes whose GEMM columns are tap-major (column tap*C + c)
constexpr bool wgrad_tap(int pass) { return pass == PASS_WGRAD_TAP || pass == PASS_WGRAD_TAP4 || pass == PASS_WGRAD_ANYC; }
constexpr bool dgrad_tap(int pass) { return pass == PASS_DGRAD_TAP || pass == PASS_DGRAD_TAPW; }

// Wp[a][tap][b] = W[..] so that the tap-major K index tap*CH + ch is contiguous:
//   mode 0 (forward, and the data gradient when C % 4 == 0): Wp[o][tap][c] = W[o][c][tap]
//   mode 2: the same from weights stored with their channel axes swapped, W[c][o][tap] (a transposed
//           convolution keeps its kernel that way)
//   mode 1 (dgrad, other C): Wp[c][t][o] = W[o][c][tap_t], t over the taps of the pixel class
__device__ __forceinline__ void permute_one(float* wp, const float* w, int O, int C, int KK, int mode, const ConvGeom& g,
                                            const PixelClass& pc, int i) {
  if (mode == 0 || mode == 2) {
    if (i >= O * C * KK) return;
    const int b = i % C, tap = (i / C) % KK, a = i / (C * KK);
    wp[i] = mode == 0 ? w[((size_t)a * C + b) * KK + tap] : w[((size_t)b * O + a) * KK + tap];
  } else {
    const int nt = pc.nkh * pc.nkw;
    if (i >= O * C * nt) return;
    const int b = i % O, t = (i / O) % nt, a = i / (O * nt);
    const int jh = t / pc.nkw, jw = t - jh * pc.nkw;
    const int tap = nth_tap(g.KH, g.D, g.S, pc.rh, jh) * g.KW + nth_tap(g.KW, g.D, g.S, pc.rw, jw);
    wp[i] = w[((size_t)b * C + a) * KK + tap];
  }
}
__global__ void permute_weights(float* wp, const float* w, int O, int C, int KK, int mode, ConvGeom g, PixelClass pc) {
  permute_one(wp, w, O, C, KK, mode, g, pc, blockIdx.x * blockDim.x + threadIdx.x);
}
// Modes 0 and 2 through LDS: a block moves 64 channels of one output row, so that its reads and its writes both run
// along contiguous floats (the element-wise kernel above reads with a stride of KK floats, or of O * KK).
constexpr int kPermuteMaxKK = 200;   // 64 * (KK | 1) floats of LDS
__global__ __launch_bounds__(256) void permute_weights_tiled(float* wp, const float* w, int O, int C, int KK, int mode) {
  extern __shared__ float permute_tile[];
  const int kkp = KK | 1;   // odd row pitch: the transposed reads spread over the banks
  const int cblocks = (C + 63) / 64;
  const int o = blockIdx.x / cblocks, c0 = (blockIdx.x - o * cblocks) * 64;
  const int nc = C - c0 < 64 ? C - c0 : 64;
  const int n = nc * KK;
  const float* src = w + ((size_t)o * C + c0) * KK;
  for (int j = threadIdx.x; j < n; j += 256) {
    const int cl = j / KK, tap = j - cl * KK;
    permute_tile[cl * kkp + tap] = mode == 0 ? src[j] : w[((size_t)(c0 + cl) * O + o) * KK + tap];
  }
  __syncthreads();
  for (int j = threadIdx.x; j < 64 * KK; j += 256) {
    const int tap = j >> 6, cl = j & 63;
    if (cl < nc) wp[((size_t)o * KK + tap) * C + c0 + cl] = permute_tile[cl * kkp + tap];
  }
}
// mode 1 for up to four pixel classes at once: blockIdx.y = class
struct PermuteBatch {
  float* wp[4];
  PixelClass pc[4];
};
__global__ void permute_weights_classes(PermuteBatch b, const float* w, int O, int C, int KK, ConvGeom g) {
  permute_one(b.wp[blockIdx.y], w, O, C, KK, 1, g, b.pc[blockIdx.y], blockIdx.x * blockDim.x + threadIdx.x);
}

template <int PASS, int WM, int NTMAX, bool FLAG>
struct ConvCfg {
  static constexpr int WN = 4 / WM, BM = 32 * WM, BNMAX = 32 * WN * 2 * NTMAX;
  // the tap-major passes send both operands straight into unpadded LDS tiles, three stages deep
  static constexpr bool DIRECT = PASS == PASS_FWD_TAP || PASS == PASS_FWD_ANYC || dgrad_tap(PASS) || wgrad_tap(PASS);
  // A side is K-contiguous in LDS for all passes.
  static constexpr int SA = DIRECT ? BM * BK : LdsSize<true, BM>::value;
  // B side: pixel-contiguous gathers (fwd, dgrad) or K-contiguous (wgrad).
  static constexpr int SB = DIRECT ? BNMAX * BK : LdsSize<PASS == PASS_WGRAD, BNMAX>::value;
  static constexpr int STAGES = DIRECT ? 3 : 2;
};

// Loader selection and initialisation per pass.  FLAG:
//   PASS_WGRAD(_TAP) 128-bit loads of dY (OHW % 4 == 0)
template <int PASS, bool FLAG, int ST>
struct ConvProblem;

struct ConvProblemBase {
  ConvGeom g;
  const KEntry* tab;
  rsrc_t rx, rw, rc;
  int M, Ncols, K, kbeg, kend, beta;
  OutMap om;
  PostOp post;
};

template <bool FLAG, int ST>
struct ConvProblem<PASS_FWD_ANYC, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  // few channels mean few K steps per sub-tile (a 7x7 stem on RGB: 5), each short: the transfers need the extra
  // step in flight
  static constexpr bool REQUEST_FIRST = true;
  template <int R> using LA = DirectKC4<R>;
  template <int R> using LB = ConvFwdBDirect<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, K, row0, M, K); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, tab, col0, Ncols, kbeg); }
};
template <bool FLAG, int ST>
struct ConvProblem<PASS_FWD_TAP, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  template <int R> using LA = ConvFwdATap<R>;            // permuted weights [O][KK*C]
  template <int R> using LB = ConvFwdBTap<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, row0, M, kbeg); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, col0, Ncols, kbeg); }
};
template <bool FLAG, int ST>
struct ConvProblem<PASS_DGRAD, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  template <int R> using LA = ConvDgradA<R>;
  template <int R> using LB = ConvDgradB<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, tab, row0, kbeg); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, tab, col0, Ncols, kbeg); }
};
template <bool FLAG, int ST>
struct ConvProblem<PASS_DGRAD_TAP, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  template <int R> using LA = DirectKC<R>;               // permuted weights [C][taps*O]
  template <int R> using LB = ConvDgradBTap<R, false>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, K, row0, M, K); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, tab, col0, Ncols, kbeg); }
};
template <bool FLAG, int ST>
struct ConvProblem<PASS_DGRAD_TAPW, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  template <int R> using LA = ConvDgradATapMC<R>;        // the forward pass's permuted weights [O][KK*C]
  template <int R> using LB = ConvDgradBTap<R, true>;
  // K = O * (taps of the pixel class)
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, tab, row0, kbeg, K / g.O); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, tab, col0, Ncols, kbeg, K / g.O); }
};
template <bool FLAG, int ST>
struct ConvProblem<PASS_WGRAD, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  template <int R> using LA = ConvWgradA<R, FLAG>;
  template <int R> using LB = ConvWgradB<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, row0, kend); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A&) const { l.init(rx, g, tab, col0, Ncols, kend); }
};

template <bool FLAG, int ST>
struct ConvProblem<PASS_WGRAD_TAP, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  static constexpr bool STREAM_UNROLL = false;   // measured: slower with constant stages (config 3: 0.235 -> 0.247 ms)
  static constexpr bool STREAM_REGIONS = true;
  template <int R> using LA = typename std::conditional<FLAG, ConvWgradTapA4Direct<R>, ConvWgradTapADirect<R>>::type;
  template <int R> using LB = ConvWgradTapBDirect<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, row0, kend, kbeg); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A& la) const { l.init(rx, g, col0, la, kend, kbeg); }
};

template <bool FLAG, int ST>
struct ConvProblem<PASS_WGRAD_ANYC, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  static constexpr bool STREAM_UNROLL = false;   // measured: slower with constant stages (config 3: 0.235 -> 0.247 ms)
  static constexpr bool STREAM_REGIONS = true;
  template <int R> using LA = typename std::conditional<FLAG, ConvWgradTapA4Direct<R>, ConvWgradTapADirect<R>>::type;
  template <int R> using LB = ConvWgradBAnyC<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, row0, kend, kbeg); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A& la) const { l.init(rx, g, col0, Ncols, la, kend, kbeg); }
};

template <bool FLAG, int ST>
struct ConvProblem<PASS_WGRAD_TAP4, FLAG, ST> : ConvProblemBase {
  static constexpr int STAGES = ST;
  static constexpr bool STREAM_UNROLL = false;   // measured: slower with constant stages (config 3: 0.235 -> 0.247 ms)
  static constexpr bool STREAM_REGIONS = true;
  template <int R> using LA = ConvWgradTapA4Direct<R>;
  template <int R> using LB = ConvWgradTapB4Direct<R>;
  template <int R> __device__ __forceinline__ void init_a(LA<R>& l, int row0) const { l.init(rw, g, row0, kend, kbeg); }
  template <int R, class A> __device__ __forceinline__ void init_b(LB<R>& l, int col0, A& la) const { l.init(rx, g, col0, la, kend, kbeg); }
};

// Where GEMM element (m, column) of a pass lives in its output tensor.
__host__ __device__ inline OutMap plain_map(int ncols) {
  OutMap om;
  om.nchw = 0; om.ld = ncols; om.mtot = 0; om.dHW = FastDiv{0, 0, 1};
  om.dCW = FastDiv{0, 0, 1}; om.s = 0; om.iw = 0; om.org = 0;
  return om;
}
template <int PASS>
__host__ __device__ inline OutMap final_map(const ConvArgs& a) {
  OutMap om = plain_map(a.Ncols);
  if (PASS == PASS_FWD_TAP || PASS == PASS_FWD_ANYC) {
    om.nchw = 1; om.ld = a.g.OHW; om.mtot = a.g.O; om.dHW = a.g.dOHW;
  } else if (PASS == PASS_DGRAD || dgrad_tap(PASS)) {
    om.nchw = 3; om.ld = a.full_IHW; om.mtot = a.g.C; om.dHW = a.g.dIHW;
    om.dCW = a.g.dIW; om.s = a.cls_s; om.iw = a.full_IW; om.org = a.cls_org;
  } else if (wgrad_tap(PASS)) {
    // GEMM column tap*C + c lands in dW[o][c][tap], or in dW[c][o][tap] for a gradient kept with swapped channel axes
    om.nchw = 2; om.ld = a.Ncols; om.mtot = a.g.KK; om.dHW = a.dC;
    if (a.w_iohw) { om.ld = a.g.KK; om.mtot = a.g.O * a.g.KK; }
  }
  return om;
}

// (bx, by): this workgroup's position in the problem's own grid (x: share of the output, y: K slice)
// Consecutive workgroups of a launch go to the eight XCDs in turn, each with its own L2.  For workgroup b of n
// (counted from a workgroup that went to any XCD) this returns an index in [0, n) such that the workgroups of one XCD
// hold a contiguous range of indices: work items that share operands are numbered side by side and then meet in one L2.
__device__ __forceinline__ int xcd_contiguous(int b, int n) {
  const int x = b & 7, i = b >> 3, q = n >> 3, r = n & 7;
  return x * q + (x < r ? x : r) + i;
}

template <int PASS, int WM, int NTMAX, bool FLAG>
__device__ __forceinline__ void conv_body(const ConvArgs& a, int bx, int by) {
  using Cfg = ConvCfg<PASS, WM, NTMAX, FLAG>;
  __shared__ __attribute__((aligned(16))) float lds[Cfg::STAGES * (Cfg::SA + Cfg::SB)];
  ConvProblem<PASS, FLAG, Cfg::STAGES> p;
  p.g = a.g;
  p.tab = a.tab;
  p.rx = make_rsrc(a.X, a.bytesX);
  p.rw = make_rsrc(a.W, a.bytesW);
  p.M = a.M; p.Ncols = a.Ncols; p.K = a.K; p.beta = a.beta;
  p.kbeg = 0;
  p.kend = a.K;
  float* out = a.Out;
  int chunk_i = bx;
  const bool eq = wgrad_tap(PASS) && a.eq_wgs > 0;
  if (a.ksplit > 1 && !eq) {
    // K slice of this workgroup: slices are in gridDim.y, except that the tap-major wgrad pass has a flat
    // grid in which the last chunk, if it holds less work, is cut into proportionally fewer slices
    int slice = by, ns = a.ksplit;
    if (wgrad_tap(PASS)) {
      // The chunks of one K slice read the same pixels (the same dY, and X windows a few rows apart), so the full
      // chunks' workgroups are taken slice by slice and every XCD gets a contiguous run of that order: the chunks of
      // a slice run side by side on one XCD (two, where a run ends inside a slice) and meet their operands in its L2
      // (3x3 dilated on 64 channels, 9 tap columns in 5 chunks: 162 -> 78 MB fetched per launch; the time does not move).
      const int b = bx, nc = a.n_chunks - 1, nfull = nc * a.ksplit;
      if (b < nfull) {
        const int j = xcd_contiguous(b, nfull);
        slice = j / nc;
        chunk_i = j - slice * nc;
      } else {
        chunk_i = a.n_chunks - 1;
        slice = b - nfull;
        ns = a.ks_last;
      }
    }
    const int nkt = (a.K + BK - 1) / BK;
    const int t0 = (int)((long long)nkt * slice / ns);
    const int t1 = (int)((long long)nkt * (slice + 1) / ns);
    p.kbeg = t0 * BK;
    p.kend = t1 * BK < a.K ? t1 * BK : a.K;
    out += (size_t)slice * a.M * a.Ncols;
  }
  p.rc = make_rsrc(out, a.bytesOut);
  // split-K partials stay in GEMM order (coalesced); the slice reduction applies the final mapping
  p.om = a.ksplit > 1 ? plain_map(a.Ncols) : final_map<PASS>(a);
  p.post = a.post;
  if (a.ksplit > 1) { p.post.bias = nullptr; p.post.act = 0; }   // applied by the slice reduction
  if (wgrad_tap(PASS)) {
    // one chunk over one K slice - or, with equal K shares, this workgroup's run of the end-to-end K steps, piece
    // by piece: the rest of the chunk it begins in, whole chunks, the beginning of the chunk it ends in
    const int nkt = (a.K + BK - 1) / BK;
    long long s0 = 0, s1 = 1;
    const int run = bx;
    if (eq) {
      const long long T = (long long)a.n_chunks * nkt;
      s0 = T * run / a.eq_wgs;
      s1 = T * (run + 1) / a.eq_wgs;
    }
    int piece = 0;
    while (s0 < s1) {
      long long adv = 1;
      if (eq) {
        constexpr int WN = 4 / WM, BM = 32 * WM;
        const int place = (int)(s0 / nkt);
        chunk_i = a.eq_d > 0 ? (place % a.eq_d) * a.eq_g + place / a.eq_d : place;
        const int t0 = (int)(s0 - (long long)place * nkt);
        const int t1 = s1 - s0 < nkt - t0 ? t0 + (int)(s1 - s0) : nkt;
        p.kbeg = t0 * BK;
        p.kend = t1 * BK < a.K ? t1 * BK : a.K;
        // element (m, n) of the chunk at (m - mt*BM) * CW + (n - n0) of the piece's block: a plain map of pitch CW
        // over a buffer that begins that much before the block
        const int CW = a.chunk_units * 32 * WN, per_mt = a.seg_units * a.segs_per_mt;
        const int u0 = chunk_i * a.chunk_units, mt = u0 / per_mt, n0 = (u0 - mt * per_mt) * 32 * WN;
        const int shift = mt * BM * CW + n0;
        p.rc = make_rsrc(a.Out + (size_t)(2 * run + piece) * (BM * CW) - shift, (uint32_t)(shift + BM * CW) * 4u);
        p.om = plain_map(CW);
        adv = t1 - t0;
        ++piece;
      }
      walk_units_seg<WM, NTMAX>(p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, a.seg_units, a.segs_per_mt,
                                a.total_units, a.chunk_units, chunk_i, eq ? a.chunk_units >> 1 : NTMAX);
      s0 += adv;
    }
  } else if (a.tail_units == 0) {
    walk_units<WM, NTMAX>(p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, a.n_units, a.total_units,
                          bx, a.grid_x);
  } else {
    walk_units<WM, NTMAX>(p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, a.n_units, a.main_units,
                          bx, a.grid_x);
    if (bx < a.tail_units * a.tail_split) {
      constexpr int WN = 4 / WM, BM = 32 * WM, UW = 32 * WN;
      const int j = bx / a.tail_split, slice = bx - j * a.tail_split;
      const int u = a.main_units + j, mt = u / a.n_units, n0 = (u - mt * a.n_units) * UW;
      const int nkt = (a.K + BK - 1) / BK;
      const int t0 = (int)((long long)nkt * slice / a.tail_split), t1 = (int)((long long)nkt * (slice + 1) / a.tail_split);
      p.kbeg = t0 * BK;
      p.kend = t1 * BK < a.K ? t1 * BK : a.K;
      // element (m, n) of the unit at (m - mt*BM) * UW + (n - n0) of its block: a plain map of pitch UW over a
      // buffer that begins that much before the block
      const int shift = mt * BM * UW + n0;
      p.rc = make_rsrc(a.tail_part + (size_t)(slice * a.tail_units + j) * (BM * UW) - shift, (uint32_t)(shift + BM * UW) * 4u);
      p.om = plain_map(UW);
      p.beta = 0;
      p.post.bias = nullptr; p.post.act = 0;   // applied by reduce_tail
      run_pair<WM, NTMAX, false>(1, 0, p, lds, lds + Cfg::STAGES * Cfg::SA, Cfg::SA, Cfg::SB, mt * BM, n0, n0 + UW);
    }
  }
}

// Sum of the K slices of the tail units (see ConvArgs), one thread per element, slices added in order; applies the
// final output mapping, '+=' and the bias / activation epilogue.
struct TailArgs {
  const float* part;
  int tail_units, tail_split, main_units, n_units, M, Ncols, beta, bm, uw;
  OutMap om;
  PostOp post;
};
__global__ __launch_bounds__(256) void reduce_tail(float* out, TailArgs t) {
  const int per = t.bm * t.uw;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= t.tail_units * per) return;
  const int j = i / per, e = i - j * per, row = e / t.uw, col = e - row * t.uw;
  const int u = t.main_units + j, mt = u / t.n_units;
  const int m = mt * t.bm + row, n = (u - mt * t.n_units) * t.uw + col;
  if (m >= t.M || n >= t.Ncols) return;
  float v = 0.0f;
  for (int s = 0; s < t.tail_split; ++s) v += t.part[(size_t)(s * t.tail_units + j) * per + e];
  float* dst = out + ((size_t)t.om.col((uint32_t)n) + (size_t)m * t.om.ld);
  if (t.beta) v += *dst;
  else if (t.post.any()) v = t.post.apply(v, t.post.bias != nullptr ? t.post.bias[t.post.bias_col ? n : m] : 0.0f);
  *dst = v;
}

template <int PASS, int WM, int NTMAX, bool FLAG>
__global__ __launch_bounds__(512, 2) void conv_kernel(ConvArgs a) {
  int bx = blockIdx.x, by = blockIdx.y;
  if (!wgrad_tap(PASS) && PASS != PASS_WGRAD && a.ksplit > 1) {
    // forward / data gradient cut along K: the sub-tiles of one K slice and one row of tiles read the same weights,
    // those of one slice the same activations; numbered slice by slice and handed to the XCDs in contiguous runs,
    // each weight is fetched by one XCD or two instead of all eight (256 -> 512 channels 5x5 stride 2 on 16 x 16
    // pixels, batch 16: 110 -> 18 MB fetched per launch; the pass takes 1-2 % longer, the sub-tiles of an XCD now
    // waiting for the same lines at the same time)
    const int j = xcd_contiguous(by * (int)gridDim.x + bx, (int)(gridDim.x * gridDim.y));
    by = j / (int)gridDim.x;
    bx = j - by * (int)gridDim.x;
  }
  conv_body<PASS, WM, NTMAX, FLAG>(a, bx, by);
}

// Several independent problems of one pass in one launch (the pixel classes of a strided dgrad).  The grid is
// flat and holds exactly the workgroups the problems asked for, problem after problem (first[i] = where problem
// i's begin): a launch that also carried workgroups with nothing to do would, when the useful ones number as many
// as the chip has compute units, leave some unit with two of them in a row.
constexpr int kMaxBatch = 4;
struct ConvArgsBatch {
  ConvArgs c[kMaxBatch];
  int first[kMaxBatch + 1];
};
template <int PASS, int WM, int NTMAX>
__global__ __launch_bounds__(512, 2) void conv_kernel_batch(ConvArgsBatch b) {
  const int lin = blockIdx.x;
  int i = 0;
#pragma unroll
  for (int q = 1; q < kMaxBatch; ++q) i += lin >= b.first[q];
  const int gx = b.c[i].grid_x;
  int local = lin - b.first[i];
  if (b.c[i].ksplit > 1) local = xcd_contiguous(local, b.first[i + 1] - b.first[i]);   // as in conv_kernel
  const int by = local / gx, bx = local - by * gx;
  conv_body<PASS, WM, NTMAX, true>(b.c[i], bx, by);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static int fill_geom(const lnn_conv2d_desc* d, ConvGeom& g) {
  if (!d) return set_error(LNN_ERR_INVALID, "conv2d: null descriptor");
  const int v[] = {d->N, d->C, d->IH, d->IW, d->O, d->KH, d->KW, d->OH, d->OW, d->stride, d->dilation};
  for (int x : v)
    if (x <= 0) return set_error(LNN_ERR_INVALID, "conv2d: non-positive dimension in descriptor");
  if (d->PADL < 0 || d->PADT < 0) return set_error(LNN_ERR_INVALID, "conv2d: negative padding");
  g.N = d->N; g.C = d->C; g.IH = d->IH; g.IW = d->IW; g.O = d->O; g.KH = d->KH; g.KW = d->KW;
  g.OH = d->OH; g.OW = d->OW; g.PADL = d->PADL; g.PADT = d->PADT; g.S = d->stride; g.D = d->dilation;
  const uint64_t ihw = (uint64_t)d->IH * d->IW, ohw = (uint64_t)d->OH * d->OW, kk = (uint64_t)d->KH * d->KW;
  const uint64_t xb = (uint64_t)d->N * d->C * ihw * 4, yb = (uint64_t)d->N * d->O * ohw * 4;
  const uint64_t wb = (uint64_t)d->O * d->C * kk * 4;
  if (xb > kMaxTensorBytes || yb > kMaxTensorBytes || wb > kMaxTensorBytes)
    return set_error(LNN_ERR_UNSUPPORTED, "conv2d: a tensor of 2 GiB or more");
  // coordinates must stay far below the sentinel used for masked elements
  if ((uint64_t)d->OH * d->stride + (uint64_t)d->KH * d->dilation + d->PADT + d->IH >= (uint64_t)BIG / 2 ||
      (uint64_t)d->OW * d->stride + (uint64_t)d->KW * d->dilation + d->PADL + d->IW >= (uint64_t)BIG / 2)
    return set_error(LNN_ERR_UNSUPPORTED, "conv2d: coordinate range too large");
  g.IHW = (int)ihw; g.OHW = (int)ohw; g.KK = (int)kk;
  g.dOW = make_fastdiv(g.OW); g.dOHW = make_fastdiv(g.OHW);
  g.dIW = make_fastdiv(g.IW); g.dIHW = make_fastdiv(g.IHW);
  g.dS = make_fastdiv(g.S);
  return LNN_OK;
}

// Bound the table cache: before a call that may add up to n tables, drop everything once the work queued so
// far is done.  Never in the middle of a call: its earlier tables must stay valid until it has launched.
static int reserve_tables(DeviceCtx* ctx, size_t n) {
  if (ctx->no_alloc || ctx->tables.size() + n <= 256) return LNN_OK;
  LNN_HIP(hipStreamSynchronize(ctx->stream));
  for (auto& kv : ctx->tables) (void)hipFree(kv.second);
  ctx->tables.clear();
  return LNN_OK;
}

// mode 0: forward / wgrad table; 1, 2: dgrad tables of pixel class pc (per k / per tap)
static int get_table(DeviceCtx* ctx, const ConvGeom& g, int mode, const PixelClass& pc, const KEntry** out) {
  const int nt = pc.nkh * pc.nkw;
  const int K = mode == 0 ? g.C * g.KK : (mode == 1 ? g.O * nt : nt);
  // readers prefetch one K step (mode 2: one tap) past the end
  const int Kpad = mode == 2 ? K + 2 : ((K + BK - 1) / BK) * BK + BK;
  const std::array<int, 16> key = {mode, g.C,  g.O,  g.KH, g.KW,   g.D,    g.IH,  g.IW,
                                   g.OH, g.OW, g.S, g.PADT, g.PADL, pc.rh, pc.rw, 0};
  if (ctx->no_alloc) {
    // from the tail of the fixed scratch array, built anew by every call (the next call reuses the memory)
    const size_t tb = ((size_t)Kpad * sizeof(KEntry) + 255) & ~(size_t)255;
    if (tb > ctx->ws_bytes)
      return set_error(LNN_ERR_UNSUPPORTED, "conv2d: the gather table does not fit the allocation-free entry point's scratch");
    ctx->ws_bytes -= tb;
    KEntry* t = reinterpret_cast<KEntry*>(static_cast<char*>(ctx->ws) + ctx->ws_bytes);
    hipLaunchKernelGGL(build_ktable, dim3((Kpad + 255) / 256), dim3(256), 0, ctx->stream, t, K, Kpad, mode, g, pc);
    LNN_HIP(hipGetLastError());
    *out = t;
    return LNN_OK;
  }
  auto it = ctx->tables.find(key);
  if (it != ctx->tables.end()) {
    *out = it->second;
    return LNN_OK;
  }
  KEntry* tab = nullptr;
  hipError_t e = hipMalloc((void**)&tab, (size_t)Kpad * sizeof(KEntry));
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    return set_error(LNN_ERR_OOM, "conv2d: out of device memory for the gather table");
  }
  LNN_HIP(e);
  hipLaunchKernelGGL(build_ktable, dim3((Kpad + 255) / 256), dim3(256), 0, ctx->stream, tab, K, Kpad, mode, g, pc);
  LNN_HIP(hipGetLastError());
  ctx->tables[key] = tab;
  *out = tab;
  return LNN_OK;
}

// Weights into a permuted layout (modes as in permute_one).
static int launch_permute(DeviceCtx* ctx, float* wp, const float* W, const ConvGeom& g, int mode, const PixelClass& pc) {
  if (mode != 1 && g.KK <= kPermuteMaxKK) {
    const int blocks = g.O * ((g.C + 63) / 64);
    hipLaunchKernelGGL(permute_weights_tiled, dim3(blocks), dim3(256), (size_t)64 * (g.KK | 1) * sizeof(float), ctx->stream,
                       wp, W, g.O, g.C, g.KK, mode);
  } else {
    const int n = g.O * g.C * (mode == 1 ? pc.nkh * pc.nkw : g.KK);
    hipLaunchKernelGGL(permute_weights, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, wp, W, g.O, g.C, g.KK, mode, g, pc);
  }
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// Channel-permuted copy of the weights in the library's scratch buffer (valid
// until the next call that uses scratch; the stream orders it before its reader).
static int permuted_weights(DeviceCtx* ctx, const ConvGeom& g, const float* W, int mode, const PixelClass& pc,
                            const float** out, size_t* used) {
  const int n = g.O * g.C * (mode == 0 ? g.KK : pc.nkh * pc.nkw);
  *used = ((size_t)(n > 0 ? n : 1) * sizeof(float) + 255) & ~(size_t)255;
  // leave room behind the weights for the split-K partial sums of the same call (at most one full
  // 32768-element sub-tile per workgroup slot), so that the buffer is not reallocated under them
  int st = ensure_workspace(ctx, *used + (size_t)ctx->cus * 32768 * sizeof(float));
  if (st != LNN_OK) return st;
  if (n > 0) {
    st = launch_permute(ctx, static_cast<float*>(ctx->ws), W, g, mode, pc);
    if (st != LNN_OK) return st;
  }
  *out = static_cast<const float*>(ctx->ws);
  return LNN_OK;
}

// Slice reduction of a split-K problem into its final tensor.
template <int PASS, int WM>
static ReduceArgs reduce_args(const ConvArgs& a, int final_beta) {
  constexpr int WN = 4 / WM;
  ReduceArgs r = {};
  r.n = a.M * a.Ncols; r.slices = a.ksplit; r.slices_last = a.ksplit; r.beta = final_beta; r.ncols = a.Ncols;
  r.bm_log = WM == 4 ? 7 : (WM == 2 ? 6 : 5); r.uw_log = WN == 4 ? 7 : (WN == 2 ? 6 : 5);
  r.per_mt = 0; r.last_unit0 = 0x7fffffff;
  r.kk = 0;
  if (wgrad_tap(PASS)) {
    r.kk = a.g.KK;
    r.slices_last = a.ks_last;
    r.per_mt = a.seg_units * a.segs_per_mt;
    r.last_unit0 = (a.n_chunks - 1) * a.chunk_units;
    if (a.eq_wgs > 0) {
      r.eq_wgs = a.eq_wgs; r.eq_nkt = (a.K + BK - 1) / BK; r.eq_chunk = a.chunk_units; r.eq_chunks = a.n_chunks;
      r.eq_cw_log = r.uw_log + (a.chunk_units == 2 ? 1 : (a.chunk_units == 4 ? 2 : 3));
      r.eq_d = a.eq_d; r.eq_g = a.eq_g;
    }
  }
  r.dN = make_fastdiv((uint32_t)a.Ncols);
  r.om = final_map<PASS>(a);
  r.post = a.post;
  return r;
}

template <int PASS, int WM>
static int launch_reduce(DeviceCtx* ctx, const ConvArgs& a, float* final_out, int final_beta) {
  const ReduceArgs r = reduce_args<PASS, WM>(a, final_beta);
  if (wgrad_tap(PASS) && a.Ncols % 4 == 0 && a.Ncols >= 256 && (size_t)a.Ncols * sizeof(float) <= 64 * 1024 && !r.post.any()) {
    // rows fewer than four times the compute units: several blocks per row, each a run of channels
    int parts = 1;
    if (a.g.C % 4 == 0)
      while (parts < 8 && a.M * parts < 4 * ctx->cus && a.g.C / (2 * parts) >= 16) parts *= 2;
    hipLaunchKernelGGL(reduce_partials_rows, dim3(a.M, parts), dim3(256), (size_t)a.Ncols * sizeof(float), ctx->stream, final_out,
                       static_cast<const float*>(a.Out), r);
  }
  else if (a.Ncols % 4 == 0)   // partial buffers start 256-byte aligned
    hipLaunchKernelGGL(reduce_partials4, dim3((r.n + reduce4_block(r) - 1) / reduce4_block(r)), dim3(256), 0, ctx->stream, final_out,
                       static_cast<const float*>(a.Out), r);
  else
    hipLaunchKernelGGL(reduce_partials, dim3((r.n + 31) / 32), dim3(256), 0, ctx->stream, final_out,
                       static_cast<const float*>(a.Out), r);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// Forward / dgrad: units, grid and K split of one problem that may use `slots` workgroups.
// Returns the bytes of partial sums it needs (0 without a K split).
template <int WM, int NTMAX>
static size_t plan_tiles(ConvArgs& a, long long slots, bool allow_tail = false) {
  constexpr int WN = 4 / WM, BM = 32 * WM;
  const int m_tiles = (a.M + BM - 1) / BM;
  a.n_units = (a.Ncols + 32 * WN - 1) / (32 * WN);
  const long long total = (long long)m_tiles * a.n_units;
  a.total_units = total > 0x7fffffffll ? -1 : (int)total;
  a.chunk_units = 0;
  a.n_chunks = 1;
  a.ks_last = 1;
  a.ksplit = 1;
  a.grid_x = (int)(total < slots ? total : slots);
  a.main_units = a.total_units; a.tail_units = 0; a.tail_split = 1; a.tail_part = nullptr;
  // Few output tiles (small images, deep layers): a workgroup's share would be a sliver of a sub-tile and
  // most of its time data movement.  Cut the output into full sub-tiles instead and split K over the
  // workgroups that are left, as wgrad does.
  const int chunk = NTMAX > 1 ? NTMAX : 2;
  const long long chunks = (total + chunk - 1) / chunk;
  const int nkt = (a.K + BK - 1) / BK;
  if (total < slots * (NTMAX + 1) && chunks * 2 <= slots && nkt >= 16) {
    long long s = slots / chunks;
    if (s > nkt / 8) s = nkt / 8;
    if (s > 1) {
      a.ksplit = (int)s;
      a.grid_x = (int)chunks;
      return (size_t)a.ksplit * a.M * a.Ncols * sizeof(float);
    }
  }
  // A few units per workgroup and a remainder: the workgroups that would take one unit more set the pace
  // (3136 units on 256 workgroups: 13 against 12.25).  Cut the remainder along K instead, one slice per workgroup.
  if (allow_tail && total > slots && total <= 64 * slots) {
    const long long q = total / slots, r = total - q * slots;
    long long ts = r > 0 ? slots / r : 0;
    if (ts > nkt / 6) ts = nkt / 6;   // a slice should still hold a handful of K steps
    if (ts >= 2) {
      a.main_units = (int)(q * slots);
      a.tail_units = (int)r;
      a.tail_split = (int)ts;
      return (size_t)ts * r * BM * (32 * WN) * sizeof(float);
    }
  }
  return 0;
}

// Tap-major weight gradient: when the plan "whole chunks x K slices" would leave much of the chip idle (200 sub-tiles
// of 16 K steps on 256 compute units), cut the K steps of all chunks, laid end to end, into one equal run per
// workgroup slot instead (ConvArgs::eq_wgs).  Chunks are half-width sub-tiles then (both groups at half their
// accumulators: half the partial sums per piece).  Taken only when a run is shorter than a chunk's K (so a workgroup
// has at most two pieces), its estimated time - steps per workgroup plus a refill of the pipeline for the second
// piece - beats the plan it replaces by a tenth, and the slice sum can run row-wise.  The pieces' blocks take
// 2 * slots * BM * (chunk width) floats whatever the problem: 32 MiB on 256 compute units.
template <int WM, int NTMAX>
static void plan_equal_shares(ConvArgs& a, long long slots, int nkt) {
  constexpr int WN = 4 / WM;
  if (a.post.any() || a.Ncols % 4 != 0 || a.Ncols < 256 || (size_t)a.Ncols * sizeof(float) > 64 * 1024) return;
  const int half = a.chunk_units / 2, per_mt = a.seg_units * a.segs_per_mt;
  if (half < 2 || half % 2 != 0 || half * 32 * WN < 128) return;
  if (a.total_units % half != 0 || per_mt % half != 0) return;   // whole chunks, none across two rows of tiles
  const long long chunks = a.total_units / half, T = chunks * nkt;
  if (T < 8 * slots || nkt < 16 || chunks > slots) return;
  // time in K steps of a half-width chunk: now, and with equal shares
  const long long rounds = (a.grid_x + slots - 1) / slots;
  const long long now = rounds * ((nkt + a.ksplit - 1) / a.ksplit) * 2;
  const long long then = (T + slots - 1) / slots + 2;
  if (then * 11 > now * 10) return;
  a.eq_wgs = (int)slots;
  // Runs w and w + P stand at the same K position all along when S * P is a multiple of nkt (S steps per run), and
  // with 8 | P they also share an XCD (workgroups go to the XCDs in turn).  Their places in the end-to-end order lie
  // D = S * P / nkt apart, so the order takes the chunks with a stride: the W / P runs that move through K together
  // work on neighbouring chunks - neighbouring taps of one row of tiles, which read the same dY rows and X rows a
  // few pixels apart - and meet their operands in that XCD's L2.
  a.eq_d = a.eq_g = 0;
  if (T % slots == 0) {
    const long long S = T / slots;
    long long gcd = S, r = nkt;
    while (r) { const long long t = gcd % r; gcd = r; r = t; }
    const long long P = nkt / gcd, D = S * P / nkt;
    if (P % 8 == 0 && slots % P == 0 && D * (slots / P) == chunks) {
      a.eq_d = (int)D;
      a.eq_g = (int)(slots / P);
    }
  }
  a.chunk_units = half;
  a.n_chunks = (int)chunks;
  a.ksplit = 2;
  a.ks_last = 2;
  a.grid_x = (int)slots;
}

template <int PASS, int WM, int NTMAX>
static int launch_pass(DeviceCtx* ctx, ConvArgs& a, bool flag) {
  constexpr int WN = 4 / WM, BM = 32 * WM;
  // one 512-thread workgroup per compute unit; two of the 64 x 128 tiles, whose three LDS stages take 72 KB
  const long long slots = (long long)ctx->cus * (WM == 2 && NTMAX == 1 ? 2 : 1);
  float* final_out = a.Out;
  const int final_beta = a.beta;
  int grid_y = 1;
  a.main_units = 0; a.tail_units = 0; a.tail_split = 1; a.tail_part = nullptr;
  if (PASS == PASS_WGRAD || wgrad_tap(PASS)) {
    const int m_tiles = (a.M + BM - 1) / BM;
    a.n_units = (a.Ncols + 32 * WN - 1) / (32 * WN);
    long long total = (long long)m_tiles * a.n_units;
    a.chunk_units = 0;
    if (wgrad_tap(PASS)) {
      // columns are tap-major.  The loaders that keep one tap per group see KK segments of C / (32*WN) units per M
      // tile, and a workgroup takes one sub-tile's worth of whole segments (or of one segment's halves); for the
      // loader whose columns may span taps the whole row is one segment and every sub-tile is full.
      if (PASS == PASS_WGRAD_ANYC) {
        a.seg_units = a.n_units;
        a.segs_per_mt = 1;
        a.chunk_units = a.seg_units < 2 * NTMAX ? a.seg_units : 2 * NTMAX;
      } else {
        a.seg_units = a.g.C / (32 * WN);
        a.segs_per_mt = a.g.KK;
        a.chunk_units = 2 * (a.seg_units < NTMAX ? a.seg_units : NTMAX);
      }
      a.n_units = a.seg_units;
      total = (long long)m_tiles * a.segs_per_mt * a.seg_units;
      a.dC = make_fastdiv((uint32_t)a.g.C);
    }
    if (total > 0x7fffffffll) return set_error(LNN_ERR_UNSUPPORTED, "conv2d: too many tiles");
    a.total_units = (int)total;
    a.n_chunks = 1;
    a.ks_last = 1;
    // one full-width sub-tile per workgroup, then as many K slices as fill the chip
    const int chunk = wgrad_tap(PASS) ? a.chunk_units : 2 * NTMAX;
    int grid = (int)((total + chunk - 1) / chunk);
    const int nkt = (a.K + BK - 1) / BK;
    long long s = wgrad_tap(PASS) ? slots * chunk / total : slots / grid;
    if (s > nkt / 4) s = nkt / 4;
    if (s > 1024) s = 1024;
    if (s < 1) s = 1;
    int ksplit = (int)s;
    grid_y = ksplit;
    if (wgrad_tap(PASS)) {
      // the last chunk holds rem <= chunk units: give it the matching share of the slices.  A K step of u
      // units costs about (o + u) with a fixed part o worth an eighth of a full chunk (measured: a half
      // chunk's step takes 0.56 of a full one), so that is the ratio of the slice counts.
      const int rem = (int)(total - (long long)(grid - 1) * chunk);
      const int o = chunk >= 8 ? chunk / 8 : 1;
      auto last = [&](int sf) { const int l = (sf * (o + rem) + o + chunk - 1) / (o + chunk); return l < 1 ? 1 : (l > sf ? sf : l); };
      while (ksplit > 1 && (long long)(grid - 1) * ksplit + last(ksplit) > slots) --ksplit;
      a.n_chunks = grid;
      a.ks_last = last(ksplit);
      if (ksplit > 1) grid = (grid - 1) * ksplit + a.ks_last;
      grid_y = 1;
    }
    a.ksplit = ksplit;
    a.grid_x = grid;
    a.eq_wgs = 0;
    if (wgrad_tap(PASS) && PASS != PASS_WGRAD_ANYC) plan_equal_shares<WM, NTMAX>(a, slots, nkt);
    ksplit = a.ksplit;
    grid = a.grid_x;
    if (ksplit > 1) {
      const size_t need = a.eq_wgs > 0 ? (size_t)2 * a.eq_wgs * BM * (a.chunk_units * 32 * WN) * sizeof(float)
                                       : (size_t)ksplit * a.M * a.Ncols * sizeof(float);
      int st = ensure_workspace(ctx, need);
      if (st != LNN_OK) return st;
      a.Out = static_cast<float*>(ctx->ws);
      a.beta = 0;
    }
  } else {
    const size_t need = plan_tiles<WM, NTMAX>(a, slots, true);
    if (a.total_units < 0) return set_error(LNN_ERR_UNSUPPORTED, "conv2d: too many tiles");
    if (need) {
      // the scratch buffer may already hold this call's permuted weights: keep them in front
      int st = ensure_workspace(ctx, a.ws_used + need);
      if (st != LNN_OK) return st;
      float* scratch = reinterpret_cast<float*>(static_cast<char*>(ctx->ws) + a.ws_used);
      if (a.tail_units > 0) {
        a.tail_part = scratch;
      } else {
        a.Out = scratch;
        a.beta = 0;
        grid_y = a.ksplit;
      }
    }
  }
  if (PASS == PASS_WGRAD || wgrad_tap(PASS)) {
    ctx->last_wgrad_plan[0] = a.grid_x * grid_y;
    ctx->last_wgrad_plan[1] = a.ksplit;
    ctx->last_wgrad_plan[2] = wgrad_tap(PASS) && a.eq_wgs > 0 ? 1 : 0;
    ctx->last_wgrad_plan[3] = BM;
  }
  dim3 g(a.grid_x, grid_y, 1), b(512, 1, 1);
  constexpr bool kUsesFlag = PASS == PASS_WGRAD || PASS == PASS_WGRAD_TAP || PASS == PASS_WGRAD_ANYC;   // the other passes have one variant
  if (flag || !kUsesFlag) {
    hipLaunchKernelGGL((conv_kernel<PASS, WM, NTMAX, true>), g, b, 0, ctx->stream, a);
  } else if constexpr (kUsesFlag) {
    hipLaunchKernelGGL((conv_kernel<PASS, WM, NTMAX, false>), g, b, 0, ctx->stream, a);
  }
  LNN_HIP(hipGetLastError());
  if (a.ksplit > 1) return launch_reduce<PASS, WM>(ctx, a, final_out, final_beta);
  if (a.tail_units > 0) {
    TailArgs t;
    t.part = a.tail_part;
    t.tail_units = a.tail_units; t.tail_split = a.tail_split; t.main_units = a.main_units; t.n_units = a.n_units;
    t.M = a.M; t.Ncols = a.Ncols; t.beta = final_beta; t.bm = BM; t.uw = 32 * WN;
    t.om = final_map<PASS>(a);
    t.post = a.post;
    const int n = a.tail_units * BM * 32 * WN;
    hipLaunchKernelGGL(reduce_tail, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, final_out, t);
    LNN_HIP(hipGetLastError());
  }
  return LNN_OK;
}

// The pixel classes of one strided dgrad (all the same M, hence the same tile shape): planned for an equal
// share of the chip each, launched kMaxBatch at a time, partial sums behind `ws_off` in the scratch buffer
// (which the caller has sized), then reduced one by one.
template <int PASS, int WM, int NTMAX>
static int launch_classes(DeviceCtx* ctx, std::vector<ConvArgs>& cls, size_t ws_off) {
  const int n = (int)cls.size();
  const int per_batch = n < kMaxBatch ? n : kMaxBatch;
  // equal shares of the chip; the 64 x 128 tile's three LDS stages (72 KB) fit twice on a compute unit
  const long long chip = (long long)ctx->cus * (WM == 2 && NTMAX == 1 ? 2 : 1);
  const long long equal = chip / per_batch > 0 ? chip / per_batch : 1;
  // The classes of one launch differ in their number of taps (5x5 stride 2: 9, 6, 6 and 4): with the tap-major
  // kernels, whose time follows the multiply-adds, each gets workgroups in proportion to its work instead
  // (256 -> 512 channels at 16 x 16: 77 -> 63 us).
  std::vector<long long> share(n, equal);
  if (dgrad_tap(PASS) && n <= kMaxBatch) {
    // Only where every class is cut along K anyway (few output tiles: any share divides into whole sub-tiles times
    // K slices).  Classes with many tiles and no K split lose more to the narrow sub-tiles of an odd share than
    // they gain (64 -> 128 channels at 64 x 64: 82 -> 121 us).
    bool all_split = true;
    std::vector<long long> chunks(n), nkt(n);
    for (int i = 0; i < n; ++i) {
      ConvArgs a = cls[i];
      plan_tiles<WM, NTMAX>(a, equal);
      all_split = all_split && a.total_units >= 0 && a.ksplit > 1;
      chunks[i] = a.grid_x;                       // full sub-tiles of this class
      nkt[i] = (cls[i].K + BK - 1) / BK;
    }
    if (all_split) {
      // K slices per class so that the longest slice of any class is as short as the chip allows: start from one
      // slice each and keep giving one more to the class whose slices are longest while workgroups are left
      // (5x5 stride 2, 256 -> 512 channels at 16 x 16: 72 / 48 / 48 / 32 K steps in 5 / 4 / 4 / 3 slices instead of
      // the 5 / 3 / 3 / 2 that shares in proportion to the work round down to)
      std::vector<long long> ks(n, 1);
      long long used = 0;
      for (int i = 0; i < n; ++i) used += chunks[i];
      for (;;) {
        int best = -1;
        for (int i = 0; i < n; ++i) {
          if (used + chunks[i] > chip || ks[i] + 1 > nkt[i] / 8) continue;   // plan_tiles caps slices at nkt / 8
          if (best < 0 || nkt[i] * ks[best] > nkt[best] * ks[i]) best = i;
        }
        if (best < 0) break;
        // stop when the class with the longest slices cannot be helped: more slices elsewhere shorten nothing
        int longest = 0;
        for (int i = 1; i < n; ++i)
          if (nkt[i] * ks[longest] > nkt[longest] * ks[i]) longest = i;
        if (best != longest) break;
        ++ks[best];
        used += chunks[best];
      }
      for (int i = 0; i < n; ++i) share[i] = chunks[i] * ks[i];
    }
  }
  std::vector<float*> final_out(n);
  std::vector<int> final_beta(n);
  for (int i = 0; i < n; ++i) {
    ConvArgs& a = cls[i];
    const size_t need = plan_tiles<WM, NTMAX>(a, share[i]);
    if (a.total_units < 0) return set_error(LNN_ERR_UNSUPPORTED, "conv2d: too many tiles");
    final_out[i] = a.Out;
    final_beta[i] = a.beta;
    if (need) {
      a.Out = reinterpret_cast<float*>(static_cast<char*>(ctx->ws) + ws_off);
      a.beta = 0;
      ws_off += (need + 255) & ~(size_t)255;
    }
  }
  if (ws_off > ctx->ws_bytes) return set_error(LNN_ERR_HIP, "conv2d_dgrad: scratch buffer smaller than planned");
  for (int i0 = 0; i0 < n; i0 += kMaxBatch) {
    const int nb = n - i0 < kMaxBatch ? n - i0 : kMaxBatch;
    ConvArgsBatch b;
    int total = 0;
    for (int i = 0; i < kMaxBatch; ++i) {
      b.c[i] = cls[i0 + (i < nb ? i : 0)];
      b.first[i] = total;
      if (i < nb) total += b.c[i].grid_x * (b.c[i].ksplit > 1 ? b.c[i].ksplit : 1);
    }
    b.first[kMaxBatch] = total;
    if (total > 0) {
      hipLaunchKernelGGL((conv_kernel_batch<PASS, WM, NTMAX>), dim3(total), dim3(512, 1, 1), 0, ctx->stream, b);
      LNN_HIP(hipGetLastError());
    }
  }
  // the K-split classes' reductions, kMaxReduceBatch per launch
  ReduceBatch rb;
  int nr = 0;
  unsigned gx = 1;
  auto flush = [&]() {
    if (nr == 0) return;
    hipLaunchKernelGGL(reduce_partials_batch, dim3(gx, nr), dim3(256), 0, ctx->stream, rb);
    nr = 0;
    gx = 1;
  };
  for (int i = 0; i < n; ++i)
    if (cls[i].ksplit > 1) {
      rb.r[nr] = reduce_args<PASS, WM>(cls[i], final_beta[i]);
      rb.out[nr] = final_out[i];
      rb.part[nr] = cls[i].Out;
      rb.vec[nr] = cls[i].Ncols % 4 == 0;
      const unsigned per_block = rb.vec[nr] ? (unsigned)reduce4_block(rb.r[nr]) : 32u;
      const unsigned blocks = ((unsigned)rb.r[nr].n + per_block - 1) / per_block;
      gx = blocks > gx ? blocks : gx;
      if (++nr == kMaxReduceBatch) flush();
    }
  flush();
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

template <int PASS>
static int launch_classes_by_m(DeviceCtx* ctx, std::vector<ConvArgs>& cls, size_t ws_off) {
  const int M = cls[0].M;
  if (PASS == PASS_DGRAD_TAPW && M > 64 && cls.size() == 4) {
    // Four classes of a deep layer (few pixels, long K): every workgroup's piece is a handful of K steps, and filling
    // and draining the pipeline costs as much as computing.  On 64 x 128 tiles two workgroups share a compute unit and
    // one computes while the other fills or stores (128 -> 256 and 256 -> 512 channels, 5x5 stride 2, at 16 x 16 and
    // 8 x 8: 80 -> 73 and 74 -> 69 us; 64 x 256 tiles, one workgroup per compute unit: 82 and 83).
    bool few = true;
    for (const ConvArgs& a : cls) few = few && (long long)((a.M + 127) / 128) * ((a.Ncols + 31) / 32) < ctx->cus;
    if (few) {
      std::sort(cls.begin(), cls.end(), [](const ConvArgs& x, const ConvArgs& y) { return x.K > y.K; });
      std::swap(cls[2], cls[3]);
      return launch_classes<PASS, 2, 1>(ctx, cls, ws_off);
    }
  }
  if (M > 64) return launch_classes<PASS, 4, 4>(ctx, cls, ws_off);
  if (PASS == PASS_DGRAD_TAPW && M > 32 && cls.size() == 4) {
    // Four classes with many tiles each and different K lengths (5x5 stride 2: 9, 6, 6 and 4 taps): on 64 x 128
    // tiles two workgroups share a compute unit, and with the classes in the order longest, second, shortest, third
    // workgroups b and b + (number of compute units) - which land on the same one - are a long and a short piece.
    bool plain = true;
    for (const ConvArgs& a : cls) {
      const long long units = (a.Ncols + 63) / 64;
      plain = plain && units >= 2ll * ctx->cus / 4 * 2;   // at least one full 2-unit sub-tile per workgroup: no K split
    }
    if (plain) {
      std::sort(cls.begin(), cls.end(), [](const ConvArgs& x, const ConvArgs& y) { return x.K > y.K; });
      std::swap(cls[2], cls[3]);
      return launch_classes<PASS, 2, 1>(ctx, cls, ws_off);
    }
  }
  if (M > 32) return launch_classes<PASS, 2, 2>(ctx, cls, ws_off);
  return launch_classes<PASS, 1, 1>(ctx, cls, ws_off);
}

template <int PASS>
static int launch_by_m(DeviceCtx* ctx, ConvArgs& a, bool flag) {
  if (PASS == PASS_WGRAD_TAP && a.M > 64 && a.g.C % 64 == 0) {
    // A weight gradient whose 128 x 256 tiles would each be cut into many short K slices (a deep layer: large weight
    // tensor, few output pixels): on 64 x 128 tiles two workgroups share a compute unit, one computing while the other
    // fills its pipeline or stores its partial sums (128 -> 256 channels 5x5 at 16 x 16 pixels, batch 16: 79 -> 74 us;
    // with long slices, or hardly any K split, the larger tile's better operand reuse wins)
    const int seg = a.g.C / 32, chunk = 2 * (seg < 4 ? seg : 4);
    const long long total = (long long)((a.M + 127) / 128) * a.g.KK * seg;
    const long long slices = (long long)ctx->cus * chunk / total, nkt = (a.K + BK - 1) / BK;
    if (slices >= 4 && nkt < 14 * slices) return launch_pass<PASS, 2, 1>(ctx, a, flag);
  }
  if (a.M > 64) return launch_pass<PASS, 4, 4>(ctx, a, flag);
  if (a.M > 32) return launch_pass<PASS, 2, 2>(ctx, a, flag);
  return launch_pass<PASS, 1, 1>(ctx, a, flag);
}

// The weight gradient's pixel walkers move a lane's pixel by one K step with single wrap tests: an image must hold a
// K step of pixels, and a K step must not wrap around an image more than once.  (Tiny images outside this take the
// table-driven kernel.)
static bool wgrad_walkers_fit(const ConvGeom& g) { return g.OHW >= BK && BK / g.OW + 1 <= g.OH; }
// ... and the loaders that keep one tap per group want the channels to fill whole units of the tile shape chosen for
// O, enough of them for full sub-tiles (fewer channels: the loader whose columns span taps).
static bool wgrad_one_tap_per_group(const ConvGeom& g) {
  const int unit = g.O > 64 ? 32 : (g.O > 32 ? 64 : 128);
  return wgrad_walkers_fit(g) && g.C % unit == 0;
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace
}  // namespace lnn
