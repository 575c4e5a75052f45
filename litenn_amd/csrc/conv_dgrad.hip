// Convolution data gradient: pixel classes on the MFMA engine, and the vector-ALU kernel for very few input channels.
#include "conv_common.hpp"


namespace lnn {
namespace {

// ---- data gradient for very few input channels (image stems, the last layer of a decoder) ----------------------
// With C <= 4 the GEMM of the data gradient has at most 4 rows, and an MFMA tile would work on 32.  This kernel
// computes it on the vector ALU instead.  Stride S, dilation 1, square K x K kernel: the input pixels with the same
// rh = (ih + PADT) % S, rw = (iw + PADW) % S form a class that sees the taps kh = rh, rh + S, ... (NKH of them) and
// kw = rw, rw + S, ..., spaced one output pixel apart:
//   dX[n][c][h0 + S*y][w0 + S*x] (+)= sum over o, jh, jw of dY[n][o][y + ah - jh][x + aw - jw] * W[o][c][rh + S*jh][rw + S*jw]
// A block owns the 16 x 16 pixels (y, x) of ALL S*S classes of one image, i.e. one region of dY; each of its four
// wavefronts sums a quarter of the output channels over that region, on its own: it brings its channels' planes of
// the region to its own part of LDS, kDsOC at a time (global -> LDS transfers of 64 consecutive tile elements, all in
// flight together), and waits for nobody but itself.  A lane owns 2 x 2 pixels of every class: per output channel
// and class it reads its (NKH+1) x (NKW+1) window once; the weights (4 floats per tap, channels past C zero) travel
// to LDS with the planes and are read from there, the same address in every lane (through the scalar cache, whose
// loads return out of order, every pair of taps waited for its own load: 0.242 against 0.224 ms for a 7 x 7 stride 2
// stem at batch 32).  4 * NKH * NKW * C multiply-adds per window.
// At the end wavefronts 1..3 hand their sums over through LDS, one after the other, and wavefront 0 adds them in
// that order and stores.
// (A block of 32 x 32 pixels with one wavefront per 8 rows was measured first: a 112 x 112 class plane is 3.5 such
// tiles wide and tall, and 31 % of the lanes worked on pixels that do not exist.)
constexpr int kDsOC = 4, kDsTile = 16;
struct SmallDgradArgs {
  const float* dY;
  const float* wc;        // [O][K*K taps, class by class][4]
  float* dX;
  int N, O, C, OH, OW, IH, IW;
  int h0[4], w0[4];       // per class (rh*S + rw): origin, ...
  int ph[4], pw[4];       // ... plane size (0: no such pixels), ...
  int dh[4], dw[4];       // ... and tile row / column of output pixel (y + ah, x + aw) for y = x = 0
  int oh_base, ow_base;   // output pixel under tile element (0, 0) of block (0, 0)
  int th, tw;             // tile rows / columns in use
  int tiles_x, beta;
};
// number of taps k < K with k % S == r, and the number of taps in the classes before class (rh, rw)
constexpr int ds_nk(int K, int S, int r) { return r < K ? (K - r + S - 1) / S : 0; }
constexpr int ds_tap_base(int K, int S, int cls) {
  int n = 0;
  for (int q = 0; q < cls; ++q) n += ds_nk(K, S, q / S) * ds_nk(K, S, q % S);
  return n;
}
// Wc[o][t][c]: t runs over the classes' taps in class order, c < 4 (zero for c >= C)
__global__ void small_dgrad_weights(float* wc, const float* w, int O, int C, int K, int S) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x, KK = K * K;
  if (i >= O * KK * 4) return;
  const int c = i & 3, t = (i >> 2) % KK, o = (i >> 2) / KK;
  int rest = t, kh = 0, kw = 0;
  for (int cls = 0; cls < S * S; ++cls) {
    const int rh = cls / S, rw = cls % S;
    const int nh = rh < K ? (K - rh + S - 1) / S : 0, nw = rw < K ? (K - rw + S - 1) / S : 0;
    if (rest < nh * nw) {
      kh = rh + S * (rest / nw);
      kw = rw + S * (rest % nw);
      break;
    }
    rest -= nh * nw;
  }
  wc[i] = c < C ? w[((size_t)o * C + c) * KK + kh * K + kw] : 0.0f;
}

template <int S, int K, int CN, int CLS>
struct SmallDgradClass {
  static constexpr int RH = CLS / S, RW = CLS % S, NKH = ds_nk(K, S, RH), NKW = ds_nk(K, S, RW);
  static constexpr int TAP0 = ds_tap_base(K, S, CLS);
  // adds output channel o's contribution to the 2 x 2 pixels of this class
  static __device__ __forceinline__ void accumulate(const SmallDgradArgs& a, const float* tile, int pitch, const float* wo,
                                                    int ty, int tx, float (&acc)[2][2][CN]) {
    if constexpr (NKH > 0 && NKW > 0) {
      // tile element of output pixel (y + ah - jh, x + aw - jw): row dh + y - jh
      const float* base = tile + (a.dh[CLS] + 2 * ty - (NKH - 1)) * pitch + a.dw[CLS] + 2 * tx - (NKW - 1);
      float win[NKH + 1][NKW + 1];
#pragma unroll
      for (int i = 0; i <= NKH; ++i)
#pragma unroll
        for (int j = 0; j <= NKW; ++j) win[i][j] = base[i * pitch + j];
#pragma unroll
      for (int jh = 0; jh < NKH; ++jh)
#pragma unroll
        for (int jw = 0; jw < NKW; ++jw) {
          const f32x4 w4 = *reinterpret_cast<const f32x4*>(wo + (TAP0 + jh * NKW + jw) * 4);   // LDS, same address in every lane
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float v = win[i + NKH - 1 - jh][j + NKW - 1 - jw];
#pragma unroll
              for (int c = 0; c < CN; ++c) acc[i][j][c] += v * w4[c];
            }
        }
    }
  }
  static __device__ __forceinline__ void store(const SmallDgradArgs& a, int n, int y0, int x0, int ty, int tx,
                                               const float (&acc)[2][2][CN]) {
    if constexpr (NKH > 0 && NKW > 0) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int y = y0 + 2 * ty + i, x = x0 + 2 * tx + j;
          if (y >= a.ph[CLS] || x >= a.pw[CLS]) continue;
#pragma unroll
          for (int c = 0; c < CN; ++c) {
            if (c >= a.C) continue;
            float* dst = a.dX + ((size_t)n * a.C + c) * a.IH * a.IW + (size_t)(a.h0[CLS] + S * y) * a.IW + a.w0[CLS] + S * x;
            *dst = a.beta ? *dst + acc[i][j][c] : acc[i][j][c];
          }
        }
    }
  }
};

template <int S, int K, int CN>
__global__ __launch_bounds__(256) void small_dgrad_kernel(SmallDgradArgs a) {
  constexpr int NCLS = S * S, KK = K * K;
  constexpr int TMAX = kDsTile + (K + S - 1) / S + 1, PITCH = TMAX | 1, PLANE = TMAX * PITCH;
  constexpr int CHUNK = kDsOC * PLANE, NTR = (CHUNK + 63) / 64;   // floats / transfers per chunk of channels
  constexpr int WCH = kDsOC * KK * 4, NTW = (WCH + 63) / 64;       // the chunk's weights
  constexpr int NACC = NCLS * 4 * CN;                              // sums per lane
  constexpr int WOFF = NTR * 64;                                   // weights behind the planes (16-byte aligned)
  constexpr int WAVE_LDS = WOFF + NTW * 64;
  static_assert(NACC * 64 <= 4 * WAVE_LDS, "one wavefront's sums fit the block's LDS");
  __shared__ float lds[4 * WAVE_LDS];
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int tx = lane & 7, ty = lane >> 3;
  const int by = blockIdx.x / a.tiles_x, bx = blockIdx.x - by * a.tiles_x, n = blockIdx.y;
  const int y0 = by * kDsTile, x0 = bx * kDsTile;
  const int oh0 = a.oh_base + y0, ow0 = a.ow_base + x0;
  float* const tile = lds + wave * WAVE_LDS;
  float acc[NCLS][2][2][CN];
#pragma unroll
  for (int q = 0; q < NCLS; ++q)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int c = 0; c < CN; ++c) acc[q][i][j][c] = 0.0f;
  const uint32_t plane = (uint32_t)a.OH * a.OW;
  // this image's dY
  const rsrc_t rs = make_rsrc(a.dY + (size_t)n * a.O * plane, (uint32_t)a.O * plane * 4u);
  // where this lane's element of each transfer lies in dY, relative to the chunk's first channel
  uint32_t voff[NTR];
#pragma unroll
  for (int t = 0; t < NTR; ++t) {
    const int f = t * 64 + lane, o = f / PLANE, rem = f - o * PLANE, r = rem / PITCH, c = rem - r * PITCH;
    const int oh = oh0 + r, ow = ow0 + c;
    const bool ok = f < CHUNK && r < a.th && c < a.tw && (uint32_t)oh < (uint32_t)a.OH && (uint32_t)ow < (uint32_t)a.OW;
    voff[t] = ok ? ((uint32_t)o * plane + (uint32_t)oh * a.OW + (uint32_t)ow) * 4u : OOB;
  }
  // the weights Wc[o][tap][4] of a chunk are WCH consecutive floats
  const rsrc_t rw = make_rsrc(a.wc, (uint32_t)a.O * KK * 16u);
  uint32_t woff[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) woff[t] = t * 64 + lane < WCH ? (uint32_t)(t * 64 + lane) * 4u : OOB;
  // this wavefront's output channels: [obeg, oend), whole chunks except at the end
  const int per = ((a.O + 3) / 4 + kDsOC - 1) / kDsOC * kDsOC;
  const int obeg = wave * per, oend = obeg + per < a.O ? obeg + per : a.O;
  for (int o0 = obeg; o0 < oend; o0 += kDsOC) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the previous chunk has been read
    const uint32_t soff = (uint32_t)o0 * plane * 4u;
    // a last chunk with fewer than kDsOC channels: the lanes of the missing ones ask for nothing (their range test is
    // made on the vector offset, whatever the hardware does with the scalar one)
    const int live = a.O - o0;
#pragma unroll
    for (int t = 0; t < NTR; ++t)
      buf_load_lds4(rs, tile + t * 64, live >= kDsOC || (t * 64 + lane) / PLANE < live ? voff[t] : OOB, soff);
#pragma unroll
    for (int t = 0; t < NTW; ++t)
      buf_load_lds4(rw, tile + WOFF + t * 64, live >= kDsOC || (t * 64 + lane) / (KK * 4) < live ? woff[t] : OOB,
                    (uint32_t)o0 * KK * 16u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const int on = oend - o0 < kDsOC ? oend - o0 : kDsOC;
#pragma unroll 1
    for (int o = 0; o < on; ++o) {
      const float* t = tile + o * PLANE;
      const float* wo = tile + WOFF + o * KK * 4;
      SmallDgradClass<S, K, CN, 0>::accumulate(a, t, PITCH, wo, ty, tx, acc[0]);
      if constexpr (NCLS > 1) {
        SmallDgradClass<S, K, CN, 1>::accumulate(a, t, PITCH, wo, ty, tx, acc[1]);
        SmallDgradClass<S, K, CN, 2>::accumulate(a, t, PITCH, wo, ty, tx, acc[2]);
        SmallDgradClass<S, K, CN, 3>::accumulate(a, t, PITCH, wo, ty, tx, acc[3]);
      }
    }
  }
  // sums of wavefronts 1..3 to wavefront 0, one after the other through the (now idle) planes, added in that order
  __syncthreads();
#pragma unroll 1
  for (int w = 1; w < 4; ++w) {
    if (wave == w) {
      int k = 0;
#pragma unroll
      for (int q = 0; q < NCLS; ++q)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int c = 0; c < CN; ++c, ++k) lds[k * 64 + lane] = acc[q][i][j][c];
    }
    __syncthreads();
    if (wave == 0) {
      int k = 0;
#pragma unroll
      for (int q = 0; q < NCLS; ++q)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int c = 0; c < CN; ++c, ++k) acc[q][i][j][c] += lds[k * 64 + lane];
    }
    __syncthreads();
  }
  if (wave != 0) return;
  SmallDgradClass<S, K, CN, 0>::store(a, n, y0, x0, ty, tx, acc[0]);
  if constexpr (NCLS > 1) {
    SmallDgradClass<S, K, CN, 1>::store(a, n, y0, x0, ty, tx, acc[1]);
    SmallDgradClass<S, K, CN, 2>::store(a, n, y0, x0, ty, tx, acc[2]);
    SmallDgradClass<S, K, CN, 3>::store(a, n, y0, x0, ty, tx, acc[3]);
  }
}

}  // namespace

// The vector-ALU data gradient serves C <= 4, dilation 1, stride 1 (K = 1, 3, 5) or 2 (K = 3, 4, 5, 7), when there
// are enough tiles to occupy the chip (a small problem is quicker on the MFMA path, whose tiles are finer).
static bool small_dgrad_applies(int cus, const ConvGeom& g) {
  if (g.C > 4 || g.D != 1 || g.KH != g.KW) return false;
  const int K = g.KH;
  const bool shape = (g.S == 1 && (K == 1 || K == 3 || K == 5)) || (g.S == 2 && (K == 3 || K == 4 || K == 5 || K == 7));
  if (!shape) return false;
  const long long ph = (g.IH + g.S - 1) / g.S, pw = (g.IW + g.S - 1) / g.S;
  const long long blocks = ((ph + kDsTile - 1) / kDsTile) * ((pw + kDsTile - 1) / kDsTile) * g.N;
  if ((uint64_t)g.N * g.O * g.OHW * 4 > kMaxTensorBytes) return false;
  return blocks >= cus;   // at least one block of four wavefronts per compute unit
}

constexpr int kNotHere = 1;   // plan_small_dgrad: a geometry it leaves to the general path (no error)
// Tile geometry of the vector-ALU data gradient (host only; the pointers of `a` are left alone).
static int plan_small_dgrad(const ConvGeom& g, int beta, SmallDgradArgs& a, int* grid_x) {
  const int K = g.KH, S = g.S;
  a.N = g.N; a.O = g.O; a.C = g.C; a.OH = g.OH; a.OW = g.OW; a.IH = g.IH; a.IW = g.IW;
  int ah[4], aw[4], lo_h = 1 << 30, lo_w = 1 << 30, hi_h = -(1 << 30), hi_w = -(1 << 30), max_ph = 0, max_pw = 0;
  for (int cls = 0; cls < 4; ++cls) {
    a.h0[cls] = a.w0[cls] = a.ph[cls] = a.pw[cls] = a.dh[cls] = a.dw[cls] = 0;
    ah[cls] = aw[cls] = 0;
  }
  for (int cls = 0; cls < S * S; ++cls) {
    const int rh = cls / S, rw = cls % S;
    const int nkh = rh < K ? (K - rh + S - 1) / S : 0, nkw = rw < K ? (K - rw + S - 1) / S : 0;
    const int h0 = ((rh - g.PADT) % S + S) % S, w0 = ((rw - g.PADL) % S + S) % S;
    a.h0[cls] = h0; a.w0[cls] = w0;
    a.ph[cls] = h0 < g.IH ? (g.IH - h0 + S - 1) / S : 0;
    a.pw[cls] = w0 < g.IW ? (g.IW - w0 + S - 1) / S : 0;
    if (nkh == 0 || nkw == 0) {
      if (!beta && a.ph[cls] > 0 && a.pw[cls] > 0) return kNotHere;   // a class without taps would need a zero fill
      a.ph[cls] = a.pw[cls] = 0;
      continue;
    }
    ah[cls] = (h0 + g.PADT - rh) / S;   // exact: h0 + PADT = rh (mod S)
    aw[cls] = (w0 + g.PADL - rw) / S;
    lo_h = std::min(lo_h, ah[cls] - (nkh - 1)); hi_h = std::max(hi_h, ah[cls]);
    lo_w = std::min(lo_w, aw[cls] - (nkw - 1)); hi_w = std::max(hi_w, aw[cls]);
    max_ph = std::max(max_ph, a.ph[cls]); max_pw = std::max(max_pw, a.pw[cls]);
  }
  *grid_x = 0;
  a.th = a.tw = a.tiles_x = 0;
  a.oh_base = a.ow_base = 0;
  a.beta = beta ? 1 : 0;
  if (max_ph == 0 || max_pw == 0) return LNN_OK;   // nothing to compute
  for (int cls = 0; cls < S * S; ++cls) { a.dh[cls] = ah[cls] - lo_h; a.dw[cls] = aw[cls] - lo_w; }
  a.oh_base = lo_h; a.ow_base = lo_w;
  a.th = kDsTile + hi_h - lo_h; a.tw = kDsTile + hi_w - lo_w;
  const int tmax = kDsTile + (K + S - 1) / S + 1;
  if (a.th > tmax || a.tw > tmax) return kNotHere;
  a.tiles_x = (max_pw + kDsTile - 1) / kDsTile;
  *grid_x = a.tiles_x * ((max_ph + kDsTile - 1) / kDsTile);
  return LNN_OK;
}

static int launch_small_dgrad(DeviceCtx* ctx, const ConvGeom& g, const float* dY, const float* W, float* dX, int beta) {
  SmallDgradArgs a;
  int grid_x = 0;
  if (plan_small_dgrad(g, beta, a, &grid_x) == kNotHere) return kNotHere;
  if (grid_x == 0) return LNN_OK;
  const int K = g.KH, S = g.S, n_w = g.O * K * K * 4;
  int st = ensure_workspace(ctx, (size_t)n_w * sizeof(float));
  if (st != LNN_OK) return st;
  float* wc = static_cast<float*>(ctx->ws);
  hipLaunchKernelGGL(small_dgrad_weights, dim3((n_w + 255) / 256), dim3(256), 0, ctx->stream, wc, W, g.O, g.C, K, S);
  LNN_HIP(hipGetLastError());
  a.dY = dY; a.wc = wc; a.dX = dX;
  const dim3 grid((unsigned)grid_x, (unsigned)g.N), block(256);
#define LNN_DS(S_, K_)                                                                                        \
  do {                                                                                                        \
    if (g.C == 3) hipLaunchKernelGGL((small_dgrad_kernel<S_, K_, 3>), grid, block, 0, ctx->stream, a);         \
    else hipLaunchKernelGGL((small_dgrad_kernel<S_, K_, 4>), grid, block, 0, ctx->stream, a);                  \
  } while (0)
  if (S == 1) { if (K == 1) LNN_DS(1, 1); else if (K == 3) LNN_DS(1, 3); else LNN_DS(1, 5); }
  else { if (K == 3) LNN_DS(2, 3); else if (K == 4) LNN_DS(2, 4); else if (K == 5) LNN_DS(2, 5); else LNN_DS(2, 7); }
#undef LNN_DS
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int conv_dgrad_path(const lnn_conv2d_desc* d, int beta, int compute_units, int* path, int32_t* tile_info) {
  ConvGeom g;
  int st = fill_geom(d, g);
  if (st != LNN_OK) return st;
  if (!path || compute_units <= 0) return set_error(LNN_ERR_INVALID, "conv2d_dgrad_path: null result pointer or no compute units");
  *path = g.O % BK == 0 ? LNN_DGRAD_PATH_MFMA_TAP : LNN_DGRAD_PATH_MFMA_TABLE;
  if (tile_info)
    for (int i = 0; i < 7; ++i) tile_info[i] = 0;
  if (stem_dgrad_applies(d, compute_units)) {
    *path = LNN_DGRAD_PATH_STEM_MFMA;
    return LNN_OK;
  }
  if (small_dgrad_applies(compute_units, g)) {
    SmallDgradArgs a;
    int grid_x = 0;
    if (plan_small_dgrad(g, beta, a, &grid_x) != kNotHere) {
      *path = LNN_DGRAD_PATH_VECTOR;
      if (tile_info && grid_x > 0) {
        const int K = g.KH, S = g.S;
        int lo_r = 1 << 30, lo_c = 1 << 30, hi_r = -1, hi_c = -1;
        for (int cls = 0; cls < S * S; ++cls) {
          const int nkh = ds_nk(K, S, cls / S), nkw = ds_nk(K, S, cls % S);
          if (nkh == 0 || nkw == 0) continue;
          // lane (ty, tx), ty, tx < 8, reads rows dh + 2*ty - (nkh-1) ... dh + 2*ty + 1, likewise columns
          lo_r = std::min(lo_r, a.dh[cls] - (nkh - 1)); hi_r = std::max(hi_r, a.dh[cls] + 2 * 7 + 1);
          lo_c = std::min(lo_c, a.dw[cls] - (nkw - 1)); hi_c = std::max(hi_c, a.dw[cls] + 2 * 7 + 1);
        }
        tile_info[0] = a.th; tile_info[1] = a.tw; tile_info[2] = kDsTile + (K + S - 1) / S + 1;
        tile_info[3] = lo_r; tile_info[4] = lo_c; tile_info[5] = hi_r; tile_info[6] = hi_c;
      }
    }
  }
  return LNN_OK;
}

// Whether the data gradient of this geometry reads the weights in the forward pass's permuted layout
// Wp[o][tap][c] (shared with the forward pass, made once per weight update by the caller or per call here).
bool dgrad_reads_permuted(const ConvGeom& g) { return g.O % BK == 0 && g.C % 4 == 0 && g.C > 4; }

int launch_conv_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* W, float* dX, int beta,
                      const float* Wp) {
  ConvGeom full;
  int st = fill_geom(d, full);
  if (st != LNN_OK) return st;
  const bool tapw = dgrad_reads_permuted(full);
  if (Wp && !tapw) return set_error(LNN_ERR_INVALID, "conv2d_dgrad: this geometry does not read permuted weights");
  if (Wp && !aligned16(Wp)) return set_error(LNN_ERR_INVALID, "conv2d_dgrad: permuted weights must be 16-byte aligned");
  if (!dY || (!W && !Wp) || !dX) return set_error(LNN_ERR_INVALID, "conv2d_dgrad: null pointer");
  const int S = full.S;
  if (S > 15) return set_error(LNN_ERR_UNSUPPORTED, "conv2d_dgrad: stride > 15");
  if (!Wp && stem_dgrad_applies(d, ctx->cus)) return launch_stem_dgrad(ctx, d, dY, W, dX, beta);
  if (!tapw && small_dgrad_applies(ctx->cus, full)) {
    st = launch_small_dgrad(ctx, full, dY, W, dX, beta);
    if (st != kNotHere) return st;
  }
  st = reserve_tables(ctx, (size_t)S * S);
  if (st != LNN_OK) return st;
  const bool tap = full.O % BK == 0;
  // one stride-1 problem per class of input pixels (see ConvDgradB)
  std::vector<ConvArgs> cls;
  std::vector<PixelClass> pcs;
  std::vector<size_t> w_off;   // where each class's permuted weights start in the scratch buffer
  size_t w_bytes = 0;          // permuted weights of all classes, back to back
  for (int rh = 0; rh < S; ++rh)
    for (int rw = 0; rw < S; ++rw) {
      PixelClass pc;
      pc.rh = rh; pc.rw = rw;
      pc.h0 = ((rh - full.PADT) % S + S) % S;
      pc.w0 = ((rw - full.PADL) % S + S) % S;
      if (pc.h0 >= full.IH || pc.w0 >= full.IW) continue;   // no such pixels
      pc.nkh = pc.nkw = 0;
      for (int k = 0; k < full.KH; ++k) pc.nkh += k * full.D % S == rh;
      for (int k = 0; k < full.KW; ++k) pc.nkw += k * full.D % S == rw;
      const int nt = pc.nkh * pc.nkw;
      if (nt == 0 && beta) continue;                        // nothing to add; without beta the class is zero-filled
      ConvArgs a;
      a.ws_used = 0;
      a.w_iohw = 0;
      a.post = PostOp{nullptr, 0, 0.0f};
      a.g = full;
      ConvGeom& g = a.g;
      g.IH = (full.IH - pc.h0 + S - 1) / S;
      g.IW = (full.IW - pc.w0 + S - 1) / S;
      g.IHW = g.IH * g.IW;
      g.dIW = make_fastdiv(g.IW); g.dIHW = make_fastdiv(g.IHW);
      a.full_IW = full.IW; a.full_IHW = full.IHW; a.cls_s = S; a.cls_org = pc.h0 * full.IW + pc.w0;
      a.tab = nullptr;
      a.X = dY; a.W = W; a.Out = dX;
      a.bytesX = (uint32_t)((uint64_t)g.N * g.O * g.OHW * 4);
      a.bytesW = (uint32_t)((uint64_t)g.O * g.C * (tap && !tapw ? nt : g.KK) * 4);
      a.bytesOut = (uint32_t)((uint64_t)g.N * g.C * full.IHW * 4);
      a.M = g.C; a.Ncols = g.N * g.IHW; a.K = g.O * nt;
      a.beta = beta ? 1 : 0;
      a.dC = make_fastdiv(1);
      st = get_table(ctx, full, tap ? 2 : 1, pc, &a.tab);
      if (st != LNN_OK) return st;
      if (tap && !tapw) {
        w_off.push_back(w_bytes);
        w_bytes += ((size_t)(a.bytesW ? a.bytesW : 4) + 255) & ~(size_t)255;
      }
      cls.push_back(a);
      pcs.push_back(pc);
    }
  if (cls.empty()) return LNN_OK;
  // scratch: permuted weights of every class, then room for the split-K partial sums of one batch of
  // classes (at most one full 32768-element sub-tile per workgroup slot)
  const int nc = (int)cls.size();
  const size_t part_bytes = (size_t)ctx->cus * 32768 * sizeof(float) + 256 * (size_t)nc;
  // A class that fills the chip on its own (several units of output per workgroup) gains nothing from
  // sharing it; neither do more classes than one launch holds (stride > 2).
  const int unit_cols = cls[0].M > 64 ? 32 : (cls[0].M > 32 ? 64 : 128);
  const long long units0 = (long long)((cls[0].M + 127) / 128) * ((cls[0].Ncols + unit_cols - 1) / unit_cols);
  const bool one_by_one = nc > kMaxBatch || units0 >= 4ll * ctx->cus;
  if (tapw) {
    // every class reads the same copy of the weights, Wp[o][tap][c]: the caller's, the weights themselves (a 1x1
    // kernel already has that layout), or one made here at the front of the scratch buffer
    const float* wsrc = Wp ? Wp : (full.KK == 1 && aligned16(W) ? W : nullptr);
    if (!wsrc) w_bytes = ((size_t)full.O * full.C * full.KK * sizeof(float) + 255) & ~(size_t)255;
    st = ensure_workspace(ctx, w_bytes + part_bytes);
    if (st != LNN_OK) return st;
    if (!wsrc) {
      size_t used = 0;
      st = permuted_weights(ctx, full, W, 0, PixelClass{}, &wsrc, &used);
      if (st != LNN_OK) return st;
    }
    for (int i = 0; i < nc; ++i) {
      cls[i].W = wsrc;
      cls[i].ws_used = w_bytes;
    }
    if (!one_by_one) return launch_classes_by_m<PASS_DGRAD_TAPW>(ctx, cls, w_bytes);
    for (int i = 0; i < nc; ++i) {
      st = launch_by_m<PASS_DGRAD_TAPW>(ctx, cls[i], true);
      if (st != LNN_OK) return st;
    }
    return LNN_OK;
  }
  if (one_by_one) {
    // one after the other, each with the whole chip.  All the scratch any class needs (its permuted weights,
    // then partial sums) is reserved before the first launch: a failed allocation then leaves dX untouched, so
    // the caller may free memory and repeat the call.
    size_t w_most = 0;
    for (int i = 0; i < nc; ++i) w_most = std::max<size_t>(w_most, ((size_t)(cls[i].bytesW ? cls[i].bytesW : 4) + 255) & ~(size_t)255);
    st = ensure_workspace(ctx, w_most + part_bytes);
    if (st != LNN_OK) return st;
    for (int i = 0; i < nc; ++i) {
      ConvArgs& a = cls[i];
      if (tap) {
        st = permuted_weights(ctx, full, W, 1, pcs[i], &a.W, &a.ws_used);
        if (st != LNN_OK) return st;
        st = launch_by_m<PASS_DGRAD_TAP>(ctx, a, true);
      } else {
        a.ws_used = 0;
        st = launch_by_m<PASS_DGRAD>(ctx, a, true);
      }
      if (st != LNN_OK) return st;
    }
    return LNN_OK;
  }
  st = ensure_workspace(ctx, w_bytes + part_bytes);
  if (st != LNN_OK) return st;
  if (tap) {
    // every class's weights in one launch (nc <= kMaxBatch <= 4 here)
    PermuteBatch pb;
    int most = 0;
    for (int i = 0; i < 4; ++i) {
      const int j = i < nc ? i : 0;
      pb.wp[i] = reinterpret_cast<float*>(static_cast<char*>(ctx->ws) + w_off[j]);
      pb.pc[i] = pcs[j];
      if (i < nc) {
        const int n = full.O * full.C * pcs[i].nkh * pcs[i].nkw;
        most = n > most ? n : most;
        cls[i].W = pb.wp[i];
      }
    }
    if (most > 0) {
      hipLaunchKernelGGL(permute_weights_classes, dim3((most + 255) / 256, nc), dim3(256), 0, ctx->stream, pb, W, full.O,
                         full.C, full.KK, full);
      LNN_HIP(hipGetLastError());
    }
  }
  return tap ? launch_classes_by_m<PASS_DGRAD_TAP>(ctx, cls, w_bytes) : launch_classes_by_m<PASS_DGRAD>(ctx, cls, w_bytes);
}

}  // namespace lnn
