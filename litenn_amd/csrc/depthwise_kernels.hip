// Depthwise convolution: one filter per channel, no contraction over channels,
// so there is no GEMM in it and nothing for the matrix cores: 2*KH*KW flop per
// output element against 8 bytes of compulsory traffic.  Three bandwidth-bound
// kernels with one thread per produced element.
//
//   forward  Y[n,c,oh,ow]  = sum_{kh,kw} X[n,c,oh*S-PT+kh*D, ow*S-PL+kw*D] * K[c,kh,kw]
//   dgrad    dX[n,c,ih,iw] = sum over the taps with (ih+PT-kh*D) % S == 0 (likewise w) of
//                            dY[n,c,(ih+PT-kh*D)/S,(iw+PL-kw*D)/S] * K[c,kh,kw]
//   wgrad    dK[c,kh,kw]   = sum_{n,oh,ow} X[n,c,oh*S-PT+kh*D, ow*S-PL+kw*D] * dY[n,c,oh,ow]
//
// Consecutive threads own consecutive pixels of one image row, so every tap is
// a coalesced, shifted read of that row; the KH*KW re-reads of a row hit L1/L2.
#include "common.hpp"
#include "tile_engine.hpp"

// the tap loops carry an unroll request that only the compile-time filter sizes can honour
#pragma clang diagnostic ignored "-Wpass-failed"

namespace lnn {

struct DwGeom {
  int N, C, IH, IW, KH, KW, OH, OW, PADL, PADT, S, D;
  FastDiv dOW, dIW, dS;
};

// All three kernels work on one band of rows of one (image, channel) plane per block: the rows of the
// source plane(s) that the band touches are copied to LDS once with coalesced reads, then every thread
// produces elements from LDS.  Each input element leaves HBM once.
// LDSF floats of source rows per block: 4096 (16 KB, eight blocks per compute unit hide the copy latency)
// when a useful band fits, else 32768 (128 KB, one block) for very wide rows.
constexpr int kDwSmall = 4096, kDwLarge = 32768;
// kernel gradient with very wide rows: X rows and dY rows share the LDS (120 KB), both multiples of 256 floats
constexpr int kDwWgradX = 20480, kDwWgradY = 10240;

// Rows row_lo..row_hi of a plane are one contiguous run of floats.  They go to LDS with global->LDS transfers,
// which occupy no registers and are all in flight at once: one memory latency per block.  A transfer that
// starts inside the run and ends past it deposits zeros, so the LDS array must hold the run rounded up to
// 256 floats.  dw_copy_wait() before the block barrier.
__device__ __forceinline__ void dw_copy_rows(float* lds, const float* __restrict__ plane, int row_lo, int row_hi, int W) {
  const int n = (row_hi - row_lo + 1) * W;
  const float* src = plane + (size_t)row_lo * W;
  const rsrc_t rs = make_rsrc(src, (uint32_t)n * 4u);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (((reinterpret_cast<uintptr_t>(src) | (uintptr_t)(n * 4)) & 15) == 0) {   // block-uniform
    for (int c = wave * 256; c < n; c += 1024) buf_load_lds16(rs, lds + c, (uint32_t)(c + lane * 4) * 4u, 0);
  } else {
    for (int c = wave * 64; c < n; c += 256) buf_load_lds4(rs, lds + c, (uint32_t)(c + lane) * 4u, 0);
  }
}
__device__ __forceinline__ void dw_copy_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// KS > 0: square KS x KS filter known at compile time (tap loops unrolled, filter in registers);
// KS == 0: any KH x KW, filter read from LDS.
template <int KS>
struct DwFilter {
  float k[KS > 0 ? KS * KS : 1];
  const float* lk;
  int KH, KW;
  __device__ __forceinline__ void load(const float* __restrict__ kp, float* ldsk, int kh, int kw) {
    KH = KS > 0 ? KS : kh;
    KW = KS > 0 ? KS : kw;
    if (KS > 0) {
#pragma unroll
      for (int i = 0; i < KS * KS; ++i) k[i] = kp[i];
    } else {
      for (int i = threadIdx.x; i < kh * kw; i += 256) ldsk[i] = kp[i];
      lk = ldsk;
    }
  }
  __device__ __forceinline__ float at(int kh, int kw) const { return KS > 0 ? k[kh * KS + kw] : lk[kh * KW + kw]; }
};
constexpr int kDwMaxTaps = 1024;   // runtime-sized filters of up to 32 x 32 taps

// Stride 1, dilation 1, compile-time filter: dst[r][c] = sum over (a, b) of src[r - pt + a][c - pl + b] * w(a, b).
// A thread keeps one column and a contiguous run of the band's rows, and slides a KS x KS window of source values
// down the column: a produced element costs KS LDS reads instead of KS * KS.  A source element outside the plane
// reads element 0 of the band and is replaced by zero.
template <int KS>
struct DwColumn {
  int cw[KS > 0 ? KS : 1];
  bool okw[KS > 0 ? KS : 1];
  __device__ __forceinline__ void init(int c, int pl, int srcW) {
#pragma unroll
    for (int b = 0; b < KS; ++b) {
      const int s = c - pl + b;
      okw[b] = (uint32_t)s < (uint32_t)srcW;
      cw[b] = okw[b] ? s : 0;
    }
  }
  __device__ __forceinline__ void load_row(const float* lds, int lo, int srcH, int srcW, int sr, float* out) const {
    const bool okh = (uint32_t)sr < (uint32_t)srcH;
    const float* row = lds + (okh ? (sr - lo) * srcW : 0);
    // the reads stay unconditional (the empty statement uses every value), so a row's reads are in flight together
    float x[KS > 0 ? KS : 1];
#pragma unroll
    for (int b = 0; b < KS; ++b) x[b] = row[cw[b]];
#pragma unroll
    for (int b = 0; b < KS; ++b) asm volatile("" : "+v"(x[b]));
#pragma unroll
    for (int b = 0; b < KS; ++b) out[b] = (okh && okw[b]) ? x[b] : 0.0f;
  }
};

// rows [ra, rb) of the band for this thread's row group, and whether the thread takes part at all
__device__ __forceinline__ bool dw_row_group(int width, int r0, int r1, int& tc, int& ncol, int& ra, int& rb) {
  ncol = width < 256 ? width : 256;
  const int ngrp = 256 / ncol, tg = threadIdx.x / ncol;
  tc = threadIdx.x - tg * ncol;
  const int rpg = (r1 - r0 + ngrp - 1) / ngrp;
  ra = r0 + tg * rpg;
  rb = ra + rpg < r1 ? ra + rpg : r1;
  return tg < ngrp && ra < rb;
}

template <int KS, bool FLIP>
__device__ __forceinline__ void dw_unit_rows(const float* lds, int lo, int srcH, int srcW, int dstW, int r0, int r1,
                                             int pt, int pl, const float* k, float* __restrict__ dst, int beta) {
  constexpr int T = KS > 0 ? KS : 1;
  int tc, ncol, ra, rb;
  if (!dw_row_group(dstW, r0, r1, tc, ncol, ra, rb)) return;
  float w[T * T];
#pragma unroll
  for (int i = 0; i < KS * KS; ++i) w[i] = FLIP ? k[KS * KS - 1 - i] : k[i];
  for (int c = tc; c < dstW; c += ncol) {
    DwColumn<KS> col;
    col.init(c, pl, srcW);
    float win[T][T];
#pragma unroll
    for (int j = 0; j + 1 < KS; ++j) col.load_row(lds, lo, srcH, srcW, ra - pt + j, win[j + 1]);
    auto row = [&](int r, float old) {
#pragma unroll
      for (int j = 0; j + 1 < KS; ++j)
#pragma unroll
        for (int b = 0; b < KS; ++b) win[j][b] = win[j + 1][b];
      col.load_row(lds, lo, srcH, srcW, r - pt + KS - 1, win[T - 1]);   // T = KS in every instantiation that runs
      float v = 0.0f;
#pragma unroll
      for (int a = 0; a < KS; ++a)
#pragma unroll
        for (int b = 0; b < KS; ++b) v += win[a][b] * w[a * KS + b];
      dst[r * dstW + c] = old + v;
    };
    if (!beta) {
      for (int r = ra; r < rb; ++r) row(r, 0.0f);
    } else {
      // '+=': the old values of a run of rows are requested together, ahead of the arithmetic, so that the thread
      // waits for memory once per run and not once per row
      constexpr int RUN = 8;
      int r = ra;
      for (; r + RUN <= rb; r += RUN) {
        float old[RUN];
#pragma unroll
        for (int j = 0; j < RUN; ++j) old[j] = dst[(r + j) * dstW + c];
#pragma unroll
        for (int j = 0; j < RUN; ++j) row(r + j, old[j]);
      }
      if (r < rb) {   // the last, shorter run
        float old[RUN];
#pragma unroll
        for (int j = 0; j < RUN; ++j) old[j] = r + j < rb ? dst[(r + j) * dstW + c] : 0.0f;
#pragma unroll
        for (int j = 0; j < RUN; ++j)
          if (r + j < rb) row(r + j, old[j]);
      }
    }
  }
}

// forward: Y rows [r0, r1) of the plane from X rows [lo, hi]
template <int KS, int LDSF, bool UNIT>
__global__ __launch_bounds__(256) void dw_fwd_kernel(DwGeom g, const float* __restrict__ X, const float* __restrict__ K,
                                                     float* __restrict__ Y, int bands, int TH, int beta) {
  __shared__ __attribute__((aligned(16))) float lds[LDSF];
  __shared__ float ldsk[KS > 0 ? 1 : kDwMaxTaps];
  const int plane = blockIdx.x / bands, band = blockIdx.x - plane * bands;
  const int c = plane % g.C;
  const int r0 = band * TH, r1 = r0 + TH < g.OH ? r0 + TH : g.OH;
  int lo = r0 * g.S - g.PADT, hi = (r1 - 1) * g.S - g.PADT + (g.KH - 1) * g.D;
  lo = lo < 0 ? 0 : lo;
  hi = hi >= g.IH ? g.IH - 1 : hi;
  if (hi >= lo) dw_copy_rows(lds, X + (size_t)plane * g.IH * g.IW, lo, hi, g.IW);
  DwFilter<KS> f;
  f.load(K + (size_t)c * g.KH * g.KW, ldsk, g.KH, g.KW);
  dw_copy_wait();
  __syncthreads();
  float* yp = Y + (size_t)plane * g.OH * g.OW;
  if (KS > 0 && UNIT) {
    dw_unit_rows<KS, false>(lds, lo, g.IH, g.IW, g.OW, r0, r1, g.PADT, g.PADL, f.k, yp, beta);
    return;
  }
  if (KS > 0) {
    // A thread keeps one output column and walks down the band's rows: the column tests and offsets of the
    // KS taps are computed once, a row costs KS row tests and KS*KS guarded multiply-adds.
    const int ncol = g.OW < 256 ? g.OW : 256, ngrp = 256 / ncol;
    const int tc = threadIdx.x % ncol, tg = threadIdx.x / ncol;
    for (int ow = tc; ow < g.OW; ow += ncol) {
      if (tg >= ngrp) break;
      // a tap outside the image reads element 0 of the band instead and is dropped afterwards: every LDS
      // read of a row is unconditional, so all of them are in flight together
      int iw[KS > 0 ? KS : 1];
      bool okw[KS > 0 ? KS : 1];
#pragma unroll
      for (int kw = 0; kw < KS; ++kw) {
        const int w = ow * g.S - g.PADL + kw * g.D;
        okw[kw] = (uint32_t)w < (uint32_t)g.IW;
        iw[kw] = okw[kw] ? w : 0;
      }
      for (int oh = r0 + tg; oh < r1; oh += ngrp) {
        const int ih0 = oh * g.S - g.PADT;
        float x[KS > 0 ? KS * KS : 1];
        bool okh[KS > 0 ? KS : 1];
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) {
          const int ih = ih0 + kh * g.D;
          okh[kh] = (uint32_t)ih < (uint32_t)g.IH;
          const float* row = lds + (okh[kh] ? (ih - lo) * g.IW : 0);
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) x[kh * KS + kw] = row[iw[kw]];
        }
        float v = 0.0f;
#pragma unroll
        for (int kh = 0; kh < KS; ++kh)
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) v += (okh[kh] && okw[kw]) ? x[kh * KS + kw] * f.at(kh, kw) : 0.0f;
        const int o = oh * g.OW + ow;
        yp[o] = beta ? yp[o] + v : v;
      }
    }
    return;
  }
  const int n = (r1 - r0) * g.OW;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int r = (int)g.dOW.div((uint32_t)i), ow = i - r * g.OW, oh = r0 + r;
    const int ih0 = oh * g.S - g.PADT, iw0 = ow * g.S - g.PADL;
    float v = 0.0f;
    for (int kh = 0; kh < f.KH; ++kh) {
      const int ih = ih0 + kh * g.D;
      if ((uint32_t)ih < (uint32_t)g.IH) {
        const float* row = lds + (ih - lo) * g.IW;
        for (int kw = 0; kw < f.KW; ++kw) {
          const int iw = iw0 + kw * g.D;
          if ((uint32_t)iw < (uint32_t)g.IW) v += row[iw] * f.at(kh, kw);
        }
      }
    }
    const int o = oh * g.OW + ow;
    yp[o] = beta ? yp[o] + v : v;
  }
}
template <int KS, int LDSF, bool UNIT>
__global__ __launch_bounds__(256) void dw_dgrad_kernel(DwGeom g, const float* __restrict__ dY,
                                                       const float* __restrict__ K, float* __restrict__ dX, int bands,
                                                       int TH, int beta) {
  __shared__ __attribute__((aligned(16))) float lds[LDSF];
  const int plane = blockIdx.x / bands, band = blockIdx.x - plane * bands;
  const int c = plane % g.C;
  const int r0 = band * TH, r1 = r0 + TH < g.IH ? r0 + TH : g.IH;
  // output rows oh = (ih + PT - kh*D) / S for ih in [r0, r1)
  int lo = r0 + g.PADT - (g.KH - 1) * g.D, hi = (r1 - 1 + g.PADT) / g.S;
  lo = lo <= 0 ? 0 : (lo + g.S - 1) / g.S;
  hi = hi >= g.OH ? g.OH - 1 : hi;
  if (hi >= lo) dw_copy_rows(lds, dY + (size_t)plane * g.OH * g.OW, lo, hi, g.OW);
  __shared__ float ldsk[KS > 0 ? 1 : kDwMaxTaps];
  DwFilter<KS> f;
  f.load(K + (size_t)c * g.KH * g.KW, ldsk, g.KH, g.KW);
  dw_copy_wait();
  __syncthreads();
  float* xp = dX + (size_t)plane * g.IH * g.IW;
  if (KS > 0 && UNIT) {
    // dX[ih][iw] = sum dY[ih + PADT - kh][iw + PADL - kw] * k[kh][kw]: the same walk with the filter turned by 180 degrees
    dw_unit_rows<KS, true>(lds, lo, g.OH, g.OW, g.IW, r0, r1, KS - 1 - g.PADT, KS - 1 - g.PADL, f.k, xp, beta);
    return;
  }
  if (KS > 0) {
    // column walk as in the forward kernel: the output column of each tap and whether it exists are fixed per thread
    const int ncol = g.IW < 256 ? g.IW : 256, ngrp = 256 / ncol;
    const int tc = threadIdx.x % ncol, tg = threadIdx.x / ncol;
    for (int iw = tc; iw < g.IW; iw += ncol) {
      if (tg >= ngrp) break;
      int ow[KS > 0 ? KS : 1];
      bool okw[KS > 0 ? KS : 1];
#pragma unroll
      for (int kw = 0; kw < KS; ++kw) {
        const int nw = iw + g.PADL - kw * g.D;
        const int q = (int)g.dS.div((uint32_t)nw & 0x7fffffffu);
        okw[kw] = nw >= 0 && q * g.S == nw && q < g.OW;
        ow[kw] = okw[kw] ? q : 0;
      }
      for (int ih = r0 + tg; ih < r1; ih += ngrp) {
        float y[KS > 0 ? KS * KS : 1];
        bool okh[KS > 0 ? KS : 1];
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) {
          const int nh = ih + g.PADT - kh * g.D;
          const int oh = (int)g.dS.div((uint32_t)nh & 0x7fffffffu);
          okh[kh] = nh >= 0 && oh * g.S == nh && oh < g.OH;
          const float* row = lds + (okh[kh] ? (oh - lo) * g.OW : 0);
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) y[kh * KS + kw] = row[ow[kw]];
        }
        float v = 0.0f;
#pragma unroll
        for (int kh = 0; kh < KS; ++kh)
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) v += (okh[kh] && okw[kw]) ? y[kh * KS + kw] * f.at(kh, kw) : 0.0f;
        const int o = ih * g.IW + iw;
        xp[o] = beta ? xp[o] + v : v;
      }
    }
    return;
  }
  const int n = (r1 - r0) * g.IW;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int r = (int)g.dIW.div((uint32_t)i), iw = i - r * g.IW, ih = r0 + r;
    float v = 0.0f;
    for (int kh = 0; kh < f.KH; ++kh) {
      const int nh = ih + g.PADT - kh * g.D;
      const int oh = (int)g.dS.div((uint32_t)nh & 0x7fffffffu);
      if (nh >= 0 && oh * g.S == nh && oh < g.OH) {
        const float* row = lds + (oh - lo) * g.OW;
        for (int kw = 0; kw < f.KW; ++kw) {
          const int nw = iw + g.PADL - kw * g.D;
          const int ow = (int)g.dS.div((uint32_t)nw & 0x7fffffffu);
          if (nw >= 0 && ow * g.S == nw && ow < g.OW) v += row[ow] * f.at(kh, kw);
        }
      }
    }
    const int o = ih * g.IW + iw;
    xp[o] = beta ? xp[o] + v : v;
  }
}

// Kernel gradient, compile-time filter: adds X * dY of the dY rows [r0, r1) held in ldsy (row r0 first) and the X
// rows from lo on held in ldsx to the thread's running sum per tap.
template <int KS, bool UNIT>
__device__ __forceinline__ void dw_wgrad_accumulate(const DwGeom& g, const float* ldsx, const float* ldsy, int r0, int r1,
                                                    int lo, float* acc) {
  constexpr int T = KS > 0 ? KS * KS : 1;
  int tc, ncol, ra, rb;
  const bool active = dw_row_group(g.OW, r0, r1, tc, ncol, ra, rb);
  if (UNIT && active) {
    // the window of X slides down the column with the output row; each of its elements meets the row's dY value
    for (int ow = tc; ow < g.OW; ow += ncol) {
      DwColumn<KS> col;
      col.init(ow, g.PADL, g.IW);
      float win[KS > 0 ? KS : 1][KS > 0 ? KS : 1];
#pragma unroll
      for (int j = 0; j + 1 < KS; ++j) col.load_row(ldsx, lo, g.IH, g.IW, ra - g.PADT + j, win[j + 1]);
      for (int oh = ra; oh < rb; ++oh) {
#pragma unroll
        for (int j = 0; j + 1 < KS; ++j)
#pragma unroll
          for (int b = 0; b < KS; ++b) win[j][b] = win[j + 1][b];
        col.load_row(ldsx, lo, g.IH, g.IW, oh - g.PADT + KS - 1, win[KS - 1]);
        const float dyv = ldsy[(oh - r0) * g.OW + ow];
#pragma unroll
        for (int a = 0; a < KS; ++a)
#pragma unroll
          for (int b = 0; b < KS; ++b) acc[a * KS + b] += win[a][b] * dyv;
      }
    }
  }
  if (!UNIT) {
    const int ngrp = 256 / ncol, tg = threadIdx.x / ncol;
    for (int ow = tc; ow < g.OW; ow += ncol) {
      if (tg >= ngrp) break;
      int iw[T];
      bool okw[T];
#pragma unroll
      for (int kw = 0; kw < KS; ++kw) {
        const int w = ow * g.S - g.PADL + kw * g.D;
        okw[kw] = (uint32_t)w < (uint32_t)g.IW;
        iw[kw] = okw[kw] ? w : 0;
      }
      for (int r = tg; r < r1 - r0; r += ngrp) {
        const int ih0 = (r0 + r) * g.S - g.PADT;
        const float dyv = ldsy[r * g.OW + ow];
        float x[T];
        bool okh[T];
#pragma unroll
        for (int kh = 0; kh < KS; ++kh) {
          const int ih = ih0 + kh * g.D;
          okh[kh] = (uint32_t)ih < (uint32_t)g.IH;
          const float* row = ldsx + (okh[kh] ? (ih - lo) * g.IW : 0);
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) x[kh * KS + kw] = row[iw[kw]];
        }
#pragma unroll
        for (int kh = 0; kh < KS; ++kh)
#pragma unroll
          for (int kw = 0; kw < KS; ++kw) acc[kh * KS + kw] += (okh[kh] && okw[kw]) ? x[kh * KS + kw] * dyv : 0.0f;
      }
    }
  }
}

// Sum of every tap's running sums over the block, in a fixed order: wavefront butterflies of all taps side by side
// (their exchanges overlap), then the four wavefront sums.
template <int T>
__device__ __forceinline__ void dw_reduce_taps(float* acc, float* out) {
  __shared__ float red2[4][T];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float got[T];
#pragma unroll
    for (int t = 0; t < T; ++t) got[t] = __shfl_xor(acc[t], o, 64);
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] += got[t];
  }
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int t = 0; t < T; ++t) red2[threadIdx.x >> 6][t] = acc[t];
  }
  __syncthreads();
  if (threadIdx.x < T) out[threadIdx.x] = (red2[0][threadIdx.x] + red2[1][threadIdx.x]) + (red2[2][threadIdx.x] + red2[3][threadIdx.x]);
}

// kernel gradient: block (plane, band) holds dY rows [r0, r1) and the X rows under them and writes, per tap,
// the sum of X * dY over the band to part[(plane*bands + band)*KK + tap]
template <int KS, int LDSF, int LDSY, bool UNIT>
__global__ __launch_bounds__(256) void dw_wgrad_kernel(DwGeom g, const float* __restrict__ X,
                                                       const float* __restrict__ dY, float* __restrict__ part,
                                                       int bands, int TH) {
  __shared__ __attribute__((aligned(16))) float ldsx[LDSF];
  __shared__ __attribute__((aligned(16))) float ldsy[LDSY];
  __shared__ float red[4];
  const int plane = blockIdx.x / bands, band = blockIdx.x - plane * bands;
  const int r0 = band * TH, r1 = r0 + TH < g.OH ? r0 + TH : g.OH;
  int lo = r0 * g.S - g.PADT, hi = (r1 - 1) * g.S - g.PADT + (g.KH - 1) * g.D;
  lo = lo < 0 ? 0 : lo;
  hi = hi >= g.IH ? g.IH - 1 : hi;
  if (hi >= lo) dw_copy_rows(ldsx, X + (size_t)plane * g.IH * g.IW, lo, hi, g.IW);
  dw_copy_rows(ldsy, dY + (size_t)plane * g.OH * g.OW, r0, r1 - 1, g.OW);
  dw_copy_wait();
  __syncthreads();
  const int n = (r1 - r0) * g.OW, KK = g.KH * g.KW;
  float* out = part + ((size_t)plane * bands + band) * KK;
  if (KS > 0) {
    constexpr int T = KS > 0 ? KS * KS : 1;
    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0f;
    dw_wgrad_accumulate<KS, UNIT>(g, ldsx, ldsy, r0, r1, lo, acc);
    dw_reduce_taps<T>(acc, out);
  } else {
    for (int kh = 0; kh < g.KH; ++kh)
      for (int kw = 0; kw < g.KW; ++kw) {
        float v = 0.0f;
        for (int i = threadIdx.x; i < n; i += 256) {
          const int r = (int)g.dOW.div((uint32_t)i), ow = i - r * g.OW;
          const int ih = (r0 + r) * g.S - g.PADT + kh * g.D, iw = ow * g.S - g.PADL + kw * g.D;
          if ((uint32_t)ih < (uint32_t)g.IH && (uint32_t)iw < (uint32_t)g.IW) v += ldsx[(ih - lo) * g.IW + iw] * ldsy[i];
        }
        // wavefront butterfly, then the four wavefront sums in a fixed order
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        if (threadIdx.x == 0) out[kh * g.KW + kw] = (red[0] + red[1]) + (red[2] + red[3]);
        __syncthreads();
      }
  }
}


// Kernel gradient when a whole X plane and dY plane fit in LDS twice: block (slice, channel) walks its images'
// planes of that channel, the transfers of the next plane running while the current one is accumulated, and reduces
// once at the end: part[(slice*C + c)*KK + tap].  stage = floats per LDS stage, xf = floats reserved for the X plane.
template <int KS, bool UNIT>
__global__ __launch_bounds__(256) void dw_wgrad_planes_kernel(DwGeom g, const float* __restrict__ X,
                                                              const float* __restrict__ dY, float* __restrict__ part,
                                                              int slices, int stage, int xf) {
  extern __shared__ __attribute__((aligned(16))) float dw_lds[];
  constexpr int T = KS > 0 ? KS * KS : 1;
  const int c = blockIdx.x % g.C, sl = blockIdx.x / g.C;
  const int n0 = (int)((long long)g.N * sl / slices), n1 = (int)((long long)g.N * (sl + 1) / slices);
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.0f;
  auto fetch = [&](int n, int st) {
    const size_t plane = (size_t)n * g.C + c;
    dw_copy_rows(dw_lds + st * stage, X + plane * g.IH * g.IW, 0, g.IH - 1, g.IW);
    dw_copy_rows(dw_lds + st * stage + xf, dY + plane * g.OH * g.OW, 0, g.OH - 1, g.OW);
  };
  if (n0 < n1) fetch(n0, 0);
  for (int n = n0; n < n1; ++n) {
    const int st = (n - n0) & 1;
    dw_copy_wait();
    __syncthreads();   // plane n has landed for every wavefront, and every wavefront is done with plane n - 1
    if (n + 1 < n1) fetch(n + 1, st ^ 1);
    dw_wgrad_accumulate<KS, UNIT>(g, dw_lds + st * stage, dw_lds + st * stage + xf, 0, g.OH, 0, acc);
  }
  dw_reduce_taps<T>(acc, part + ((size_t)sl * g.C + c) * T);
}

// dK[c][tap] (+)= sum over images and bands, in a fixed order.  One block per channel: thread (j, tap) adds every
// J-th (image, band) entry of its tap, then the J running sums of a tap are added in ascending j.
__global__ __launch_bounds__(256) void dw_wgrad_finish_kernel(float* __restrict__ dK, const float* __restrict__ part,
                                                              int C, int KK, int N, int bands, int beta) {
  __shared__ float red[256];
  const int c = blockIdx.x, E = N * bands;
  for (int t0 = 0; t0 < KK; t0 += 256) {
    const int tl = KK - t0 < 256 ? KK - t0 : 256, J = 256 / tl;
    const int j = threadIdx.x / tl, tap = t0 + threadIdx.x - j * tl;
    float v = 0.0f;
    if (j < J)
      for (int e = j; e < E; e += J) {
        const int n = e / bands, b = e - n * bands;
        v += part[(((size_t)n * C + c) * bands + b) * KK + tap];
      }
    red[threadIdx.x] = v;
    __syncthreads();
    if (threadIdx.x < tl) {
      float s = 0.0f;
      for (int q = 0; q < J; ++q) s += red[q * tl + threadIdx.x];
      float* o = dK + (size_t)c * KK + tap;
      *o = beta ? *o + s : s;
    }
    __syncthreads();
  }
}

static int dw_geom(const lnn_conv2d_desc* d, DwGeom& g, const char* who) {
  if (!d) return set_error(LNN_ERR_INVALID, std::string(who) + ": null descriptor");
  const int v[] = {d->N, d->C, d->IH, d->IW, d->O, d->KH, d->KW, d->OH, d->OW, d->stride, d->dilation};
  for (int x : v)
    if (x <= 0) return set_error(LNN_ERR_INVALID, std::string(who) + ": non-positive dimension in descriptor");
  if (d->PADL < 0 || d->PADT < 0) return set_error(LNN_ERR_INVALID, std::string(who) + ": negative padding");
  if (d->O != d->C) return set_error(LNN_ERR_INVALID, std::string(who) + ": depthwise needs O == C");
  const uint64_t xb = (uint64_t)d->N * d->C * d->IH * d->IW * 4, yb = (uint64_t)d->N * d->C * d->OH * d->OW * 4;
  if (xb > kMaxTensorBytes || yb > kMaxTensorBytes)
    return set_error(LNN_ERR_UNSUPPORTED, std::string(who) + ": a tensor of 2 GiB or more");
  g.N = d->N; g.C = d->C; g.IH = d->IH; g.IW = d->IW; g.KH = d->KH; g.KW = d->KW; g.OH = d->OH; g.OW = d->OW;
  g.PADL = d->PADL; g.PADT = d->PADT; g.S = d->stride; g.D = d->dilation;
  g.dOW = make_fastdiv(g.OW); g.dIW = make_fastdiv(g.IW); g.dS = make_fastdiv(g.S);
  if ((uint64_t)d->N * d->C > 0x7fffffffull / 64) return set_error(LNN_ERR_UNSUPPORTED, std::string(who) + ": too many planes");
  return LNN_OK;
}

// Rows of the produced plane per block such that the source rows they touch fit in `floats` of LDS:
// src_rows(TH) = (TH - 1) * num / den + extra + 1 rows of `width` floats.  0 if even one row does not fit.
static int dw_band_rows(int out_rows, int width, long long num, long long den, long long extra, int floats) {
  int th = out_rows;
  while (th >= 1 && (((long long)(th - 1) * num) / den + extra + 1) * width > floats) th = th > 8 ? th * 3 / 4 : th - 1;
  return th;
}

int launch_dw_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* K, float* Y, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_fwd");
  if (st != LNN_OK) return st;
  if (!X || !K || !Y) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_fwd: null pointer");
  int TH = dw_band_rows(g.OH, g.IW, g.S, 1, (long long)(g.KH - 1) * g.D, kDwSmall);
  const bool small = TH >= 8 || TH >= g.OH;
  if (!small) TH = dw_band_rows(g.OH, g.IW, g.S, 1, (long long)(g.KH - 1) * g.D, kDwLarge);
  if (TH < 1) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d_fwd: image rows wider than the LDS band");
  const int bands = (g.OH + TH - 1) / TH;
  if (g.KH * g.KW > kDwMaxTaps) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d: more than 1024 taps");
  const dim3 grid((unsigned)(g.N * g.C * bands)), block(256);
  const int b = beta ? 1 : 0;
#define LNN_DW_LAUNCH(KS, UNIT)                                                                                  \
  do {                                                                                                     \
    if (small) hipLaunchKernelGGL((dw_fwd_kernel<KS, kDwSmall, UNIT>), grid, block, 0, ctx->stream, g, X, K, Y, bands, TH, b); \
    else hipLaunchKernelGGL((dw_fwd_kernel<KS, kDwLarge, UNIT>), grid, block, 0, ctx->stream, g, X, K, Y, bands, TH, b);       \
  } while (0)
  const bool unit = g.S == 1 && g.D == 1;   // sliding-window kernels
  if (g.KH == g.KW && g.KH == 3) { if (unit) LNN_DW_LAUNCH(3, true); else LNN_DW_LAUNCH(3, false); }
  else if (g.KH == g.KW && g.KH == 5) { if (unit) LNN_DW_LAUNCH(5, true); else LNN_DW_LAUNCH(5, false); }
  else if (g.KH == g.KW && g.KH == 1) { if (unit) LNN_DW_LAUNCH(1, true); else LNN_DW_LAUNCH(1, false); }
  else LNN_DW_LAUNCH(0, false);
#undef LNN_DW_LAUNCH
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_dw_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* K, float* dX, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_dgrad");
  if (st != LNN_OK) return st;
  if (!dY || !K || !dX) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_dgrad: null pointer");
  // TH rows of dX touch at most (TH - 1 + (KH-1)*D) / S + 2 rows of dY
  int TH = dw_band_rows(g.IH, g.OW, 1, g.S, (long long)((g.KH - 1) * g.D) / g.S + 2, kDwSmall);
  const bool small = TH >= 8 || TH >= g.IH;
  if (!small) TH = dw_band_rows(g.IH, g.OW, 1, g.S, (long long)((g.KH - 1) * g.D) / g.S + 2, kDwLarge);
  if (TH < 1) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d_dgrad: image rows wider than the LDS band");
  const int bands = (g.IH + TH - 1) / TH;
  if (g.KH * g.KW > kDwMaxTaps) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d: more than 1024 taps");
  const dim3 grid((unsigned)(g.N * g.C * bands)), block(256);
  const int b = beta ? 1 : 0;
#define LNN_DW_LAUNCH(KS, UNIT)                                                                                    \
  do {                                                                                                       \
    if (small) hipLaunchKernelGGL((dw_dgrad_kernel<KS, kDwSmall, UNIT>), grid, block, 0, ctx->stream, g, dY, K, dX, bands, TH, b); \
    else hipLaunchKernelGGL((dw_dgrad_kernel<KS, kDwLarge, UNIT>), grid, block, 0, ctx->stream, g, dY, K, dX, bands, TH, b);       \
  } while (0)
  const bool unit = g.S == 1 && g.D == 1;   // sliding-window kernels
  if (g.KH == g.KW && g.KH == 3) { if (unit) LNN_DW_LAUNCH(3, true); else LNN_DW_LAUNCH(3, false); }
  else if (g.KH == g.KW && g.KH == 5) { if (unit) LNN_DW_LAUNCH(5, true); else LNN_DW_LAUNCH(5, false); }
  else if (g.KH == g.KW && g.KH == 1) { if (unit) LNN_DW_LAUNCH(1, true); else LNN_DW_LAUNCH(1, false); }
  else LNN_DW_LAUNCH(0, false);
#undef LNN_DW_LAUNCH
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_dw_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dK, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_wgrad");
  if (st != LNN_OK) return st;
  if (!X || !dY || !dK) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_wgrad: null pointer");
  const int KK = g.KH * g.KW;
  // Whole planes twice in LDS (at most 64 KB): the pipelined kernel, one reduction per block
  const int xf = (g.IH * g.IW + 255) / 256 * 256, yf = (g.OH * g.OW + 255) / 256 * 256, stage = xf + yf;
  const bool square = g.KH == g.KW && (g.KH == 1 || g.KH == 3 || g.KH == 5);
  if (square && (long long)g.IH * g.IW <= 8192 && (long long)g.OH * g.OW <= 8192 && 2 * stage * 4 <= 65536) {
    // as many blocks as the LDS holds at once (160 KB per compute unit), each walking several planes
    int per_cu = 160 * 1024 / (2 * stage * 4);
    per_cu = per_cu > 8 ? 8 : per_cu;
    int slices = (per_cu * ctx->cus + g.C - 1) / g.C;
    slices = slices > g.N ? g.N : slices;
    st = ensure_workspace(ctx, (size_t)slices * g.C * KK * sizeof(float));
    if (st != LNN_OK) return st;
    float* part = static_cast<float*>(ctx->ws);
    const dim3 grid((unsigned)(g.C * slices)), block(256);
    const size_t lds_bytes = (size_t)2 * stage * sizeof(float);
    const bool unit = g.S == 1 && g.D == 1;
#define LNN_DW_LAUNCH(KS)                                                                                          \
  do {                                                                                                             \
    if (unit) hipLaunchKernelGGL((dw_wgrad_planes_kernel<KS, true>), grid, block, lds_bytes, ctx->stream, g, X, dY, part, slices, stage, xf); \
    else hipLaunchKernelGGL((dw_wgrad_planes_kernel<KS, false>), grid, block, lds_bytes, ctx->stream, g, X, dY, part, slices, stage, xf);    \
  } while (0)
    if (g.KH == 3) LNN_DW_LAUNCH(3);
    else if (g.KH == 5) LNN_DW_LAUNCH(5);
    else LNN_DW_LAUNCH(1);
#undef LNN_DW_LAUNCH
    LNN_HIP(hipGetLastError());
    hipLaunchKernelGGL(dw_wgrad_finish_kernel, dim3((unsigned)g.C), dim3(256), 0, ctx->stream, dK, part, g.C, KK, slices, 1,
                       beta ? 1 : 0);
    LNN_HIP(hipGetLastError());
    return LNN_OK;
  }
  auto rows = [&](int xfloats, int yfloats) {
    int th = dw_band_rows(g.OH, g.IW, g.S, 1, (long long)(g.KH - 1) * g.D, xfloats);
    while (th >= 1 && (long long)th * g.OW > yfloats) --th;
    return th;
  };
  int TH = rows(kDwSmall, kDwSmall);
  const bool small = TH >= 8 || TH >= g.OH;
  if (!small) TH = rows(kDwWgradX, kDwWgradY);
  if (TH < 1) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d_wgrad: image rows wider than the LDS band");
  const int bands = (g.OH + TH - 1) / TH;
  const size_t need = (size_t)g.N * g.C * bands * KK * sizeof(float);
  if (need > kMaxTensorBytes) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d_wgrad: partial sums of 2 GiB or more");
  st = ensure_workspace(ctx, need);
  if (st != LNN_OK) return st;
  const dim3 grid((unsigned)(g.N * g.C * bands)), block(256);
  float* part = static_cast<float*>(ctx->ws);
#define LNN_DW_LAUNCH(KS, UNIT)                                                                                      \
  do {                                                                                                         \
    if (small) hipLaunchKernelGGL((dw_wgrad_kernel<KS, kDwSmall, kDwSmall, UNIT>), grid, block, 0, ctx->stream, g, X, dY, part, bands, TH); \
    else hipLaunchKernelGGL((dw_wgrad_kernel<KS, kDwWgradX, kDwWgradY, UNIT>), grid, block, 0, ctx->stream, g, X, dY, part, bands, TH); \
  } while (0)
  const bool unit = g.S == 1 && g.D == 1;   // sliding-window kernels
  if (g.KH == g.KW && g.KH == 3) { if (unit) LNN_DW_LAUNCH(3, true); else LNN_DW_LAUNCH(3, false); }
  else if (g.KH == g.KW && g.KH == 5) { if (unit) LNN_DW_LAUNCH(5, true); else LNN_DW_LAUNCH(5, false); }
  else if (g.KH == g.KW && g.KH == 1) { if (unit) LNN_DW_LAUNCH(1, true); else LNN_DW_LAUNCH(1, false); }
  else LNN_DW_LAUNCH(0, false);
#undef LNN_DW_LAUNCH
  LNN_HIP(hipGetLastError());
  hipLaunchKernelGGL(dw_wgrad_finish_kernel, dim3((unsigned)g.C), dim3(256), 0, ctx->stream, dK,
                     static_cast<const float*>(ctx->ws), g.C, KK, g.N, bands, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

}  // namespace lnn
