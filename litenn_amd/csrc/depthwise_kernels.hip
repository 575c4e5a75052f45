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

namespace lnn {

struct DwGeom {
  int N, C, IH, IW, KH, KW, OH, OW, PADL, PADT, S, D;
  FastDiv dOW, dOH, dIW, dIH, dC;
};

__global__ __launch_bounds__(256) void dw_fwd_kernel(DwGeom g, const float* __restrict__ X, const float* __restrict__ K,
                                                     float* __restrict__ Y, uint32_t n, int beta) {
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u) {
    const uint32_t q = g.dOW.div(i), ow = i - q * g.OW;
    const uint32_t nc = g.dOH.div(q), oh = q - nc * g.OH;           // nc = n*C + c
    const uint32_t c = nc - g.dC.div(nc) * g.C;
    const float* xp = X + (size_t)nc * g.IH * g.IW;
    const float* kp = K + (size_t)c * g.KH * g.KW;
    const int ih0 = (int)oh * g.S - g.PADT, iw0 = (int)ow * g.S - g.PADL;
    float v = 0.0f;
    for (int kh = 0; kh < g.KH; ++kh) {
      const int ih = ih0 + kh * g.D;
      if ((uint32_t)ih < (uint32_t)g.IH)
        for (int kw = 0; kw < g.KW; ++kw) {
          const int iw = iw0 + kw * g.D;
          if ((uint32_t)iw < (uint32_t)g.IW) v += xp[ih * g.IW + iw] * kp[kh * g.KW + kw];
        }
    }
    Y[i] = beta ? Y[i] + v : v;
  }
}

__global__ __launch_bounds__(256) void dw_dgrad_kernel(DwGeom g, const float* __restrict__ dY,
                                                       const float* __restrict__ K, float* __restrict__ dX, uint32_t n,
                                                       int beta, FastDiv dS) {
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += gridDim.x * 256u) {
    const uint32_t q = g.dIW.div(i), iw = i - q * g.IW;
    const uint32_t nc = g.dIH.div(q), ih = q - nc * g.IH;
    const uint32_t c = nc - g.dC.div(nc) * g.C;
    const float* yp = dY + (size_t)nc * g.OH * g.OW;
    const float* kp = K + (size_t)c * g.KH * g.KW;
    float v = 0.0f;
    for (int kh = 0; kh < g.KH; ++kh) {
      const int nh = (int)ih + g.PADT - kh * g.D;
      if (nh < 0) break;                       // later taps only move further up
      const uint32_t oh = dS.div((uint32_t)nh);
      if (oh * (uint32_t)g.S != (uint32_t)nh || oh >= (uint32_t)g.OH) continue;
      for (int kw = 0; kw < g.KW; ++kw) {
        const int nw = (int)iw + g.PADL - kw * g.D;
        if (nw < 0) break;
        const uint32_t ow = dS.div((uint32_t)nw);
        if (ow * (uint32_t)g.S == (uint32_t)nw && ow < (uint32_t)g.OW) v += yp[oh * g.OW + ow] * kp[kh * g.KW + kw];
      }
    }
    dX[i] = beta ? dX[i] + v : v;
  }
}

// grid (C, splits): block (c, s) sums its share of the N*OH*OW pixels of channel c for every tap and
// writes part[(c*splits + s)*KK + tap]; the shares are contiguous pixel ranges, the order of addition is fixed.
__global__ __launch_bounds__(256) void dw_wgrad_kernel(DwGeom g, const float* __restrict__ X,
                                                       const float* __restrict__ dY, float* __restrict__ part,
                                                       int splits) {
  __shared__ float red[4];
  const int c = blockIdx.x, s = blockIdx.y;
  const uint32_t OHW = (uint32_t)g.OH * g.OW, P = (uint32_t)g.N * OHW;
  const uint32_t p0 = (uint32_t)((uint64_t)P * s / splits), p1 = (uint32_t)((uint64_t)P * (s + 1) / splits);
  const FastDiv dOHW = g.dIH;   // the host passes the divider by OH*OW in this slot for this kernel
  for (int kh = 0; kh < g.KH; ++kh)
    for (int kw = 0; kw < g.KW; ++kw) {
      float v = 0.0f;
      for (uint32_t p = p0 + threadIdx.x; p < p1; p += 256u) {
        const uint32_t img = dOHW.div(p), rem = p - img * OHW;
        const uint32_t oh = g.dOW.div(rem), ow = rem - oh * g.OW;
        const int ih = (int)oh * g.S - g.PADT + kh * g.D, iw = (int)ow * g.S - g.PADL + kw * g.D;
        if ((uint32_t)ih < (uint32_t)g.IH && (uint32_t)iw < (uint32_t)g.IW)
          v += X[((size_t)img * g.C + c) * g.IH * g.IW + ih * g.IW + iw] * dY[((size_t)img * g.C + c) * OHW + rem];
      }
      // wavefront butterfly, then the four wavefront sums in a fixed order
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
      if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
      __syncthreads();
      if (threadIdx.x == 0)
        part[((size_t)c * splits + s) * (g.KH * g.KW) + kh * g.KW + kw] = (red[0] + red[1]) + (red[2] + red[3]);
      __syncthreads();
    }
}

__global__ void dw_wgrad_finish_kernel(float* __restrict__ dK, const float* __restrict__ part, int n, int KK, int splits,
                                       int beta) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;   // i = c*KK + tap
  if (i >= n) return;
  const int c = i / KK, tap = i - c * KK;
  float v = 0.0f;
  for (int s = 0; s < splits; ++s) v += part[((size_t)c * splits + s) * KK + tap];
  dK[i] = beta ? dK[i] + v : v;
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
  g.dOW = make_fastdiv(g.OW); g.dOH = make_fastdiv(g.OH); g.dIW = make_fastdiv(g.IW); g.dIH = make_fastdiv(g.IH);
  g.dC = make_fastdiv(g.C);
  return LNN_OK;
}

static dim3 dw_grid(uint32_t n, int cus) {
  uint64_t blocks = ((uint64_t)n + 255) / 256;
  const uint64_t cap = (uint64_t)cus * 32;
  return dim3((unsigned)(blocks > cap ? cap : (blocks < 1 ? 1 : blocks)));
}

int launch_dw_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* K, float* Y, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_fwd");
  if (st != LNN_OK) return st;
  if (!X || !K || !Y) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_fwd: null pointer");
  const uint32_t n = (uint32_t)((uint64_t)g.N * g.C * g.OH * g.OW);
  hipLaunchKernelGGL(dw_fwd_kernel, dw_grid(n, ctx->cus), dim3(256), 0, ctx->stream, g, X, K, Y, n, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_dw_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* K, float* dX, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_dgrad");
  if (st != LNN_OK) return st;
  if (!dY || !K || !dX) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_dgrad: null pointer");
  const uint32_t n = (uint32_t)((uint64_t)g.N * g.C * g.IH * g.IW);
  hipLaunchKernelGGL(dw_dgrad_kernel, dw_grid(n, ctx->cus), dim3(256), 0, ctx->stream, g, dY, K, dX, n, beta ? 1 : 0,
                     make_fastdiv(g.S));
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_dw_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dK, int beta) {
  DwGeom g;
  int st = dw_geom(d, g, "depthwise_conv2d_wgrad");
  if (st != LNN_OK) return st;
  if (!X || !dY || !dK) return set_error(LNN_ERR_INVALID, "depthwise_conv2d_wgrad: null pointer");
  const int KK = g.KH * g.KW;
  const uint64_t P = (uint64_t)g.N * g.OH * g.OW;
  // enough blocks to fill the chip a few times over, each with at least a few thousand pixels
  long long splits = ((long long)ctx->cus * 8 + g.C - 1) / g.C;
  if (splits > (long long)((P + 2047) / 2048)) splits = (long long)((P + 2047) / 2048);
  if (splits < 1) splits = 1;
  if (splits > 65535) splits = 65535;
  if (g.C > 0x7fffffff / KK) return set_error(LNN_ERR_UNSUPPORTED, "depthwise_conv2d_wgrad: kernel tensor too large");
  st = ensure_workspace(ctx, (size_t)g.C * splits * KK * sizeof(float));
  if (st != LNN_OK) return st;
  g.dIH = make_fastdiv((uint32_t)(g.OH * g.OW));   // see dw_wgrad_kernel
  hipLaunchKernelGGL(dw_wgrad_kernel, dim3(g.C, (unsigned)splits), dim3(256), 0, ctx->stream, g, X, dY,
                     static_cast<float*>(ctx->ws), (int)splits);
  LNN_HIP(hipGetLastError());
  const int n = g.C * KK;
  hipLaunchKernelGGL(dw_wgrad_finish_kernel, dim3((n + 255) / 256), dim3(256), 0, ctx->stream, dK,
                     static_cast<const float*>(ctx->ws), n, KK, (int)splits, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

}  // namespace lnn
