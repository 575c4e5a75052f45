// Convolution forward pass (and its fused bias / activation epilogue).
#include "conv_common.hpp"


namespace lnn {

// Which passes of a geometry read (forward, data gradient) the weights in the permuted layout Wp[o][tap][c], or can
// write (weight gradient) a gradient whose channel axes are swapped.  Host arithmetic only.
int conv_weights_plan(const lnn_conv2d_desc* d, int pass, int* yes) {
  ConvGeom g;
  int st = fill_geom(d, g);
  if (st != LNN_OK) return st;
  if (!yes) return set_error(LNN_ERR_INVALID, "conv2d_weights_plan: null result pointer");
  if (pass == LNN_PASS_FWD) *yes = g.C % BK == 0;
  else if (pass == LNN_PASS_DGRAD) *yes = g.O % BK == 0 && g.C % 4 == 0 && g.C > 4;
  else if (pass == LNN_PASS_WGRAD) *yes = wgrad_walkers_fit(g);
  else return set_error(LNN_ERR_INVALID, "conv2d_weights_plan: unknown pass");
  return LNN_OK;
}

int conv_fwd_path(const lnn_conv2d_desc* d, int compute_units, int* path) {
  ConvGeom g;
  int st = fill_geom(d, g);
  if (st != LNN_OK) return st;
  if (!path || compute_units <= 0) return set_error(LNN_ERR_INVALID, "conv2d_fwd_path: null result pointer or no compute units");
  *path = stem_fwd_applies(d, compute_units) ? LNN_FWD_PATH_STEM_PATCH : LNN_FWD_PATH_IMPLICIT_GEMM;
  return LNN_OK;
}

// Wp[o][kh*KW + kw][c] = W[o][c][kh][kw] (w_layout LNN_W_OIHW) or W[c][o][kh][kw] (LNN_W_IOHW)
int launch_permute_weights(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* W, int w_layout, float* Wp) {
  ConvGeom g;
  int st = fill_geom(d, g);
  if (st != LNN_OK) return st;
  if (!W || !Wp) return set_error(LNN_ERR_INVALID, "conv2d_permute_weights: null pointer");
  if (w_layout != LNN_W_OIHW && w_layout != LNN_W_IOHW) return set_error(LNN_ERR_INVALID, "conv2d_permute_weights: unknown layout");
  if (!aligned16(Wp)) return set_error(LNN_ERR_INVALID, "conv2d_permute_weights: the destination must be 16-byte aligned");
  return launch_permute(ctx, Wp, W, g, w_layout == LNN_W_OIHW ? 0 : 2, PixelClass{});
}

int launch_conv_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta,
                    const float* bias, int act, float slope, const float* Wp) {
  ConvArgs a;
  a.ws_used = 0;
  a.w_iohw = 0;
  a.post = PostOp{bias, act, slope};
  if (beta && a.post.any()) return set_error(LNN_ERR_INVALID, "conv2d_fwd: bias / activation cannot be combined with accumulation");
  int st = fill_geom(d, a.g);
  if (st != LNN_OK) return st;
  if (Wp && a.g.C % BK != 0) return set_error(LNN_ERR_INVALID, "conv2d_fwd: this geometry does not read permuted weights");
  if (Wp && !aligned16(Wp)) return set_error(LNN_ERR_INVALID, "conv2d_fwd: permuted weights must be 16-byte aligned");
  if (!X || (!W && !Wp) || !Y) return set_error(LNN_ERR_INVALID, "conv2d_fwd: null pointer");
  if (!Wp && stem_fwd_applies(d, ctx->cus)) return launch_stem_fwd(ctx, d, X, W, Y, beta, bias, act, slope);
  st = reserve_tables(ctx, 1);
  if (st != LNN_OK) return st;
  a.tab = nullptr;
  const ConvGeom& g = a.g;
  a.X = X; a.W = W; a.Out = Y;
  a.bytesX = (uint32_t)((uint64_t)g.N * g.C * g.IHW * 4);
  a.bytesW = (uint32_t)((uint64_t)g.O * g.C * g.KK * 4);
  a.bytesOut = (uint32_t)((uint64_t)g.N * g.O * g.OHW * 4);
  a.M = g.O; a.Ncols = g.N * g.OHW; a.K = g.C * g.KK;
  a.beta = beta ? 1 : 0;
  if (Wp) {
    a.W = Wp;
    return launch_by_m<PASS_FWD_TAP>(ctx, a, true);
  }
  if (g.C % BK == 0 && (g.KK > 1 || aligned16(W))) {
    if (g.KK > 1) {   // a 1x1 kernel already is [O][tap][C]
      st = permuted_weights(ctx, g, W, 0, PixelClass{}, &a.W, &a.ws_used);
      if (st != LNN_OK) return st;
    }
    return launch_by_m<PASS_FWD_TAP>(ctx, a, true);
  }
  st = get_table(ctx, a.g, 0, PixelClass{}, &a.tab);
  if (st != LNN_OK) return st;
  return launch_by_m<PASS_FWD_ANYC>(ctx, a, true);
}

}  // namespace lnn
