// Convolution weight gradient (split over the output pixels, deterministic slice reduction).
#include "conv_common.hpp"


namespace lnn {

int launch_conv_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta,
                      int w_iohw) {
  ConvArgs a;
  a.w_iohw = w_iohw ? 1 : 0;
  a.ws_used = 0;
  a.post = PostOp{nullptr, 0, 0.0f};
  int st = fill_geom(d, a.g);
  if (st != LNN_OK) return st;
  if (!X || !dY || !dW) return set_error(LNN_ERR_INVALID, "conv2d_wgrad: null pointer");
  ctx->last_wgrad_plan[0] = ctx->last_wgrad_plan[1] = ctx->last_wgrad_plan[2] = ctx->last_wgrad_plan[3] = 0;   // image-stem kernel: no tile plan
  if (!w_iohw && stem_wgrad_applies(d, ctx->cus, dY)) return launch_stem_wgrad(ctx, d, X, dY, dW, beta);
  a.tab = nullptr;
  const ConvGeom& g = a.g;
  a.X = X; a.W = dY; a.Out = dW;
  a.bytesX = (uint32_t)((uint64_t)g.N * g.C * g.IHW * 4);
  a.bytesW = (uint32_t)((uint64_t)g.N * g.O * g.OHW * 4);
  a.bytesOut = (uint32_t)((uint64_t)g.O * g.C * g.KK * 4);
  a.M = g.O; a.Ncols = g.C * g.KK; a.K = g.N * g.OHW;
  a.beta = beta ? 1 : 0;
  const bool vec = g.OHW % 4 == 0 && aligned16(dY);
  if (wgrad_one_tap_per_group(g)) {
    // every tap of every output pixel reads a column inside the image: the gather can move four pixels at a time
    const bool cols_inside = g.PADL == 0 && g.OW - 1 + (g.KW - 1) * g.D <= g.IW - 1;
    if (vec && g.S == 1 && g.OW % 4 == 0 && cols_inside) return launch_by_m<PASS_WGRAD_TAP4>(ctx, a, true);
    // also with fewer channels than a full sub-tile per tap: wider sub-tiles through the loader below would mean
    // more K slices for the same chip (dilated 3x3 on 64 channels: 0.065 ms here, 0.070 ms there)
    return launch_by_m<PASS_WGRAD_TAP>(ctx, a, vec);
  }
  // any other channel count: a group's columns may span taps
  if (wgrad_walkers_fit(g)) return launch_by_m<PASS_WGRAD_ANYC>(ctx, a, vec);
  if (w_iohw) return set_error(LNN_ERR_UNSUPPORTED, "conv2d_wgrad: this geometry cannot write a gradient with swapped channel axes");
  // tiny images: the table-driven kernel with per-column gather entries
  st = reserve_tables(ctx, 1);
  if (st != LNN_OK) return st;
  st = get_table(ctx, a.g, 0, PixelClass{}, &a.tab);
  if (st != LNN_OK) return st;
  return launch_by_m<PASS_WGRAD>(ctx, a, vec);
}

}  // namespace lnn
