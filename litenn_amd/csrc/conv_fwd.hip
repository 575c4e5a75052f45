// Convolution forward pass (and its fused bias / activation epilogue).
#include "conv_common.hpp"

namespace lnn {

int launch_conv_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta,
                    const float* bias, int act, float slope) {
  ConvArgs a;
  a.ws_used = 0;
  a.post = PostOp{bias, act, slope};
  if (beta && a.post.any()) return set_error(LNN_ERR_INVALID, "conv2d_fwd: bias / activation cannot be combined with accumulation");
  int st = fill_geom(d, a.g);
  if (st != LNN_OK) return st;
  if (!X || !W || !Y) return set_error(LNN_ERR_INVALID, "conv2d_fwd: null pointer");
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
  if (g.C % BK == 0 && (g.KK > 1 || aligned16(W))) {
    if (g.KK > 1) {   // a 1x1 kernel already is [O][tap][C]
      st = permuted_weights(ctx, g, W, 0, PixelClass{}, &a.W, &a.ws_used);
      if (st != LNN_OK) return st;
    }
    return launch_by_m<PASS_FWD_TAP>(ctx, a, true);
  }
  st = get_table(ctx, a.g, 0, PixelClass{}, &a.tab);
  if (st != LNN_OK) return st;
  return launch_by_m<PASS_FWD>(ctx, a, a.K % 4 == 0 && aligned16(W));
}

}  // namespace lnn
