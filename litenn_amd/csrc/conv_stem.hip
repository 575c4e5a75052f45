// Convolution forward pass for image stems: three input channels, 33-64 output channels, a small dense kernel.
//
// The implicit-GEMM passes gather the B operand element by element, with a range test per element; with K = C*KH*KW
// of only a few K steps that address arithmetic costs as much as the matrix instructions.  Here a block brings the
// input patch under its 256 output pixels to LDS once (C planes of R rows), and the B operand of every MFMA is read
// straight from that patch: the address of tap k of a lane's pixel is the pixel's base address plus a constant known
// at compile time, so the K loop is nothing but ds_read_b32 with immediate offsets and MFMAs.  K is not padded to a
// multiple of 32 either: v_mfma_f32_32x32x2_f32 takes two k per instruction, so K = 147 costs 74 steps.
// A block lays the weights out in LDS once and walks over tiles; the next tile's patch travels global -> LDS (no
// registers) into a second buffer while the current tile is computed.
#include <utility>

#include "common.hpp"

constexpr int kStemMinTiles = 4;   // tiles of 256 pixels per compute unit from which the patch kernels are used

namespace lnn {
namespace {

// LDS row pitch of the patch.  A 32-lane block of pixels is one tile row (TW = 32) or two (TW = 16); with two, the
// second row's addresses should fall into the banks the first leaves free: S*PW = 16*S (mod 64).
constexpr int stem_pitch(int qn, int s, int tw) {
  if (tw == 32) return qn;
  int pw = qn;
  while ((s * pw) % 64 != (16 * s) % 64) ++pw;
  return pw;
}
// Two blocks share a compute unit: 80 KB of LDS each.
constexpr int kStemLdsFloats = 80 * 1024 / 4;

template <int KH_, int KW_, int S_, int TW_>
struct StemCfg {
  static constexpr int C = 3, KH = KH_, KW = KW_, S = S_, TW = TW_, TH = 256 / TW_;
  static constexpr int K = C * KH * KW, T = (K + 1) / 2;   // MFMA steps: k = 2t and 2t + 1
  static constexpr int R = (TH - 1) * S + KH;              // patch rows
  static constexpr int QN = (TW - 1) * S + KW;             // patch columns
  // weights in LDS: [t][row block][k parity][32 rows], steps 129 floats apart: a block fills them reading W in memory
  // order (lanes along k), and the odd pitch spreads those writes over the banks
  static constexpr int WPITCH = 129;
  static constexpr int WL = (T * WPITCH + 3) & ~3;
  // the conflict-free pitch where two patch buffers of it fit beside the weights, else the next multiple of 8
  static constexpr int PW_FREE = stem_pitch(QN, S, TW);
  static constexpr int PW = WL + 2 * ((C * R * PW_FREE + 63) & ~63) <= kStemLdsFloats ? PW_FREE : (QN + 7) & ~7;
  static constexpr int PLANE = R * PW;
  static constexpr int CHUNKS = (C * PLANE + 63) / 64;     // global -> LDS transfers (64 floats each) per patch
  static constexpr int PER_WAVE = (CHUNKS + 3) / 4;        // every wavefront sends as many (the surplus: zeros)
  static constexpr int PATCH = PER_WAVE * 4 * 64;
  static constexpr int LDS_FLOATS = WL + 2 * PATCH;
  // where tap k = (c, kh, kw) lies relative to a pixel's window origin
  static constexpr int off(int k) { return (k / (KH * KW)) * PLANE + ((k % (KH * KW)) / KW) * PW + k % KW; }
  // the odd k of step t relative to the even one: 1 inside a kernel row, else the jump to the next row or plane;
  // 0 for the padding k behind an odd K (its weight is zero, and it rereads an element of the pixel's own window)
  static constexpr int delta(int t) { return 2 * t + 1 < K ? off(2 * t + 1) - off(2 * t) : 0; }
  static constexpr int D_ROW = PW - (KW - 1), D_PLANE = PLANE - ((KH - 1) * PW + KW - 1);
};

struct StemArgs {
  const float* X;
  const float* W;
  float* Y;
  int N, IH, IW, O, OH, OW, PADT, PADL, tiles_w, tiles_h, tiles, beta;
  FastDiv dTW, dTH;   // divide by tiles_w, tiles_h
  uint32_t bytesX;
  PostOp post;
};

// The operands of step T: two weights (row blocks 0 and 1) and two pixels (pixel blocks 0 and 1) per lane.
template <class Cfg, int T>
__device__ __forceinline__ void stem_load(const float* wlane, const float* patch, const int (&b1)[2], const int (&br)[2],
                                          const int (&bp)[2], const int (&b0)[2], float (&a)[2], float (&b)[2]) {
  constexpr int o0 = Cfg::off(2 * T), d = Cfg::delta(T);
  a[0] = wlane[T * Cfg::WPITCH];
  a[1] = wlane[T * Cfg::WPITCH + 64];
#pragma unroll
  for (int pb = 0; pb < 2; ++pb) {
    const int base = d == 1 ? b1[pb] : (d == Cfg::D_ROW ? br[pb] : (d == Cfg::D_PLANE ? bp[pb] : b0[pb]));
    b[pb] = patch[base + o0];
  }
}
// Step T: the next step's operands are requested first, then this step's four MFMAs go out - an LDS read takes about
// as long as two MFMAs, and a wavefront that asked only when it needed the values would idle the pipe every step.
// Every step is a scheduling region of its own so that this order survives.
template <class Cfg, int T>
__device__ __forceinline__ void stem_step(const float* wlane, const float* patch, const int (&b1)[2], const int (&br)[2],
                                          const int (&bp)[2], const int (&b0)[2], float (&a)[2][2], float (&b)[2][2],
                                          f32x16 (&acc)[2][2]) {
  if (T + 1 < Cfg::T) stem_load<Cfg, (T + 1 < Cfg::T ? T + 1 : T)>(wlane, patch, b1, br, bp, b0, a[(T + 1) & 1], b[(T + 1) & 1]);
#pragma unroll
  for (int pb = 0; pb < 2; ++pb) {
    acc[0][pb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[T & 1][0], b[T & 1][pb], acc[0][pb], 0, 0, 0);
    acc[1][pb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[T & 1][1], b[T & 1][pb], acc[1][pb], 0, 0, 0);
  }
  __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);   // the LDS reads (the compiler may have paired some)
  __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);   // then the MFMAs
  __builtin_amdgcn_sched_barrier(0);
}
template <class Cfg, int... Ts>
__device__ __forceinline__ void stem_steps(std::integer_sequence<int, Ts...>, const float* wlane, const float* patch,
                                           const int (&b1)[2], const int (&br)[2], const int (&bp)[2], const int (&b0)[2],
                                           f32x16 (&acc)[2][2]) {
  float a[2][2], b[2][2];
  stem_load<Cfg, 0>(wlane, patch, b1, br, bp, b0, a[0], b[0]);
  __builtin_amdgcn_sched_barrier(0);
  (stem_step<Cfg, Ts>(wlane, patch, b1, br, bp, b0, a, b, acc), ...);
}

// A block of 256 threads walks over tiles of TH x TW output pixels (tile = blockIdx.x, + gridDim.x, ...: the tiles in
// flight at any time are a compact stretch of the output; a contiguous run of tiles per block, or pairs of
// neighbouring tiles, measured 12 % slower, and handing tiles out through a counter made no difference), all (at
// most 64) output channels each.
// Wavefront w owns the pixel blocks 2w and 2w + 1 of a tile (32 pixels each, in row-major tile order) and both row
// blocks.
template <class Cfg>
__global__ __launch_bounds__(256, 2) void stem_fwd_kernel(StemArgs a) {
  __shared__ __attribute__((aligned(16))) float smem[Cfg::LDS_FLOATS];
  float* wl = smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63, i = lane & 31, h = lane >> 5;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const rsrc_t rx = make_rsrc(a.X, a.bytesX);
  constexpr uint32_t OOB = 0x80000000u;

  // Patch transfers: chunk j of this wavefront fills LDS floats [(w + 4j)*64, +64) of a patch buffer; a lane's
  // float is element (c, r, q) of the patch (or pitch padding / the tail of the last chunk: never read, zeros).
  // rel: its offset in X relative to the patch origin; rq: r and q for the range tests of each tile.
  int rel[Cfg::PER_WAVE], rq[Cfg::PER_WAVE];
#pragma unroll
  for (int j = 0; j < Cfg::PER_WAVE; ++j) {
    const int e = (w + 4 * j) * 64 + lane;
    const int c = e / Cfg::PLANE, rem = e - c * Cfg::PLANE, r = rem / Cfg::PW, q = rem - r * Cfg::PW;
    const bool used = e < Cfg::C * Cfg::PLANE && q < Cfg::QN;
    rel[j] = (c * a.IH + r) * a.IW + q;
    rq[j] = used ? (r | (q << 16)) : -1;
  }
  // a tile index into (column of tiles, row of tiles, image), in scalar registers
  auto decode = [&](int tile, int& tw, int& th, int& n) {
    const uint32_t t = (uint32_t)__builtin_amdgcn_readfirstlane(tile);
    const uint32_t rest = a.dTW.div(t), img = a.dTH.div(rest);
    tw = (int)(t - rest * (uint32_t)a.tiles_w);
    th = (int)(rest - img * (uint32_t)a.tiles_h);
    n = (int)img;
  };
  auto request = [&](int tile, float* patch) {
    int tw, th, n;
    decode(tile, tw, th, n);
    const int ih0 = th * Cfg::TH * Cfg::S - a.PADT, iw0 = tw * Cfg::TW * Cfg::S - a.PADL;
    const int origin = (n * Cfg::C * a.IH + ih0) * a.IW + iw0;   // may be negative; valid elements are not
#pragma unroll
    for (int j = 0; j < Cfg::PER_WAVE; ++j) {
      const int ih = ih0 + (rq[j] & 0xffff), iw = iw0 + (rq[j] >> 16);
      const bool ok = rq[j] >= 0 && (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
      buf_load_lds4(rx, patch + (w + 4 * j) * 64, ok ? (uint32_t)(origin + rel[j]) * 4u : OOB, 0);
    }
  };

  // consecutive workgroups go to different XCDs (eight, each with its own L2) and neighbouring tiles share input
  // columns and output lines: number the blocks so that an XCD's blocks take neighbouring tiles
  const int bx = (gridDim.x & 7) == 0 ? (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  request(bx, smem + Cfg::WL);
  // weights: element (o, k) of W[O][K] goes to wl[k/2][o/32][k%2][o%32]; zeros for the rows past O and the padding k
  constexpr int KP = 2 * Cfg::T;
  constexpr int WITER = (64 * KP + 255) / 256;
  float wv[WITER];
#pragma unroll
  for (int it = 0; it < WITER; ++it) {   // all loads in flight together
    const int e = tid + 256 * it, o = e / KP, k = e - o * KP;
    wv[it] = (o < a.O && k < Cfg::K) ? a.W[o * Cfg::K + k] : 0.0f;
  }
#pragma unroll
  for (int it = 0; it < WITER; ++it) {
    const int e = tid + 256 * it, o = e / KP, k = e - o * KP;
    if (e < 64 * KP) wl[(k >> 1) * Cfg::WPITCH + (o >> 5) * 64 + (k & 1) * 32 + (o & 31)] = wv[it];
  }

  // lane bases inside a patch: pixel (row, col) of the tile, plus the odd k's displacement for each kind of step
  int b1[2], br[2], bp[2], b0[2];
#pragma unroll
  for (int pb = 0; pb < 2; ++pb) {
    const int pl = (2 * w + pb) * 32 + i, row = pl / Cfg::TW, col = pl % Cfg::TW;
    b0[pb] = row * Cfg::S * Cfg::PW + col * Cfg::S;
    b1[pb] = b0[pb] + h;
    br[pb] = b0[pb] + h * Cfg::D_ROW;
    bp[pb] = b0[pb] + h * Cfg::D_PLANE;
  }

  int cur = 0;
  for (int tile = bx; tile < a.tiles; tile += (int)gridDim.x, cur ^= 1) {
    // this tile's patch has landed (and this thread's stores of the last tile have left); behind the barrier every
    // wavefront is done reading the other buffer, which the next tile's patch may now overwrite
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const float* patch = smem + Cfg::WL + cur * Cfg::PATCH;
    if (tile + (int)gridDim.x < a.tiles) request(tile + (int)gridDim.x, smem + Cfg::WL + (cur ^ 1) * Cfg::PATCH);

    f32x16 acc[2][2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int pb = 0; pb < 2; ++pb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][pb][r] = 0.0f;
    stem_steps<Cfg>(std::make_integer_sequence<int, Cfg::T>{}, wl + h * 32 + i, patch, b1, br, bp, b0, acc);

    // Element r of an accumulator: channel 8*(r/4) + 4*h + r%4 of the row block, pixel i of the pixel block.  Stores
    // go through a descriptor of this image's O planes: the lane's part of the address (pixel, and 4*h channels) is
    // computed once per pixel block, the rest of the channel index travels in the scalar offset, and channels past O
    // fall outside the descriptor and are dropped - no vector arithmetic per store.
    int tw, th, n;
    decode(tile, tw, th, n);
    const int ohw = a.OH * a.OW;
    const rsrc_t ry = make_rsrc(a.Y + (size_t)n * a.O * ohw, (uint32_t)(a.O * ohw) * 4u);
#pragma unroll
    for (int pb = 0; pb < 2; ++pb) {
      const int pl = (2 * w + pb) * 32 + i, oh = th * Cfg::TH + pl / Cfg::TW, ow = tw * Cfg::TW + pl % Cfg::TW;
      const uint32_t voff = (oh < a.OH && ow < a.OW) ? (uint32_t)(oh * a.OW + ow + 4 * h * ohw) * 4u : OOB;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int mc = mb * 32 + 8 * (r >> 2) + (r & 3);   // + 4*h: this lane's channel
          const int soff = mc * ohw * 4;
          float v = acc[mb][pb][r];
          if (a.post.any()) {
            const int m = mc + 4 * h;
            v = a.post.apply(v, (a.post.bias != nullptr && m < a.O) ? a.post.bias[m] : 0.0f);
          }
          if (a.beta) v += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ry, (int)voff, soff, 0));
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), ry, (int)voff, soff, 0);
        }
    }
  }
}

template <int KH, int KW, int S>
int launch_stem_shape(DeviceCtx* ctx, StemArgs& a) {
  // the tile shape that covers the output plane with less overhang
  auto count = [&](int tw_) { return (long long)((a.OW + tw_ - 1) / tw_) * ((a.OH + 256 / tw_ - 1) / (256 / tw_)); };
  const bool wide = count(32) <= count(16);
  using Wide = StemCfg<KH, KW, S, 32>;
  using Square = StemCfg<KH, KW, S, 16>;
  static_assert(Wide::LDS_FLOATS <= kStemLdsFloats && Square::LDS_FLOATS <= kStemLdsFloats, "two blocks per compute unit");
  const int tw_ = wide ? 32 : 16, th_ = 256 / tw_;
  a.tiles_w = (a.OW + tw_ - 1) / tw_;
  a.tiles_h = (a.OH + th_ - 1) / th_;
  const long long tiles = (long long)a.N * a.tiles_w * a.tiles_h;
  if (tiles > 0x7fffffffll) return set_error(LNN_ERR_UNSUPPORTED, "conv2d: too many tiles");
  a.tiles = (int)tiles;
  a.dTW = make_fastdiv((uint32_t)a.tiles_w);
  a.dTH = make_fastdiv((uint32_t)a.tiles_h);
  const long long blocks = tiles < 2ll * ctx->cus ? tiles : 2ll * ctx->cus;   // two blocks per compute unit
  if (wide) hipLaunchKernelGGL((stem_fwd_kernel<Wide>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((stem_fwd_kernel<Square>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// Weight gradient of the same geometries: dW[o][col] = sum over pixels of dY[o][pixel] * X[window of pixel][col],
// col = (c, kh, kw).  The roles turn around: the K dimension is the pixels, two per MFMA; a lane of the B operand
// owns a column, whose offset inside a pixel's window is fixed for the whole kernel, and the pixel's position in the
// patch is the compile-time part of the address.  The A operand (dY) goes from global memory straight into registers,
// sixteen consecutive pixels per lane and row block, a tile ahead.  One block of four wavefronts per compute unit, one
// wavefront per SIMD: each keeps all 2 x NB accumulators (160 registers for 7x7) for its quarter of every tile's
// pixels and for all the block's tiles; only at the end the four wavefronts' sums are added through LDS and the
// block's partial result goes to scratch, where a small kernel adds the blocks up in a fixed order.
template <int KH_, int KW_, int S_, int TW_>
struct StemWCfg {
  static constexpr int C = 3, KH = KH_, KW = KW_, S = S_, TW = TW_, TH = 128 / TW_;
  static constexpr int K = C * KH * KW, NB = (K + 31) / 32;   // column blocks
  static constexpr int R = (TH - 1) * S + KH, QN = (TW - 1) * S + KW;
  static constexpr int PW = QN | 1, PLANE = R * PW;
  static constexpr int CHUNKS = (C * PLANE + 63) / 64, PER_WAVE = (CHUNKS + 3) / 4, PATCH = PER_WAVE * 4 * 64;
  static constexpr int LDS_FLOATS = 2 * PATCH > 4096 ? 2 * PATCH : 4096;   // the final sum needs 4 x 1024 floats
  static constexpr int PART = 2 * NB * 1024;   // floats of a block's partial result: [row block][column block][r][lane]
  // a wavefront's 32 pixels: one tile row (TW = 32: lane half h = columns 16h .. 16h+15) or two (TW = 16: h = row)
  static constexpr int H_STEP = TW == 32 ? 16 * S : S * PW;
  static constexpr int W_STEP = (TW == 32 ? 1 : 2) * S * PW;
};

struct StemWArgs {
  const float* X;
  const float* dY;
  float* part;
  int N, IH, IW, O, OH, OW, PADT, PADL, tiles_w, tiles_h, tiles;
  FastDiv dTW, dTH;   // divide by tiles_w, tiles_h
  uint32_t bytesX, bytesY;
};

template <class Cfg>
__global__ __launch_bounds__(256, 1) void stem_wgrad_kernel(StemWArgs a) {
  __shared__ __attribute__((aligned(16))) float smem[Cfg::LDS_FLOATS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, i = lane & 31, h = lane >> 5;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const rsrc_t rx = make_rsrc(a.X, a.bytesX), ry = make_rsrc(a.dY, a.bytesY);
  constexpr uint32_t OOB = 0x80000000u;
  constexpr int NB = Cfg::NB;

  int rel[Cfg::PER_WAVE], rq[Cfg::PER_WAVE];
#pragma unroll
  for (int j = 0; j < Cfg::PER_WAVE; ++j) {
    const int e = (w + 4 * j) * 64 + lane;
    const int c = e / Cfg::PLANE, rem = e - c * Cfg::PLANE, r = rem / Cfg::PW, q = rem - r * Cfg::PW;
    const bool used = e < Cfg::C * Cfg::PLANE && q < Cfg::QN;
    rel[j] = (c * a.IH + r) * a.IW + q;
    rq[j] = used ? (r | (q << 16)) : -1;
  }
  auto request = [&](int tw, int th, int n, float* patch) {
    const int ih0 = th * Cfg::TH * Cfg::S - a.PADT, iw0 = tw * Cfg::TW * Cfg::S - a.PADL;
    const int origin = (n * Cfg::C * a.IH + ih0) * a.IW + iw0;
#pragma unroll
    for (int j = 0; j < Cfg::PER_WAVE; ++j) {
      const int ih = ih0 + (rq[j] & 0xffff), iw = iw0 + (rq[j] >> 16);
      const bool ok = rq[j] >= 0 && (unsigned)ih < (unsigned)a.IH && (unsigned)iw < (unsigned)a.IW;
      buf_load_lds4(rx, patch + (w + 4 * j) * 64, ok ? (uint32_t)(origin + rel[j]) * 4u : OOB, 0);
    }
  };
  // dY of a tile: this lane's sixteen pixels (row oh, columns ow .. ow + 15) of channels i and 32 + i.  Pixels past
  // the row's end are read as whatever follows in memory (or zero past the tensor) and cleared afterwards.
  f32x4 an[2][4];
  auto load_a = [&](int tw, int th, int n) {
    const int oh = th * Cfg::TH + (Cfg::TW == 32 ? w : 2 * w + h), ow = tw * Cfg::TW + (Cfg::TW == 32 ? 16 * h : 0);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int o = mb * 32 + i;
      const bool ok = o < a.O && oh < a.OH && ow < a.OW;
      const uint32_t voff = ok ? (uint32_t)(((n * a.O + o) * a.OH + oh) * a.OW + ow) * 4u : OOB;
#pragma unroll
      for (int q = 0; q < 4; ++q) an[mb][q] = buf_load4_s(ry, voff, (uint32_t)(16 * q));
    }
    return ow;
  };

  // the column of lane i in each column block: where its tap lies inside a pixel's window; plus this wavefront's and
  // this lane half's pixels
  int bbase[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    int col = nb * 32 + i;
    if (col >= Cfg::K) col = 0;   // padding columns compute something nobody stores
    const int c = col / (Cfg::KH * Cfg::KW), r = col - c * (Cfg::KH * Cfg::KW), kh = r / Cfg::KW, kw = r - kh * Cfg::KW;
    bbase[nb] = c * Cfg::PLANE + kh * Cfg::PW + kw + w * Cfg::W_STEP + h * Cfg::H_STEP;
  }
  f32x16 acc[2][NB];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.0f;

  // a tile index into (column of tiles, row of tiles, image), in scalar registers
  auto fetch = [&](int tile, float* patch) {
    const uint32_t t = (uint32_t)__builtin_amdgcn_readfirstlane(tile);
    const uint32_t rest = a.dTW.div(t), tw = t - rest * (uint32_t)a.tiles_w, n = a.dTH.div(rest), th = rest - n * (uint32_t)a.tiles_h;
    request((int)tw, (int)th, (int)n, patch);
    return load_a((int)tw, (int)th, (int)n);
  };
  int cur = 0;
  // this block's tiles: a contiguous run [first, last) (neighbouring tiles share lines of dY and columns of X); the
  // grid never has more blocks than tiles
  const int first = (int)((long long)a.tiles * blockIdx.x / gridDim.x), last = (int)((long long)a.tiles * (blockIdx.x + 1) / gridDim.x);
  int ow_next = fetch(first, smem);
  for (int tile = first; tile < last; ++tile, cur ^= 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // this tile's dY, pixels past the end of the row cleared
    float av[2][16];
    const int left = a.OW - ow_next;   // pixels of this lane's run that exist
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) av[mb][4 * q + e] = 4 * q + e < left ? an[mb][q][e] : 0.0f;
    const float* patch = smem + cur * Cfg::PATCH;
    // the next tile's operands (behind the last tile: that tile once more, into the buffer nobody reads again - no
    // branch, so that these instructions can be spread among the MFMAs below)
    ow_next = fetch(tile + 1 < last ? tile + 1 : tile, smem + (cur ^ 1) * Cfg::PATCH);
    // sixteen steps: the pixel t (lane half 0) and t + 16 or the pixel below (lane half 1)
    float b[2][NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) b[0][nb] = patch[bbase[nb]];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      if (t + 1 < 16) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) b[(t + 1) & 1][nb] = patch[bbase[nb] + (t + 1) * Cfg::S];
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        acc[0][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[0][t], b[t & 1][nb], acc[0][nb], 0, 0, 0);
        acc[1][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[1][t], b[t & 1][nb], acc[1][nb], 0, 0, 0);
      }
    }
  }

  // the four wavefronts' sums, one accumulator at a time: [wave][r][lane] in LDS, thread (r4, lane) adds four values
  // (wavefronts in order) for r = 4*r4 .. 4*r4 + 3
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  float* part = a.part + (size_t)blockIdx.x * Cfg::PART;
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 16; ++r) smem[w * 1024 + r * 64 + lane] = acc[mb][nb][r];
      __syncthreads();
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int e = tid + 256 * q;
        part[(mb * NB + nb) * 1024 + e] = ((smem[e] + smem[1024 + e]) + smem[2048 + e]) + smem[3072 + e];
      }
    }
}

// dW[o][col] (+)= sum over the blocks' partial results, blocks added in a fixed order: 32 consecutive elements per
// block of 256 threads, eight lanes per element striding over the blocks.
__global__ __launch_bounds__(256) void stem_wgrad_reduce(float* dW, const float* part, int nblocks, int per_block, int NB,
                                                         int O, int K, int beta) {
  __shared__ float red[8][33];
  const int li = threadIdx.x & 31, ls = threadIdx.x >> 5;
  const int e = blockIdx.x * 32 + li;
  float s = 0.0f;
  if (e < per_block) {
#pragma unroll 8
    for (int b = ls; b < nblocks; b += 8) s += part[(size_t)b * per_block + e];
  }
  red[ls][li] = s;
  __syncthreads();
  if (ls == 0 && e < per_block) {
#pragma unroll
    for (int k = 1; k < 8; ++k) s += red[k][li];
    // element e of a partial result = (row block, column block, r, lane)
    const int lane = e & 63, r = (e >> 6) & 15, pair = e >> 10, mb = pair / NB, nb = pair - mb * NB;
    const int o = mb * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3), col = nb * 32 + (lane & 31);
    if (o < O && col < K) {
      float* dst = dW + (size_t)o * K + col;
      *dst = beta ? *dst + s : s;
    }
  }
}

template <int KH, int KW, int S>
int launch_stem_wgrad_shape(DeviceCtx* ctx, StemWArgs& a, float* dW, int beta) {
  auto count = [&](int tw_) { return (long long)((a.OW + tw_ - 1) / tw_) * ((a.OH + 128 / tw_ - 1) / (128 / tw_)); };
  const bool wide = count(32) <= count(16);
  using Wide = StemWCfg<KH, KW, S, 32>;
  using Square = StemWCfg<KH, KW, S, 16>;
  const int tw_ = wide ? 32 : 16, th_ = 128 / tw_;
  a.tiles_w = (a.OW + tw_ - 1) / tw_;
  a.tiles_h = (a.OH + th_ - 1) / th_;
  const long long tiles = (long long)a.N * a.tiles_w * a.tiles_h;
  if (tiles > 0x7fffffffll) return set_error(LNN_ERR_UNSUPPORTED, "conv2d: too many tiles");
  a.tiles = (int)tiles;
  a.dTW = make_fastdiv((uint32_t)a.tiles_w);
  a.dTH = make_fastdiv((uint32_t)a.tiles_h);
  const int blocks = (int)(tiles < ctx->cus ? tiles : ctx->cus);   // one block per compute unit
  int st = ensure_workspace(ctx, (size_t)blocks * Wide::PART * sizeof(float));
  if (st != LNN_OK) return st;
  a.part = static_cast<float*>(ctx->ws);
  if (wide) hipLaunchKernelGGL((stem_wgrad_kernel<Wide>), dim3(blocks), dim3(256), 0, ctx->stream, a);
  else hipLaunchKernelGGL((stem_wgrad_kernel<Square>), dim3(blocks), dim3(256), 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  hipLaunchKernelGGL(stem_wgrad_reduce, dim3((Wide::PART + 31) / 32), dim3(256), 0, ctx->stream, dW, a.part, blocks,
                     Wide::PART, Wide::NB, a.O, Wide::K, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// ---------------------------------------------------------------------------------------------------------------
// Data gradient of stride-2 convolutions with at most 4 input channels (the image gradient of a stem).  Seen from a
// 2 x 2 block of input pixels (2i + a, 2j + b), every tap reads dY at (i + dh, j + dw) with dh, dw from a window of
// at most four values each, and which tap that is depends only on (a, dh) and (b, dw).  So
//     dX[(c, a, b)][i, j] = sum over o, sh, sw of dY[o][i + DH0 + sh][j + DW0 + sw] * Wt[(c, a, b)][o][sh][sw]
// is a stride-1 4 x 4 convolution of dY with C * 4 <= 16 output rows and zeros where a (parity, slot) pair has no
// tap: a GEMM with 16 rows, K = 16 * O, computed with v_mfma_f32_16x16x4_f32 (the four k of an instruction = the four
// sw of one (o, sh)).  A block of four wavefronts computes 16 x 16 coarse pixels; dY travels global -> LDS eight
// channels at a time (19 x 19 patch each, next chunk during the current one), the B operand is read from the patch at
// lane base + immediate, the A operand from the rearranged weights of the same eight channels.
constexpr int kDgTile = 16, kDgRows = kDgTile + 3, kDgPitch = 20, kDgPlane = kDgRows * kDgPitch, kDgChunk = 8;
constexpr int kDgPatch = 3072;   // 8 planes of 380 floats, rounded up to whole transfers of 64 (48 = 12 per wavefront)
constexpr int kDgWt = kDgChunk * 256;   // [o][sh][row][sw] of eight channels

struct StemDArgs {
  const float* dY;
  const float* Wt;
  float* dX;
  int N, C, IH, IW, O, OH, OW, DH0, DW0, tiles_w, tiles_h, tiles, per_xcd, beta, pairs;
  uint32_t bytesY, bytesWt, bytesX;
};
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Wt[o][sh][row = c*4 + a*2 + b][sw] = W[o][c][kh][kw] with kh = a + PADT - 2*(DH0 + sh), kw likewise; 0 without a tap
__global__ void stem_dgrad_weights_kernel(float* wt, const float* w, int O, int C, int KH, int KW, int PADT, int PADL,
                                          int DH0, int DW0) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= O * 256) return;
  const int sw = e & 3, row = (e >> 2) & 15, sh = (e >> 6) & 3, o = e >> 8;
  const int c = row >> 2, a = (row >> 1) & 1, b = row & 1;
  const int kh = a + PADT - 2 * (DH0 + sh), kw = b + PADL - 2 * (DW0 + sw);
  wt[e] = (c < C && kh >= 0 && kh < KH && kw >= 0 && kw < KW) ? w[((size_t)(o * C + c) * KH + kh) * KW + kw] : 0.0f;
}

template <int OL, int SH>
__device__ __forceinline__ void stem_dgrad_step(const float* wt, const float* patch, int abase, const int (&bbase)[4],
                                                f32x4 (&acc)[4]) {
  const float a = wt[abase + (OL * 4 + SH) * 64];
  float b[4];
#pragma unroll
  for (int cb = 0; cb < 4; ++cb) b[cb] = patch[bbase[cb] + OL * kDgPlane + SH * kDgPitch];
#pragma unroll
  for (int cb = 0; cb < 4; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[cb], acc[cb], 0, 0, 0);
}
template <int... Is>
__device__ __forceinline__ void stem_dgrad_chunk(std::integer_sequence<int, Is...>, const float* wt, const float* patch,
                                                 int abase, const int (&bbase)[4], f32x4 (&acc)[4]) {
  (stem_dgrad_step<Is / 4, Is % 4>(wt, patch, abase, bbase, acc), ...);
}

__global__ __launch_bounds__(256, 3) void stem_dgrad_kernel(StemDArgs a) {
  __shared__ __attribute__((aligned(16))) float smem[2 * (kDgPatch + kDgWt)];
  const int tid = threadIdx.x, lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const rsrc_t ry = make_rsrc(a.dY, a.bytesY), rw = make_rsrc(a.Wt, a.bytesWt), rx = make_rsrc(a.dX, a.bytesX);
  constexpr uint32_t OOB = 0x80000000u;
  // Consecutive workgroups go to different XCDs (eight, each with its own L2), neighbouring tiles share lines of dY:
  // workgroup b takes tile (b % 8) * per_xcd + b / 8, so that an XCD walks a contiguous run of tiles.
  int bid = (int)(blockIdx.x & 7) * a.per_xcd + (int)(blockIdx.x >> 3);
  if (bid >= a.tiles) return;   // the whole block leaves together
  const int tw = bid % a.tiles_w;
  bid /= a.tiles_w;
  const int th = bid % a.tiles_h, n = bid / a.tiles_h;
  const int i0 = th * kDgTile, j0 = tw * kDgTile;   // coarse origin of the tile
  const int ohw = a.OH * a.OW;

  // dY patch transfers of one chunk: transfer t of this wavefront fills floats [(w + 4t)*64, +64) of the patch buffer,
  // element (channel ol, row r, column q) of the chunk; the chunk's first channel travels in the scalar offset
  uint32_t voff[12];
#pragma unroll
  for (int t = 0; t < 12; ++t) {
    const int e = (w + 4 * t) * 64 + lane;
    const int ol = e / kDgPlane, rem = e - ol * kDgPlane, r = rem / kDgPitch, q = rem - r * kDgPitch;
    const int oh = i0 + a.DH0 + r, ow = j0 + a.DW0 + q;
    const bool ok = ol < kDgChunk && q < kDgRows && (unsigned)oh < (unsigned)a.OH && (unsigned)ow < (unsigned)a.OW;
    voff[t] = ok ? (uint32_t)(((n * a.O + ol) * a.OH + oh) * a.OW + ow) * 4u : OOB;
  }
  auto request = [&](int chunk, float* buf) {
    const uint32_t sy = (uint32_t)(chunk * kDgChunk * ohw) * 4u, sw_ = (uint32_t)(chunk * kDgWt) * 4u;
#pragma unroll
    for (int t = 0; t < 12; ++t) buf_load_lds4(ry, buf + (w + 4 * t) * 64, voff[t], sy);
#pragma unroll
    for (int t = 0; t < 8; ++t) buf_load_lds4(rw, buf + kDgPatch + (w + 4 * t) * 64, (uint32_t)((w + 4 * t) * 64 + lane) * 4u, sw_);
  };

  // lane (x = lane % 16, kq = lane / 16): row x of the A operand / column x of the B operand, k = kq (= sw)
  const int x = lane & 15, kq = lane >> 4;
  const int abase = x * 4 + kq;
  int bbase[4];
#pragma unroll
  for (int cb = 0; cb < 4; ++cb) bbase[cb] = (4 * w + cb) * kDgPitch + x + kq;
  f32x4 acc[4];
#pragma unroll
  for (int cb = 0; cb < 4; ++cb) acc[cb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  const int nch = a.O / kDgChunk;
  request(0, smem);
  for (int ch = 0, cur = 0; ch < nch; ++ch, cur ^= 1) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const float* buf = smem + cur * (kDgPatch + kDgWt);
    if (ch + 1 < nch) request(ch + 1, smem + (cur ^ 1) * (kDgPatch + kDgWt));
    stem_dgrad_chunk(std::make_integer_sequence<int, kDgChunk * 4>{}, buf + kDgPatch, buf, abase, bbase, acc);
  }

  // accumulator element r of lane (x, g = lane / 16): row 4g + r = channel g, pixel parity (a, b) = (r / 2, r % 2),
  // coarse pixel (i0 + 4w + cb, j0 + x)
  const int c = kq;
  if (c < a.C) {
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
      const int i = i0 + 4 * w + cb, j = j0 + x;
      if (a.pairs) {   // even row length, 8-byte aligned tensor: the two pixels of a row in one 64-bit access
#pragma unroll
        for (int pa = 0; pa < 2; ++pa) {
          const int ih = 2 * i + pa, iw = 2 * j;
          const uint32_t off = (ih < a.IH && iw < a.IW) ? (uint32_t)(((n * a.C + c) * a.IH + ih) * a.IW + iw) * 4u : OOB;
          f32x2 v = {acc[cb][2 * pa], acc[cb][2 * pa + 1]};
          if (a.beta) v += __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rx, (int)off, 0, 0));
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, v), rx, (int)off, 0, 0);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int ih = 2 * i + (r >> 1), iw = 2 * j + (r & 1);
          const uint32_t off = (ih < a.IH && iw < a.IW) ? (uint32_t)(((n * a.C + c) * a.IH + ih) * a.IW + iw) * 4u : OOB;
          float v = acc[cb][r];
          if (a.beta) v += buf_load(rx, off);
          buf_store(rx, off, v);
        }
      }
    }
  }
}

}  // namespace

// Geometries the patch kernels take.  With fewer than four tiles per compute unit the implicit-GEMM passes, which cut
// the work more finely, are about as fast (16 x 3 x 128 x 128, 5x5 stride 2, one tile per compute unit: forward and
// weight gradient together within 2 us either way).
bool stem_fwd_applies(const lnn_conv2d_desc* d, int compute_units) {
  if (d->C != 3 || d->O <= 32 || d->O > 64 || d->dilation != 1 || d->KH != d->KW) return false;
  const int k = d->KH, s = d->stride;
  if (!((k == 7 && s == 2) || (k == 5 && s == 2) || (k == 3 && (s == 1 || s == 2)))) return false;
  return (long long)d->N * (((long long)d->OH * d->OW + 255) / 256) >= (long long)kStemMinTiles * compute_units;
}

// Y (+)= conv(X, W) with the bias / activation epilogue, for the geometries stem_fwd_applies() accepts
int launch_stem_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta,
                    const float* bias, int act, float slope) {
  StemArgs a;
  a.X = X; a.W = W; a.Y = Y;
  a.N = d->N; a.IH = d->IH; a.IW = d->IW; a.O = d->O; a.OH = d->OH; a.OW = d->OW; a.PADT = d->PADT; a.PADL = d->PADL;
  a.beta = beta ? 1 : 0;
  a.bytesX = (uint32_t)((uint64_t)d->N * d->C * d->IH * d->IW * 4);
  a.post = PostOp{bias, act, slope};
  const int k = d->KH, s = d->stride;
  if (k == 7 && s == 2) return launch_stem_shape<7, 7, 2>(ctx, a);
  if (k == 5 && s == 2) return launch_stem_shape<5, 5, 2>(ctx, a);
  if (k == 3 && s == 1) return launch_stem_shape<3, 3, 1>(ctx, a);
  if (k == 3 && s == 2) return launch_stem_shape<3, 3, 2>(ctx, a);
  return set_error(LNN_ERR_INVALID, "conv2d_fwd: not a stem geometry");
}

// The weight gradient of the same geometries; rows of dY must be 16-byte aligned for the 128-bit loads.
bool stem_wgrad_applies(const lnn_conv2d_desc* d, int compute_units, const float* dY) {
  if (!stem_fwd_applies(d, compute_units)) return false;
  return d->OW % 4 == 0 && (reinterpret_cast<uintptr_t>(dY) & 15) == 0;
}

// dW (+)= wgrad(X, dY) for the geometries stem_wgrad_applies() accepts
int launch_stem_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta) {
  StemWArgs a;
  a.X = X; a.dY = dY; a.part = nullptr;
  a.N = d->N; a.IH = d->IH; a.IW = d->IW; a.O = d->O; a.OH = d->OH; a.OW = d->OW; a.PADT = d->PADT; a.PADL = d->PADL;
  a.bytesX = (uint32_t)((uint64_t)d->N * d->C * d->IH * d->IW * 4);
  a.bytesY = (uint32_t)((uint64_t)d->N * d->O * d->OH * d->OW * 4);
  const int k = d->KH, s = d->stride;
  if (k == 7 && s == 2) return launch_stem_wgrad_shape<7, 7, 2>(ctx, a, dW, beta);
  if (k == 5 && s == 2) return launch_stem_wgrad_shape<5, 5, 2>(ctx, a, dW, beta);
  if (k == 3 && s == 1) return launch_stem_wgrad_shape<3, 3, 1>(ctx, a, dW, beta);
  if (k == 3 && s == 2) return launch_stem_wgrad_shape<3, 3, 2>(ctx, a, dW, beta);
  return set_error(LNN_ERR_INVALID, "conv2d_wgrad: not a stem geometry");
}

// floor(a / 2) for negative a too
static int half_floor(int a) { return a >= 0 ? a / 2 : -((-a + 1) / 2); }

// The data gradient above: stride 2, no dilation, at most 4 input channels, output channels a multiple of 8 (from 32),
// at most four dY rows and columns per input pixel pair (kernels up to 8 x 8), at least two tiles per compute unit.
bool stem_dgrad_applies(const lnn_conv2d_desc* d, int compute_units) {
  if (d->C > 4 || d->stride != 2 || d->dilation != 1 || d->O % kDgChunk != 0 || d->O < 32) return false;
  const int dh0 = -half_floor(d->KH - 1 - d->PADT), dw0 = -half_floor(d->KW - 1 - d->PADL);
  if (half_floor(1 + d->PADT) - dh0 + 1 > 4 || half_floor(1 + d->PADL) - dw0 + 1 > 4) return false;
  const long long tiles = (long long)d->N * (((d->IH + 1) / 2 + kDgTile - 1) / kDgTile) * (((d->IW + 1) / 2 + kDgTile - 1) / kDgTile);
  return tiles >= 2ll * compute_units && tiles <= 0x7fffffffll;
}

// dX (+)= dgrad(dY, W) for the geometries stem_dgrad_applies() accepts
int launch_stem_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* W, float* dX, int beta) {
  StemDArgs a;
  a.dY = dY; a.dX = dX;
  a.N = d->N; a.C = d->C; a.IH = d->IH; a.IW = d->IW; a.O = d->O; a.OH = d->OH; a.OW = d->OW;
  a.DH0 = -half_floor(d->KH - 1 - d->PADT);
  a.DW0 = -half_floor(d->KW - 1 - d->PADL);
  a.tiles_h = ((d->IH + 1) / 2 + kDgTile - 1) / kDgTile;
  a.tiles_w = ((d->IW + 1) / 2 + kDgTile - 1) / kDgTile;
  a.beta = beta ? 1 : 0;
  a.pairs = d->IW % 2 == 0 && (reinterpret_cast<uintptr_t>(dX) & 7) == 0;
  a.bytesY = (uint32_t)((uint64_t)d->N * d->O * d->OH * d->OW * 4);
  a.bytesX = (uint32_t)((uint64_t)d->N * d->C * d->IH * d->IW * 4);
  a.bytesWt = (uint32_t)((uint64_t)d->O * 256 * 4);
  int st = ensure_workspace(ctx, a.bytesWt);
  if (st != LNN_OK) return st;
  float* wt = static_cast<float*>(ctx->ws);
  hipLaunchKernelGGL(stem_dgrad_weights_kernel, dim3((d->O * 256 + 255) / 256), dim3(256), 0, ctx->stream, wt, W, d->O, d->C,
                     d->KH, d->KW, d->PADT, d->PADL, a.DH0, a.DW0);
  LNN_HIP(hipGetLastError());
  a.Wt = wt;
  const long long tiles = (long long)a.N * a.tiles_w * a.tiles_h;
  a.tiles = (int)tiles;
  a.per_xcd = (int)((tiles + 7) / 8);
  hipLaunchKernelGGL(stem_dgrad_kernel, dim3((unsigned)(8 * a.per_xcd)), dim3(256), 0, ctx->stream, a);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

}  // namespace lnn
