// fp32 MFMA tile engine for gfx950 (CDNA4): one kernel skeleton shared by the
// plain GEMM and by the three implicit-GEMM convolution passes.
//
//   C[m, n] (+)= sum_k A(m, k) * B(k, n)
//
// A workgroup has 256 threads = 4 wavefronts of 64 lanes arranged WM x WN.
// Each wavefront owns a 32 x (32*NT) slab of the output held in NT
// v_mfma_f32_32x32x2_f32 accumulators.  Operand tiles are staged through LDS
// (double buffered, one barrier per K step of BK) by "loader" objects which
// differ only in how they turn (row, k) into a global address: plain strided
// matrices or on-the-fly im2col gathers.  All global traffic uses raw buffer
// instructions so that an out-of-range or masked element is a hardware zero
// (loads) or a dropped write (stores) instead of a branch or a fault.
//
// Work distribution: the output is cut into "units" of 32*WN columns per
// M-tile; the launch gives every workgroup a contiguous, nearly equal range of
// units (so all compute units finish together regardless of how the problem
// size divides into tiles) and the workgroup walks its range in sub-tiles of
// 1..NTMAX units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lnn {

constexpr int BK = 16;            // K extent of one LDS stage
constexpr int LDK = BK + 4;       // row stride (floats) of a K-contiguous LDS tile
constexpr uint32_t OOB = 0x80000000u;  // byte offset beyond every buffer (< 2 GiB each)
constexpr int BIG = 0x40000000;   // coordinate that fails every range test

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
using rsrc_t = __amdgpu_buffer_rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load(rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0));
}
__device__ __forceinline__ f32x4 buf_load4(rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
}
__device__ __forceinline__ void buf_store(rsrc_t r, uint32_t off, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, (int)off, 0, 0);
}

// Exact unsigned division of n < 2^31 by a fixed divisor via one 64-bit
// multiply: q = (n * m) >> sh with m = ceil(2^sh / d), sh = 31 + ceil(log2 d).
struct FastDiv {
  uint32_t m, sh, d;
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return (uint32_t)(((uint64_t)n * m) >> sh);
  }
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.sh = 31 + s;
  f.m = (uint32_t)(((1ull << f.sh) + d - 1) / d);
  f.d = d;
  return f;
}

// ---------------------------------------------------------------------------
// Loaders.  Common interface:
//   KC            LDS layout: true  -> tile[row][LDK]   (k contiguous)
//                             false -> tile[k][R]       (row contiguous)
//   init(...)     per sub-tile set-up (row0 = first row of the tile)
//   fetch(k0)     global -> registers for K range [k0, k0 + BK)
//   commit(lds)   registers -> LDS stage
// R is the number of tile rows (BM for the A side, BN for the B side).
// ---------------------------------------------------------------------------

// Plain strided matrix, element (r, k) at r*ld + k.
template <int R, bool VEC>
struct PlainKC {
  static constexpr bool KC = true;
  static constexpr int E = (R * 4 + 255) / 256;
  rsrc_t rs;
  uint32_t base[E];
  int kend;
  f32x4 v[E];
  __device__ __forceinline__ void init(rsrc_t r, int ld, int row0, int rows_total, int kend_) {
    rs = r;
    kend = kend_;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2, kg = s & 3;
      const bool ok = row < R && row0 + row < rows_total;
      base[e] = ok ? (uint32_t)((row0 + row) * ld + 4 * kg) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    const int kg = threadIdx.x & 3;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      if (VEC) {
        const uint32_t off = (k0 + 4 * kg < kend) ? base[e] + (uint32_t)k0 * 4u : OOB;
        v[e] = buf_load4(rs, off);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t off = (k0 + 4 * kg + j < kend) ? base[e] + (uint32_t)(k0 + j) * 4u : OOB;
          v[e][j] = buf_load(rs, off);
        }
      }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2, kg = s & 3;
      if (R * 4 % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[row * LDK + 4 * kg]) = v[e];
    }
  }
};

// Plain strided matrix stored K-major, element (r, k) at k*ld + r.
template <int R, bool VEC>
struct PlainMC {
  static constexpr bool KC = false;
  static constexpr int G = R / 4;  // float4 groups per k row
  static constexpr int E = (BK * G + 255) / 256;
  rsrc_t rs;
  uint32_t base[E];
  int nval[E];
  int ld, kend;
  f32x4 v[E];
  __device__ __forceinline__ void init(rsrc_t r, int ld_, int row0, int rows_total, int kend_) {
    rs = r;
    ld = ld_;
    kend = kend_;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, ks = s / G, rg = s - ks * G;
      const int left = rows_total - (row0 + 4 * rg);
      nval[e] = ks < BK ? (left < 0 ? 0 : (left > 4 ? 4 : left)) : 0;
      base[e] = nval[e] > 0 ? (uint32_t)(ks * ld + row0 + 4 * rg) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, ks = s / G;
      const uint32_t off = (k0 + ks < kend) ? base[e] + (uint32_t)(k0 * ld) * 4u : OOB;
      if (VEC) {
        v[e] = buf_load4(rs, off);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[e][j] = buf_load(rs, j < nval[e] ? off + 4u * j : OOB);
      }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, ks = s / G, rg = s - ks * G;
      if (BK * G % 256 == 0 || ks < BK) *reinterpret_cast<f32x4*>(&lds[ks * R + 4 * rg]) = v[e];
    }
  }
};

// Geometry of one convolution, shared by host and device.
struct ConvGeom {
  int N, C, IH, IW, O, KH, KW, OH, OW, PADL, PADT, S, D;
  int IHW, OHW, KK;
  FastDiv dOW, dOHW, dIW, dIHW, dS;
};

// Per-k table entry of an implicit-GEMM gather.  Built once per geometry.
//   fwd / wgrad (k = (c, kh, kw)):  x = c*IH*IW + kh*D*IW + kw*D, y = kh*D, z = kw*D
//   dgrad       (k = (o, kh, kw)):  x = o*OH*OW,                  y = kh*D, z = kw*D,
//                                   w = o*C*KK + kh*KW + kw
// Entries past the last k carry y = BIG (fails the row range test) and
// w = 0x20000000 (byte offset 2 GiB: out of range).
struct __attribute__((aligned(16))) KEntry { int x, y, z, w; };

// The table is read through the constant address space with wave-uniform
// indices so that entries arrive in scalar registers (s_load), one K step
// ahead of their use: a loader's fetch(k0) consumes the entries fetched by the
// previous call and requests those of k0 + BK.
typedef const __attribute__((address_space(4))) KEntry* ktab_t;
__device__ __forceinline__ ktab_t as_ktab(const KEntry* p) {
  return reinterpret_cast<ktab_t>(reinterpret_cast<uintptr_t>(p));
}

// Forward im2col gather: element (pixel p, k) = X[n, c, oh*S-PT+kh*D, ow*S-PL+kw*D].
// Each wavefront fetches 4 of the 16 k rows; lanes run over pixels so that
// global reads follow the image rows and k stays wave-uniform.
template <int R>
struct ConvFwdB {
  static constexpr bool KC = false;
  static constexpr int CC = (R + 63) / 64;
  rsrc_t rs;
  ktab_t tab;
  int IH, IW;
  int base[CC], ih0[CC], iw0[CC];
  int tx[4], ty[4], tz[4];   // table entries of the next fetch (scalar registers)
  float v[4][CC];
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const ktab_t t = tab + (k0 + wave + 4 * e);
      tx[e] = t->x; ty[e] = t->y; tz[e] = t->z;
    }
  }
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab_, int p0, int P, int kbeg) {
    rs = r;
    tab = as_ktab(tab_);
    load_entries(kbeg);
    IH = g.IH;
    IW = g.IW;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dOHW.div(pp), rem = pp - img * g.OHW;
      const uint32_t oh = g.dOW.div(rem), ow = rem - oh * g.OW;
      ih0[c] = (int)oh * g.S - g.PADT;
      iw0[c] = ok ? (int)ow * g.S - g.PADL : -BIG;
      base[c] = ((int)img * g.C * g.IH + ih0[c]) * g.IW + ((int)ow * g.S - g.PADL);
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
#pragma unroll
      for (int c = 0; c < CC; ++c) {
        const bool ok = (uint32_t)(ih0[c] + ty[e]) < (uint32_t)IH && (uint32_t)(iw0[c] + tz[e]) < (uint32_t)IW;
        v[e][c] = buf_load(rs, ok ? (uint32_t)(base[c] + tx[e]) * 4u : OOB);
      }
    }
    load_entries(k0 + BK);
  }
  __device__ __forceinline__ void commit(float* lds) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < CC; ++c)
        if (R % 64 == 0 || lane + 64 * c < R) lds[(wave + 4 * e) * R + lane + 64 * c] = v[e][c];
  }
};

// Tap-major variants of the two pixel gathers, for channel counts that are a
// multiple of BK.  K is ordered k = tap*CH + ch (tap = kh*KW + kw), so one K
// step is BK consecutive channels of a single tap: the pixel part of the
// address and its range test depend on the tap only and live in a VGPR, the
// channel part is wave-uniform and rides in the scalar offset of the buffer
// instruction.  No table, no per-element arithmetic.  fetch() must be called
// with consecutive K steps starting at the kbeg given to init().
__device__ __forceinline__ float buf_load_s(rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0));
}

template <int R>
struct ConvFwdBTap {
  static constexpr bool KC = false;
  static constexpr int CC = (R + 63) / 64;
  rsrc_t rs;
  int IH, IW, IHW, C, D, KW;
  int base[CC], ih0[CC], iw0[CC];
  int c0, kh, kw;   // K position of the next fetch
  float v[4][CC];
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int p0, int P, int kbeg) {
    rs = r;
    IH = g.IH; IW = g.IW; IHW = g.IHW; C = g.C; D = g.D; KW = g.KW;
    const int tap = kbeg / g.C;
    c0 = kbeg - tap * g.C;
    kh = tap / g.KW;
    kw = tap - kh * g.KW;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dOHW.div(pp), rem = pp - img * g.OHW;
      const uint32_t oh = g.dOW.div(rem), ow = rem - oh * g.OW;
      ih0[c] = (int)oh * g.S - g.PADT;
      iw0[c] = ok ? (int)ow * g.S - g.PADL : -BIG;
      base[c] = ((int)img * g.C * g.IH + ih0[c]) * g.IW + ((int)ow * g.S - g.PADL);
    }
  }
  __device__ __forceinline__ void fetch(int) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dh = kh * D, dw = kw * D, tapoff = dh * IW + dw;
    uint32_t voff[CC];
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const bool ok = (uint32_t)(ih0[c] + dh) < (uint32_t)IH && (uint32_t)(iw0[c] + dw) < (uint32_t)IW;
      voff[c] = ok ? (uint32_t)(base[c] + tapoff) * 4u : OOB;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t soff = (uint32_t)((c0 + wave + 4 * e) * IHW) * 4u;
#pragma unroll
      for (int c = 0; c < CC; ++c) v[e][c] = buf_load_s(rs, voff[c], soff);
    }
    c0 += BK;
    if (c0 >= C) {
      c0 = 0;
      ++kw;
      if (kw == KW) { kw = 0; ++kh; }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < CC; ++c)
        if (R % 64 == 0 || lane + 64 * c < R) lds[(wave + 4 * e) * R + lane + 64 * c] = v[e][c];
  }
};

template <int R, bool STRIDE1>
struct ConvDgradBTap {
  static constexpr bool KC = false;
  static constexpr int CC = (R + 63) / 64;
  rsrc_t rs;
  int OH, OW, OHW, O, S, D, KW;
  FastDiv dS;
  int base[CC], a0[CC], b0[CC];
  int o0, kh, kw;
  float v[4][CC];
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int p0, int P, int kbeg) {
    rs = r;
    OH = g.OH; OW = g.OW; OHW = g.OHW; O = g.O; S = g.S; D = g.D; KW = g.KW;
    dS = g.dS;
    const int tap = kbeg / g.O;
    o0 = kbeg - tap * g.O;
    kh = tap / g.KW;
    kw = tap - kh * g.KW;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dIHW.div(pp), rem = pp - img * g.IHW;
      const uint32_t ih = g.dIW.div(rem), iw = rem - ih * g.IW;
      a0[c] = (int)ih + g.PADT;
      b0[c] = ok ? (int)iw + g.PADL : -BIG;
      base[c] = (int)img * g.O * g.OHW;
    }
  }
  __device__ __forceinline__ void fetch(int) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int dh = kh * D, dw = kw * D;
    uint32_t voff[CC];
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int nh = a0[c] - dh, nw = b0[c] - dw;
      bool ok;
      int oh, ow;
      if (STRIDE1) {
        oh = nh;
        ow = nw;
        ok = (uint32_t)nh < (uint32_t)OH && (uint32_t)nw < (uint32_t)OW;
      } else {
        oh = (int)dS.div((uint32_t)nh & 0x7fffffffu);
        ow = (int)dS.div((uint32_t)nw & 0x7fffffffu);
        ok = nh >= 0 && nw >= 0 && oh * S == nh && ow * S == nw && oh < OH && ow < OW;
      }
      voff[c] = ok ? (uint32_t)(base[c] + oh * OW + ow) * 4u : OOB;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t soff = (uint32_t)((o0 + wave + 4 * e) * OHW) * 4u;
#pragma unroll
      for (int c = 0; c < CC; ++c) v[e][c] = buf_load_s(rs, voff[c], soff);
    }
    o0 += BK;
    if (o0 >= O) {
      o0 = 0;
      ++kw;
      if (kw == KW) { kw = 0; ++kh; }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < CC; ++c)
        if (R % 64 == 0 || lane + 64 * c < R) lds[(wave + 4 * e) * R + lane + 64 * c] = v[e][c];
  }
};

// dgrad gather of dY: element (input pixel (n, ih, iw), k = (o, kh, kw)) =
// dY[n, o, (ih+PT-kh*D)/S, (iw+PL-kw*D)/S] when both quotients are exact and
// in range, else 0.
template <int R, bool STRIDE1>
struct ConvDgradB {
  static constexpr bool KC = false;
  static constexpr int CC = (R + 63) / 64;
  rsrc_t rs;
  ktab_t tab;
  int OH, OW, S;
  FastDiv dS;
  int base[CC], a0[CC], b0[CC];
  int tx[4], ty[4], tz[4];
  float v[4][CC];
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const ktab_t t = tab + (k0 + wave + 4 * e);
      tx[e] = t->x; ty[e] = t->y; tz[e] = t->z;
    }
  }
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab_, int p0, int P, int kbeg) {
    rs = r;
    tab = as_ktab(tab_);
    load_entries(kbeg);
    OH = g.OH;
    OW = g.OW;
    S = g.S;
    dS = g.dS;
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dIHW.div(pp), rem = pp - img * g.IHW;
      const uint32_t ih = g.dIW.div(rem), iw = rem - ih * g.IW;
      a0[c] = (int)ih + g.PADT;
      b0[c] = ok ? (int)iw + g.PADL : -BIG;
      base[c] = (int)img * g.O * g.OHW;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int t_x = tx[e];
#pragma unroll
      for (int c = 0; c < CC; ++c) {
        const int nh = a0[c] - ty[e], nw = b0[c] - tz[e];
        bool ok;
        int oh, ow;
        if (STRIDE1) {
          oh = nh;
          ow = nw;
          ok = (uint32_t)nh < (uint32_t)OH && (uint32_t)nw < (uint32_t)OW;
        } else {
          oh = (int)dS.div((uint32_t)nh & 0x7fffffffu);
          ow = (int)dS.div((uint32_t)nw & 0x7fffffffu);
          ok = nh >= 0 && nw >= 0 && oh * S == nh && ow * S == nw && oh < OH && ow < OW;
        }
        v[e][c] = buf_load(rs, ok ? (uint32_t)(base[c] + t_x + oh * OW + ow) * 4u : OOB);
      }
    }
    load_entries(k0 + BK);
  }
  __device__ __forceinline__ void commit(float* lds) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int c = 0; c < CC; ++c)
        if (R % 64 == 0 || lane + 64 * c < R) lds[(wave + 4 * e) * R + lane + 64 * c] = v[e][c];
  }
};

// dgrad weight gather: element (c, k = (o, kh, kw)) = W[o, c, kh, kw].
// Wavefront w fetches k columns 4w..4w+3 (wave-uniform table entries); lanes
// run over the channel rows.
template <int R>
struct ConvDgradA {
  static constexpr bool KC = true;
  static constexpr int E = (R + 63) / 64;
  rsrc_t rs;
  ktab_t tab;
  uint32_t cb[E];
  uint32_t tw[4];
  f32x4 v[E];
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
#pragma unroll
    for (int j = 0; j < 4; ++j) tw[j] = (uint32_t)(tab + (k0 + 4 * wave + j))->w;
  }
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab_, int c0, int kbeg) {
    rs = r;
    tab = as_ktab(tab_);
    load_entries(kbeg);
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int row = lane + 64 * e;
      cb[e] = (row < R && c0 + row < g.C) ? (uint32_t)((c0 + row) * g.KK) : 0x20000000u;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = tw[j];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        // either term alone is >= 2^29 elements (2 GiB) when invalid; clamp the sum
        const uint32_t idx = cb[e] + w;
        v[e][j] = buf_load(rs, idx >= 0x20000000u ? OOB : idx * 4u);
      }
    }
    load_entries(k0 + BK);
  }
  __device__ __forceinline__ void commit(float* lds) const {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (R % 64 == 0 || lane + 64 * e < R)
        *reinterpret_cast<f32x4*>(&lds[(lane + 64 * e) * LDK + 4 * wave]) = v[e];
  }
};

// wgrad A side: dY viewed as [O][P], k = p = (n, oh, ow); element (o, p) at
// (n*O + o)*OHW + (p mod OHW).  VEC requires OHW % 4 == 0.
template <int R, bool VEC>
struct ConvWgradA {
  static constexpr bool KC = true;
  static constexpr int E = (R * 4 + 255) / 256;
  rsrc_t rs;
  uint32_t rb[E];
  int O, OHW, kend;
  FastDiv dOHW;
  f32x4 v[E];
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int o0, int kend_) {
    rs = r;
    O = g.O;
    OHW = g.OHW;
    dOHW = g.dOHW;
    kend = kend_;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2;
      rb[e] = (row < R && o0 + row < g.O) ? (uint32_t)((o0 + row) * g.OHW) : 0x20000000u;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    const int kg = threadIdx.x & 3;
    if (VEC) {
      const uint32_t p = (uint32_t)(k0 + 4 * kg);
      const uint32_t img = dOHW.div(p), rem = p - img * OHW;
      const uint32_t pb = (p < (uint32_t)kend) ? img * (uint32_t)(O * OHW) + rem : 0x20000000u;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const uint32_t idx = rb[e] + pb;
        v[e] = buf_load4(rs, idx >= 0x20000000u ? OOB : idx * 4u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t p = (uint32_t)(k0 + 4 * kg + j);
        const uint32_t img = dOHW.div(p), rem = p - img * OHW;
        const uint32_t pb = (p < (uint32_t)kend) ? img * (uint32_t)(O * OHW) + rem : 0x20000000u;
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const uint32_t idx = rb[e] + pb;
          v[e][j] = buf_load(rs, idx >= 0x20000000u ? OOB : idx * 4u);
        }
      }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2, kg = s & 3;
      if (R * 4 % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[row * LDK + 4 * kg]) = v[e];
    }
  }
};

// wgrad B side: im2row gather with k = p; element (q = (c, kh, kw), p) =
// X[n, c, oh*S-PT+kh*D, ow*S-PL+kw*D].
template <int R>
struct ConvWgradB {
  static constexpr bool KC = true;
  static constexpr int E = (R * 4 + 255) / 256;
  rsrc_t rs;
  int xo[E], dh[E], dw[E];
  int C, IH, IW, IHW, OHW, OW, S, PADL, PADT, kend;
  FastDiv dOHW, dOW;
  f32x4 v[E];
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab, int q0, int Q, int kend_) {
    rs = r;
    C = g.C; IH = g.IH; IW = g.IW; IHW = g.IHW; OHW = g.OHW; OW = g.OW;
    S = g.S; PADL = g.PADL; PADT = g.PADT;
    dOHW = g.dOHW; dOW = g.dOW;
    kend = kend_;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2;
      const bool ok = row < R && q0 + row < Q;
      const KEntry t = tab[ok ? q0 + row : 0];
      xo[e] = t.x;
      dh[e] = ok ? t.y : BIG;
      dw[e] = t.z;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    const int kg = threadIdx.x & 3;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t p = (uint32_t)(k0 + 4 * kg + j);
      const bool pok = p < (uint32_t)kend;
      const uint32_t pp = pok ? p : 0u;
      const uint32_t img = dOHW.div(pp), rem = pp - img * OHW;
      const uint32_t oh = dOW.div(rem), ow = rem - oh * OW;
      const int ih0 = (int)oh * S - PADT;
      const int iw0 = pok ? (int)ow * S - PADL : -BIG;
      const int pb = ((int)img * C * IH + ih0) * IW + ((int)ow * S - PADL);
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const bool ok = (uint32_t)(ih0 + dh[e]) < (uint32_t)IH && (uint32_t)(iw0 + dw[e]) < (uint32_t)IW;
        v[e][j] = buf_load(rs, ok ? (uint32_t)(pb + xo[e]) * 4u : OOB);
      }
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = threadIdx.x + 256 * e, row = s >> 2, kg = s & 3;
      if (R * 4 % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[row * LDK + 4 * kg]) = v[e];
    }
  }
};

// ---------------------------------------------------------------------------
// Output mapping.  plain: off = m*ld + n.  NCHW image tensor with the GEMM
// column n = (img, pixel): off = (img*Mtot + m)*HW + pixel.
// ---------------------------------------------------------------------------
struct OutMap {
  int nchw;    // 0 plain, 1 image layout
  int ld;      // plain: leading dimension; nchw: HW
  int mtot;    // nchw: channel count
  FastDiv dHW;
  __device__ __forceinline__ uint32_t col(uint32_t n) const {
    if (!nchw) return n;
    const uint32_t img = dHW.div(n);
    return img * (uint32_t)(mtot * ld) + (n - img * ld);
  }
};

// ---------------------------------------------------------------------------
// The MFMA step: both operands come from LDS in one of two layouts.
// Lane (i = lane % 32, h = lane / 32) feeds row i of the 32-row fragment; in
// each group of 8 k values lane half h supplies k = 8*kk + 4*h + t to the
// t-th MFMA.  A and B use the same k assignment, so any k permutation cancels.
// ---------------------------------------------------------------------------
template <int NT, bool A_KC, bool B_KC, int RA, int RB>
__device__ __forceinline__ void load_frags(const float* __restrict__ As, const float* __restrict__ Bs, int arow,
                                           int brow, int kk, float (&a)[4], float (&b)[NT][4]) {
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  const int kb = kk * 8 + h * 4;
  if (A_KC) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(&As[(arow + i) * LDK + kb]);
    a[0] = t[0]; a[1] = t[1]; a[2] = t[2]; a[3] = t[3];
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) a[t] = As[(kb + t) * RA + arow + i];
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (B_KC) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(&Bs[(brow + 32 * j + i) * LDK + kb]);
      b[j][0] = t[0]; b[j][1] = t[1]; b[j][2] = t[2]; b[j][3] = t[3];
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) b[j][t] = Bs[(kb + t) * RB + brow + 32 * j + i];
    }
  }
}

// One LDS stage = BK/8 groups of 4*NT MFMAs.  The fragments of group kk+1 are
// read from LDS before the MFMAs of group kk are issued, so the LDS latency is
// covered by a full group of matrix work instead of stalling every group.
template <int NT, bool A_KC, bool B_KC, int RA, int RB>
__device__ __forceinline__ void mma_stage(const float* __restrict__ As, const float* __restrict__ Bs,
                                          f32x16 (&acc)[NT], int arow, int brow) {
  float a[2][4], b[2][NT][4];
  load_frags<NT, A_KC, B_KC, RA, RB>(As, Bs, arow, brow, 0, a[0], b[0]);
#pragma unroll
  for (int kk = 0; kk < BK / 8; ++kk) {
    const int cur = kk & 1;
    if (kk + 1 < BK / 8) load_frags<NT, A_KC, B_KC, RA, RB>(As, Bs, arow, brow, kk + 1, a[cur ^ 1], b[cur ^ 1]);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][t], b[cur][j][t], acc[j], 0, 0, 0);
  }
}

template <bool KC, int R>
struct LdsSize { static constexpr int value = KC ? R * LDK : BK * R; };

// One output sub-tile: BM x BN with BM = 32*WM, BN = 32*WN*NT.
// The loaders must already be initialised for this tile.
template <int WM, int NT, class LA, class LB>
__device__ __forceinline__ void run_tile(LA& la, LB& lb, float* ldsA, float* ldsB, int strideA, int strideB,
                                         int kbeg, int kend, rsrc_t rc, const OutMap& om, int m0, int n0,
                                         int M, int Ncols, int beta) {
  constexpr int WN = 4 / WM, BM = 32 * WM, BN = 32 * WN * NT;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave % WM, wn = wave / WM;
  f32x16 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

  const int nk = (kend - kbeg + BK - 1) / BK;
  if (nk > 0) {
    la.fetch(kbeg);
    lb.fetch(kbeg);
    la.commit(ldsA);
    lb.commit(ldsB);
  }
  __syncthreads();
  // Steady state: the global loads of K step it+1 are issued first, so that
  // they (and their address arithmetic) share one scheduling region with the
  // MFMAs of step it; the data is parked in LDS after the MFMAs.
  for (int it = 0; it + 1 < nk; ++it) {
    const int cur = it & 1;
    la.fetch(kbeg + (it + 1) * BK);
    lb.fetch(kbeg + (it + 1) * BK);
    __builtin_amdgcn_sched_barrier(0);   // keep the loads ahead of the matrix work
    mma_stage<NT, LA::KC, LB::KC, BM, BN>(ldsA + cur * strideA, ldsB + cur * strideB, acc, wm * 32, wn * NT * 32);
    __builtin_amdgcn_sched_barrier(0);
    la.commit(ldsA + (cur ^ 1) * strideA);
    lb.commit(ldsB + (cur ^ 1) * strideB);
    __syncthreads();
  }
  if (nk > 0) {
    const int cur = (nk - 1) & 1;
    mma_stage<NT, LA::KC, LB::KC, BM, BN>(ldsA + cur * strideA, ldsB + cur * strideB, acc, wm * 32, wn * NT * 32);
    __syncthreads();   // the next sub-tile's prologue overwrites stage 0
  }

  // epilogue: acc[j][r] is C[m0 + wm*32 + 8*(r/4) + 4*(lane/32) + r%4][n0 + (wn*NT + j)*32 + lane%32]
  const int i = lane & 31, h = lane >> 5;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n0 + (wn * NT + j) * 32 + i;
    const bool nok = n < Ncols;
    const uint32_t cb = om.col(nok ? (uint32_t)n : 0u);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      const uint32_t off = (nok && m < M) ? (cb + (uint32_t)(m * om.ld)) * 4u : OOB;
      float val = acc[j][r];
      if (beta) val += buf_load(rc, off);
      buf_store(rc, off, val);
    }
  }
}

// Sub-tile width policy for a remaining run of cnt units.
template <int NTMAX>
__device__ __forceinline__ int pick_units(int cnt) {
  if (cnt <= NTMAX) return cnt;
  if (cnt >= 2 * NTMAX) return NTMAX;
  return (cnt + 1) >> 1;
}

}  // namespace lnn
