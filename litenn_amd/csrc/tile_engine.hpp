// fp32 MFMA tile engine for gfx950 (CDNA4): one kernel skeleton shared by the
// plain GEMM and by the three implicit-GEMM convolution passes.
//
//   C[m, n] (+)= sum_k A(m, k) * B(k, n)
//
// A workgroup has 512 threads: two groups of 4 wavefronts (arranged WM x WN
// inside a group).  The two groups share one compute unit's four SIMDs, one
// wavefront of each group per SIMD, and run in opposite phases separated by
// workgroup barriers ("ping-pong"): while one group issues the MFMAs of a K
// step, the other parks its previously fetched operands in LDS and issues the
// global loads of a later step, so the matrix pipe of every SIMD always has
// one wavefront feeding it.  Both groups work on the same M tile and K step
// (they share the A operand tile in LDS) and on adjacent column ranges: group
// g owns NT_g accumulators of v_mfma_f32_32x32x2_f32 per wavefront, i.e. a
// 32 x (32*NT_g) slab.  Operand tiles are double buffered in LDS and filled by
// "loader" objects which differ only in how they turn (row, k) into a global
// address: plain strided matrices or on-the-fly im2col gathers.  All global
// traffic uses raw buffer instructions so that an out-of-range or masked
// element is a hardware zero (loads) or a dropped write (stores) instead of a
// branch or a fault.
//
// Work distribution: the output is cut into "units" of 32*WN columns per
// M-tile; the launch gives every workgroup a contiguous, nearly equal range of
// units (so all compute units finish together regardless of how the problem
// size divides into tiles) and the workgroup walks its range in sub-tiles of
// 1..2*NTMAX units, split between the two groups.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace lnn {

constexpr int BK = 32;            // K extent of one LDS stage
constexpr int KG = BK / 4;        // float4 groups along K
constexpr int KR = BK / 4;        // K rows fetched per wavefront of a group in the pixel-major gathers
constexpr int LDK = BK + 4;       // row stride (floats) of a K-contiguous LDS tile
constexpr uint32_t OOB = 0x80000000u;  // byte offset beyond every buffer (< 2 GiB each)
constexpr int BIG = 0x40000000;   // coordinate that fails every range test

// LDS tile layouts.  R = rows of the tile (BM on the A side, a group's columns on the B side).
//   LAY_KC        tile[row][LDK]: k contiguous, rows padded to LDK floats
//   LAY_KC_SWZ    tile[row][BK]:  k contiguous, no padding, 4-float group g of row r in slot g ^ (r % 8)
//   LAY_MC        tile[k][R]:     row contiguous, one tile shared by both groups
//   LAY_MC_SPLIT  one tile[k][R'] per group, back to back: a group's slab of R' rows
//                 starting at tile row `off` begins at float off*BK
enum { LAY_KC = 0, LAY_KC_SWZ = 1, LAY_MC = 2, LAY_MC_SPLIT = 3, LAY_KC_SWZP = 4 };
//   LAY_KC_SWZP   the same with group g of row r in slot g ^ ((r / 2) % 8).  LDS has 64 banks of 4 bytes and serves a
//                 128-bit read 16 lanes at a time; rows of 128 bytes alternate between the two bank halves, so 16
//                 consecutive rows reading the same group are conflict free only if the eight rows of each parity sit
//                 in eight different slots.  Keyed by r % 8 (LAY_KC_SWZ) rows r and r + 8 collide: measured 32 cycles
//                 per ds_read_b128 against 16.  Loaders that move 16 bytes per lane use this key; those that move 4
//                 bytes per lane fill a row pair per instruction and need one key per wavefront, which only the r % 8
//                 key gives them.
constexpr bool lay_kc(int l) { return l == LAY_KC || l == LAY_KC_SWZ || l == LAY_KC_SWZP; }
constexpr bool lay_swz(int l) { return l == LAY_KC_SWZ || l == LAY_KC_SWZP; }

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
using rsrc_t = __amdgpu_buffer_rsrc_t;

// thread / wavefront index inside a group of 256 threads
__device__ __forceinline__ int gtid() { return threadIdx.x & 255; }
__device__ __forceinline__ int gwave() { return (threadIdx.x >> 6) & 3; }

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load(rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0));
}
__device__ __forceinline__ f32x4 buf_load4(rsrc_t r, uint32_t off) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
}
// voff is per lane; soff is wave-uniform and travels in a scalar register, so
// a K step can advance the address without any vector arithmetic.
__device__ __forceinline__ float buf_load_s(rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0));
}
__device__ __forceinline__ f32x4 buf_load4_s(rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}
// Global -> LDS without passing through registers: lane l of the wavefront
// deposits its 4 (16) bytes at lds + 4*l (16*l).  lds must be wave-uniform.
// An out-of-range lane writes zeros, an inactive lane writes nothing.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
__device__ __forceinline__ void buf_load_lds4(rsrc_t r, float* lds, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)lds, 4, (int)voff, (int)soff, 0, 0);
}
__device__ __forceinline__ void buf_load_lds16(rsrc_t r, float* lds, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)lds, 16, (int)voff, (int)soff, 0, 0);
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
  static constexpr int E = (R * KG + 255) / 256;
  rsrc_t rs;
  uint32_t base[E];
  int kend;
  f32x4 v[E];
  __device__ __forceinline__ void init(rsrc_t r, int ld, int row0, int rows_total, int kend_) {
    rs = r;
    kend = kend_;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, row = s / KG, kg = s % KG;
      const bool ok = row < R && row0 + row < rows_total;
      base[e] = ok ? (uint32_t)((row0 + row) * ld + 4 * kg) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    if (k0 + BK <= kend) {   // whole K step in range (wave-uniform): no per-lane arithmetic
      const uint32_t soff = (uint32_t)k0 * 4u;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (VEC) {
          v[e] = buf_load4_s(rs, base[e], soff);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[e][j] = buf_load_s(rs, base[e] + 4u * j, soff);
        }
      }
      return;
    }
    const int kg = gtid() % KG;
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
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, row = s / KG, kg = s % KG;
      if (R * KG % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[(off + row) * LDK + 4 * kg]) = v[e];
    }
  }
};

// Plain strided matrix, K-contiguous, straight into LDS (needs K % BK == 0 and
// 16-byte aligned rows).  The LDS tile is [row][BK] without padding; to keep
// the 128-bit fragment reads conflict free the k groups of a row are stored
// XOR-swizzled: group g of row r sits in slot g ^ ((r / 2) % 8) (LAY_KC_SWZP).  One instruction
// moves 8 rows (1 KiB): lane l carries slot l % 8 of row l / 8.
template <int R>
struct DirectKC {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZP;
  static constexpr int NB = R / 8, E = (NB + 3) / 4;
  static constexpr int NLD = NB % 4 == 0 ? E : -1;   // transfers per wavefront and K step (-1: differs between wavefronts)
  static_assert(R % 8 == 0, "whole 8-row blocks");
  rsrc_t rs;
  uint32_t voff[E];
  __device__ __forceinline__ void init(rsrc_t r, int ld, int row0, int M, int) {
    rs = r;
    // tile row = 8 * (wave + 4e) + rb (plus the group's offset, a multiple of 16): (row / 2) % 8 is the same for all e
    const int wave = gwave(), lane = threadIdx.x & 63, rb = lane >> 3, kg = (lane & 7) ^ (((wave & 1) << 2) | (rb >> 1));
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int row = row0 + (wave + 4 * e) * 8 + rb;
      voff[e] = row < M ? (uint32_t)(row * ld + kg * 4) * 4u : OOB;
    }
  }
  // off: first tile row of this group.  Returns the number of transfers this wavefront issued.
  // issue_part<PART, NPARTS> sends the PART-th of NPARTS shares of a K step's transfers (all loaders: the shares of
  // one K step are asked for in order, and the loader moves on to the next K step with the last one).
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int k0, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    int n = 0;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e) {
      const int blk = wave + 4 * e;
      if (NB % 4 == 0 || blk < NB) { buf_load_lds16(rs, lds + (off + blk * 8) * BK, voff[e], (uint32_t)k0 * 4u); ++n; }
    }
    return n;
  }
};

// Plain strided matrix stored K-major (element (r, k) at k*ld + r), straight
// into LDS with 128-bit transfers (16-byte aligned rows, row count % 4 == 0).
// One instruction moves 256 consecutive floats of the group's [BK][R] slab.
// K rows past the end lie beyond the buffer and arrive as zeros.
template <int R>
struct DirectMC {
  static constexpr bool KC = false, DIRECT = true;
  static constexpr int LAYOUT = LAY_MC_SPLIT;
  static constexpr int NI = BK * R / 256, E = (NI + 3) / 4;
  static constexpr int NLD = NI % 4 == 0 ? E : -1;
  static_assert(R % 8 == 0, "whole 256-float transfers");
  rsrc_t rs;
  uint32_t voff[E];
  int ld;
  __device__ __forceinline__ void init(rsrc_t r, int ld_, int row0, int M, int) {
    rs = r;
    ld = ld_;
    const int wave = gwave(), lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int f = (wave + 4 * e) * 256 + lane * 4, k = f / R, n = f - k * R;
      voff[e] = (k < BK && row0 + n < M) ? (uint32_t)(k * ld + row0 + n) * 4u : OOB;
    }
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld_, int off) { return issue_part<0, 1>(k0, lds, ld_, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int k0, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const uint32_t soff = (uint32_t)(k0 * ld) * 4u;
    int n = 0;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e) {
      const int q = wave + 4 * e;
      if (NI % 4 == 0 || q < NI) { buf_load_lds16(rs, lds + off * BK + q * 256, voff[e], soff); ++n; }
    }
    return n;
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
      const int s = gtid() + 256 * e, ks = s / G, rg = s - ks * G;
      const int left = rows_total - (row0 + 4 * rg);
      nval[e] = ks < BK ? (left < 0 ? 0 : (left > 4 ? 4 : left)) : 0;
      base[e] = nval[e] > 0 ? (uint32_t)(ks * ld + row0 + 4 * rg) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    if (k0 + BK <= kend) {   // whole K step in range (wave-uniform)
      const uint32_t soff = (uint32_t)(k0 * ld) * 4u;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (VEC) {
          v[e] = buf_load4_s(rs, base[e], soff);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[e][j] = buf_load_s(rs, j < nval[e] ? base[e] + 4u * j : OOB, soff);
        }
      }
      return;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, ks = s / G;
      const uint32_t off = (k0 + ks < kend) ? base[e] + (uint32_t)(k0 * ld) * 4u : OOB;
      if (VEC) {
        v[e] = buf_load4(rs, off);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[e][j] = buf_load(rs, j < nval[e] ? off + 4u * j : OOB);
      }
    }
  }
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, ks = s / G, rg = s - ks * G;
      if (BK * G % 256 == 0 || ks < BK) *reinterpret_cast<f32x4*>(&lds[ks * ld + off + 4 * rg]) = v[e];
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

// The forward pass's weight operand Wp[o][tap][c], rows of K = KK*C floats, read in the K order of ConvFwdBTap
// (see there): K step (channel block, tap) sits at row offset tap*C + block*BK.
template <int R>
struct ConvFwdATap : DirectKC<R> {
  int C, KK, c0, tap;
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int row0, int M, int kbeg) {
    DirectKC<R>::init(r, g.C * g.KK, row0, M, 0);
    C = g.C; KK = g.KK;
    const int t0 = kbeg / BK, cb = t0 / g.KK;
    tap = t0 - cb * g.KK;
    c0 = cb * BK;
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int ld, int off) {
    const int n = DirectKC<R>::template issue_part<PART, NPARTS>(tap * C + c0, lds, ld, off);
    if (PART == NPARTS - 1) {
      if (++tap == KK) { tap = 0; c0 += BK; }
    }
    return n;
  }
};

// Plain strided matrix, K-contiguous, any K and any alignment, straight into a swizzled LDS tile with 4-byte
// transfers (the layout of DirectKC, filled like ConvWgradTapADirect fills it: one transfer = two adjacent tile rows,
// lanes 0..31 the even one, and a lane's swizzled position is one fixed k of the K step).  K positions past the end
// of a row arrive as zeros.
__device__ __forceinline__ int direct_k4() {   // k (0..BK-1) whose swizzled position this lane fills
  const int lane = threadIdx.x & 63, pos = lane & 31, key = 2 * gwave() + (lane >> 5);
  return (((pos >> 2) ^ key) << 2) | (pos & 3);
}
template <int R>
struct DirectKC4 {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZ;
  static constexpr int E = R / 8, NLD = E;
  static_assert(R % 8 == 0, "whole row pairs for all four wavefronts");
  rsrc_t rs;
  uint32_t roff[E];   // byte offset of (this lane's row of transfer e, this lane's k), or OOB for a row past the end
  int kk, K;
  __device__ __forceinline__ void init(rsrc_t r, int ld, int row0, int M, int K_) {
    rs = r;
    K = K_;
    kk = direct_k4();
    const int half = (int)((threadIdx.x & 63) >> 5);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int row = row0 + 8 * e + 2 * gwave() + half;
      roff[e] = row < M ? (uint32_t)(row * ld + kk) * 4u : OOB;
    }
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int k0, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const bool kok = k0 + kk < K;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e)
      buf_load_lds4(rs, lds + (off + 8 * e + 2 * wave) * BK, kok ? roff[e] : OOB, (uint32_t)k0 * 4u);
    return E * (PART + 1) / NPARTS - E * PART / NPARTS;
  }
};

// ConvFwdB with the gathered elements sent straight into the LDS stage (element (k = wave + 4e, column lane + 64c)
// of the row-contiguous tile), no staging registers and no LDS writes.
template <int R>
struct ConvFwdBDirect {
  static constexpr bool KC = false, DIRECT = true;
  static constexpr int CC = (R + 63) / 64;
  static constexpr int NLD = KR * CC;
  rsrc_t rs;
  ktab_t tab;
  int IH, IW;
  int base[CC], ih0[CC], iw0[CC];
  int tx[KR], ty[KR], tz[KR];   // table entries of the next K step (scalar registers)
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int e = 0; e < KR; ++e) {
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
  // must be called with consecutive K steps starting at the kbeg given to init()
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int k0, float* lds, int ld, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int e = KR * PART / NPARTS; e < KR * (PART + 1) / NPARTS; ++e) {
#pragma unroll
      for (int c = 0; c < CC; ++c) {
        const bool ok = (uint32_t)(ih0[c] + ty[e]) < (uint32_t)IH && (uint32_t)(iw0[c] + tz[e]) < (uint32_t)IW;
        // all 64 lanes, also where the group is narrower (see run_tile): no lane mask around a transfer
        buf_load_lds4(rs, lds + (wave + 4 * e) * ld + off + 64 * c, ok ? (uint32_t)(base[c] + tx[e]) * 4u : OOB, 0);
      }
    }
    if (PART == NPARTS - 1) load_entries(k0 + BK);
    return (KR * (PART + 1) / NPARTS - KR * PART / NPARTS) * CC;
  }
};

// Tap-major variants of the two pixel gathers, for channel counts that are a
// multiple of BK.  K is ordered k = tap*CH + ch (tap = kh*KW + kw), so one K
// step is BK consecutive channels of a single tap: the pixel part of the
// address and its range test depend on the tap only and live in a VGPR, the
// channel part is wave-uniform and rides in the scalar offset of the buffer
// instruction.  No table, no per-element arithmetic.  issue() must be called
// with consecutive K steps starting at the kbeg given to init().
// K order: the channel block is the outer loop and the taps the inner one (k-step t = block * KK +
// tap), so that the KK consecutive steps of one block of BK channels re-read the same pixels, shifted, while they
// are still in the L2 of the XCD; tap-major order (all channels of a tap, then the next tap) revisits a pixel only
// after the whole channel range, by when a 4 MB L2 shared by 32 workgroups has dropped it.
template <int R>
struct ConvFwdBTap {
  static constexpr bool KC = false, DIRECT = true;
  static constexpr int CC = (R + 63) / 64;
  static constexpr int NLD = KR * CC;
  rsrc_t rs;
  int IH, IW, IHW, C, D, KW, KH;
  int base[CC], ih0[CC], iw0[CC];
  uint32_t voff[CC];   // per-pixel byte offset for the current tap, or OOB
  int c0, kh, kw;   // K position of the next transfer
  __device__ __forceinline__ void set_tap() {
    const int dh = kh * D, dw = kw * D, tapoff = dh * IW + dw;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const bool ok = (uint32_t)(ih0[c] + dh) < (uint32_t)IH && (uint32_t)(iw0[c] + dw) < (uint32_t)IW;
      voff[c] = ok ? (uint32_t)(base[c] + tapoff) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int p0, int P, int kbeg) {
    rs = r;
    IH = g.IH; IW = g.IW; IHW = g.IHW; C = g.C; D = g.D; KW = g.KW; KH = g.KH;
    const int t0 = kbeg / BK, cb = t0 / g.KK, tap = t0 - cb * g.KK;
    c0 = cb * BK;
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
    set_tap();
  }
  __device__ __forceinline__ void advance() {
    ++kw;                                   // next tap of the same channel block ...
    if (kw == KW) {
      kw = 0;
      ++kh;
      if (kh == KH) { kh = 0; c0 += BK; }   // ... then the next block, from the first tap
    }
    set_tap();
  }
  // straight into the LDS stage: element (k = wave + 4e, column lane + 64c)
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int ld, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int e = KR * PART / NPARTS; e < KR * (PART + 1) / NPARTS; ++e) {
      const uint32_t soff = (uint32_t)((c0 + wave + 4 * e) * IHW) * 4u;
#pragma unroll
      for (int c = 0; c < CC; ++c)
        buf_load_lds4(rs, lds + (wave + 4 * e) * ld + off + 64 * c, voff[c], soff);   // all 64 lanes (see run_tile)
    }
    if (PART == NPARTS - 1) advance();
    return (KR * (PART + 1) / NPARTS - KR * PART / NPARTS) * CC;
  }
};

// OBM: K order with the block of BK output channels as the outer loop and the class's taps as the inner one (the
// counterpart of the K order of ConvFwdBTap, for the same reason); otherwise tap-major.
template <int R, bool OBM>
struct ConvDgradBTap {
  static constexpr bool KC = false, DIRECT = true;
  static constexpr int CC = (R + 63) / 64;
  static constexpr int NLD = KR * CC;
  rsrc_t rs;
  ktab_t tab;           // one entry per tap of the pixel class: y, z (see ConvDgradB)
  int OH, OW, OHW, O, nt;
  int base[CC], a0[CC], b0[CC];
  uint32_t voff[CC];
  int o0, tap;          // K position of the next fetch
  int cy, cz, ny, nz;   // (y, z) of the current tap and of the one after it
  __device__ __forceinline__ void set_tap() {
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int oh = a0[c] - cy, ow = b0[c] - cz;
      const bool ok = (uint32_t)oh < (uint32_t)OH && (uint32_t)ow < (uint32_t)OW;
      voff[c] = ok ? (uint32_t)(base[c] + oh * OW + ow) * 4u : OOB;
    }
  }
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab_, int p0, int P, int kbeg, int nt_ = 0) {
    rs = r;
    tab = as_ktab(tab_);
    OH = g.OH; OW = g.OW; OHW = g.OHW; O = g.O; nt = nt_;
    if (OBM) {
      const int t0 = kbeg / BK, ob = nt > 0 ? t0 / nt : 0;
      tap = t0 - ob * nt;
      o0 = ob * BK;
      const int nx = tap + 1 == nt ? 0 : tap + 1;
      cy = (tab + tap)->y; cz = (tab + tap)->z;
      ny = (tab + nx)->y; nz = (tab + nx)->z;
    } else {
      tap = kbeg / g.O;
      o0 = kbeg - tap * g.O;
      cy = (tab + tap)->y; cz = (tab + tap)->z;
      ny = (tab + tap + 1)->y; nz = (tab + tap + 1)->z;
    }
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dIHW.div(pp), rem = pp - img * g.IHW;
      const uint32_t ih = g.dIW.div(rem), iw = rem - ih * g.IW;
      a0[c] = (int)ih;
      b0[c] = ok ? (int)iw : -BIG;
      base[c] = (int)img * g.O * g.OHW;
    }
    set_tap();
  }
  __device__ __forceinline__ void advance() {
    if (OBM) {
      if (++tap == nt) { tap = 0; o0 += BK; }
      cy = ny; cz = nz;
      set_tap();
      const int nx = tap + 1 == nt ? 0 : tap + 1;
      ny = (tab + nx)->y; nz = (tab + nx)->z;
    } else {
      o0 += BK;
      if (o0 >= O) {   // wave-uniform: next tap
        o0 = 0;
        ++tap;
        cy = ny; cz = nz;
        set_tap();
        ny = (tab + tap + 1)->y; nz = (tab + tap + 1)->z;
      }
    }
  }
  // straight into the LDS stage: element (k = wave + 4e, column lane + 64c)
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int ld, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int e = KR * PART / NPARTS; e < KR * (PART + 1) / NPARTS; ++e) {
      const uint32_t soff = (uint32_t)((o0 + wave + 4 * e) * OHW) * 4u;
#pragma unroll
      for (int c = 0; c < CC; ++c)
        buf_load_lds4(rs, lds + (wave + 4 * e) * ld + off + 64 * c, voff[c], soff);   // all 64 lanes (see run_tile)
    }
    if (PART == NPARTS - 1) advance();
    return (KR * (PART + 1) / NPARTS - KR * PART / NPARTS) * CC;
  }
};

// dgrad weight operand read from the weights in the layout the tap-major forward pass reads,
// Wp[o][tap][c] (tap = kh*KW + kw): element (row c, k = (tap, o)) sits at o*ld + tap*C + c with ld = KK*C, so for
// one tap the 32 output channels of a K step are 32 rows of C contiguous floats: a K-major stored matrix, moved
// with 128-bit transfers into the group's [BK][R] slab exactly as DirectMC moves one (C % 4 == 0, 16-byte
// aligned Wp).  The K advance (next 32 output channels, then the class's next tap, whose index the per-tap table
// carries in .w) rides in the scalar offset.  Forward and data gradient thus share one permuted copy of the
// weights, whatever the stride and the pixel class.
template <int R>
struct ConvDgradATapMC {
  static constexpr bool KC = false, DIRECT = true;
  static constexpr int LAYOUT = LAY_MC_SPLIT;
  static constexpr int NI = BK * R / 256, E = (NI + 3) / 4;
  static constexpr int NLD = NI % 4 == 0 ? E : -1;
  static_assert(R % 8 == 0, "whole 256-float transfers");
  rsrc_t rs;
  ktab_t tab;           // one entry per tap of the pixel class: .w = kh*KW + kw
  uint32_t voff[E];
  int ld, O, C, nt;
  int o0, tap, cw, nw;  // K position of the next transfer; tap index of the current tap and of the one after it
  // nt_: taps of the pixel class.  K order as in ConvDgradBTap<R, DIR, true>: output-channel block outer, taps inner.
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, const KEntry* tab_, int row0, int kbeg, int nt_) {
    rs = r;
    tab = as_ktab(tab_);
    ld = g.KK * g.C; O = g.O; C = g.C; nt = nt_;
    const int t0 = kbeg / BK, ob = nt > 0 ? t0 / nt : 0;
    tap = t0 - ob * nt;
    o0 = ob * BK;
    cw = (tab + tap)->w;
    nw = (tab + (tap + 1 == nt ? 0 : tap + 1))->w;
    const int wave = gwave(), lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int f = (wave + 4 * e) * 256 + lane * 4, k = f / R, n = f - k * R;
      voff[e] = (k < BK && row0 + n < g.C) ? (uint32_t)(k * ld + row0 + n) * 4u : OOB;
    }
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld_, int off) { return issue_part<0, 1>(k0, lds, ld_, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const uint32_t soff = (uint32_t)(o0 * ld + cw * C) * 4u;
    int n = 0;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e) {
      const int q = wave + 4 * e;
      if (NI % 4 == 0 || q < NI) { buf_load_lds16(rs, lds + off * BK + q * 256, voff[e], soff); ++n; }
    }
    if (PART == NPARTS - 1) {
      if (++tap == nt) { tap = 0; o0 += BK; }
      cw = nw;
      nw = (tab + (tap + 1 == nt ? 0 : tap + 1))->w;
    }
    return n;
  }
};

// dgrad gather of dY.  A strided convolution is handled as S*S independent
// stride-1 problems, one per class of input pixels with equal
// ((ih + PT) mod S, (iw + PL) mod S): inside a class only the taps with
// kh*D = (ih + PT) (mod S) contribute, and for those
//   oh = (ih + PT - kh*D) / S = ihc - y,   ih = h0 + S*ihc,  y = (kh*D - PT - h0) / S
// exactly (likewise ow = iwc - z).  The geometry handed to the loader is that
// of the class (IH, IW = class grid) and the table lists the class's taps:
// element (class pixel (n, ihc, iwc), k = (o, tap)) = dY[n, o, ihc - y, iwc - z]
// when in range, else 0.  Stride 1 is the single class h0 = w0 = 0.
template <int R>
struct ConvDgradB {
  static constexpr bool KC = false;
  static constexpr int CC = (R + 63) / 64;
  rsrc_t rs;
  ktab_t tab;
  int OH, OW;
  int base[CC], a0[CC], b0[CC];
  int tx[KR], ty[KR], tz[KR];
  float v[KR][CC];
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int e = 0; e < KR; ++e) {
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
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const int col = lane + 64 * c, p = p0 + col;
      const bool ok = col < R && p < P;
      const uint32_t pp = ok ? (uint32_t)p : 0u;
      const uint32_t img = g.dIHW.div(pp), rem = pp - img * g.IHW;
      const uint32_t ih = g.dIW.div(rem), iw = rem - ih * g.IW;
      a0[c] = (int)ih;
      b0[c] = ok ? (int)iw : -BIG;
      base[c] = (int)img * g.O * g.OHW;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int e = 0; e < KR; ++e) {
      const int t_x = tx[e];
#pragma unroll
      for (int c = 0; c < CC; ++c) {
        const int oh = a0[c] - ty[e], ow = b0[c] - tz[e];
        const bool ok = (uint32_t)oh < (uint32_t)OH && (uint32_t)ow < (uint32_t)OW;
        v[e][c] = buf_load(rs, ok ? (uint32_t)(base[c] + t_x + oh * OW + ow) * 4u : OOB);
      }
    }
    load_entries(k0 + BK);
  }
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
    const int wave = gwave(), lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < KR; ++e)
#pragma unroll
      for (int c = 0; c < CC; ++c)
        if (R % 64 == 0 || lane + 64 * c < R) lds[(wave + 4 * e) * ld + off + lane + 64 * c] = v[e][c];
  }
};

// dgrad weight gather: element (c, k = (o, kh, kw)) = W[o, c, kh, kw].
// Wavefront w fetches the k groups w, w+4, ... (four k each, wave-uniform table
// entries); lanes run over the channel rows.
template <int R>
struct ConvDgradA {
  static constexpr bool KC = true;
  static constexpr int E = (R + 63) / 64;
  static constexpr int NG = KG / 4;     // k groups per wavefront
  rsrc_t rs;
  ktab_t tab;
  uint32_t cb[E];
  uint32_t tw[NG][4];
  f32x4 v[E][NG];
  __device__ __forceinline__ void load_entries(int k0) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
#pragma unroll
    for (int q = 0; q < NG; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) tw[q][j] = (uint32_t)(tab + (k0 + 4 * (wave + 4 * q) + j))->w;
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
    for (int q = 0; q < NG; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t w = tw[q][j];
#pragma unroll
        for (int e = 0; e < E; ++e) {
          // either term alone is >= 2^29 elements (2 GiB) when invalid; clamp the sum
          const uint32_t idx = cb[e] + w;
          v[e][q][j] = buf_load(rs, idx >= 0x20000000u ? OOB : idx * 4u);
        }
      }
    load_entries(k0 + BK);
  }
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
    const int wave = gwave(), lane = threadIdx.x & 63;
#pragma unroll
    for (int e = 0; e < E; ++e)
#pragma unroll
      for (int q = 0; q < NG; ++q)
        if (R % 64 == 0 || lane + 64 * e < R)
          *reinterpret_cast<f32x4*>(&lds[(off + lane + 64 * e) * LDK + 4 * (wave + 4 * q)]) = v[e][q];
  }
};

// wgrad A side: dY viewed as [O][P], k = p = (n, oh, ow); element (o, p) at
// (n*O + o)*OHW + (p mod OHW).  VEC requires OHW % 4 == 0.
template <int R, bool VEC>
struct ConvWgradA {
  static constexpr bool KC = true;
  static constexpr int E = (R * KG + 255) / 256;
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
      const int s = gtid() + 256 * e, row = s / KG;
      rb[e] = (row < R && o0 + row < g.O) ? (uint32_t)((o0 + row) * g.OHW) : 0x20000000u;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    const int kg = gtid() % KG;
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
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, row = s / KG, kg = s % KG;
      if (R * KG % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[(off + row) * LDK + 4 * kg]) = v[e];
    }
  }
};

// wgrad B side: im2row gather with k = p; element (q = (c, kh, kw), p) =
// X[n, c, oh*S-PT+kh*D, ow*S-PL+kw*D].
template <int R>
struct ConvWgradB {
  static constexpr bool KC = true;
  static constexpr int E = (R * KG + 255) / 256;
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
      const int s = gtid() + 256 * e, row = s / KG;
      const bool ok = row < R && q0 + row < Q;
      const KEntry t = tab[ok ? q0 + row : 0];
      xo[e] = t.x;
      dh[e] = ok ? t.y : BIG;
      dw[e] = t.z;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
    const int kg = gtid() % KG;
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
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int s = gtid() + 256 * e, row = s / KG, kg = s % KG;
      if (R * KG % 256 == 0 || row < R) *reinterpret_cast<f32x4*>(&lds[(off + row) * LDK + 4 * kg]) = v[e];
    }
  }
};

// Pixel-major wgrad loaders for channel counts that fill whole units: K = the
// output pixel p, and the GEMM columns are ordered tap-major (column = tap*C + c)
// so that all columns of a group belong to one tap.  Lane (tid % 32) owns one
// pixel of the K step, tid / 32 selects a row subgroup; the rows of a thread
// are sub + 8*e and differ only by a wave-uniform multiple of the plane size,
// which rides in the scalar offset.  Per K step a thread decomposes its pixel
// once (shared by both loaders), tests the padding once, and issues its loads.
template <int R>
struct ConvWgradTapA {
  static constexpr bool KC = true;
  static constexpr int E = R / 8;       // rows per thread (R is a multiple of 8)
  rsrc_t rs;
  int OHW, OOHW, kend;
  FastDiv dOHW;
  uint32_t rowoff;          // (first row of this thread) * OHW
  uint32_t img, rem;        // decomposition of this thread's pixel in the last fetch
  bool pok;
  float v[E];
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int o0, int kend_) {
    rs = r;
    OHW = g.OHW;
    OOHW = g.O * g.OHW;
    dOHW = g.dOHW;
    kend = kend_;
    rowoff = (uint32_t)((o0 + (gtid() >> 5)) * g.OHW);
  }
  __device__ __forceinline__ void fetch(int k0) {
    const uint32_t p = (uint32_t)(k0 + (gtid() & 31));
    pok = p < (uint32_t)kend;
    img = dOHW.div(p);
    rem = p - img * OHW;
    // rows past the last output channel are never stored, so they need no mask
    const uint32_t voff = pok ? (img * (uint32_t)OOHW + rem + rowoff) * 4u : OOB;
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = buf_load_s(rs, voff, (uint32_t)(8 * e * OHW) * 4u);
  }
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
    const int l = gtid() & 31, sub = gtid() >> 5;
#pragma unroll
    for (int e = 0; e < E; ++e) lds[(off + sub + 8 * e) * LDK + l] = v[e];
  }
};

template <int R>
struct ConvWgradTapB {
  static constexpr bool KC = true;
  static constexpr bool NEEDS_A = true;
  static constexpr int E = R / 8;
  rsrc_t rs;
  int C, IH, IW, IHW, OW, S;
  FastDiv dOW;
  int dh, dw;               // kh*D - PADT, kw*D - PADL of this group's tap
  uint32_t chanoff;         // (first channel of this thread) * IHW
  float v[E];
  template <class LA>
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int col0, const LA&) {
    rs = r;
    C = g.C; IH = g.IH; IW = g.IW; IHW = g.IHW; OW = g.OW; S = g.S;
    dOW = g.dOW;
    const int tap = col0 / g.C, c0 = col0 - tap * g.C;
    const int kh = tap / g.KW, kw = tap - kh * g.KW;
    dh = kh * g.D - g.PADT;
    dw = kw * g.D - g.PADL;
    chanoff = (uint32_t)((c0 + (gtid() >> 5)) * g.IHW);
  }
  template <class LA>
  __device__ __forceinline__ void fetch(int, const LA& la) {
    const uint32_t oh = dOW.div(la.rem), ow = la.rem - oh * OW;
    const int ih = (int)oh * S + dh, iw = (int)ow * S + dw;
    const bool ok = la.pok && (uint32_t)ih < (uint32_t)IH && (uint32_t)iw < (uint32_t)IW;
    const uint32_t voff = ok ? (la.img * (uint32_t)(C * IHW) + (uint32_t)(ih * IW + iw) + chanoff) * 4u : OOB;
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = buf_load_s(rs, voff, (uint32_t)(8 * e * IHW) * 4u);
  }
  __device__ __forceinline__ void commit(float* lds, int ld, int off) const {
    const int l = gtid() & 31, sub = gtid() >> 5;
#pragma unroll
    for (int e = 0; e < E; ++e) lds[(off + sub + 8 * e) * LDK + l] = v[e];
  }
};

// The same two operands sent straight into swizzled K-contiguous LDS tiles
// (LAY_KC_SWZ).  One transfer fills two adjacent tile rows: lanes 0..31 the
// even one, lanes 32..63 the odd one.  Wavefront w owns the row pairs
// w, w+4, w+8, ..., so every row a lane ever fills has the same r % 8 = 2w +
// lane/32: the lane's swizzled position corresponds to one fixed k of the K
// step, i.e. one pixel to decompose per step, and its rows differ by
// wave-uniform multiples of 8 planes which ride in the scalar offset.
__device__ __forceinline__ int wgrad_direct_k() {   // k (0..BK-1) whose swizzled position this lane fills
  const int lane = threadIdx.x & 63, pos = lane & 31, key = 2 * gwave() + (lane >> 5);
  return (((pos >> 2) ^ key) << 2) | (pos & 3);
}
//
// The lane's pixel advances by BK per K step.  Its coordinates and the
// element offsets derived from them are carried along with additions and
// single wrap tests (which is why these loaders need BK/OW + 1 <= OH): no
// division or multiplication in the K loop.
template <int R>
struct ConvWgradTapADirect {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZ;
  static constexpr int E = R / 8, NLD = E;
  static_assert(R % 8 == 0, "whole row pairs for all four wavefronts");
  rsrc_t rs;
  int OHW, kend, p, rem, aoff, awrap;   // aoff = img*O*OHW + rem + (row of this lane)*OHW
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int o0, int kend_, int k0) {
    rs = r;
    OHW = g.OHW;
    kend = kend_;
    awrap = g.O * g.OHW - g.OHW;   // to the same pixel offset in the next image
    p = k0 + wgrad_direct_k();
    const uint32_t img = g.dOHW.div((uint32_t)p);
    rem = p - (int)img * g.OHW;
    aoff = (int)img * g.O * g.OHW + rem + (o0 + 2 * gwave() + (int)((threadIdx.x & 63) >> 5)) * g.OHW;
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    // rows past the last output channel are never stored, so they need no mask
    const uint32_t voff = p < kend ? (uint32_t)aoff * 4u : OOB;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e)
      buf_load_lds4(rs, lds + (off + 8 * e + 2 * wave) * BK, voff, (uint32_t)(8 * e * OHW) * 4u);
    if (PART == NPARTS - 1) {
      p += BK; rem += BK; aoff += BK;
      if (rem >= OHW) { rem -= OHW; aoff += awrap; }
    }
    return E * (PART + 1) / NPARTS - E * PART / NPARTS;
  }
};

// The same with 128-bit transfers, for OH*OW % 4 == 0 and a 16-byte aligned dY:
// lane l carries 4-pixel group (l % 8) ^ (l / 8) of row l / 8 of an 8-row block
// (the layout of DirectKC), wavefront w the blocks w, w+4, ...
template <int R>
struct ConvWgradTapA4Direct {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZP;
  static constexpr int NB = R / 8, E = (NB + 3) / 4;
  static constexpr int NLD = NB % 4 == 0 ? E : -1;
  static_assert(R % 8 == 0, "whole 8-row blocks");
  rsrc_t rs;
  int OHW, kend, p, rem, aoff, awrap;
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int o0, int kend_, int k0) {
    rs = r;
    OHW = g.OHW;
    kend = kend_;
    awrap = g.O * g.OHW - g.OHW;
    const int lane = threadIdx.x & 63, rb = lane >> 3;
    p = k0 + 4 * ((lane & 7) ^ ((((int)gwave() & 1) << 2) | (rb >> 1)));   // LAY_KC_SWZP: key (row / 2) % 8
    const uint32_t img = g.dOHW.div((uint32_t)p);
    rem = p - (int)img * g.OHW;
    aoff = (int)img * g.O * g.OHW + rem + (o0 + 8 * gwave() + rb) * g.OHW;
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const uint32_t voff = p < kend ? (uint32_t)aoff * 4u : OOB;   // kend is a multiple of 4 here: whole groups
    int n = 0;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e)
      if (NB % 4 == 0 || wave + 4 * e < NB) {
        buf_load_lds16(rs, lds + (off + (wave + 4 * e) * 8) * BK, voff, (uint32_t)(32 * e * OHW) * 4u);
        ++n;
      }
    if (PART == NPARTS - 1) {
      p += BK; rem += BK; aoff += BK;
      if (rem >= OHW) { rem -= OHW; aoff += awrap; }
    }
    return n;
  }
};

template <int R>
struct ConvWgradTapBDirect {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZ;
  static constexpr int E = R / 8, NLD = E;
  static_assert(R % 8 == 0, "whole row pairs for all four wavefronts");
  rsrc_t rs;
  int IH, IW, IHW, OH, OW, kend;
  int p, oh, ow;            // this lane's output pixel, its row and column inside the image
  int ih, iw;               // oh*S + kh*D - PADT, ow*S + kw*D - PADL: the input pixel under this group's tap
  int xoff;                 // its element offset (for the channel of this lane)
  int qh, rw;               // a K step moves the pixel qh rows and rw columns ahead ...
  int s_q, s_r, x_step;     // ... i.e. ih by S*qh, iw by S*rw, xoff by S*qh*IW + S*rw
  int s_OW, s_OH, S, xwrap_w, xwrap_h;   // corrections when the column / the row wraps
  template <class LA>
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int col0, const LA&, int kend_, int k0) {
    rs = r;
    IH = g.IH; IW = g.IW; IHW = g.IHW; OH = g.OH; OW = g.OW; S = g.S;
    kend = kend_;
    const int tap = col0 / g.C, c0 = col0 - tap * g.C;
    const int kh = tap / g.KW, kw = tap - kh * g.KW;
    qh = BK / g.OW; rw = BK - qh * g.OW;
    s_q = g.S * qh; s_r = g.S * rw; s_OW = g.S * g.OW; s_OH = g.S * g.OH;
    x_step = s_q * g.IW + s_r;
    xwrap_w = g.S * g.IW - s_OW;              // column wrap: one row down, OW columns back
    xwrap_h = g.C * g.IHW - s_OH * g.IW;      // row wrap: next image, OH rows back
    p = k0 + wgrad_direct_k();
    const uint32_t img = g.dOHW.div((uint32_t)p), rem = (uint32_t)p - img * g.OHW;
    oh = (int)g.dOW.div(rem);
    ow = (int)rem - oh * g.OW;
    ih = oh * g.S + kh * g.D - g.PADT;
    iw = ow * g.S + kw * g.D - g.PADL;
    xoff = ((int)img * g.C + c0 + 2 * gwave() + (int)((threadIdx.x & 63) >> 5)) * g.IHW + ih * g.IW + iw;
  }
  __device__ __forceinline__ int issue(int, float* lds, int, int off) { go<0, 1>(lds, off); return E; }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    go<PART, NPARTS>(lds, off);
    return E * (PART + 1) / NPARTS - E * PART / NPARTS;
  }
  template <int PART, int NPARTS>
  __device__ __forceinline__ void go(float* lds, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const bool ok = p < kend && (uint32_t)ih < (uint32_t)IH && (uint32_t)iw < (uint32_t)IW;
    const uint32_t voff = ok ? (uint32_t)xoff * 4u : OOB;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e) {
      buf_load_lds4(rs, lds + (off + 8 * e + 2 * wave) * BK, voff, (uint32_t)(8 * e * IHW) * 4u);
    }
    if (PART == NPARTS - 1) {
      p += BK; oh += qh; ow += rw; ih += s_q; iw += s_r; xoff += x_step;
      if (ow >= OW) { ow -= OW; ++oh; iw -= s_OW; ih += S; xoff += xwrap_w; }
      if (oh >= OH) { oh -= OH; ih -= s_OH; xoff += xwrap_h; }
    }
  }
};

// The pixel gather with 128-bit transfers, for stride 1, OW % 4 == 0 and no padding at the left or right edge
// (1x1 kernels, 'valid' convolutions): the four pixels p..p+3 (p % 4 == 0) of a lane sit in one output row, so the
// input pixels under a tap are four consecutive floats of one input row (at any 4-byte alignment), all inside the
// image or - above / below it - all outside.  Same block / lane layout as ConvWgradTapA4Direct: lane l carries
// 4-pixel group (l % 8) ^ (l / 8) for channel l / 8 of an 8-channel block, wavefront w the blocks w, w+4, ...
// With padded columns one group per image row and off-centre tap hangs over the edge; repairing it after the
// transfer (zeros over the outside elements) was measured and cost more than the wider transfers gain.
template <int R>
struct ConvWgradTapB4Direct {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZP;
  static constexpr int NB = R / 8, E = (NB + 3) / 4;
  static constexpr int NLD = NB % 4 == 0 ? E : -1;
  static_assert(R % 8 == 0, "whole 8-row blocks");
  rsrc_t rs;
  int IH, IHW, OH, OW, kend;
  int p, oh, ow, ih, xoff;
  int qh, rw, x_step, xwrap_w, xwrap_h;
  template <class LA>
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int col0, const LA&, int kend_, int k0) {
    rs = r;
    IH = g.IH; IHW = g.IHW; OH = g.OH; OW = g.OW;
    kend = kend_;
    const int tap = col0 / g.C, c0 = col0 - tap * g.C;
    const int kh = tap / g.KW, kw = tap - kh * g.KW;
    qh = BK / g.OW; rw = BK - qh * g.OW;
    x_step = qh * g.IW + rw;
    xwrap_w = g.IW - g.OW;
    xwrap_h = g.C * g.IHW - g.OH * g.IW;
    const int lane = threadIdx.x & 63, rb = lane >> 3;
    p = k0 + 4 * ((lane & 7) ^ ((((int)gwave() & 1) << 2) | (rb >> 1)));   // LAY_KC_SWZP: key (row / 2) % 8
    const uint32_t img = g.dOHW.div((uint32_t)p), rem = (uint32_t)p - img * g.OHW;
    oh = (int)g.dOW.div(rem);
    ow = (int)rem - oh * g.OW;
    ih = oh + kh * g.D - g.PADT;
    xoff = ((int)img * g.C + c0 + 8 * gwave() + rb) * g.IHW + ih * g.IW + ow + kw * g.D;
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const uint32_t voff = p < kend && (uint32_t)ih < (uint32_t)IH ? (uint32_t)xoff * 4u : OOB;
    int n = 0;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e)
      if (NB % 4 == 0 || wave + 4 * e < NB) {
        buf_load_lds16(rs, lds + (off + (wave + 4 * e) * 8) * BK, voff, (uint32_t)(32 * e * IHW) * 4u);
        ++n;
      }
    if (PART == NPARTS - 1) {
      p += BK; oh += qh; ow += rw; ih += qh; xoff += x_step;
      if (ow >= OW) { ow -= OW; ++oh; ++ih; xoff += xwrap_w; }
      if (oh >= OH) { oh -= OH; ih -= OH; xoff += xwrap_h; }
    }
    return n;
  }
};

// wgrad pixel gather for any channel count, GEMM columns tap-major (q = tap*C + c) like the other pixel-major
// loaders but free to span taps inside a group, sent straight
// into a swizzled K-contiguous LDS tile like ConvWgradTapBDirect: a lane owns one fixed pixel position of the K
// step (carried forward by additions and single wrap tests) and, per transfer, one column - lanes 0..31 the even
// row of the pair, lanes 32..63 the odd one - whose three constants (element offset from the window's origin, row
// and column displacement of its tap for the padding test) it keeps in registers for the whole kernel.  Lanes run
// over consecutive output pixels, so a transfer reads a run of image-row floats S apart: a handful of cache lines,
// where lanes over the columns of one pixel touch some thirty.  Columns past C*KH*KW arrive as zeros.
template <int R>
struct ConvWgradBAnyC {
  static constexpr bool KC = true, DIRECT = true;
  static constexpr int LAYOUT = LAY_KC_SWZ;
  static constexpr int E = R / 8, NLD = E;
  static_assert(R % 8 == 0, "whole row pairs for all four wavefronts");
  rsrc_t rs;
  int IH, IW, OH, OW, kend;
  int coff[E], yy[E], zz[E];   // this lane's column of transfer e
  int p, oh, ow;               // this lane's output pixel, its row and column inside the image
  int ih, iw;                  // oh*S - PADT, ow*S - PADL: origin of the pixel's window
  int xoff;                    // its element offset (channel 0)
  int qh, rw, s_q, s_r, x_step, s_OW, s_OH, S, xwrap_w, xwrap_h;   // see ConvWgradTapBDirect
  template <class LA>
  __device__ __forceinline__ void init(rsrc_t r, const ConvGeom& g, int col0, int Q, const LA&, int kend_, int k0) {
    rs = r;
    IH = g.IH; IW = g.IW; OH = g.OH; OW = g.OW; S = g.S;
    kend = kend_;
    const int half = (int)((threadIdx.x & 63) >> 5);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int q = col0 + 8 * e + 2 * gwave() + half;
      const bool ok = q < Q;
      const int qq = ok ? q : 0;
      const int tap = qq / g.C, ch = qq - tap * g.C, kh = tap / g.KW, kw = tap - kh * g.KW;
      yy[e] = ok ? kh * g.D : BIG;
      zz[e] = kw * g.D;
      coff[e] = ch * g.IHW + kh * g.D * g.IW + kw * g.D;
    }
    qh = BK / g.OW; rw = BK - qh * g.OW;
    s_q = g.S * qh; s_r = g.S * rw; s_OW = g.S * g.OW; s_OH = g.S * g.OH;
    x_step = s_q * g.IW + s_r;
    xwrap_w = g.S * g.IW - s_OW;              // column wrap: one row down, OW columns back
    xwrap_h = g.C * g.IHW - s_OH * g.IW;      // row wrap: next image, OH rows back
    p = k0 + wgrad_direct_k();
    const uint32_t img = g.dOHW.div((uint32_t)p), rem = (uint32_t)p - img * g.OHW;
    oh = (int)g.dOW.div(rem);
    ow = (int)rem - oh * g.OW;
    ih = oh * g.S - g.PADT;
    iw = ow * g.S - g.PADL;
    xoff = (int)img * g.C * g.IHW + ih * g.IW + iw;
  }
  __device__ __forceinline__ int issue(int k0, float* lds, int ld, int off) { return issue_part<0, 1>(k0, lds, ld, off); }
  template <int PART, int NPARTS>
  __device__ __forceinline__ int issue_part(int, float* lds, int, int off) {
    const int wave = __builtin_amdgcn_readfirstlane(gwave());
    const int ihm = p < kend ? ih : BIG;
#pragma unroll
    for (int e = E * PART / NPARTS; e < E * (PART + 1) / NPARTS; ++e) {
      const bool ok = (uint32_t)(ihm + yy[e]) < (uint32_t)IH && (uint32_t)(iw + zz[e]) < (uint32_t)IW;
      buf_load_lds4(rs, lds + (off + 8 * e + 2 * wave) * BK, ok ? (uint32_t)(xoff + coff[e]) * 4u : OOB, 0);
    }
    if (PART == NPARTS - 1) {
      p += BK; oh += qh; ow += rw; ih += s_q; iw += s_r; xoff += x_step;
      if (ow >= OW) { ow -= OW; ++oh; iw -= s_OW; ih += S; xoff += xwrap_w; }
      if (oh >= OH) { oh -= OH; ih -= s_OH; xoff += xwrap_h; }
    }
    return E * (PART + 1) / NPARTS - E * PART / NPARTS;
  }
};

// Optional per-row bias and activation applied to a finished element before
// it is stored ('=' only): y = f(acc + bias[m]), f = identity or leaky ReLU
// (x >= 0 ? x : slope * x, the same selection the pointwise kernel makes).
struct PostOp {
  const float* bias;   // one value per output row m (per column n with bias_col), or null
  int act;             // 0 none, 1 leaky ReLU
  float slope;
  int bias_col;        // 0: bias[m] (a convolution's output channel), 1: bias[n] (a dense layer's output feature)
  __host__ __device__ bool any() const { return bias != nullptr || act != 0; }
  __device__ __forceinline__ float apply(float v, float b) const {
    v += b;
    return (act == 0 || v >= 0.0f) ? v : slope * v;
  }
};

// ---------------------------------------------------------------------------
// Output mapping.  plain: off = m*ld + n.  NCHW image tensor with the GEMM
// column n = (img, pixel): off = (img*Mtot + m)*HW + pixel.
// ---------------------------------------------------------------------------
struct OutMap {
  int nchw;    // 0 plain, 1 image layout, 2 tap-major weight columns, 3 strided pixel class of an image layout
  int ld;      // plain / tap-major: leading dimension; nchw: HW
  int mtot;    // nchw: channel count; tap-major: KK
  FastDiv dHW; // nchw: divide by HW (class: by the class plane); tap-major: divide by the channel count C
  // class: column (img, ihc, iwc) is pixel (h0 + s*ihc, w0 + s*iwc) of a plane of width iw; org = h0*iw + w0
  FastDiv dCW;
  int s, iw, org;
  __device__ __forceinline__ uint32_t col(uint32_t n) const {
    if (nchw == 0) return n;
    const uint32_t q = dHW.div(n);
    if (nchw == 1) return q * (uint32_t)(mtot * ld) + (n - q * ld);   // q = image
    if (nchw == 2) return (n - q * dHW.d) * (uint32_t)mtot + q;       // q = tap: column tap*C + c -> c*KK + tap
    const uint32_t rem = n - q * dHW.d, r = dCW.div(rem), c = rem - r * dCW.d;
    return q * (uint32_t)(mtot * ld) + (uint32_t)org + (r * (uint32_t)iw + c) * (uint32_t)s;
  }
};

// ---------------------------------------------------------------------------
// The MFMA step: both operands come from LDS in one of two layouts.
// Lane (i = lane % 32, h = lane / 32) feeds row i of the 32-row fragment; in
// each group of 8 k values lane half h supplies k = 8*kk + 4*h + t to the
// t-th MFMA.  A and B use the same k assignment, so any k permutation cancels.
// ---------------------------------------------------------------------------
template <int NT, int LAY_A, int LAY_B, int RA, int RB>
__device__ __forceinline__ void load_frags(const float* __restrict__ As, const float* __restrict__ Bs, int arow,
                                           int brow, int kk, float (&a)[4], float (&b)[NT][4]) {
  const int lane = threadIdx.x & 63, i = lane & 31, h = lane >> 5;
  const int kb = kk * 8 + h * 4;
  // swizzled position of k group 2*kk + h; row offsets are multiples of 32
  const int sw = ((2 * kk + h) ^ (i & 7)) << 2, swp = ((2 * kk + h) ^ ((i >> 1) & 7)) << 2;
  if (lay_kc(LAY_A)) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(LAY_A == LAY_KC ? &As[(arow + i) * LDK + kb] : &As[(arow + i) * BK + (LAY_A == LAY_KC_SWZP ? swp : sw)]);
    a[0] = t[0]; a[1] = t[1]; a[2] = t[2]; a[3] = t[3];
  } else if (LAY_A == LAY_MC) {
    const float* ap = As + (arow + i + h * (4 * RA));   // one address per lane, k as immediate offsets
#pragma unroll
    for (int t = 0; t < 4; ++t) a[t] = ap[(kk * 8 + t) * RA];
  } else {   // two [BK][RA/2] slabs
    constexpr int H = RA / 2;
    const int r = arow + i;
    // one address per lane, the four k as immediate offsets (they pair into two-dword reads)
    const float* ap = As + ((r / H) * (BK * H) + r % H + h * (4 * H)) + kk * (8 * H);
#pragma unroll
    for (int t = 0; t < 4; ++t) a[t] = ap[t * H];
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    if (lay_kc(LAY_B)) {
      const int r = brow + 32 * j + i;
      const f32x4 t = *reinterpret_cast<const f32x4*>(LAY_B == LAY_KC ? &Bs[r * LDK + kb] : &Bs[r * BK + (LAY_B == LAY_KC_SWZP ? swp : sw)]);
      b[j][0] = t[0]; b[j][1] = t[1]; b[j][2] = t[2]; b[j][3] = t[3];
    } else {   // shared tile or the group's own slab: the caller passes the matching base, pitch and brow
      // one address per lane and accumulator tile; kk and t are immediate offsets, so with RB a multiple
      // of 64 the four reads pair into two-dword reads without any address arithmetic in the K loop
      const float* bp = Bs + (brow + 32 * j + i + h * (4 * RB));
#pragma unroll
      for (int t = 0; t < 4; ++t) b[j][t] = bp[(kk * 8 + t) * RB];
    }
  }
}

// One LDS stage = BK/8 groups of 4*NT MFMAs.  The fragments of the first
// group are read up front; the reads of each following group are slotted one
// by one between the MFMAs of the group before it, so the matrix pipe does
// not wait for LDS within the stage.
template <int NT, int LAY_A, int LAY_B, int RA, int RB>
__device__ __forceinline__ void mma_stage(const float* __restrict__ As, const float* __restrict__ Bs,
                                          f32x16 (&acc)[NT], int arow, int brow) {
  constexpr int NG = BK / 8;
  float fa[2][4], fb[2][NT][4];
  // LDS read instructions per group: A is one b128 or four b32; B is NT b128 or 4*NT b32 (paired into read2)
  constexpr int RD = (lay_kc(LAY_A) ? 1 : 2) + (lay_kc(LAY_B) ? NT : 2 * NT);
  load_frags<NT, LAY_A, LAY_B, RA, RB>(As, Bs, arow, brow, 0, fa[0], fb[0]);
  __builtin_amdgcn_sched_group_barrier(0x100, RD, 0);              // DS reads of group 0
#pragma unroll
  for (int kk = 0; kk < NG; ++kk) {
    const int cur = kk & 1;
    if (kk + 1 < NG) load_frags<NT, LAY_A, LAY_B, RA, RB>(As, Bs, arow, brow, kk + 1, fa[cur ^ 1], fb[cur ^ 1]);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][t], fb[cur][j][t], acc[j], 0, 0, 0);
    if (kk + 1 < NG) {
#pragma unroll
      for (int i = 0; i < RD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);         // one MFMA of group kk
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);         // one DS read of group kk+1
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * NT - RD, 0);  // the remaining MFMAs of group kk
    } else {
      __builtin_amdgcn_sched_group_barrier(0x008, 4 * NT, 0);       // last group
    }
  }
}

// One LDS stage of a pipeline that never leaves the MFMA stream (BK / 8 = 4 groups of 4*NT MFMAs).  On entry
// fa[0] / fb[0] hold the fragments of the stage's first group, read by the previous stage (or by the prologue).
// The global -> LDS transfers that refill the stage read one K step ago go out in four shares, send(share), one per
// group, slotted between the MFMAs that carry no fragment read.  Late in the last group comes the K step's only
// barrier, mid(): behind it the next stage is complete in LDS and this one is no longer read by anybody, so the
// step's last MFMAs carry the reads of the next stage's first group (NEXT) and the next step may refill this stage.
// Vector-memory and LDS instructions cost the matrix pipe nothing while they sit between the MFMAs of the same
// wavefront; vector-ALU instructions stop it, and so does anything the other wavefront of the SIMD wants to issue.
// NV: transfers per wavefront and K step if known (0: unknown or none).
template <int N> using ic = std::integral_constant<int, N>;
template <int NT, int LAY_A, int LAY_B, int RA, int RB, int NV, bool NEXT, bool REGIONS, class MID, class SEND>
__device__ __forceinline__ void mma_stage_stream(const float* __restrict__ As, const float* __restrict__ Bs,
                                                 const float* __restrict__ Asn, const float* __restrict__ Bsn,
                                                 f32x16 (&acc)[NT], float (&fa)[2][4], float (&fb)[2][NT][4], int arow,
                                                 int brow, MID mid, SEND send) {
  constexpr int NG = BK / 8;
  static_assert(NG == 4, "four groups, four shares of transfers; the next stage's first group lands in buffer 0");
  constexpr int RD = (lay_kc(LAY_A) ? 1 : 2) + (lay_kc(LAY_B) ? NT : 2 * NT);
  constexpr int G = 4 * NT;                       // MFMAs per group
  constexpr int PAIRS = RD < G ? RD : G;          // MFMAs of a group that carry a fragment read
  constexpr int FREE = G - PAIRS;                 // ... and those that do not
  // transfers slotted into one group (the scheduler takes them in program order, whichever share they belong to)
  constexpr int SHARE = (NV + NG - 1) / NG;
  constexpr int PER = FREE > 0 ? (SHARE + FREE - 1) / FREE : SHARE;
  auto mfmas = [&](auto curc, auto loc, auto hic) {
    constexpr int cur = decltype(curc)::value, lo = decltype(loc)::value, hi = decltype(hic)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        if (t * NT + j >= lo && t * NT + j < hi)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][t], fb[cur][j][t], acc[j], 0, 0, 0);
  };
  auto read_slots = [&] {
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if (RD > G) __builtin_amdgcn_sched_group_barrier(0x100, RD - G, 0);
  };
  auto transfer_slots = [&] {
    if (NV > 0) {
#pragma unroll
      for (int i = 0; i < FREE; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (i * PER < SHARE) __builtin_amdgcn_sched_group_barrier(0x020, PER, 0);   // the last one may stay short
      }
      if (FREE == 0) __builtin_amdgcn_sched_group_barrier(0x020, SHARE, 0);
    } else if (FREE > 0) {
      __builtin_amdgcn_sched_group_barrier(0x008, FREE, 0);
    }
  };
  auto group = [&](auto kkc) {
    constexpr int kk = decltype(kkc)::value, cur = kk & 1;
    if constexpr (kk + 1 < NG) {
      load_frags<NT, LAY_A, LAY_B, RA, RB>(As, Bs, arow, brow, kk + 1, fa[cur ^ 1], fb[cur ^ 1]);
      mfmas(ic<cur>(), ic<0>(), ic<G>());
      send(kkc);
      read_slots();
      transfer_slots();
      // REGIONS (the loops that keep a running stage index): each group is a scheduling region of its own.  With
      // the whole stage in one region their slots were honoured for the first share only and the other transfers
      // went out in one burst (config 3 wgrad 0.242 -> 0.235 ms); the unrolled loops schedule well as one region
      if (REGIONS) __builtin_amdgcn_sched_barrier(0);
    } else {
      mfmas(ic<cur>(), ic<0>(), ic<FREE>());
      send(kkc);
      transfer_slots();
      __builtin_amdgcn_sched_barrier(0);
      mid();
      __builtin_amdgcn_sched_barrier(0);
      if (NEXT) load_frags<NT, LAY_A, LAY_B, RA, RB>(Asn, Bsn, arow, brow, 0, fa[cur ^ 1], fb[cur ^ 1]);
      mfmas(ic<cur>(), ic<FREE>(), ic<G>());
      if (NEXT) read_slots(); else __builtin_amdgcn_sched_group_barrier(0x008, PAIRS, 0);
    }
  };
  if (REGIONS)
  // vector-ALU instructions of the step (fragment addresses, the loaders' address walks) in one batch at the start:
  // one alone between two MFMAs costs the matrix pipe 13-18 cycles, in a batch 5-9 each
    __builtin_amdgcn_sched_group_barrier(0x002, 64, 0);
  group(ic<0>());
  group(ic<1>());
  group(ic<2>());
  group(ic<3>());
}

template <bool KC, int R>
struct LdsSize { static constexpr int value = KC ? R * LDK : BK * R; };

// What a kernel hands to the engine: loader types (templates over the row
// count) and how to initialise them for one sub-tile.
//
//   struct Problem {
//     template <int R> using LA = ...;   template <int R> using LB = ...;
//     template <int R> void init_a(LA<R>&, int row0) const;
//     template <int R, class A> void init_b(LB<R>&, int col0, A& la) const;   (la: this group's A loader)
//     int kbeg, kend, M, Ncols, beta;  rsrc_t rc;  OutMap om;  PostOp post;
//   };

// A B-side loader that shares per-step state with its group's A loader
// declares `static constexpr bool NEEDS_A = true` and takes the A loader in fetch().
template <class T, class = void>
struct needs_a : std::false_type {};
template <class T>
struct needs_a<T, std::void_t<decltype(T::NEEDS_A)>> : std::true_type {};
template <class LB, class LA>
__device__ __forceinline__ void fetch_b(LB& lb, int k0, const LA& la) {
  if constexpr (needs_a<LB>::value)
    lb.fetch(k0, la);
  else
    lb.fetch(k0);
}

// A loader that moves global memory straight into LDS declares
// `static constexpr bool DIRECT = true` and provides issue(k0, lds, ld, off)
// instead of fetch() / commit().
template <class T, class = void>
struct is_direct : std::false_type {};
template <class T>
struct is_direct<T, std::void_t<decltype(T::DIRECT)>> : std::integral_constant<bool, T::DIRECT> {};
// LDS layout a loader fills: T::LAYOUT if declared, else padded K-contiguous or shared row-contiguous by T::KC
template <class T, class = void>
struct layout_of : std::integral_constant<int, T::KC ? LAY_KC : LAY_MC> {};
template <class T>
struct layout_of<T, std::void_t<decltype(T::LAYOUT)>> : std::integral_constant<int, T::LAYOUT> {};

// End of a phase.  The barrier is issued by hand so that it waits for exactly
// what the schedule needs: LDS operations of this wavefront (fragment reads,
// parked operands) always; its global -> LDS transfers only where stated.
// Nothing may be scheduled across it: the MFMAs of a phase must not sink into
// the other group's phase.
__device__ __forceinline__ void barrier_after_compute() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ void barrier_after_issue() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
// All global -> LDS transfers of this wavefront have landed (the compiler
// tracks register loads by itself, not these).
template <bool ANY_DIRECT>
__device__ __forceinline__ void wait_transfers() {
  if (ANY_DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// All global -> LDS transfers of this wavefront have landed except the n it issued last (they complete in order).
// n is wave-uniform and, after inlining, a constant in nearly every instantiation.
__device__ __forceinline__ void wait_transfers_but(int n) {
#define LNN_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
  switch (n) {
    LNN_W(1) LNN_W(2) LNN_W(3) LNN_W(4) LNN_W(5) LNN_W(6) LNN_W(7) LNN_W(8) LNN_W(9) LNN_W(10) LNN_W(11) LNN_W(12)
    LNN_W(13) LNN_W(14) LNN_W(15) LNN_W(16) LNN_W(17) LNN_W(18) LNN_W(19) LNN_W(20) LNN_W(21) LNN_W(22) LNN_W(23) LNN_W(24)
    LNN_W(25) LNN_W(26) LNN_W(27) LNN_W(28) LNN_W(29) LNN_W(30) LNN_W(31) LNN_W(32)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;   // none issued, or more than the counter is trusted for
  }
#undef LNN_W
}

// A problem whose transfers come a long way relative to its K steps (short steps, operands not resident in L2)
// declares `static constexpr bool REQUEST_FIRST = true`: its three-stage pipeline then sends K step t+2 off before it
// waits for step t+1.
template <class T, class = void>
struct request_first : std::false_type {};
template <class T>
struct request_first<T, std::void_t<decltype(T::REQUEST_FIRST)>> : std::integral_constant<bool, T::REQUEST_FIRST> {};

// A problem whose streaming loop should keep a running stage index (no threefold unrolling: register pressure or code
// size cost it more than the address arithmetic) declares `static constexpr bool STREAM_UNROLL = false`.
template <class T, class = void>
struct stream_unroll : std::true_type {};
template <class T>
struct stream_unroll<T, std::void_t<decltype(T::STREAM_UNROLL)>> : std::integral_constant<bool, T::STREAM_UNROLL> {};

// Whether the streaming stage makes each MFMA group a scheduling region of its own (see mma_stage_stream): by default
// the loops that are not unrolled; a problem overrides it with `static constexpr bool STREAM_REGIONS`.
template <class T, class = void>
struct stream_regions : std::integral_constant<bool, !stream_unroll<T>::value> {};
template <class T>
struct stream_regions<T, std::void_t<decltype(T::STREAM_REGIONS)>> : std::integral_constant<bool, T::STREAM_REGIONS> {};

template <class LB, class LA>
__device__ __forceinline__ int issue_b(LB& lb, int k0, float* lds, int ld, int off, LA& la) {
  if constexpr (needs_a<LB>::value)
    return lb.issue(k0, lds, ld, off, la);
  else
    return lb.issue(k0, lds, ld, off);
}

// Body of one group (G = 0 or 1) for one sub-tile: BM = 32*WM rows shared by
// both groups, 32*WN*NT columns of its own starting at column offset COFF of
// the sub-tile; BNTOT is the column count of both groups together.
template <int WM, int NT, int G, int COFF, int BNTOT, class P>
__device__ __forceinline__ void group_body(const P& p, float* ldsA, float* ldsB, int strideA, int strideB, int m0,
                                           int ng) {   // ng: first global column of this group
  constexpr int WN = 4 / WM, BM = 32 * WM, HALF = BM / 2, NTC = NT > 0 ? NT : 1, BN = 32 * WN * NTC;
  using LA = typename P::template LA<HALF>;
  using LB = typename P::template LB<BN>;
  constexpr int LAY_A = layout_of<LA>::value, LAY_B = layout_of<LB>::value;
  constexpr int LDA = LAY_A == LAY_KC ? LDK : (lay_swz(LAY_A) ? BK : BM);
  constexpr int LDB = LAY_B == LAY_KC ? LDK : (lay_swz(LAY_B) ? BK : BNTOT);
  const int wave = gwave(), lane = threadIdx.x & 63;
  const int wm = wave % WM, wn = wave / WM;
  // fragment addressing: a split B tile is read through the group's own slab
  constexpr int RB = LAY_B == LAY_MC_SPLIT ? BN : BNTOT;
  const int arow = wm * 32, brow = (LAY_B == LAY_MC_SPLIT ? 0 : COFF) + wn * NT * 32;
  const float* const ldsBr = ldsB + (LAY_B == LAY_MC_SPLIT ? COFF * BK : 0);
  LA la;
  LB lb;
  p.template init_a<HALF>(la, m0 + G * HALF);
  if (NT > 0) p.template init_b<BN>(lb, ng, la);
  f32x16 acc[NTC];
#pragma unroll
  for (int j = 0; j < NTC; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

  const int kbeg = p.kbeg;
  const int nk = (p.kend - kbeg + BK - 1) / BK;

  // Each K step t has two phases separated by barriers.  Group 0 computes in
  // the first and moves data in the second; group 1 the other way round.
  constexpr int ST = P::STAGES;
  constexpr bool DA = is_direct<LA>::value, DB = is_direct<LB>::value;
  static_assert(ST == 3 || (!DA && !DB) || (DA && DB), "a mix of direct and register-staged loaders needs three stages");
  // request: ask global memory for a K step, into an LDS stage (direct loader) or into registers;
  // land: park a register-staged K step in its LDS stage
  auto request = [&](int k0, int stage) -> int {   // number of global -> LDS transfers issued by this wavefront
    int n = 0;
    if constexpr (DA) n += la.issue(k0, ldsA + stage * strideA, LDA, G * HALF); else la.fetch(k0);
    if constexpr (NT > 0) {
      if constexpr (DB) n += issue_b(lb, k0, ldsB + stage * strideB, LDB, COFF, la); else fetch_b(lb, k0, la);
    }
    return n;
  };
  auto land = [&](int stage) {
    if constexpr (!DA) la.commit(ldsA + stage * strideA, LDA, G * HALF);
    if constexpr (NT > 0 && !DB) lb.commit(ldsB + stage * strideB, LDB, COFF);
  };
  auto compute = [&](int stage) {
    if constexpr (NT > 0)
      mma_stage<NTC, LAY_A, LAY_B, BM, RB>(ldsA + stage * strideA, ldsBr + stage * strideB, acc, arow, brow);
  };
  if constexpr (DA && DB && ST == 2) {
    // "moving data" in step t = sending K step t+1 into the other LDS stage
    // (last read for step t-1) and waiting for it to land
    if (nk > 0) request(kbeg, 0);
    barrier_after_issue();
    for (int t = 0; t < nk; ++t) {
      const int cur = t & 1;
#pragma unroll
      for (int phase = 0; phase < 2; ++phase) {
        if (phase == G) {
          compute(cur);
          barrier_after_compute();
        } else {
          if (t + 1 < nk) request(kbeg + (t + 1) * BK, cur ^ 1);
          barrier_after_issue();
        }
      }
    }
  } else if constexpr (DA && DB && ST == 3) {
    // No phases: both groups run the same schedule side by side and share the matrix pipes as they come; whenever
    // one wavefront of a SIMD waits (for fragments, at the barrier) the other one's MFMAs fill the pipe.  During K
    // step t every wavefront sends the transfers of step t+2 off, in shares between its MFMAs, into the stage that
    // step t-1 read.  Per step there is one barrier, late in the step's MFMAs.  Before it every wavefront waits
    // until only the transfers it sent off in this step are still in flight: its part of step t+1, sent a whole
    // step earlier, has then landed.  Behind the barrier stage t+1 is therefore complete - the step's last MFMAs
    // already carry the reads of its first fragments - and stage t, which no wavefront reads any more, is free
    // for the transfers of step t+3.
    static_assert(!needs_a<LB>::value, "direct loaders stand alone");
    constexpr int NVT = (LA::NLD >= 0 && (NT == 0 || LB::NLD >= 0)) ? LA::NLD + (NT > 0 ? LB::NLD : 0) : 0;
    float fa[2][4], fb[2][NTC][4];
    int n1 = 0;
    if (nk > 0) request(kbeg, 0);
    if (nk > 1) n1 = request(kbeg + BK, 1);
    if (nk > 0) wait_transfers_but(n1);
    barrier_after_compute();
    if constexpr (NT > 0)
      if (nk > 0) load_frags<NTC, LAY_A, LAY_B, BM, RB>(ldsA, ldsBr, arow, brow, 0, fa[0], fb[0]);
    auto nothing = [](auto...) {};
    int cur = 0, t = 0;
    // one step that sends; the stage index may be a constant (then all LDS addresses of the step are loop invariants
    // or immediates, where a running index costs some twenty vector-ALU instructions a step)
    auto step = [&](auto curv) {
      const int nxt = curv + 1 == ST ? 0 : curv + 1, nn = nxt + 1 == ST ? 0 : nxt + 1;
      const int k0 = kbeg + (t + 2) * BK;
      int n = 0;   // transfers this wavefront has sent off in this step
      auto send = [&](auto share) {
        constexpr int S = decltype(share)::value;
        n += la.template issue_part<S, 4>(k0, ldsA + nn * strideA, LDA, G * HALF);
        if constexpr (NT > 0) n += lb.template issue_part<S, 4>(k0, ldsB + nn * strideB, LDB, COFF);
      };
      auto mid = [&] {
        wait_transfers_but(n);
        asm volatile("s_barrier" ::: "memory");
      };
      if constexpr (NT > 0) {
        mma_stage_stream<NTC, LAY_A, LAY_B, BM, RB, NVT, true, stream_regions<P>::value>(ldsA + curv * strideA, ldsBr + curv * strideB,
                                                              ldsA + nxt * strideA, ldsBr + nxt * strideB, acc, fa, fb,
                                                              arow, brow, mid, send);
      } else {
        send(ic<0>()); send(ic<1>()); send(ic<2>()); send(ic<3>());
        mid();
      }
      ++t;
    };
    if constexpr (stream_unroll<P>::value) {
      static_assert(ST == 3, "three steps per turn");
      while (t + 4 < nk) {   // three sending steps with constant stages: 0, 1, 2
        step(ic<0>());
        step(ic<1>());
        step(ic<2>());
      }
    }
    cur = t % ST;
    while (t + 2 < nk) {
      step(cur);
      cur = cur + 1 == ST ? 0 : cur + 1;
    }
    auto drain = [] { asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory"); };
    if (t + 1 < nk) {   // last but one step: nothing left to send
      const int nxt = cur + 1 == ST ? 0 : cur + 1;
      if constexpr (NT > 0)
        mma_stage_stream<NTC, LAY_A, LAY_B, BM, RB, 0, true, stream_regions<P>::value>(ldsA + cur * strideA, ldsBr + cur * strideB,
                                                            ldsA + nxt * strideA, ldsBr + nxt * strideB, acc, fa, fb,
                                                            arow, brow, drain, nothing);
      else
        drain();
      cur = nxt;
      ++t;
    }
    if (t < nk) {       // last step
      if constexpr (NT > 0)
        mma_stage_stream<NTC, LAY_A, LAY_B, BM, RB, 0, false, stream_regions<P>::value>(ldsA + cur * strideA, ldsBr + cur * strideB, ldsA, ldsBr,
                                                             acc, fa, fb, arow, brow, nothing, nothing);
    }
  } else {
    // "moving data" in step t = completing K step t+1 (requested in step t-1:
    // wait for the transfers, park what sits in registers) in the stage last
    // read for step t-2 (ST = 3) or t-1 (ST = 2), then requesting K step t+2;
    // a direct request targets the stage last read for step t-1, which is why
    // direct loaders need three stages here
    if (nk > 0) {
      request(kbeg, 0);
      wait_transfers<DA || DB>();
      land(0);
    }
    if (nk > 1) request(kbeg + BK, 1);
    barrier_after_compute();   // LDS writes done; transfers of step 1 stay in flight
    int cur = 0;
    for (int t = 0; t < nk; ++t) {
      const int nxt = cur + 1 == ST ? 0 : cur + 1, nn = nxt + 1 == ST ? 0 : nxt + 1;
#pragma unroll
      for (int phase = 0; phase < 2; ++phase) {
        if (phase == G) {
          compute(cur);
        } else if constexpr (DA && DB && request_first<P>::value) {
          // K step t+2 goes out first (into the stage last read for step t-1), then the wait for step t+1, which
          // has been in flight for a whole step, leaves those newest transfers outstanding: every transfer gets
          // close to two steps to land, which short steps (narrow tiles) need
          int n = 0;
          if (t + 2 < nk) n = request(kbeg + (t + 2) * BK, nn);
          if (t + 1 < nk) wait_transfers_but(n);
        } else {
          if (t + 1 < nk) {
            wait_transfers<DA || DB>();
            land(nxt);
          }
          if (t + 2 < nk) request(kbeg + (t + 2) * BK, nn);
        }
        barrier_after_compute();
      }
      cur = nxt;
    }
  }

  // epilogue: acc[j][r] is C[m0 + wm*32 + 8*(r/4) + 4*(lane/32) + r%4][ng + (wn*NT + j)*32 + lane%32]
  if (NT > 0) {
    const int i = lane & 31, h = lane >> 5;
    uint32_t roff[16];   // row part of the element offset, OOB for rows past M
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      roff[r] = m < p.M ? (uint32_t)(m * p.om.ld) : OOB;
    }
    auto col_off = [&](int j) -> uint32_t {
      const int n = ng + (wn * NT + j) * 32 + i;
      return n < p.Ncols ? p.om.col((uint32_t)n) : OOB;
    };
    auto elem = [](uint32_t cb, uint32_t ro) -> uint32_t { return ((cb | ro) & OOB) ? OOB : (cb + ro) * 4u; };
    if (p.beta) {
      // accumulate: the old values of fragment j+1 are in flight while fragment j is added and stored
      float old[2][16];
      uint32_t cb = col_off(0);
#pragma unroll
      for (int r = 0; r < 16; ++r) old[0][r] = buf_load(p.rc, elem(cb, roff[r]));
#pragma unroll
      for (int j = 0; j < NTC; ++j) {
        uint32_t cbn = 0;
        if (j + 1 < NTC) {
          cbn = col_off(j + 1);
#pragma unroll
          for (int r = 0; r < 16; ++r) old[(j + 1) & 1][r] = buf_load(p.rc, elem(cbn, roff[r]));
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) buf_store(p.rc, elem(cb, roff[r]), acc[j][r] + old[j & 1][r]);
        cb = cbn;
      }
    } else if (p.post.any() && p.post.bias_col) {
#pragma unroll
      for (int j = 0; j < NTC; ++j) {
        const uint32_t cb = col_off(j);
        const int n = ng + (wn * NT + j) * 32 + i;
        const float b = (p.post.bias != nullptr && n < p.Ncols) ? p.post.bias[n] : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) buf_store(p.rc, elem(cb, roff[r]), p.post.apply(acc[j][r], b));
      }
    } else if (p.post.any()) {
      float bv[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
        bv[r] = (p.post.bias != nullptr && m < p.M) ? p.post.bias[m] : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < NTC; ++j) {
        const uint32_t cb = col_off(j);
#pragma unroll
        for (int r = 0; r < 16; ++r) buf_store(p.rc, elem(cb, roff[r]), p.post.apply(acc[j][r], bv[r]));
      }
    } else {
#pragma unroll
      for (int j = 0; j < NTC; ++j) {
        const uint32_t cb = col_off(j);
#pragma unroll
        for (int r = 0; r < 16; ++r) buf_store(p.rc, elem(cb, roff[r]), acc[j][r]);
      }
    }
  }
}

// One output sub-tile: rows [m0, m0 + 32*WM); group 0 owns NT0 units of columns
// starting at global column n0a, group 1 owns NT1 units starting at n0b
// (normally n0a + 32*WN*NT0).  Must be called by all 512 threads.
template <int WM, int NT0, int NT1, class P>
__device__ __forceinline__ void run_tile(const P& p, float* ldsA, float* ldsB, int strideA, int strideB, int m0,
                                         int n0a, int n0b) {
  // In LDS each group's columns start at a multiple of 64 and the tile is a multiple of 64 wide: a global -> LDS
  // transfer of a pixel gather always deposits 64 lanes, so a group with an odd number of 32-column units would
  // otherwise need its last transfer masked to 32 lanes - and a lane mask around these transfers is not safe: the
  // compiler threads the code behind the branch into both paths and then takes the LDS address (M0, one per
  // wavefront) from whichever path lane 0 took.  The lanes past a group's columns carry the out-of-range offset and
  // deposit zeros in columns nobody reads.
  constexpr int WN = 4 / WM, W0 = 32 * WN * NT0, W1 = 32 * WN * NT1;
  constexpr int COFF1 = (W0 + 63) & ~63, BNTOT = COFF1 + ((W1 + 63) & ~63);
  // wave-uniform by construction; read through a scalar so the two bodies are
  // separate uniform branches (each wavefront executes exactly one of them)
  if (__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8)) == 0)
    group_body<WM, NT0, 0, 0, BNTOT>(p, ldsA, ldsB, strideA, strideB, m0, n0a);
  else
    group_body<WM, NT1, 1, COFF1, BNTOT>(p, ldsA, ldsB, strideA, strideB, m0, n0b);
  __syncthreads();   // the next sub-tile's prologue overwrites stage 0
}

// Dispatch on the unit counts of the two groups (nt0 >= nt1, 1 <= nt0 <= NTMAX).
template <int WM, int NTMAX, bool ANYPAIR, class P>
__device__ __forceinline__ void run_pair(int nt0, int nt1, const P& p, float* ldsA, float* ldsB, int strideA,
                                         int strideB, int m0, int n0a, int n0b) {
#define LNN_PAIR(A, B)                                                                                   \
  if (nt0 == A && nt1 == B) {                                                                            \
    run_tile<WM, (A <= NTMAX ? A : 1), (A <= NTMAX ? B : 0)>(p, ldsA, ldsB, strideA, strideB, m0, n0a, n0b); \
    return;                                                                                              \
  }
  LNN_PAIR(1, 0) LNN_PAIR(1, 1)
  if (NTMAX >= 2) { LNN_PAIR(2, 1) LNN_PAIR(2, 2) if (ANYPAIR) { LNN_PAIR(2, 0) } }
  if (NTMAX >= 3) { LNN_PAIR(3, 2) LNN_PAIR(3, 3) if (ANYPAIR) { LNN_PAIR(3, 0) LNN_PAIR(3, 1) } }
  if (NTMAX >= 4) { LNN_PAIR(4, 3) LNN_PAIR(4, 4) if (ANYPAIR) { LNN_PAIR(4, 0) LNN_PAIR(4, 1) LNN_PAIR(4, 2) } }
#undef LNN_PAIR
}

// Sub-tile width policy for a remaining run of cnt units (at most MAXU per sub-tile).
template <int MAXU>
__device__ __forceinline__ int pick_units(int cnt) {
  if (cnt <= MAXU) return cnt;
  // between one and two full sub-tiles: a full one first if at least half a sub-tile is left for the second
  // (measured: 8 + 4 units beat 6 + 6, but 8 + 1 loses to 5 + 4), else two halves
  if (2 * cnt >= 3 * MAXU) return MAXU;
  return (cnt + 1) >> 1;
}

// The walk of one workgroup over its share of the (M tile, unit) space.
template <int WM, int NTMAX, class P>
__device__ __forceinline__ void walk_units(const P& p, float* ldsA, float* ldsB, int strideA, int strideB,
                                           int n_units, int total_units, int wg, int n_wg) {
  constexpr int WN = 4 / WM;
  long long u0 = (long long)total_units * wg / n_wg;
  const long long u1 = (long long)total_units * (wg + 1) / n_wg;
  while (u0 < u1) {
    const int mt = (int)(u0 / n_units), un = (int)(u0 - (long long)mt * n_units);
    long long cnt = u1 - u0;
    if (cnt > n_units - un) cnt = n_units - un;
    const int nt = pick_units<2 * NTMAX>((int)cnt);
    const int nt0 = (nt + 1) >> 1, n0 = un * 32 * WN;
    run_pair<WM, NTMAX, false>(nt0, nt - nt0, p, ldsA, ldsB, strideA, strideB, mt * 32 * WM, n0, n0 + 32 * WN * nt0);
    u0 += nt;
  }
}

// Walk for column spaces made of segments of seg_units units (one segment per
// convolution tap): a group's columns never cross a segment, the two groups
// of a sub-tile may sit in different segments of the same M tile.
// Units are numbered (mt * segs_per_mt + segment) * seg_units + unit; workgroup
// chunk_index takes units [chunk_index*chunk, (chunk_index+1)*chunk); group 0 takes at most cap of them at a time
// (NTMAX, or half a chunk that is narrower than two full groups).
template <int WM, int NTMAX, class P>
__device__ __forceinline__ void walk_units_seg(const P& p, float* ldsA, float* ldsB, int strideA, int strideB,
                                               int seg_units, int segs_per_mt, int total_units, int chunk,
                                               int chunk_index, int cap) {
  constexpr int WN = 4 / WM;
  const int per_mt = seg_units * segs_per_mt;
  int pos = chunk_index * chunk;
  const int end = pos + chunk < total_units ? pos + chunk : total_units;
  while (pos < end) {
    const int mt = pos / per_mt;
    int nt0 = seg_units - pos % seg_units;
    if (nt0 > cap) nt0 = cap;
    if (nt0 > end - pos) nt0 = end - pos;
    const int p1 = pos + nt0;
    int nt1 = 0;
    if (p1 < end && p1 / per_mt == mt) {
      nt1 = seg_units - p1 % seg_units;
      if (nt1 > nt0) nt1 = nt0;
      if (nt1 > end - p1) nt1 = end - p1;
    }
    run_pair<WM, NTMAX, true>(nt0, nt1, p, ldsA, ldsB, strideA, strideB, mt * 32 * WM, (pos - mt * per_mt) * 32 * WN,
                              (p1 - mt * per_mt) * 32 * WN);
    pos = p1 + nt1;
  }
}

}  // namespace lnn
