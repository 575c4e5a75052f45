// Sum of the K slices of a split-K pass: the partial sums part[slice][m][col] of a GEMM-shaped result, added in a
// fixed order into the final tensor, with the output mapping, '+=' and the bias / activation epilogue applied there.
// Shared by the convolution passes and the plain GEMM; everything has internal linkage (each translation unit that
// includes this carries its own copy of these small kernels).
#pragma once
#include "common.hpp"

namespace lnn {
namespace {

// out[map(m, col)] (+)= sum over slices of part[slice][m][col], slices added in a
// fixed order.  A block covers 32 consecutive elements (one 128-byte line per
// slice row) with 8 lanes per element striding over the slices.  Elements of
// units >= last_unit0 (unit = (m >> bm_log) * per_mt + (col >> uw_log)) have
// only slices_last slices.
struct ReduceArgs {
  int n, slices, slices_last, beta, ncols;
  int kk;   // KH*KW when the columns are tap-major weight-gradient columns (tap*C + c), else 0
  int bm_log, uw_log, per_mt, last_unit0;
  // Equal K shares (eq_wgs > 0): the K steps of all chunks (eq_chunk units each, eq_nkt steps per chunk), laid end
  // to end, are cut into eq_wgs equal runs, one per workgroup and none longer than a chunk's; workgroup w's sums for
  // the chunk its run begins in are the block part[2w] of [1 << bm_log][eq_chunk << uw_log] floats, those for the
  // chunk it goes on in part[2w + 1].
  int eq_wgs, eq_nkt, eq_chunk, eq_chunks, eq_cw_log;   // eq_cw_log: log2 of a block's width in floats
  int eq_d, eq_g;   // the end-to-end order takes chunk (q % eq_d) * eq_g + q / eq_d at place q (eq_d = 0: chunk q)
  FastDiv dN;
  OutMap om;
  PostOp post;
};
// The workgroup whose run of K steps holds step s of the end-to-end order: runs are [T*w/W, T*(w+1)/W) for T steps
// and W workgroups, so it is the smallest w with T*(w+1)/W > s.
__host__ __device__ inline int eq_owner(long long s, long long T, long long W) { return (int)(((s + 1) * W + T - 1) / T - 1); }
// How many workgroups hold a piece of chunk c, and which is the first
__host__ __device__ inline int eq_planes(int c, int nkt, int chunks, int wgs, int* first) {
  const long long T = (long long)chunks * nkt, s = (long long)c * nkt;
  const int f = eq_owner(s, T, wgs);
  if (first) *first = f;
  return eq_owner(s + nkt - 1, T, wgs) - f + 1;
}
__device__ __forceinline__ void reduce_body(float* out, const float* part, const ReduceArgs& a) {
  __shared__ float red[8][33];
  const int li = threadIdx.x & 31, ls = threadIdx.x >> 5;
  const int i = blockIdx.x * 32 + li;
  float s = 0.0f;
  uint32_t m = 0, col = 0;
  if (i < a.n) {
    m = a.dN.div((uint32_t)i);
    col = (uint32_t)i - m * (uint32_t)a.ncols;
    const int unit = (int)(m >> a.bm_log) * a.per_mt + (int)(col >> a.uw_log);
    const int ns = unit >= a.last_unit0 ? a.slices_last : a.slices;
    // the additions stay in slice order; unrolled so that several slices' loads are in flight together (many
    // slices over a tiny output, the weight gradient of an image stem, would otherwise pay one latency per slice)
#pragma unroll 8
    for (int k = ls; k < ns; k += 8) s += part[(size_t)k * a.n + i];
  }
  red[ls][li] = s;
  __syncthreads();
  if (ls == 0 && i < a.n) {
#pragma unroll
    for (int k = 1; k < 8; ++k) s += red[k][li];
    const uint32_t o = a.om.col(col) + m * (uint32_t)a.om.ld;
    if (a.post.any()) s = a.post.apply(s, a.post.bias != nullptr ? a.post.bias[a.post.bias_col ? col : m] : 0.0f);
    out[o] = a.beta ? out[o] + s : s;
  }
}
__global__ __launch_bounds__(256) void reduce_partials(float* out, const float* part, ReduceArgs a) {
  reduce_body(out, part, a);
}

// The same for ncols % 4 == 0 with 128-bit reads: a block covers 128 consecutive
// elements, 8 lanes per group of 4 striding over the slices.
__device__ __forceinline__ void reduce_body4(float* out, const float* part, const ReduceArgs& a) {
  __shared__ float red[8][128];
  const int q = threadIdx.x & 31, ls = threadIdx.x >> 5;
  const int i4 = (blockIdx.x * 32 + q) * 4;
  f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  if (i4 < a.n) {
    const uint32_t m = a.dN.div((uint32_t)i4), col = (uint32_t)i4 - m * (uint32_t)a.ncols;
    const int unit = (int)(m >> a.bm_log) * a.per_mt + (int)(col >> a.uw_log);
    const int ns = unit >= a.last_unit0 ? a.slices_last : a.slices;
#pragma unroll 4
    for (int k = ls; k < ns; k += 8) s += *reinterpret_cast<const f32x4*>(&part[(size_t)k * a.n + i4]);
  }
  *reinterpret_cast<f32x4*>(&red[ls][4 * q]) = s;
  __syncthreads();
  const int e = threadIdx.x, i = blockIdx.x * 128 + e;
  if (e < 128 && i < a.n) {
    float t = red[0][e];
#pragma unroll
    for (int k = 1; k < 8; ++k) t += red[k][e];
    const uint32_t m = a.dN.div((uint32_t)i), col = (uint32_t)i - m * (uint32_t)a.ncols;
    const uint32_t o = a.om.col(col) + m * (uint32_t)a.om.ld;
    if (a.post.any()) t = a.post.apply(t, a.post.bias != nullptr ? a.post.bias[a.post.bias_col ? col : m] : 0.0f);
    out[o] = a.beta ? out[o] + t : t;
  }
}
// ... and with at most kFewSlices slices: nothing to gain from lanes striding over the slices (most of them would
// idle), so every thread adds up the slices of four consecutive elements itself, all its loads in flight together,
// and a block covers 1024 elements, which leave through LDS so that consecutive lanes store consecutive elements.
// The additions are the ones reduce_body4 makes, in the same order.
constexpr int kFewSlices = 8;
template <int NS>
__device__ __forceinline__ f32x4 sum_slices(const float* part, size_t n, int i4, int ns) {
  f32x4 v[NS];
#pragma unroll
  for (int k = 0; k < NS; ++k) v[k] = *reinterpret_cast<const f32x4*>(&part[(size_t)(k < ns ? k : 0) * n + i4]);
  f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int k = 0; k < NS; ++k) s += k < ns ? v[k] : zero;
  return s;
}
__device__ __forceinline__ void reduce_body4_few(float* out, const float* part, const ReduceArgs& a) {
  __shared__ float red[1024];
  const int i4 = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 4;
  f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
  if (i4 < a.n) {
    const uint32_t m = a.dN.div((uint32_t)i4), col = (uint32_t)i4 - m * (uint32_t)a.ncols;
    const int unit = (int)(m >> a.bm_log) * a.per_mt + (int)(col >> a.uw_log);
    const int ns = unit >= a.last_unit0 ? a.slices_last : a.slices;
    // the slice count of the problem is uniform: one straight run of loads per count; a unit of the last chunk,
    // which may have fewer slices, reads slice 0 again in their place and adds zeros
    switch (a.slices) {
      case 2: s = sum_slices<2>(part, (size_t)a.n, i4, ns); break;
      case 3: s = sum_slices<3>(part, (size_t)a.n, i4, ns); break;
      case 4: s = sum_slices<4>(part, (size_t)a.n, i4, ns); break;
      case 5: s = sum_slices<5>(part, (size_t)a.n, i4, ns); break;
      case 6: s = sum_slices<6>(part, (size_t)a.n, i4, ns); break;
      case 7: s = sum_slices<7>(part, (size_t)a.n, i4, ns); break;
      default: s = sum_slices<8>(part, (size_t)a.n, i4, ns); break;
    }
  }
  *reinterpret_cast<f32x4*>(&red[4 * threadIdx.x]) = s;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = (int)threadIdx.x + 256 * j, i = (int)blockIdx.x * 1024 + e;
    if (i < a.n) {
      float t = red[e];
      const uint32_t m = a.dN.div((uint32_t)i), col = (uint32_t)i - m * (uint32_t)a.ncols;
      const uint32_t o = a.om.col(col) + m * (uint32_t)a.om.ld;
      if (a.post.any()) t = a.post.apply(t, a.post.bias != nullptr ? a.post.bias[a.post.bias_col ? col : m] : 0.0f);
      out[o] = a.beta ? out[o] + t : t;
    }
  }
}
// Weight gradients (columns tap-major, tap*C + c; result stored [o][c][tap] or [c][o][tap]): one block per GEMM row.
// The element-wise kernels above store a row's elements KK floats apart, 4 bytes at a time; here the row's sums are
// parked in LDS at their permuted place c*KK + tap (KK odd for the usual kernels: no bank conflicts) and leave as one
// contiguous run (whole runs of KK floats per channel for a gradient kept with swapped channel axes).  Slices are
// added in ascending order, eight loads in flight.  ncols % 4 == 0; a row may be shared out among gridDim.y blocks by
// runs of channels (C % 4 == 0 then); (channels per block) * KK floats of dynamic LDS.
__global__ __launch_bounds__(256) void reduce_partials_rows(float* out, const float* part, ReduceArgs a) {
  extern __shared__ float reduce_row[];
  const uint32_t m = blockIdx.x, C = a.om.dHW.d;
  const size_t n = (size_t)a.n;
  // equal K shares: per chunk of this row, the first workgroup that holds a piece of it, how many do, and whether
  // that first one's piece is its second (its run began in the chunk before)
  __shared__ int eq_first[128], eq_count[128];
  if (a.eq_wgs > 0) {
    const int per_row = a.ncols >> a.eq_cw_log;
    const long long T = (long long)a.eq_chunks * a.eq_nkt;
    for (int j = threadIdx.x; j < per_row; j += 256) {
      const int c = (int)(m >> a.bm_log) * per_row + j;
      const int q = a.eq_d > 0 ? a.eq_d * (c % a.eq_g) + c / a.eq_g : c;   // the chunk's place in the end-to-end order
      int first;
      const int np = eq_planes(q, a.eq_nkt, a.eq_chunks, a.eq_wgs, &first);
      const int second = (int)(T * first / a.eq_wgs / a.eq_nkt) == q ? 0 : 1;
      eq_first[j] = first;
      eq_count[j] = np | (second << 16);
    }
    __syncthreads();
  }
  // blockIdx.y: which run of channels of the row this block sums (gridDim.y runs of cpb channels, cpb % 4 == 0)
  const uint32_t cpb = gridDim.y > 1 ? (((C + gridDim.y - 1) / gridDim.y + 3) & ~3u) : C;
  const uint32_t c0 = blockIdx.y * cpb, cn = c0 >= C ? 0u : (C - c0 < cpb ? C - c0 : cpb);
  const int mine = (int)(cn * (uint32_t)a.kk);
  for (int g = threadIdx.x; 4 * g < mine; g += 256) {
    // the g-th group of four of this block's columns (tap-major: tap * C + c0 .. c0 + cn)
    const uint32_t tap0 = gridDim.y > 1 ? (4u * g) / cn : 0u;
    const uint32_t col = gridDim.y > 1 ? tap0 * C + c0 + (4u * g - tap0 * cn) : 4u * g;
    const size_t i4 = (size_t)m * a.ncols + col;
    const int unit = (int)(m >> a.bm_log) * a.per_mt + (int)(col >> a.uw_log);
    int ns = unit >= a.last_unit0 ? a.slices_last : a.slices;
    f32x4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    int k = 0;
    if (a.eq_wgs > 0) {
      // the blocks of the workgroups whose runs touch this element's chunk, in workgroup order
      const int j = (int)(col >> a.eq_cw_log), cw = 1 << a.eq_cw_log, bm = 1 << a.bm_log;
      const size_t within = (size_t)(m & (uint32_t)(bm - 1)) * cw + (col & (uint32_t)(cw - 1));
      const int first = eq_first[j], np = eq_count[j] & 0xffff, second = eq_count[j] >> 16;
      const float* src = part + (size_t)(2 * first + second) * bm * cw + within;
      f32x4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = *reinterpret_cast<const f32x4*>(src + (size_t)(i < np ? (i ? 2 * i - second : 0) : 0) * bm * cw);
      const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int i = 0; i < 4; ++i) s += i < np ? v[i] : zero;
      for (int i = 4; i < np; ++i) s += *reinterpret_cast<const f32x4*>(src + (size_t)(2 * i - second) * bm * cw);
      ns = 0;
    }
    for (; k + 8 <= ns; k += 8) {
      f32x4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const f32x4*>(&part[(size_t)(k + j) * n + i4]);
#pragma unroll
      for (int j = 0; j < 8; ++j) s += v[j];
    }
    if (k < ns) {
      f32x4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const f32x4*>(&part[(size_t)(k + j < ns ? k + j : k) * n + i4]);
      const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < 8; ++j) s += k + j < ns ? v[j] : zero;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t cj = col + j, tap = a.om.dHW.div(cj), c = cj - tap * C;
      reduce_row[(c - c0) * a.kk + tap] = s[j];
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < mine; e += 256) {
    const uint32_t cl = (uint32_t)e / (uint32_t)a.kk, tap = (uint32_t)e - cl * (uint32_t)a.kk, c = c0 + cl;
    const size_t o = (size_t)a.om.col(tap * C + c) + (size_t)m * a.om.ld;
    const float t = reduce_row[e];
    out[o] = a.beta ? out[o] + t : t;
  }
}

// elements per block of the 128-bit reductions
__host__ __device__ inline int reduce4_block(const ReduceArgs& a) { return a.slices <= kFewSlices ? 1024 : 128; }
__global__ __launch_bounds__(256) void reduce_partials4(float* out, const float* part, ReduceArgs a) {
  if (a.slices <= kFewSlices) reduce_body4_few(out, part, a);
  else reduce_body4(out, part, a);
}

// The reductions of the pixel classes of one strided dgrad in one launch: blockIdx.y = class.
constexpr int kMaxReduceBatch = 4;
struct ReduceBatch {
  ReduceArgs r[kMaxReduceBatch];
  float* out[kMaxReduceBatch];
  const float* part[kMaxReduceBatch];
  int vec[kMaxReduceBatch];
};
__global__ __launch_bounds__(256) void reduce_partials_batch(ReduceBatch b) {
  const int c = blockIdx.y;
  const int per_block = b.vec[c] ? reduce4_block(b.r[c]) : 32;
  if ((long long)blockIdx.x * per_block >= b.r[c].n) return;   // the whole block leaves together
  if (b.vec[c] && b.r[c].slices <= kFewSlices) reduce_body4_few(b.out[c], b.part[c], b.r[c]);
  else if (b.vec[c]) reduce_body4(b.out[c], b.part[c], b.r[c]);
  else reduce_body(b.out[c], b.part[c], b.r[c]);
}

}  // namespace
}  // namespace lnn
