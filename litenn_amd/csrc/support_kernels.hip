// Bandwidth-bound helpers around the contraction kernels: fill, pointwise
// forward/backward, broadcasting binary ops, axis reductions, transpose,
// materialised unfold and the SGD update.  One grid-stride thread per element;
// element counts are below 2^31 (every tensor is smaller than 2 GiB), so index
// decomposition is done in 32-bit arithmetic.
#include "common.hpp"

namespace lnn {

constexpr int kMaxRank = 8;
struct Dims {
  int rank;
  int shape[kMaxRank];
  long long sa[kMaxRank];   // per-axis element strides of operand a (0 = broadcast)
  long long sb[kMaxRank];
};

static inline dim3 grid_for(uint64_t n, int cus) {
  uint64_t blocks = (n + 255) / 256;
  const uint64_t cap = (uint64_t)cus * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return dim3((unsigned)blocks);
}

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t v, uint64_t n) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

__device__ __forceinline__ float ew_f(int op, float x, float p0) {
  switch (op) {
    case LNN_EW_ADD_CONST: return x + p0;
    case LNN_EW_MUL_CONST: return x * p0;
    case LNN_EW_LEAKY_RELU: return x >= 0.0f ? x : p0 * x;
    case LNN_EW_SQUARE: return x * x;
    default: return x >= 0.0f ? x : 0.0f;
  }
}
__device__ __forceinline__ float ew_df(int op, float x, float p0) {
  switch (op) {
    case LNN_EW_ADD_CONST: return 1.0f;
    case LNN_EW_MUL_CONST: return p0;
    case LNN_EW_LEAKY_RELU: return x >= 0.0f ? 1.0f : p0;
    case LNN_EW_SQUARE: return 2.0f * x;
    default: return x >= 0.0f ? 1.0f : 0.0f;
  }
}

__global__ void ew_fwd_kernel(int op, uint64_t n, const float* in, float* out, float p0, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const float r = ew_f(op, in[i], p0);
    out[i] = beta ? out[i] + r : r;
  }
}

__global__ void ew_bwd_kernel(int op, uint64_t n, const float* in, const float* dout, float* din, float p0, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const float g = dout[i] * ew_df(op, in[i], p0);
    din[i] = beta ? din[i] + g : g;
  }
}

__global__ void binary_bcast_kernel(int op, Dims d, uint64_t n, const float* a, const float* b, float* out, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    uint32_t g = (uint32_t)i;
    long long oa = 0, ob = 0;
    for (int ax = d.rank - 1; ax >= 0; --ax) {
      const uint32_t x = g % (uint32_t)d.shape[ax];
      g /= (uint32_t)d.shape[ax];
      oa += (long long)x * d.sa[ax];
      ob += (long long)x * d.sb[ax];
    }
    const float x = a[oa], y = b[ob];
    const float r = op == 0 ? x + y : (op == 1 ? x - y : x * y);
    out[i] = beta ? out[i] + r : r;
  }
}

// Reduction plan: kept axes index the output (row-major in axis order), reduced
// axes are walked by the threads of one workgroup (and, for long reductions,
// by several workgroups that leave partial sums for a second pass).
struct RedPlan {
  int nk, nr;
  int kshape[kMaxRank], rshape[kMaxRank];
  long long kstride[kMaxRank], rstride[kMaxRank];
  uint64_t outs, red;
  int flat;   // the reduced axes are the trailing ones: element r of a reduction lies r floats behind its first
};

__device__ __forceinline__ long long offset_of(uint32_t idx, int n, const int* shape, const long long* stride) {
  long long off = 0;
  for (int ax = n - 1; ax >= 0; --ax) {
    const uint32_t x = idx % (uint32_t)shape[ax];
    idx /= (uint32_t)shape[ax];
    off += (long long)x * stride[ax];
  }
  return off;
}

// grid = (outs, parts).  dst[o*parts + part] = partial sum (parts > 1) or the
// finished value (parts == 1: scaled, optionally accumulated).
__global__ void reduce_sum_kernel(RedPlan p, const float* in, float* dst, int parts, float scale, int beta) {
  __shared__ float sh[256];
  const uint64_t o = blockIdx.x;
  const int part = blockIdx.y;
  const long long base = offset_of((uint32_t)o, p.nk, p.kshape, p.kstride);
  const uint64_t r0 = p.red * part / parts, r1 = p.red * (part + 1) / parts;
  float s = 0.0f;
  if (p.flat) {   // same elements in the same order, without the index arithmetic
    for (uint64_t r = r0 + threadIdx.x; r < r1; r += 256) s += in[base + (long long)r];
  } else {
    for (uint64_t r = r0 + threadIdx.x; r < r1; r += 256) s += in[base + offset_of((uint32_t)r, p.nr, p.rshape, p.rstride)];
  }
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) sh[threadIdx.x] += sh[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (parts > 1) {
      dst[o * parts + part] = sh[0];
    } else {
      const float r = sh[0] * scale;
      dst[o] = beta ? dst[o] + r : r;
    }
  }
}

// one wavefront per output: lane l adds parts l, l + 64, ..., then a butterfly (fixed order)
__global__ __launch_bounds__(64) void reduce_finish_kernel(const float* part, float* out, uint64_t outs, int parts,
                                                           float scale, int beta) {
  const uint64_t o = blockIdx.x;
  float s = 0.0f;
  for (int k = threadIdx.x; k < parts; k += 64) s += part[o * parts + k];
#pragma unroll
  for (int w = 32; w > 0; w >>= 1) s += __shfl_xor(s, w, 64);
  if (threadIdx.x == 0) {
    s *= scale;
    out[o] = beta ? out[o] + s : s;
  }
}

// din[idx] (+)= scale * dout[kept part of idx]
__global__ void reduce_bwd_kernel(Dims d, uint64_t n, float scale, const float* dout, float* din, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    uint32_t g = (uint32_t)i;
    long long oa = 0;
    for (int ax = d.rank - 1; ax >= 0; --ax) {
      const uint32_t x = g % (uint32_t)d.shape[ax];
      g /= (uint32_t)d.shape[ax];
      oa += (long long)x * d.sa[ax];
    }
    const float v = scale * dout[oa];
    din[i] = beta ? din[i] + v : v;
  }
}

// out[perm(idx)] (+)= in[idx]; d.sa holds, per input axis, the stride of that axis in the output.
__global__ void transpose_kernel(Dims d, uint64_t n, const float* in, float* out, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    uint32_t g = (uint32_t)i;
    long long oo = 0;
    for (int ax = d.rank - 1; ax >= 0; --ax) {
      const uint32_t x = g % (uint32_t)d.shape[ax];
      g /= (uint32_t)d.shape[ax];
      oo += (long long)x * d.sa[ax];
    }
    out[oo] = beta ? out[oo] + in[i] : in[i];
  }
}

struct UnfoldArgs {
  int N, C, H, W, OH, OW, KH, KW, PADL, PADT, D, S, order, transposed;
};

// One thread per element of the unfolded matrix, written in row-major order
// of the symbol string (last symbol fastest).
__global__ void unfold2d_kernel(UnfoldArgs a, uint64_t n, const float* in, float* out, int beta) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    uint32_t g = (uint32_t)i;
    int on, oc, oh, ow, oj, oi;
    if (a.order == 0) {   // C J I N H W
      ow = (int)(g % a.OW); g /= a.OW;
      oh = (int)(g % a.OH); g /= a.OH;
      on = (int)(g % a.N);  g /= a.N;
      oi = (int)(g % a.KW); g /= a.KW;
      oj = (int)(g % a.KH); g /= a.KH;
      oc = (int)g;
    } else {              // N H W C J I
      oi = (int)(g % a.KW); g /= a.KW;
      oj = (int)(g % a.KH); g /= a.KH;
      oc = (int)(g % a.C);  g /= a.C;
      ow = (int)(g % a.OW); g /= a.OW;
      oh = (int)(g % a.OH); g /= a.OH;
      on = (int)g;
    }
    int ih, iw;
    bool ok;
    if (!a.transposed) {
      ih = -a.PADT + oj * a.D + oh * a.S;
      iw = -a.PADL + oi * a.D + ow * a.S;
      ok = ih >= 0 && ih < a.H && iw >= 0 && iw < a.W;
    } else {
      const int nh = a.PADT + oh - oj * a.D, nw = a.PADL + ow - oi * a.D;
      ih = nh >= 0 ? nh / a.S : 0;
      iw = nw >= 0 ? nw / a.S : 0;
      ok = nh >= 0 && nw >= 0 && ih * a.S == nh && iw * a.S == nw && ih < a.H && iw < a.W;
    }
    const float v = ok ? in[(((size_t)on * a.C + oc) * a.H + ih) * a.W + iw] : 0.0f;
    out[i] = beta ? out[i] + v : v;
  }
}

__global__ void sgd_kernel(uint64_t n, float* v, const float* g, float* acc, float momentum, float lr, int nesterov) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const float a = momentum * acc[i] - lr * g[i];
    acc[i] = a;
    v[i] += nesterov ? momentum * a - lr * g[i] : a;
  }
}

// m = b1*m + (1-b1)*g;  v2 = b2*v2 + (1-b2)*g*g;  t -= lr*m / (sqrt(v2) + 1e-7)   (no bias correction)
__global__ void adam_kernel(uint64_t n, float* t, const float* g, float* m, float* v2, float beta1, float beta2,
                            float lr) {
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const float gi = g[i];
    const float mi = beta1 * m[i] + (1.0f - beta1) * gi;
    const float vi = beta2 * v2[i] + (1.0f - beta2) * gi * gi;
    m[i] = mi;
    v2[i] = vi;
    t[i] += -lr * mi / (sqrtf(vi) + 1e-7f);
  }
}

// The optimizer step of up to kMultiMax tensors in one launch: blockIdx.y = tensor.  A model has a handful of
// parameter tensors, most of them small, and one launch per tensor costs more than the update itself.
constexpr int kMultiMax = 16;
struct MultiArgs {
  uint64_t n[kMultiMax];
  float* t[kMultiMax];          // the parameter
  const float* g[kMultiMax];    // its gradient
  float* s0[kMultiMax];         // optimizer state (SGD: accumulator; Adam: m)
  float* s1[kMultiMax];         // Adam: v
  // a convolution kernel's copy in the layout the tap-major passes read, Wp[o][tap][c] (or null): the update writes
  // the new value there too, so that the copy need not be made again before the next forward pass
  float* wp[kMultiMax];
  FastDiv dKK[kMultiMax], dIn[kMultiMax];   // divide by KH*KW, by the inner of the tensor's two channel axes
  int wp_c[kMultiMax];                      // C of the copy; negative: the tensor is stored [C][O][tap]
  // learning-rate dropout (Optimizer.py:199-202): seeds of the tensor's state-update and value-update kernels
  uint32_t seed0[kMultiMax], seed1[kMultiMax];
};
__device__ __forceinline__ uint32_t hash_u32(uint32_t v);
// lr, or 0 where the counter hash of (element + seed), scaled to [0, 1], does not exceed `drop`
// (Optimizer.py:199-202: if (hash_float_uint(gid + seed) <= lr_dropout) lr = 0; drop == 0 compiles the test out there)
__device__ __forceinline__ float dropped_lr(float lr, float drop, uint64_t i, uint32_t seed) {
  if (drop == 0.0f) return lr;
  const float u = (float)hash_u32((uint32_t)(i + seed)) * (1.0f / 4294967296.0f);
  return u <= drop ? 0.0f : lr;
}
// parameter element i = (o*C + c)*KK + tap (or (c*O + o)*KK + tap for a tensor stored with swapped channel axes, as
// a transposed convolution keeps its kernel) goes to Wp[(o*KK + tap)*C + c]
__device__ __forceinline__ void store_permuted(const MultiArgs& a, int k, uint64_t i, float value) {
  const uint32_t oc = a.dKK[k].div((uint32_t)i), tap = (uint32_t)i - oc * a.dKK[k].d;
  const uint32_t hi = a.dIn[k].div(oc), lo = oc - hi * a.dIn[k].d;
  const bool swapped = a.wp_c[k] < 0;
  const uint32_t C = (uint32_t)(swapped ? -a.wp_c[k] : a.wp_c[k]), o = swapped ? lo : hi, c = swapped ? hi : lo;
  a.wp[k][((size_t)o * a.dKK[k].d + tap) * C + c] = value;
}
// One element of the SGD step (SGD.py:42-74): returns the new parameter value.  With momentum 0 the accumulator's old
// value has no weight and is not read.
__device__ __forceinline__ float sgd_element(const MultiArgs& a, int k, uint64_t i, float momentum, float lr, int nesterov,
                                             float drop) {
  // the reference's two kernels per tensor draw their dropout masks from separate seeds
  const float gi = a.g[k][i];
  const float lr0 = dropped_lr(lr, drop, i, a.seed0[k]);
  float x;
  if (momentum != 0.0f) x = momentum * a.s0[k][i] - lr0 * gi;
  else x = -(lr0 * gi);
  a.s0[k][i] = x;
  const float nv = a.t[k][i] + (nesterov ? momentum * x - dropped_lr(lr, drop, i, a.seed1[k]) * gi : x);
  a.t[k][i] = nv;
  return nv;
}
// One element of the Adam step (Adam.py:44-69)
__device__ __forceinline__ float adam_element(const MultiArgs& a, int k, uint64_t i, float beta1, float beta2, float lr,
                                              float drop) {
  const float gi = a.g[k][i];
  const float mi = beta1 * a.s0[k][i] + (1.0f - beta1) * gi;
  const float vi = beta2 * a.s1[k][i] + (1.0f - beta2) * gi * gi;
  a.s0[k][i] = mi;
  a.s1[k][i] = vi;
  const float nt = a.t[k][i] + -dropped_lr(lr, drop, i, a.seed0[k]) * mi / (sqrtf(vi) + 1e-7f);
  a.t[k][i] = nt;
  return nt;
}
// The walk both optimizers share.  A tensor without a permuted copy: a grid-stride loop.  One stored [O][C][tap] with
// a copy Wp[o][tap][c]: tiles of one o and up to 64 channels, kMultiTile floats at most - a contiguous run of the
// tensor, updated in order and parked in LDS, then written to the copy tap by tap, so that the copy too is stored in
// runs of consecutive channels instead of single floats a whole row apart.  Other copies are stored element by
// element.
constexpr int kMultiTile = 4096;
template <class F>
__device__ __forceinline__ void update_walk(const MultiArgs& a, F&& element) {
  const int k = blockIdx.y;
  const uint64_t n = a.n[k];
  const int KK = (int)a.dKK[k].d, C = a.wp_c[k];
  if (a.wp[k] && C > 0 && KK * (C < 64 ? C : 64) <= kMultiTile) {
    __shared__ float tile[kMultiTile];
    const int TL = C < 64 ? C : 64, per_o = (C + TL - 1) / TL;
    const uint32_t tiles = (uint32_t)(n / ((uint64_t)C * KK)) * per_o;
    for (uint32_t t = blockIdx.x; t < tiles; t += gridDim.x) {
      const uint32_t o = t / per_o, c0 = (t - o * per_o) * TL;
      const int tl = (int)(C - c0) < TL ? (int)(C - c0) : TL, len = tl * KK;
      const uint64_t base = ((uint64_t)o * C + c0) * KK;
      for (int e = threadIdx.x; e < len; e += blockDim.x) tile[e] = element(k, base + e);
      __syncthreads();
      float* dst = a.wp[k] + (size_t)o * KK * C + c0;
      for (int e = threadIdx.x; e < len; e += blockDim.x) {
        const int tap = e / tl, cl = e - tap * tl;
        dst[(size_t)tap * C + cl] = tile[cl * KK + tap];
      }
      __syncthreads();
    }
    return;
  }
  for (uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
    const float nv = element(k, i);
    if (a.wp[k]) store_permuted(a, k, i, nv);
  }
}
__global__ __launch_bounds__(256) void sgd_multi_kernel(MultiArgs a, float momentum, float lr, int nesterov, float drop) {
  update_walk(a, [&](int k, uint64_t i) { return sgd_element(a, k, i, momentum, lr, nesterov, drop); });
}
__global__ __launch_bounds__(256) void adam_multi_kernel(MultiArgs a, float beta1, float beta2, float lr, float drop) {
  update_walk(a, [&](int k, uint64_t i) { return adam_element(a, k, i, beta1, beta2, lr, drop); });
}

// ---------------------------------------------------------------------------
// host launchers (called from the C ABI)
// ---------------------------------------------------------------------------
int launch_fill_u32(DeviceCtx* ctx, void* dst, uint32_t pattern, uint64_t count) {
  if (count == 0) return LNN_OK;
  hipLaunchKernelGGL(fill_u32_kernel, grid_for(count, ctx->cus), dim3(256), 0, ctx->stream,
                     static_cast<uint32_t*>(dst), pattern, count);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_ew_fwd(DeviceCtx* ctx, int op, uint64_t n, const float* in, float* out, float p0, int beta) {
  if (op < 0 || op > LNN_EW_RELU) return set_error(LNN_ERR_INVALID, "ew_fwd: unknown op");
  if (n == 0) return LNN_OK;
  hipLaunchKernelGGL(ew_fwd_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, op, n, in, out, p0, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_ew_bwd(DeviceCtx* ctx, int op, uint64_t n, const float* in, const float* dout, float* din, float p0,
                  int beta) {
  if (op < 0 || op > LNN_EW_RELU) return set_error(LNN_ERR_INVALID, "ew_bwd: unknown op");
  if (n == 0) return LNN_OK;
  hipLaunchKernelGGL(ew_bwd_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, op, n, in, dout, din, p0, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

static int check_rank(int rank, const int32_t* shape, const char* who) {
  if (rank < 1 || rank > kMaxRank || !shape) return set_error(LNN_ERR_INVALID, std::string(who) + ": rank must be 1..8");
  for (int i = 0; i < rank; ++i)
    if (shape[i] <= 0) return set_error(LNN_ERR_INVALID, std::string(who) + ": non-positive extent");
  return LNN_OK;
}

int launch_binary_bcast(DeviceCtx* ctx, int op, int rank, const int32_t* os, const int32_t* as, const int32_t* bs,
                        const float* a, const float* b, float* out, int beta) {
  if (op < 0 || op > 2) return set_error(LNN_ERR_INVALID, "binary_bcast: unknown op");
  int st = check_rank(rank, os, "binary_bcast");
  if (st != LNN_OK) return st;
  Dims d;
  d.rank = rank;
  uint64_t n = 1;
  long long ca = 1, cb = 1;
  for (int ax = rank - 1; ax >= 0; --ax) {
    if ((as[ax] != os[ax] && as[ax] != 1) || (bs[ax] != os[ax] && bs[ax] != 1))
      return set_error(LNN_ERR_INVALID, "binary_bcast: shapes do not broadcast");
    d.shape[ax] = os[ax];
    d.sa[ax] = as[ax] == 1 ? 0 : ca;
    d.sb[ax] = bs[ax] == 1 ? 0 : cb;
    ca *= as[ax];
    cb *= bs[ax];
    n *= (uint64_t)os[ax];
  }
  hipLaunchKernelGGL(binary_bcast_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, op, d, n, a, b, out,
                     beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_reduce_sum(DeviceCtx* ctx, int rank, const int32_t* shape, uint32_t mask, float scale, const float* in,
                      float* out, int beta) {
  int st = check_rank(rank, shape, "reduce_sum");
  if (st != LNN_OK) return st;
  RedPlan p;
  p.nk = p.nr = 0;
  p.outs = p.red = 1;
  long long stride = 1;
  long long strides[kMaxRank];
  for (int ax = rank - 1; ax >= 0; --ax) {
    strides[ax] = stride;
    stride *= shape[ax];
  }
  for (int ax = 0; ax < rank; ++ax) {
    if (mask & (1u << ax)) {
      p.rshape[p.nr] = shape[ax];
      p.rstride[p.nr++] = strides[ax];
      p.red *= (uint64_t)shape[ax];
    } else {
      p.kshape[p.nk] = shape[ax];
      p.kstride[p.nk++] = strides[ax];
      p.outs *= (uint64_t)shape[ax];
    }
  }
  if (p.outs > 0x7fffffffull) return set_error(LNN_ERR_UNSUPPORTED, "reduce_sum: too many outputs");
  p.flat = p.nr > 0 && p.rstride[p.nr - 1] == 1;
  for (int i = 0; i + 1 < p.nr; ++i) p.flat = p.flat && p.rstride[i] == p.rstride[i + 1] * p.rshape[i + 1];
  // long reductions with few outputs are split so the whole chip takes part
  int parts = 1;
  if (p.red >= 8192) {
    uint64_t want = (uint64_t)ctx->cus * 4 / p.outs;
    uint64_t most = p.red / 2048;
    if (want > most) want = most;
    if (want > 1024) want = 1024;
    if (want > 1) parts = (int)want;
  }
  float* dst = out;
  if (parts > 1) {
    st = ensure_workspace(ctx, (size_t)p.outs * parts * sizeof(float));
    if (st != LNN_OK) return st;
    dst = static_cast<float*>(ctx->ws);
  }
  hipLaunchKernelGGL(reduce_sum_kernel, dim3((unsigned)p.outs, parts), dim3(256), 0, ctx->stream, p, in, dst, parts,
                     scale, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  if (parts > 1) {
    hipLaunchKernelGGL(reduce_finish_kernel, dim3((unsigned)p.outs), dim3(64), 0, ctx->stream,
                       static_cast<const float*>(dst), out, p.outs, parts, scale, beta ? 1 : 0);
    LNN_HIP(hipGetLastError());
  }
  return LNN_OK;
}

int launch_reduce_sum_bwd(DeviceCtx* ctx, int rank, const int32_t* shape, uint32_t mask, float scale,
                          const float* dout, float* din, int beta) {
  int st = check_rank(rank, shape, "reduce_sum_bwd");
  if (st != LNN_OK) return st;
  Dims d;
  d.rank = rank;
  uint64_t n = 1;
  long long c = 1;
  for (int ax = rank - 1; ax >= 0; --ax) {
    d.shape[ax] = shape[ax];
    const bool red = mask & (1u << ax);
    d.sa[ax] = red ? 0 : c;
    d.sb[ax] = 0;
    if (!red) c *= shape[ax];
    n *= (uint64_t)shape[ax];
  }
  hipLaunchKernelGGL(reduce_bwd_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, d, n, scale, dout, din, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_transpose(DeviceCtx* ctx, int rank, const int32_t* shape, const int32_t* axes, const float* in, float* out,
                     int beta) {
  int st = check_rank(rank, shape, "transpose");
  if (st != LNN_OK) return st;
  bool seen[kMaxRank] = {false};
  for (int i = 0; i < rank; ++i) {
    if (axes[i] < 0 || axes[i] >= rank || seen[axes[i]]) return set_error(LNN_ERR_INVALID, "transpose: axes are not a permutation");
    seen[axes[i]] = true;
  }
  Dims d;
  d.rank = rank;
  uint64_t n = 1;
  long long ostride[kMaxRank];
  long long c = 1;
  for (int i = rank - 1; i >= 0; --i) {   // output axis i has extent shape[axes[i]]
    ostride[i] = c;
    c *= shape[axes[i]];
  }
  for (int i = 0; i < rank; ++i) {
    d.shape[i] = shape[i];
    d.sb[i] = 0;
    n *= (uint64_t)shape[i];
  }
  for (int i = 0; i < rank; ++i) d.sa[axes[i]] = ostride[i];
  hipLaunchKernelGGL(transpose_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, d, n, in, out, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_unfold2d(DeviceCtx* ctx, int N, int C, int H, int W, int OH, int OW, int KH, int KW, int PADL, int PADT,
                    int D, int S, int order, int transposed, const float* in, float* out, int beta) {
  const int v[] = {N, C, H, W, OH, OW, KH, KW, D, S};
  for (int x : v)
    if (x <= 0) return set_error(LNN_ERR_INVALID, "unfold2d: non-positive dimension");
  if (order != 0 && order != 1) return set_error(LNN_ERR_INVALID, "unfold2d: order must be 0 or 1");
  UnfoldArgs a = {N, C, H, W, OH, OW, KH, KW, PADL, PADT, D, S, order, transposed ? 1 : 0};
  const uint64_t n = (uint64_t)N * C * OH * OW * KH * KW;
  hipLaunchKernelGGL(unfold2d_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, a, n, in, out, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_sgd(DeviceCtx* ctx, uint64_t n, float* v, const float* g, float* acc, float momentum, float lr, int nesterov) {
  if (n == 0) return LNN_OK;
  hipLaunchKernelGGL(sgd_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, n, v, g, acc, momentum, lr,
                     nesterov ? 1 : 0);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// ---- backward of the fused conv epilogue --------------------------------------------------------------------
// One pass over Y and dY (both [N][O][HW]) gives the gradient before the activation, dpre = dY * f'(Y), and the
// bias gradient dbias[o] (+)= sum over n and pixels of dpre: the separate activation-gradient kernel and the
// reduction that follow it in the reference (element_wise_op.py:211, dual_wise_op.py:110-130) read dpre again.
// Channel o's elements are cut into pieces of 2048 consecutive floats of one plane; block (slice, o) walks a
// contiguous range of pieces, so the sums are formed in a fixed order whatever the grid.
constexpr int kEpiPiece = 2048;

__global__ __launch_bounds__(256) void bias_act_bwd_kernel(int N, int O, int HW, int ppp, int slices,
                                                           const float* __restrict__ y, const float* dy,
                                                           int act, float slope, float* dpre,
                                                           float* __restrict__ part, int vec, float* dbias, int beta) {
  const int o = blockIdx.y, sl = blockIdx.x;
  const long long total = (long long)N * ppp;
  const long long p0 = total * sl / slices, p1 = total * (sl + 1) / slices;
  float acc = 0.0f;
  for (long long p = p0; p < p1; ++p) {
    const int n = (int)(p / ppp), piece = (int)(p - (long long)n * ppp);
    const size_t base = ((size_t)n * O + o) * HW + (size_t)piece * kEpiPiece;
    const int len = HW - piece * kEpiPiece < kEpiPiece ? HW - piece * kEpiPiece : kEpiPiece;
    if (vec) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e = (h * 256 + threadIdx.x) * 4;
        if (e < len) {
          f32x4 g = *reinterpret_cast<const f32x4*>(dy + base + e);
          if (act == LNN_ACT_LEAKY_RELU) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(y + base + e);
#pragma unroll
            for (int c = 0; c < 4; ++c) g[c] *= v[c] >= 0.0f ? 1.0f : slope;
          }
          if (dpre) *reinterpret_cast<f32x4*>(dpre + base + e) = g;
          acc += (g[0] + g[1]) + (g[2] + g[3]);
        }
      }
    } else {
      for (int e = threadIdx.x; e < len; e += 256) {
        float g = dy[base + e];
        if (act == LNN_ACT_LEAKY_RELU) g *= y[base + e] >= 0.0f ? 1.0f : slope;
        if (dpre) dpre[base + e] = g;
        acc += g;
      }
    }
  }
  if (!part && !dbias) return;
  __shared__ float red[4];
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) acc += __shfl_xor(acc, s, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x != 0) return;
  const float sum = (red[0] + red[1]) + (red[2] + red[3]);
  if (dbias) dbias[o] = beta ? dbias[o] + sum : sum;   // the channel's only slice: no partial sums to add up
  else part[(size_t)o * slices + sl] = sum;
}

// The same for planes of one element, a dense layer's y[rows][O]: a thread owns a feature and walks down its
// slice of the rows (consecutive threads read consecutive floats of a row).
__global__ __launch_bounds__(256) void bias_act_bwd_rows_kernel(int N, int O, int slices, const float* __restrict__ y,
                                                                const float* dy, int act, float slope, float* dpre,
                                                                float* __restrict__ part) {
  const int o = blockIdx.x * 256 + threadIdx.x, sl = blockIdx.y;
  if (o >= O) return;
  const int r0 = (int)((long long)N * sl / slices), r1 = (int)((long long)N * (sl + 1) / slices);
  float acc = 0.0f;
  for (int r = r0; r < r1; ++r) {
    const size_t e = (size_t)r * O + o;
    float g = dy[e];
    if (act == LNN_ACT_LEAKY_RELU) g *= y[e] >= 0.0f ? 1.0f : slope;
    if (dpre) dpre[e] = g;
    acc += g;
  }
  if (part) part[(size_t)sl * O + o] = acc;   // [slice][feature]: the finishing kernel's threads read side by side
}

// dbias[o] (+)= the slices' sums of channel o, in slice order; element (o, s) lies at part[o * so + s * ss]
__global__ void bias_act_bwd_finish_kernel(int O, int slices, const float* __restrict__ part, float* __restrict__ dbias,
                                           int beta, int so, int ss) {
  const int o = blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= O) return;
  float v = 0.0f;
  for (int s = 0; s < slices; ++s) v += part[(size_t)o * so + (size_t)s * ss];
  dbias[o] = beta ? dbias[o] + v : v;
}

int launch_bias_act_bwd(DeviceCtx* ctx, int N, int O, int HW, const float* y, const float* dy, int act, float slope,
                        float* dpre, float* dbias, int beta) {
  if (N <= 0 || O <= 0 || HW <= 0) return set_error(LNN_ERR_INVALID, "bias_act_bwd: non-positive dimension");
  if (act != LNN_ACT_NONE && act != LNN_ACT_LEAKY_RELU) return set_error(LNN_ERR_INVALID, "bias_act_bwd: unknown activation");
  if (!dy || (act != LNN_ACT_NONE && !y)) return set_error(LNN_ERR_INVALID, "bias_act_bwd: null pointer");
  if (!dpre && !dbias) return set_error(LNN_ERR_INVALID, "bias_act_bwd: nothing to compute");
  if ((uint64_t)N * O * HW * 4 > kMaxTensorBytes) return set_error(LNN_ERR_UNSUPPORTED, "bias_act_bwd: a tensor of 2 GiB or more");
  if (HW == 1) {
    const int blocks = (O + 255) / 256;
    long long sl = ((long long)ctx->cus * 4 + blocks - 1) / blocks;
    if (sl > N) sl = N;
    if (sl > 64) sl = 64;
    float* part1 = nullptr;
    if (dbias) {
      int st = ensure_workspace(ctx, (size_t)O * sl * sizeof(float));
      if (st != LNN_OK) return st;
      part1 = static_cast<float*>(ctx->ws);
    }
    hipLaunchKernelGGL(bias_act_bwd_rows_kernel, dim3((unsigned)blocks, (unsigned)sl), dim3(256), 0, ctx->stream, N, O, (int)sl, y,
                       dy, act, slope, dpre, part1);
    LNN_HIP(hipGetLastError());
    if (dbias) {
      hipLaunchKernelGGL(bias_act_bwd_finish_kernel, dim3((O + 255) / 256), dim3(256), 0, ctx->stream, O, (int)sl, part1,
                         dbias, beta ? 1 : 0, 1, O);
      LNN_HIP(hipGetLastError());
    }
    return LNN_OK;
  }
  if (O > 65535) return set_error(LNN_ERR_UNSUPPORTED, "bias_act_bwd: more than 65535 channels");
  const int ppp = (HW + kEpiPiece - 1) / kEpiPiece;
  const long long total = (long long)N * ppp;
  long long slices = ((long long)ctx->cus * 8 + O - 1) / O;
  if (slices > total) slices = total;
  // a block per channel already fills the device and a channel is short: the block stores the bias gradient itself
  if (O >= ctx->cus && (long long)N * HW <= 8192) slices = 1;
  if (slices < 1) slices = 1;
  const bool direct = dbias && slices == 1;
  float* part = nullptr;
  if (dbias && !direct) {
    int st = ensure_workspace(ctx, (size_t)O * slices * sizeof(float));
    if (st != LNN_OK) return st;
    part = static_cast<float*>(ctx->ws);
  }
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const int vec = HW % 4 == 0 && aligned(dy) && aligned(y) && aligned(dpre);
  hipLaunchKernelGGL(bias_act_bwd_kernel, dim3((unsigned)slices, (unsigned)O), dim3(256), 0, ctx->stream, N, O, HW, ppp,
                     (int)slices, y, dy, act, slope, dpre, part, vec, direct ? dbias : nullptr, beta ? 1 : 0);
  LNN_HIP(hipGetLastError());
  if (dbias && !direct) {
    hipLaunchKernelGGL(bias_act_bwd_finish_kernel, dim3((O + 255) / 256), dim3(256), 0, ctx->stream, O, (int)slices, part,
                       dbias, beta ? 1 : 0, (int)slices, 1);
    LNN_HIP(hipGetLastError());
  }
  return LNN_OK;
}

// ---- on-device random initialisers ------------------------------------------------------------------------
// The reference fills a fresh parameter tensor on the device from a counter hash: element i draws from
// hash(i + seed), seed a host-side 31-bit integer (initializer/RandomUniform.py:13-27, RandomNormal.py:10-30).
// The two PCG hashes follow the reference's device helper text (CLKernelHelper.py:210-228); unsigned 32-bit
// arithmetic throughout, so the integer stream is reproducible bit for bit.
__device__ __forceinline__ uint32_t hash_u32(uint32_t v) {
  const uint32_t state = v * 747796405u + 2891336453u;
  const uint32_t word = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
  return (word >> 22u) ^ word;
}
__device__ __forceinline__ void hash_u32x2(uint32_t& x, uint32_t& y) {
  x = x * 1664525u + 1013904223u;
  y = y * 1664525u + 1013904223u;
  x += y * 1664525u;
  y += x * 1664525u;
  x ^= x >> 16u;
  y ^= y >> 16u;
  x += y * 1664525u;
  y += x * 1664525u;
  x ^= x >> 16u;
  y ^= y >> 16u;
}
// (float)h * 2^-32: the reference multiplies by 1.0 / (float)0xffffffffU, and (float)0xffffffffU rounds to 2^32
constexpr float kUnitScale = 1.0f / 4294967296.0f;

// out[i] = u * (high - low) + low (RandomUniform.py:17-21).  The reference builds every kernel with
// -cl-single-precision-constant (CLDevice.py:93), so low and high are float literals there and the whole expression
// is single precision: span = (float)high - (float)low is rounded once, and the multiply-add is contracted into one
// fused operation, which OpenCL C permits by default and GPU compilers do.
__global__ void random_uniform_kernel(float* __restrict__ out, uint64_t n, uint32_t seed, float span, float low) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
    const float u = (float)hash_u32((uint32_t)(i + seed)) * kUnitScale;
    out[i] = __builtin_fmaf(u, span, low);
  }
}
// Box-Muller on the two halves of the 2-D hash of (i + seed, 1) (RandomNormal.py:14-24), all in single precision:
// sqrt(-2*log(x)) * cos((2*PI_F)*y), then mean + normal*stddev with float mean / stddev as one fused multiply-add
__global__ void random_normal_kernel(float* __restrict__ out, uint64_t n, uint32_t seed, float mean, float stddev) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) {
    uint32_t x = (uint32_t)(i + seed), y = 1u;
    hash_u32x2(x, y);
    const float fx = (float)x * kUnitScale, fy = (float)y * kUnitScale;
    const float normal = sqrtf(-2.0f * logf(fx)) * cosf((2.0f * 3.14159274101257f) * fy);
    out[i] = __builtin_fmaf(normal, stddev, mean);
  }
}

int launch_random_uniform(DeviceCtx* ctx, float* out, uint64_t n, uint32_t seed, double low, double high) {
  if (n == 0) return LNN_OK;
  if (!out) return set_error(LNN_ERR_INVALID, "random_uniform: null pointer");
  hipLaunchKernelGGL(random_uniform_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, out, n, seed, (float)high - (float)low, (float)low);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

int launch_random_normal(DeviceCtx* ctx, float* out, uint64_t n, uint32_t seed, double mean, double stddev) {
  if (n == 0) return LNN_OK;
  if (!out) return set_error(LNN_ERR_INVALID, "random_normal: null pointer");
  hipLaunchKernelGGL(random_normal_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, out, n, seed, (float)mean, (float)stddev);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

// kind 0: SGD (p0 momentum, p1 unused, flag nesterov), kind 1: Adam (p0 beta1, p1 beta2)
// wp / wp_c / wp_kk / wp_layout (all null, or arrays of count; wp_layout may be null = all LNN_W_OIHW): tensor i's
// permuted copy Wp[o][tap][c] or null, its C and KH*KW, and how the tensor itself is stored
int launch_update_multi(DeviceCtx* ctx, int kind, int count, const uint64_t* n, float* const* t, const float* const* g,
                        float* const* s0, float* const* s1, float p0, float p1, float lr, int flag, float* const* wp,
                        const int32_t* wp_c, const int32_t* wp_kk, const int32_t* wp_layout, float drop,
                        const uint32_t* seeds) {
  const char* who = kind ? "adam_update_multi" : "sgd_update_multi";
  if (count < 0) return set_error(LNN_ERR_INVALID, std::string(who) + ": negative count");
  if (count == 0) return LNN_OK;
  if (!n || !t || !g || !s0 || (kind && !s1)) return set_error(LNN_ERR_INVALID, std::string(who) + ": null array");
  if (!(drop >= 0.0f && drop <= 1.0f)) return set_error(LNN_ERR_INVALID, std::string(who) + ": lr_dropout outside [0, 1]");
  if (drop != 0.0f && !seeds) return set_error(LNN_ERR_INVALID, std::string(who) + ": lr_dropout needs seeds");
  const int per = kind ? 1 : 2;   // seeds per tensor: SGD's two kernels, Adam's one
  for (int i0 = 0; i0 < count; i0 += kMultiMax) {
    const int nb = count - i0 < kMultiMax ? count - i0 : kMultiMax;
    MultiArgs a = {};
    uint64_t most = 0;
    for (int i = 0; i < nb; ++i) {
      a.n[i] = n[i0 + i];
      a.t[i] = t[i0 + i]; a.g[i] = g[i0 + i]; a.s0[i] = s0[i0 + i]; a.s1[i] = kind ? s1[i0 + i] : nullptr;
      if (a.n[i] && (!a.t[i] || !a.g[i] || !a.s0[i] || (kind && !a.s1[i])))
        return set_error(LNN_ERR_INVALID, std::string(who) + ": null pointer");
      most = a.n[i] > most ? a.n[i] : most;
      a.dKK[i] = a.dIn[i] = FastDiv{0, 0, 1};
      a.wp_c[i] = 0;
      a.seed0[i] = seeds ? seeds[per * (i0 + i)] : 0u;
      a.seed1[i] = (seeds && per == 2) ? seeds[per * (i0 + i) + 1] : 0u;
      if (wp && wp[i0 + i] && a.n[i]) {
        if (!wp_c || !wp_kk || wp_c[i0 + i] <= 0 || wp_kk[i0 + i] <= 0 || a.n[i] % ((uint64_t)wp_c[i0 + i] * wp_kk[i0 + i]) != 0 ||
            a.n[i] > 0x7fffffffull)
          return set_error(LNN_ERR_INVALID, std::string(who) + ": a permuted copy whose channel and tap counts do not divide the tensor");
        const int layout = wp_layout ? wp_layout[i0 + i] : LNN_W_OIHW;
        if (layout != LNN_W_OIHW && layout != LNN_W_IOHW) return set_error(LNN_ERR_INVALID, std::string(who) + ": unknown weight layout");
        const uint32_t C = (uint32_t)wp_c[i0 + i], O = (uint32_t)(a.n[i] / ((uint64_t)C * wp_kk[i0 + i]));
        a.wp[i] = wp[i0 + i];
        a.dKK[i] = make_fastdiv((uint32_t)wp_kk[i0 + i]);
        a.dIn[i] = make_fastdiv(layout == LNN_W_OIHW ? C : O);
        a.wp_c[i] = layout == LNN_W_OIHW ? (int)C : -(int)C;
      }
    }
    if (most == 0) continue;
    const dim3 grid(grid_for(most, ctx->cus / 2).x, (unsigned)nb);
    if (kind) hipLaunchKernelGGL(adam_multi_kernel, grid, dim3(256), 0, ctx->stream, a, p0, p1, lr, drop);
    else hipLaunchKernelGGL(sgd_multi_kernel, grid, dim3(256), 0, ctx->stream, a, p0, lr, flag ? 1 : 0, drop);
    LNN_HIP(hipGetLastError());
  }
  return LNN_OK;
}

int launch_adam(DeviceCtx* ctx, uint64_t n, float* t, const float* g, float* m, float* v2, float beta1, float beta2,
                float lr) {
  if (n == 0) return LNN_OK;
  if (!t || !g || !m || !v2) return set_error(LNN_ERR_INVALID, "adam_update: null pointer");
  hipLaunchKernelGGL(adam_kernel, grid_for(n, ctx->cus), dim3(256), 0, ctx->stream, n, t, g, m, v2, beta1, beta2, lr);
  LNN_HIP(hipGetLastError());
  return LNN_OK;
}

}  // namespace lnn
