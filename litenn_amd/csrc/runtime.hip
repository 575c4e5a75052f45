// Device contexts, memory, events and the extern "C" entry points.
#include <mutex>

#include "common.hpp"

namespace lnn {

int launch_fill_u32(DeviceCtx*, void*, uint32_t, uint64_t);
int launch_ew_fwd(DeviceCtx*, int, uint64_t, const float*, float*, float, int);
int launch_ew_bwd(DeviceCtx*, int, uint64_t, const float*, const float*, float*, float, int);
int launch_binary_bcast(DeviceCtx*, int, int, const int32_t*, const int32_t*, const int32_t*, const float*,
                        const float*, float*, int);
int launch_reduce_sum(DeviceCtx*, int, const int32_t*, uint32_t, float, const float*, float*, int);
int launch_reduce_sum_bwd(DeviceCtx*, int, const int32_t*, uint32_t, float, const float*, float*, int);
int launch_transpose(DeviceCtx*, int, const int32_t*, const int32_t*, const float*, float*, int);
int launch_unfold2d(DeviceCtx*, int, int, int, int, int, int, int, int, int, int, int, int, int, int, const float*,
                    float*, int);
int launch_sgd(DeviceCtx*, uint64_t, float*, const float*, float*, float, float, int);
int launch_adam(DeviceCtx*, uint64_t, float*, const float*, float*, float*, float, float, float);
int launch_random_uniform(DeviceCtx*, float*, uint64_t, uint32_t, double, double);
int launch_update_multi(DeviceCtx*, int, int, const uint64_t*, float* const*, const float* const*, float* const*, float* const*,
                        float, float, float, int, float* const*, const int32_t*, const int32_t*, const int32_t*, float = 0.0f,
                        const uint32_t* = nullptr);
int launch_bias_act_bwd(DeviceCtx*, int, int, int, const float*, const float*, int, float, float*, float*, int);
int launch_random_normal(DeviceCtx*, float*, uint64_t, uint32_t, double, double);

// Scratch of the allocation-free entry point (lnn_conv2d_wgrad_noalloc_f32): split-K partial sums and, for
// geometries that need one, the gather table.  Every GPU the library runs on holds its own copy of this array
// from the time the code object is loaded until the process ends.  In host code the name `scratch` is only a
// handle for hipGetSymbolAddress; the device address kept in DeviceCtx::static_ws is what kernels receive.
constexpr size_t kStaticScratchBytes = LNN_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

static thread_local std::string g_error;
constexpr int kMaxDevices = 64;
static DeviceCtx g_ctx[kMaxDevices];
static std::mutex g_mutex;

int set_error(int code, const std::string& msg) {
  g_error = msg;
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  (void)hipGetLastError();   // clear the sticky error so later calls are judged on their own
  const int code = e == hipErrorOutOfMemory ? LNN_ERR_OOM
                   : (e == hipErrorNoDevice || e == hipErrorInvalidDevice) ? LNN_ERR_NO_DEVICE
                                                                            : LNN_ERR_HIP;
  return set_error(code, std::string(what) + ": " + hipGetErrorString(e));
}

static int device_count_raw(int* n) {
  // the number of devices of a process does not change once it has been read successfully
  static int known = -1;
  if (known > 0) {
    *n = known;
    return LNN_OK;
  }
  hipError_t e = hipGetDeviceCount(n);
  if (e == hipSuccess && *n > 0) known = *n;
  if (e == hipErrorNoDevice) {
    (void)hipGetLastError();
    *n = 0;
    return LNN_OK;
  }
  if (e != hipSuccess) {
    *n = 0;
    return hip_fail(e, "hipGetDeviceCount");
  }
  return LNN_OK;
}

DeviceCtx* get_ctx(int dev, int* status) {
  int n = 0;
  *status = device_count_raw(&n);
  if (*status != LNN_OK) return nullptr;
  if (dev < 0 || dev >= n || dev >= kMaxDevices) {
    *status = set_error(LNN_ERR_NO_DEVICE, "no HIP device with index " + std::to_string(dev));
    return nullptr;
  }
  hipError_t e = hipSetDevice(dev);
  if (e != hipSuccess) {
    *status = hip_fail(e, "hipSetDevice");
    return nullptr;
  }
  DeviceCtx* c = &g_ctx[dev];
  if (!c->ready) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!c->ready) {
      hipDeviceProp_t prop;
      e = hipGetDeviceProperties(&prop, dev);
      if (e != hipSuccess) {
        *status = hip_fail(e, "hipGetDeviceProperties");
        return nullptr;
      }
      if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0) {
        *status = set_error(LNN_ERR_NO_DEVICE, std::string("device is ") + prop.gcnArchName +
                                                   "; this library contains gfx950 code only");
        return nullptr;
      }
      e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
      if (e != hipSuccess) {
        *status = hip_fail(e, "hipStreamCreateWithFlags");
        return nullptr;
      }
      // device `dev` is current here: its copy of the scratch array
      void* sp = nullptr;
      e = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));
      if (e != hipSuccess || sp == nullptr) {
        (void)hipStreamDestroy(c->stream);
        c->stream = nullptr;
        *status = e != hipSuccess ? hip_fail(e, "hipGetSymbolAddress(scratch)")
                                  : set_error(LNN_ERR_HIP, "hipGetSymbolAddress(scratch) returned a null address");
        return nullptr;
      }
      c->static_ws = sp;
      c->index = dev;
      c->cus = prop.multiProcessorCount;
      c->ready = true;
    }
  }
  *status = LNN_OK;
  return c;
}

int ensure_workspace(DeviceCtx* ctx, size_t bytes) {
  if (bytes <= ctx->ws_bytes) return LNN_OK;
  if (ctx->no_alloc)
    return set_error(LNN_ERR_UNSUPPORTED, "this problem needs " + std::to_string(bytes) + " bytes of scratch; the allocation-free "
                     "entry point has " + std::to_string(ctx->ws_bytes) + " (use the allocating entry point)");
  // earlier launches may still read the old buffer
  LNN_HIP(hipStreamSynchronize(ctx->stream));
  if (ctx->ws) {
    (void)hipFree(ctx->ws);
    ctx->ws = nullptr;
    ctx->ws_bytes = 0;
  }
  const size_t want = (bytes + (bytes >> 2) + 0xfffff) & ~(size_t)0xfffff;
  hipError_t e = hipMalloc(&ctx->ws, want);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    return set_error(LNN_ERR_OOM, "out of device memory for " + std::to_string(want) + " bytes of scratch");
  }
  LNN_HIP(e);
  ctx->ws_bytes = want;
  return LNN_OK;
}

}  // namespace lnn

using namespace lnn;

#define CTX(dev)                     \
  int st_ = LNN_OK;                  \
  DeviceCtx* ctx = get_ctx(dev, &st_); \
  if (!ctx) return st_;

static int check_count(uint64_t n, const char* who) {
  if (n * 4 > kMaxTensorBytes) return set_error(LNN_ERR_UNSUPPORTED, std::string(who) + ": tensor of 2 GiB or more");
  return LNN_OK;
}

extern "C" {

const char* lnn_last_error(void) { return g_error.c_str(); }

int lnn_device_count(int* count) {
  if (!count) return set_error(LNN_ERR_INVALID, "device_count: null pointer");
  return device_count_raw(count);
}

int lnn_device_info(int dev, char* name, int name_cap, uint64_t* total_mem_bytes, int* compute_units, int* clock_khz) {
  int n = 0, st = device_count_raw(&n);
  if (st != LNN_OK) return st;
  if (dev < 0 || dev >= n) return set_error(LNN_ERR_NO_DEVICE, "no HIP device with index " + std::to_string(dev));
  hipDeviceProp_t prop;
  LNN_HIP(hipGetDeviceProperties(&prop, dev));
  if (name && name_cap > 0) {
    std::string s = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    snprintf(name, (size_t)name_cap, "%s", s.c_str());
  }
  if (total_mem_bytes) *total_mem_bytes = prop.totalGlobalMem;
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (clock_khz) *clock_khz = prop.clockRate;
  return LNN_OK;
}

int lnn_release_device(int dev) {
  if (dev < 0 || dev >= kMaxDevices) return set_error(LNN_ERR_NO_DEVICE, "bad device index");
  DeviceCtx* c = &g_ctx[dev];
  if (!c->ready) return LNN_OK;
  LNN_HIP(hipSetDevice(dev));
  LNN_HIP(hipStreamSynchronize(c->stream));
  for (auto& kv : c->tables) (void)hipFree(kv.second);
  c->tables.clear();
  if (c->ws) (void)hipFree(c->ws);
  c->ws = nullptr;
  c->ws_bytes = 0;
  (void)hipStreamDestroy(c->stream);
  c->stream = nullptr;
  c->ready = false;
  return LNN_OK;
}

int lnn_malloc(int dev, uint64_t bytes, void** out) {
  if (!out || bytes == 0) return set_error(LNN_ERR_INVALID, "malloc: null result pointer or zero size");
  CTX(dev);
  *out = nullptr;
  hipError_t e = hipMalloc(out, bytes);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    return set_error(LNN_ERR_OOM, "out of device memory allocating " + std::to_string(bytes) + " bytes");
  }
  LNN_HIP(e);
  return LNN_OK;
}

int lnn_free(int dev, void* ptr) {
  if (!ptr) return LNN_OK;
  CTX(dev);
  // queued kernels may still use the buffer: hipFree waits for the device
  LNN_HIP(hipFree(ptr));
  return LNN_OK;
}

int lnn_mem_info(int dev, uint64_t* free_bytes, uint64_t* total_bytes) {
  CTX(dev);
  size_t f = 0, t = 0;
  LNN_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return LNN_OK;
}

int lnn_memcpy_h2d(int dev, void* dst, const void* src, uint64_t bytes) {
  if (bytes == 0) return LNN_OK;
  if (!dst || !src) return set_error(LNN_ERR_INVALID, "memcpy_h2d: null pointer");
  CTX(dev);
  LNN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  LNN_HIP(hipStreamSynchronize(ctx->stream));
  return LNN_OK;
}

int lnn_memcpy_d2h(int dev, void* dst, const void* src, uint64_t bytes) {
  if (bytes == 0) return LNN_OK;
  if (!dst || !src) return set_error(LNN_ERR_INVALID, "memcpy_d2h: null pointer");
  CTX(dev);
  LNN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  LNN_HIP(hipStreamSynchronize(ctx->stream));
  return LNN_OK;
}

int lnn_memcpy_d2d(int dev, void* dst, const void* src, uint64_t bytes) {
  if (bytes == 0) return LNN_OK;
  if (!dst || !src) return set_error(LNN_ERR_INVALID, "memcpy_d2d: null pointer");
  CTX(dev);
  LNN_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return LNN_OK;
}

int lnn_fill_u32(int dev, void* dst, uint32_t pattern, uint64_t count) {
  if (count == 0) return LNN_OK;
  if (!dst) return set_error(LNN_ERR_INVALID, "fill_u32: null pointer");
  CTX(dev);
  return launch_fill_u32(ctx, dst, pattern, count);
}

int lnn_synchronize(int dev) {
  CTX(dev);
  LNN_HIP(hipStreamSynchronize(ctx->stream));
  return LNN_OK;
}

int lnn_event_create(int dev, void** event) {
  if (!event) return set_error(LNN_ERR_INVALID, "event_create: null pointer");
  CTX(dev);
  hipEvent_t ev;
  LNN_HIP(hipEventCreate(&ev));
  *event = ev;
  return LNN_OK;
}

int lnn_event_record(int dev, void* event) {
  if (!event) return set_error(LNN_ERR_INVALID, "event_record: null event");
  CTX(dev);
  LNN_HIP(hipEventRecord(static_cast<hipEvent_t>(event), ctx->stream));
  return LNN_OK;
}

int lnn_event_elapsed_ms(int dev, void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return set_error(LNN_ERR_INVALID, "event_elapsed_ms: null pointer");
  CTX(dev);
  LNN_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  LNN_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return LNN_OK;
}

int lnn_event_destroy(int dev, void* event) {
  if (!event) return LNN_OK;
  CTX(dev);
  LNN_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return LNN_OK;
}

int lnn_gemm_f32(int dev, int trans_a, int trans_b, int batch, int M, int N, int K, const float* A, int lda,
                 int64_t stride_a, const float* B, int ldb, int64_t stride_b, float* C, int ldc, int64_t stride_c,
                 int beta) {
  CTX(dev);
  return launch_gemm(ctx, trans_a, trans_b, batch, M, N, K, A, lda, stride_a, B, ldb, stride_b, C, ldc, stride_c, beta);
}

int lnn_gemm_bias_act_f32(int dev, int trans_a, int trans_b, int batch, int M, int N, int K, const float* A, int lda,
                          int64_t stride_a, const float* B, int ldb, int64_t stride_b, const float* bias, int act,
                          float slope, float* C, int ldc, int64_t stride_c) {
  CTX(dev);
  if (act != LNN_ACT_NONE && act != LNN_ACT_LEAKY_RELU) return set_error(LNN_ERR_INVALID, "gemm_bias_act: unknown activation");
  return launch_gemm(ctx, trans_a, trans_b, batch, M, N, K, A, lda, stride_a, B, ldb, stride_b, C, ldc, stride_c, 0, bias,
                     act, slope);
}

int lnn_conv2d_fwd_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta) {
  CTX(dev);
  return launch_conv_fwd(ctx, d, X, W, Y, beta, nullptr, 0, 0.0f);
}

int lnn_conv2d_fwd_bias_act_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* W, const float* bias,
                                int act, float slope, float* Y) {
  CTX(dev);
  if (act != LNN_ACT_NONE && act != LNN_ACT_LEAKY_RELU) return set_error(LNN_ERR_INVALID, "conv2d_fwd_bias_act: unknown activation");
  return launch_conv_fwd(ctx, d, X, W, Y, 0, bias, act, slope);
}

int lnn_depthwise_conv2d_fwd_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* K, float* Y, int beta) {
  CTX(dev);
  return launch_dw_fwd(ctx, d, X, K, Y, beta);
}

int lnn_depthwise_conv2d_dgrad_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* K, float* dX,
                                   int beta) {
  CTX(dev);
  return launch_dw_dgrad(ctx, d, dY, K, dX, beta);
}

int lnn_depthwise_conv2d_wgrad_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dK,
                                   int beta) {
  CTX(dev);
  return launch_dw_wgrad(ctx, d, X, dY, dK, beta);
}

int lnn_conv2d_dgrad_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* W, float* dX, int beta) {
  CTX(dev);
  return launch_conv_dgrad(ctx, d, dY, W, dX, beta);
}

int lnn_conv2d_weights_plan(const lnn_conv2d_desc* d, int pass, int* yes) { return conv_weights_plan(d, pass, yes); }

int lnn_conv2d_permute_weights_f32(int dev, const lnn_conv2d_desc* d, const float* W, int w_layout, float* Wp) {
  CTX(dev);
  return launch_permute_weights(ctx, d, W, w_layout, Wp);
}

int lnn_conv2d_fwd_pw_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* Wp, const float* bias, int act,
                          float slope, float* Y, int beta) {
  CTX(dev);
  if (!Wp) return set_error(LNN_ERR_INVALID, "conv2d_fwd_pw: null pointer");
  if (act != LNN_ACT_NONE && act != LNN_ACT_LEAKY_RELU) return set_error(LNN_ERR_INVALID, "conv2d_fwd_pw: unknown activation");
  return launch_conv_fwd(ctx, d, X, nullptr, Y, beta, bias, act, slope, Wp);
}

int lnn_conv2d_dgrad_pw_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* Wp, float* dX, int beta) {
  CTX(dev);
  if (!Wp) return set_error(LNN_ERR_INVALID, "conv2d_dgrad_pw: null pointer");
  return launch_conv_dgrad(ctx, d, dY, nullptr, dX, beta, Wp);
}

int lnn_conv2d_wgrad_iohw_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta) {
  CTX(dev);
  return launch_conv_wgrad(ctx, d, X, dY, dW, beta, 1);
}

int lnn_conv2d_fwd_path(const lnn_conv2d_desc* d, int compute_units, int* path) {
  return conv_fwd_path(d, compute_units, path);
}

int lnn_conv2d_dgrad_path(const lnn_conv2d_desc* d, int beta, int compute_units, int* path, int32_t* tile_info) {
  return conv_dgrad_path(d, beta, compute_units, path, tile_info);
}

int lnn_conv2d_wgrad_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta) {
  CTX(dev);
  return launch_conv_wgrad(ctx, d, X, dY, dW, beta);
}

int lnn_conv2d_wgrad_last_plan(int dev, int32_t* info) {
  CTX(dev);
  if (!info) return set_error(LNN_ERR_INVALID, "conv2d_wgrad_last_plan: null pointer");
  for (int i = 0; i < 4; ++i) info[i] = ctx->last_wgrad_plan[i];
  return LNN_OK;
}

namespace {
// For the duration of one call the device's scratch is the fixed array (single-threaded callers per device).
struct FixedScratch {
  DeviceCtx* c;
  void* ws;
  size_t bytes;
  explicit FixedScratch(DeviceCtx* ctx) : c(ctx), ws(ctx->ws), bytes(ctx->ws_bytes) {
    c->ws = c->static_ws;
    c->ws_bytes = kStaticScratchBytes;
    c->no_alloc = true;
  }
  ~FixedScratch() {
    c->ws = ws;
    c->ws_bytes = bytes;
    c->no_alloc = false;
  }
};
}  // namespace

int lnn_conv2d_wgrad_noalloc_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta) {
  CTX(dev);
  FixedScratch fixed(ctx);
  return launch_conv_wgrad(ctx, d, X, dY, dW, beta);
}

int lnn_unfold2d_f32(int dev, int N, int C, int H, int W, int OH, int OW, int KH, int KW, int PADL, int PADT,
                     int dilation, int stride, int order, int is_transpose, const float* in, float* out, int beta) {
  if (!in || !out) return set_error(LNN_ERR_INVALID, "unfold2d: null pointer");
  if (N > 0 && C > 0 && OH > 0 && OW > 0 && KH > 0 && KW > 0) {
    int st = check_count((uint64_t)N * C * OH * OW * KH * KW, "unfold2d");
    if (st != LNN_OK) return st;
  }
  CTX(dev);
  return launch_unfold2d(ctx, N, C, H, W, OH, OW, KH, KW, PADL, PADT, dilation, stride, order, is_transpose, in, out,
                         beta);
}

int lnn_transpose_f32(int dev, int rank, const int32_t* shape, const int32_t* axes, const float* in, float* out,
                      int beta) {
  if (!shape || !axes || !in || !out) return set_error(LNN_ERR_INVALID, "transpose: null pointer");
  CTX(dev);
  return launch_transpose(ctx, rank, shape, axes, in, out, beta);
}

int lnn_ew_fwd_f32(int dev, int op, uint64_t n, const float* in, float* out, float p0, int beta) {
  if (n && (!in || !out)) return set_error(LNN_ERR_INVALID, "ew_fwd: null pointer");
  int st = check_count(n, "ew_fwd");
  if (st != LNN_OK) return st;
  CTX(dev);
  return launch_ew_fwd(ctx, op, n, in, out, p0, beta);
}

int lnn_ew_bwd_f32(int dev, int op, uint64_t n, const float* in, const float* dout, float* din, float p0, int beta) {
  if (n && (!in || !dout || !din)) return set_error(LNN_ERR_INVALID, "ew_bwd: null pointer");
  int st = check_count(n, "ew_bwd");
  if (st != LNN_OK) return st;
  CTX(dev);
  return launch_ew_bwd(ctx, op, n, in, dout, din, p0, beta);
}

int lnn_binary_bcast_f32(int dev, int op, int rank, const int32_t* out_shape, const int32_t* a_shape,
                         const int32_t* b_shape, const float* a, const float* b, float* out, int beta) {
  if (!out_shape || !a_shape || !b_shape || !a || !b || !out) return set_error(LNN_ERR_INVALID, "binary_bcast: null pointer");
  CTX(dev);
  return launch_binary_bcast(ctx, op, rank, out_shape, a_shape, b_shape, a, b, out, beta);
}

int lnn_reduce_sum_f32(int dev, int rank, const int32_t* shape, uint32_t reduce_mask, float scale, const float* in,
                       float* out, int beta) {
  if (!shape || !in || !out) return set_error(LNN_ERR_INVALID, "reduce_sum: null pointer");
  CTX(dev);
  return launch_reduce_sum(ctx, rank, shape, reduce_mask, scale, in, out, beta);
}

int lnn_reduce_sum_bwd_f32(int dev, int rank, const int32_t* shape, uint32_t reduce_mask, float scale,
                           const float* dout, float* din, int beta) {
  if (!shape || !dout || !din) return set_error(LNN_ERR_INVALID, "reduce_sum_bwd: null pointer");
  CTX(dev);
  return launch_reduce_sum_bwd(ctx, rank, shape, reduce_mask, scale, dout, din, beta);
}

int lnn_sgd_update_f32(int dev, uint64_t n, float* v, const float* g, float* acc, float momentum, float lr,
                       int nesterov) {
  if (n && (!v || !g || !acc)) return set_error(LNN_ERR_INVALID, "sgd_update: null pointer");
  CTX(dev);
  return launch_sgd(ctx, n, v, g, acc, momentum, lr, nesterov);
}

int lnn_adam_update_f32(int dev, uint64_t n, float* t, const float* g, float* m, float* v, float beta1, float beta2,
                        float lr) {
  CTX(dev);
  return launch_adam(ctx, n, t, g, m, v, beta1, beta2, lr);
}

int lnn_sgd_update_multi_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g, float* const* acc,
                             float momentum, float lr, int nesterov) {
  CTX(dev);
  return launch_update_multi(ctx, 0, count, n, v, g, acc, nullptr, momentum, 0.0f, lr, nesterov, nullptr, nullptr, nullptr, nullptr);
}

int lnn_sgd_update_multi_wp_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g,
                                float* const* acc, float momentum, float lr, int nesterov, float* const* wp,
                                const int32_t* wp_c, const int32_t* wp_kk, const int32_t* wp_layout) {
  CTX(dev);
  return launch_update_multi(ctx, 0, count, n, v, g, acc, nullptr, momentum, 0.0f, lr, nesterov, wp, wp_c, wp_kk, wp_layout);
}

int lnn_adam_update_multi_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g, float* const* m,
                              float* const* v, float beta1, float beta2, float lr) {
  CTX(dev);
  return launch_update_multi(ctx, 1, count, n, t, g, m, v, beta1, beta2, lr, 0, nullptr, nullptr, nullptr, nullptr);
}

int lnn_adam_update_multi_wp_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g,
                                 float* const* m, float* const* v, float beta1, float beta2, float lr, float* const* wp,
                                 const int32_t* wp_c, const int32_t* wp_kk, const int32_t* wp_layout) {
  CTX(dev);
  return launch_update_multi(ctx, 1, count, n, t, g, m, v, beta1, beta2, lr, 0, wp, wp_c, wp_kk, wp_layout);
}

int lnn_sgd_update_multi_lrd_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g,
                                 float* const* acc, float momentum, float lr, int nesterov, float lr_dropout,
                                 const uint32_t* seeds, float* const* wp, const int32_t* wp_c, const int32_t* wp_kk,
                                 const int32_t* wp_layout) {
  CTX(dev);
  return launch_update_multi(ctx, 0, count, n, v, g, acc, nullptr, momentum, 0.0f, lr, nesterov, wp, wp_c, wp_kk, wp_layout,
                             lr_dropout, seeds);
}

int lnn_adam_update_multi_lrd_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g,
                                  float* const* m, float* const* v, float beta1, float beta2, float lr, float lr_dropout,
                                  const uint32_t* seeds, float* const* wp, const int32_t* wp_c, const int32_t* wp_kk,
                                  const int32_t* wp_layout) {
  CTX(dev);
  return launch_update_multi(ctx, 1, count, n, t, g, m, v, beta1, beta2, lr, 0, wp, wp_c, wp_kk, wp_layout, lr_dropout, seeds);
}

int lnn_bias_act_bwd_f32(int dev, int N, int O, int HW, const float* y, const float* dy, int act, float slope,
                         float* dpre, float* dbias, int beta_bias) {
  CTX(dev);
  return launch_bias_act_bwd(ctx, N, O, HW, y, dy, act, slope, dpre, dbias, beta_bias);
}

int lnn_random_uniform_f32(int dev, float* out, uint64_t n, uint32_t seed, double low, double high) {
  CTX(dev);
  return launch_random_uniform(ctx, out, n, seed, low, high);
}

int lnn_random_normal_f32(int dev, float* out, uint64_t n, uint32_t seed, double mean, double stddev) {
  CTX(dev);
  return launch_random_normal(ctx, out, n, seed, mean, stddev);
}

}  // extern "C"
