// Shared host-side declarations of the HIP library (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <array>
#include <map>
#include <string>
#include <vector>

#include "../../include/litenn_hip.h"
#include "tile_engine.hpp"

namespace lnn {

struct DeviceCtx {
  int index = -1;
  bool ready = false;
  hipStream_t stream = nullptr;
  int cus = 0;
  // grow-only scratch owned by the library (split-K partial sums)
  void* ws = nullptr;
  size_t ws_bytes = 0;
  // gather tables, one per (geometry, kind)
  std::map<std::array<int, 16>, KEntry*> tables;
  // this device's copy of the library's fixed scratch array (device address, looked up once per device)
  void* static_ws = nullptr;
  // true while an allocation-free entry point runs: ws / ws_bytes then describe the fixed array, requests that do
  // not fit fail instead of allocating, and gather tables are carved from its tail instead of being cached
  bool no_alloc = false;
  // the plan of the most recent weight-gradient launch: {workgroups of the main kernel, K slices (1: none),
  // 1 if the K steps were dealt out in equal runs across chunk borders, rows of its tiles}
  int last_wgrad_plan[4] = {0, 0, 0, 0};
};

int set_error(int code, const std::string& msg);
int hip_fail(hipError_t e, const char* what);
DeviceCtx* get_ctx(int dev, int* status);          // makes dev current, creates the stream
int ensure_workspace(DeviceCtx* ctx, size_t bytes);

#define LNN_HIP(call)                                   \
  do {                                                  \
    hipError_t e_ = (call);                             \
    if (e_ != hipSuccess) return hip_fail(e_, #call);   \
  } while (0)

constexpr uint64_t kMaxTensorBytes = 0x7fffffffull;   // raw buffer descriptors address < 2 GiB

// launchers implemented in the kernel translation units
int launch_gemm(DeviceCtx* ctx, int ta, int tb, int batch, int M, int N, int K, const float* A, int lda,
                long long sA, const float* B, int ldb, long long sB, float* C, int ldc, long long sC, int beta,
                const float* bias = nullptr, int act = 0, float slope = 0.0f);   // bias: one value per column of C
// Wp: the weights in the permuted layout (made by launch_permute_weights), or null; W may be null when Wp is given
int launch_conv_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta,
                    const float* bias, int act, float slope, const float* Wp = nullptr);
// image stems (3 input channels, 33-64 output channels, 3x3 / 5x5 / 7x7, enough tiles): forward from an input patch in LDS
bool stem_fwd_applies(const lnn_conv2d_desc* d, int compute_units);
int launch_stem_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* W, float* Y, int beta,
                    const float* bias, int act, float slope);
bool stem_wgrad_applies(const lnn_conv2d_desc* d, int compute_units, const float* dY);
int launch_stem_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta);
bool stem_dgrad_applies(const lnn_conv2d_desc* d, int compute_units);
int launch_stem_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* W, float* dX, int beta);
int conv_fwd_path(const lnn_conv2d_desc* d, int compute_units, int* path);
int conv_weights_plan(const lnn_conv2d_desc* d, int pass, int* yes);
int launch_permute_weights(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* W, int w_layout, float* Wp);
int launch_dw_fwd(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* K, float* Y, int beta);
int launch_dw_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* K, float* dX, int beta);
int launch_dw_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dK, int beta);
int launch_conv_dgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* dY, const float* W, float* dX, int beta,
                      const float* Wp = nullptr);
int conv_dgrad_path(const lnn_conv2d_desc* d, int beta, int compute_units, int* path, int32_t* tile_info);
int launch_conv_wgrad(DeviceCtx* ctx, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW, int beta,
                      int w_iohw = 0);

}  // namespace lnn
