/* C ABI of liblitenn_hip.so: the MI355X (gfx950) device layer behind LiteNN's
 * operator API for nn.conv2D / nn.matmul and their backward passes.
 *
 * It takes the place of the 26 OpenCL entry points LiteNN binds through
 * ctypes (litenn/core/minicl/api/OpenCL/OpenCL.py:214-668) plus the kernels
 * LiteNN generates as OpenCL C text at run time.  Conventions:
 *   - every function returns an int status: 0 on success, negative on error;
 *     lnn_last_error() gives the message of the calling thread's last failure
 *     (the role of CLException/ERROR codes, OpenCL.py:175-198);
 *   - LNN_ERR_OOM is distinct so a caller-side buffer pool can evict and retry
 *     (CLDevice.py:134-164 does this on MEM_OBJECT_ALLOCATION_FAILURE);
 *   - pointers are raw device addresses owned by the caller; the library keeps
 *     no per-tensor state.  It owns, per device, one stream (all launches are
 *     asynchronous and in order, like the in-order command queue of
 *     CLDevice.py:186-190), a grow-only scratch buffer for split-K partial
 *     sums, and small cached gather tables keyed by convolution geometry;
 *   - all tensors are dense fp32; every tensor must be smaller than 2 GiB;
 *   - single-threaded callers per device; no callbacks.
 *   - `beta` is 0 (overwrite) or 1 (accumulate: out += result), the two forms
 *     LiteNN selects with is_add_to_output (matmul.py:162, unfold2D.py:110).
 */
#ifndef LITENN_HIP_H
#define LITENN_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LNN_OK 0
#define LNN_ERR_INVALID (-1)     /* bad argument (shape, alignment, null pointer) */
#define LNN_ERR_OOM (-2)         /* device allocation failed */
#define LNN_ERR_NO_DEVICE (-3)   /* no usable HIP device / bad device index */
#define LNN_ERR_HIP (-4)         /* any other HIP runtime failure */
#define LNN_ERR_UNSUPPORTED (-5) /* valid request outside the library's limits */

/* Message of the last failing call on this thread ("" if none). */
const char* lnn_last_error(void);

/* ---- devices: replaces clGetPlatformIDs/clGetDeviceIDs/clGetDeviceInfo
 *      (OpenCL.py:214-310) as used by devices.get_all (devices.py:88-105). */
int lnn_device_count(int* count);
int lnn_device_info(int dev, char* name, int name_cap, uint64_t* total_mem_bytes,
                    int* compute_units, int* clock_khz);
/* Frees the stream, scratch and cached tables of a device: the counterpart of
 * dropping the context/queue in CLDevice._cleanup (CLDevice.py:107-118). */
int lnn_release_device(int dev);

/* ---- memory: replaces clCreateBuffer / clReleaseMemObject and the
 *      clEnqueue{Write,Read,Copy,Fill}Buffer calls (OpenCL.py:376-456) behind
 *      CLDevice._mem_alloc (CLDevice.py:120-165) and CLBuffer.set/fill/np
 *      (CLBuffer.py:50-115). */
int lnn_malloc(int dev, uint64_t bytes, void** out);
int lnn_free(int dev, void* ptr);
int lnn_mem_info(int dev, uint64_t* free_bytes, uint64_t* total_bytes);
/* host -> device; returns after the host buffer may be reused (CLBuffer.py:78-80) */
int lnn_memcpy_h2d(int dev, void* dst, const void* src, uint64_t bytes);
/* device -> host; returns after the data has arrived (CLBuffer.py:112-113) */
int lnn_memcpy_d2h(int dev, void* dst, const void* src, uint64_t bytes);
/* device -> device on the device's stream, asynchronous (CLBuffer.py:66-67) */
int lnn_memcpy_d2d(int dev, void* dst, const void* src, uint64_t bytes);
/* fills `count` 32-bit words with `pattern` (CLBuffer.fill, CLBuffer.py:83-96) */
int lnn_fill_u32(int dev, void* dst, uint32_t pattern, uint64_t count);
/* waits for all work queued on the device: clFinish (CLDevice.py:51-55) */
int lnn_synchronize(int dev);

/* ---- timing on the device's stream (no counterpart in the reference, whose
 *      queue is created without profiling, OpenCL.py:349-351). */
int lnn_event_create(int dev, void** event);
int lnn_event_record(int dev, void* event);
int lnn_event_elapsed_ms(int dev, void* start, void* stop, float* ms); /* waits for `stop` */
int lnn_event_destroy(int dev, void* event);

/* ---- GEMM: replaces the generated "GeMM" kernel (matmul.py:127-164) and the
 *      transposes its gradients materialise (matmul.py:64-72).
 *   C[b] (+)= op(A[b]) * op(B[b]),  op(A) is M x K, op(B) is K x N, C is M x N,
 *   all row-major with leading dimensions lda/ldb/ldc (elements) and batch
 *   strides (elements).  trans_a: A is stored K x M.  trans_b: B is stored
 *   N x K.  nn.matmul forward is (0,0); dA = dC * B^T is (0,1); dB = A^T * dC
 *   is (1,0). */
int lnn_gemm_f32(int dev, int trans_a, int trans_b, int batch, int M, int N, int K,
                 const float* A, int lda, int64_t stride_a,
                 const float* B, int ldb, int64_t stride_b,
                 float* C, int ldc, int64_t stride_c, int beta);
/* C[b] = act(op(A[b]) * op(B[b]) + bias[n])   the product and the broadcast bias add that follows it in a dense
 * layer (module/Dense.py:44-48: nn.matmul(x, weight) + bias; dual_wise_op.py:110-130 for the broadcast operand),
 * and optionally the activation users put behind it (element_wise_op.py:208-222), in the product's only store:
 * bit-identical to the separate kernels.  bias holds N values, one per column of C (the same for every batch
 * item), or is NULL; act / slope as for lnn_conv2d_fwd_bias_act_f32 (declared below). */
int lnn_gemm_bias_act_f32(int dev, int trans_a, int trans_b, int batch, int M, int N, int K,
                          const float* A, int lda, int64_t stride_a,
                          const float* B, int ldb, int64_t stride_b,
                          const float* bias, int act, float slope,
                          float* C, int ldc, int64_t stride_c);

/* ---- convolution: replaces unfold2D + GeMM + transpose of conv2D.py:39-54.
 * Geometry as computed by InfoConv2D (InfoConv2D.py:41-77); only the left/top
 * pads enter the kernels (unfold2D.py:85-137).  X is [N,C,IH,IW], W is
 * [O,C,KH,KW], Y is [N,O,OH,OW], all NCHW row-major. */
typedef struct lnn_conv2d_desc {
  int32_t N, C, IH, IW;
  int32_t O, KH, KW;
  int32_t OH, OW;
  int32_t PADL, PADT;
  int32_t stride, dilation;
} lnn_conv2d_desc;

/* Y (+)= conv(X, W)                      conv2D.py:39-42 */
int lnn_conv2d_fwd_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* W,
                       float* Y, int beta);
/* Y = act(conv(X, W) + bias[o])          the convolution, the bias add that follows it in every layer
 * (module/Conv2D.py:59-62: x + bias.reshape(1,-1,1,1), dual_wise_op.py:110-130) and the activation users
 * put after it (element_wise_op.py:208-222: leaky_relu O = I*(I>=0) + alpha*I*(I<0)) in one pass: the
 * epilogue adds bias[o] (bias may be NULL) and applies act to the fp32 accumulator before the only store,
 * which gives bit-identical results to the three separate kernels. */
#define LNN_ACT_NONE 0
#define LNN_ACT_LEAKY_RELU 1
int lnn_conv2d_fwd_bias_act_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* W,
                                const float* bias, int act, float slope, float* Y);
/* Backward of that epilogue in one pass over y and dy, both [N][O][HW] (the layer's bias add is
 * dual_wise_op.py:110-130 for the broadcast operand, the activation gradient element_wise_op.py:211):
 *   dpre = dy * (y >= 0 ? 1 : slope)       (act == LNN_ACT_LEAKY_RELU; slope > 0 so y has the sign of the
 *                                            pre-activation)   or   dpre = dy   (LNN_ACT_NONE, y unused)
 *   dbias[o] = (beta_bias ? dbias[o] : 0) + sum over n and pixels of dpre
 * dpre may be NULL (only the bias gradient is wanted) or equal dy (in place); dbias may be NULL. */
int lnn_bias_act_bwd_f32(int dev, int N, int O, int HW, const float* y, const float* dy, int act, float slope,
                         float* dpre, float* dbias, int beta_bias);
/* dX (+)= dgrad(dY, W)                   conv2D.py:46-50 (the reference always accumulates) */
int lnn_conv2d_dgrad_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* W,
                         float* dX, int beta);
/* Which kernel family lnn_conv2d_dgrad_f32 uses for a geometry on a device with `compute_units` compute units
 * (lnn_device_info reports them).  Host arithmetic only: works without a device.  No counterpart in the reference,
 * whose data gradient always runs unfold + GeMM + transposes (conv2D.py:46-50); it lets a caller, or a test, see
 * which code a shape exercises.  For LNN_DGRAD_PATH_VECTOR tile_info (7 values, may be NULL) receives the dY tile of
 * one block: rows and columns brought to LDS, the largest extent the kernel's LDS plane holds, and the smallest /
 * largest row and column any thread reads: {rows, cols, max_extent, min_row, min_col, max_row, max_col}. */
#define LNN_DGRAD_PATH_MFMA_TABLE 0 /* implicit GEMM on the matrix cores, K = (o, tap) through a gather table */
#define LNN_DGRAD_PATH_MFMA_TAP 1   /* implicit GEMM, tap-major K over channel-permuted weights (O % 32 == 0) */
#define LNN_DGRAD_PATH_VECTOR 2     /* C <= 4: vector-ALU kernel, all pixel classes of a 32 x 32 tile per block */
#define LNN_DGRAD_PATH_STEM_MFMA 3  /* C <= 4, stride 2, O a multiple of 8 from 32, kernels up to 8 x 8, at least two
                                       32 x 32-pixel tiles per compute unit: the 2 x 2 pixel parities as rows of a
                                       16-row GEMM over a dY patch in LDS */
int lnn_conv2d_dgrad_path(const lnn_conv2d_desc* d, int beta, int compute_units, int* path, int32_t* tile_info);
/* Which kernel family lnn_conv2d_fwd_f32 / lnn_conv2d_fwd_bias_act_f32 use for a geometry on a device with
 * `compute_units` compute units.  Host arithmetic only: works without a device.  No counterpart in the reference,
 * whose forward pass always runs unfold + GeMM (conv2D.py:39-42); it lets a caller, or a test, see which code a
 * shape exercises. */
#define LNN_FWD_PATH_IMPLICIT_GEMM 0 /* implicit GEMM on the matrix cores, operands gathered tile by tile */
#define LNN_FWD_PATH_STEM_PATCH 1    /* 3 input channels, 33-64 output channels, 3x3 / 5x5 / 7x7: MFMA operands read
                                        from an input patch in LDS (problems with at least 4 tiles per compute unit);
                                        lnn_conv2d_wgrad_f32 takes the matching kernel for such a geometry when
                                        OW % 4 == 0 and dY is 16-byte aligned */
int lnn_conv2d_fwd_path(const lnn_conv2d_desc* d, int compute_units, int* path);
/* dW (+)= wgrad(X, dY)                   conv2D.py:52-54 (the reference always accumulates) */
int lnn_conv2d_wgrad_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY,
                         float* dW, int beta);
/* How the most recent weight gradient on `dev` (any of its entry points) was laid out on the chip:
 * info = {workgroups of the main kernel, K slices (1: none; 2 with equal runs), 1 if the K steps of all sub-tiles
 * were dealt out in equal runs that cross sub-tile borders, rows of a tile}; all 0 after an image-stem kernel.
 * No counterpart in the reference (one GeMM launch per gradient, matmul.py:127-164); for tests and tuning. */
int lnn_conv2d_wgrad_last_plan(int dev, int32_t* info);

/* ---- weights kept in the kernels' own layout.  The kernels for channel counts that are multiples of 32 read the
 * weights as Wp[o][kh*KW + kw][c]; lnn_conv2d_fwd_f32 / lnn_conv2d_dgrad_f32 make that copy in scratch on every
 * call.  A caller that knows when its weights change (once per optimizer step) makes the copy once with
 * lnn_conv2d_permute_weights_f32 and hands it to the *_pw entry points: forward and data gradient then share it.
 * The reference has the same need and no such cache: conv2D_dI_gradfn transposes the kernel to (O, KH, KW, C) on
 * every backward pass (conv2D.py:48), and conv2DTranspose swaps the kernel's channel axes in every pass
 * (conv2DTranspose.py:33-47).  w_layout LNN_W_IOHW reads weights stored [C][O][KH][KW] - how a transposed
 * convolution, whose passes are this convolution's passes with the roles swapped, keeps its kernel - so that no
 * swapped copy is needed; lnn_conv2d_wgrad_iohw_f32 writes the weight gradient in that layout.
 * lnn_conv2d_weights_plan (host arithmetic, no device needed) says for pass LNN_PASS_FWD / LNN_PASS_DGRAD whether
 * the geometry's kernels read Wp (only then may the *_pw entry point be used), and for LNN_PASS_WGRAD whether
 * lnn_conv2d_wgrad_iohw_f32 serves it.  Wp holds O*C*KH*KW floats and must be 16-byte aligned; for a 1x1 kernel
 * stored OIHW the weights themselves are a valid Wp. */
#define LNN_W_OIHW 0
#define LNN_W_IOHW 1
#define LNN_PASS_FWD 0
#define LNN_PASS_DGRAD 1
#define LNN_PASS_WGRAD 2
int lnn_conv2d_weights_plan(const lnn_conv2d_desc* d, int pass, int* yes);
int lnn_conv2d_permute_weights_f32(int dev, const lnn_conv2d_desc* d, const float* W, int w_layout, float* Wp);
/* Y (+)= act(conv(X, W) + bias)   with W given as Wp; bias may be NULL; bias / act need beta == 0 */
int lnn_conv2d_fwd_pw_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* Wp, const float* bias,
                          int act, float slope, float* Y, int beta);
/* dX (+)= dgrad(dY, W)            with W given as Wp */
int lnn_conv2d_dgrad_pw_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* Wp, float* dX, int beta);
/* dW[c][o][kh][kw] (+)= wgrad(X, dY)[o][c][kh][kw] */
int lnn_conv2d_wgrad_iohw_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY, float* dW,
                              int beta);

/* The same computation as lnn_conv2d_wgrad_f32, bit for bit, without any device allocation.  It has no counterpart
 * in the reference (whose buffers all come from clCreateBuffer at run time); it is for callers that cannot call
 * hipMalloc: code under HIP graph capture, tight serving or training loops, harnesses that forbid allocation.
 * The split-K partial sums (and the gather table of geometries whose channel count does not fill the pixel-major
 * tiles) live in a fixed device array of LNN_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until
 * the process ends.  A problem that needs more returns LNN_ERR_UNSUPPORTED and launches nothing; on a 256-CU
 * device the partial sums never exceed 32 MiB, so only the added table of an unusually shaped problem can.
 * The one-time set-up of a device (stream, address of the array) happens in the first call of ANY entry point on
 * that device; after it this function calls no hipMalloc / hipFree or other allocating routine.  All calls on one
 * GPU share the array: calls that overlap in time on one GPU (from two threads) race.  For its duration the call
 * also points the device's scratch bookkeeping at the array and forbids allocation on that device, so it must not
 * overlap with ANY other entry point of this library on the same GPU either: one running beside it from a second
 * thread could fail with LNN_ERR_UNSUPPORTED or place its own scratch data in the array. */
#define LNN_NOALLOC_SCRATCH_BYTES (32u << 20)
int lnn_conv2d_wgrad_noalloc_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY,
                                 float* dW, int beta);

/* ---- depthwise convolution (one KH x KW filter per channel; K is [C,KH,KW], desc.O must equal desc.C).
 * Y (+)= depthwise(X, K)                 depthwise_conv2D.py:74-96  (O_depthwise_krn)
 * dX (+)= its data gradient              depthwise_conv2D.py:98-124 (dI_depthwise_krn; the reference always accumulates)
 * dK (+)= sum over n,oh,ow of im2col(X) * dY   depthwise_conv2D.py:44-49 (unfold, broadcast multiply, reduce_sum) */
int lnn_depthwise_conv2d_fwd_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* K,
                                 float* Y, int beta);
int lnn_depthwise_conv2d_dgrad_f32(int dev, const lnn_conv2d_desc* d, const float* dY, const float* K,
                                   float* dX, int beta);
int lnn_depthwise_conv2d_wgrad_f32(int dev, const lnn_conv2d_desc* d, const float* X, const float* dY,
                                   float* dK, int beta);

/* ---- nc.op.unfold2D (unfold2D.py:6-48): materialised im2col / im2row /
 * transposed im2row.  Shares its index arithmetic with the gather loaders of
 * the convolution kernels and exists so that arithmetic can be checked bit for
 * bit.  order 0 = 'CJI_NHW', 1 = 'NHW_CJI'.  Arguments as in the reference
 * call: (H, W) source size, (OH, OW) extent of the H/W output symbols. */
int lnn_unfold2d_f32(int dev, int N, int C, int H, int W, int OH, int OW, int KH, int KW,
                     int PADL, int PADT, int dilation, int stride, int order, int is_transpose,
                     const float* in, float* out, int beta);

/* ---- nc.op.transpose (transpose.py:60-103): out[perm(idx)] (+)= in[idx],
 * rank <= 8, out shape = shape[axes]. */
int lnn_transpose_f32(int dev, int rank, const int32_t* shape, const int32_t* axes,
                      const float* in, float* out, int beta);

/* ---- pointwise / reduction helpers the training step of a conv net needs
 * around the hot path (element_wise_op.py:83-110, dual_wise_op.py:132-191,
 * reduce.py:166-301, SGD.py:42-74). */
enum {
  LNN_EW_ADD_CONST = 0,  /* out = in + p0                      element_wise_op.py:122-130 */
  LNN_EW_MUL_CONST = 1,  /* out = in * p0 */
  LNN_EW_LEAKY_RELU = 2, /* out = in >= 0 ? in : p0*in         element_wise_op.py:208-222 */
  LNN_EW_SQUARE = 3,     /* out = in*in                        element_wise_op.py:331-344 */
  LNN_EW_RELU = 4
};
/* out (+)= f(in) */
int lnn_ew_fwd_f32(int dev, int op, uint64_t n, const float* in, float* out, float p0, int beta);
/* din (+)= f'(in) * dout.  The reference always accumulates (element_wise_op.py:108) into a gradient that
 * starts as zeros; beta = 0 is that first contribution without the zero fill and the read. */
int lnn_ew_bwd_f32(int dev, int op, uint64_t n, const float* in, const float* dout, float* din,
                   float p0, int beta);
/* out (+)= a (op) b with numpy broadcasting; shapes already left-padded with
 * ones to `rank` <= 8 (dual_wise_op.py:138-152).  op: 0 add, 1 sub, 2 mul. */
int lnn_binary_bcast_f32(int dev, int op, int rank, const int32_t* out_shape,
                         const int32_t* a_shape, const int32_t* b_shape, const float* a,
                         const float* b, float* out, int beta);
/* out[kept axes] (+)= scale * sum over reduced axes of in; reduce_mask bit i
 * set = axis i is summed.  rank <= 8. */
int lnn_reduce_sum_f32(int dev, int rank, const int32_t* shape, uint32_t reduce_mask,
                       float scale, const float* in, float* out, int beta);
/* din[idx] (+)= scale * dout[idx with reduced axes set to 0]   (reduce.py:243-255; beta as above) */
int lnn_reduce_sum_bwd_f32(int dev, int rank, const int32_t* shape, uint32_t reduce_mask,
                           float scale, const float* dout, float* din, int beta);
/* SGD.py:42-74: acc = momentum*acc - lr*g;  v += nesterov ? momentum*acc - lr*g : acc */
int lnn_sgd_update_f32(int dev, uint64_t n, float* v, const float* g, float* acc, float momentum,
                       float lr, int nesterov);
/* Adam step as the reference writes it (optimizer/Adam.py:43-72, three kernels there, no bias correction):
 *   m = beta1*m + (1-beta1)*g;  v = beta2*v + (1-beta2)*g*g;  t += -lr*m / (sqrt(v) + 1e-7) */
int lnn_adam_update_f32(int dev, uint64_t n, float* t, const float* g, float* m, float* v,
                        float beta1, float beta2, float lr);

/* The same two updates for `count` tensors in one launch (an optimizer step over a model's parameters,
 * Optimizer.py:117-147 walks them one by one).  n, v/t, g, acc/m, v: host arrays of `count` element counts and
 * device pointers; tensors with n[i] == 0 are skipped. */
int lnn_sgd_update_multi_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g,
                             float* const* acc, float momentum, float lr, int nesterov);
int lnn_adam_update_multi_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g,
                              float* const* m, float* const* v, float beta1, float beta2, float lr);
/* The same, for a caller that keeps permuted copies of its convolution kernels (lnn_conv2d_permute_weights_f32):
 * wp[i] is tensor i's copy Wp[o][tap][c] or NULL, wp_c[i] / wp_kk[i] its C and KH*KW, wp_layout[i] how the tensor
 * itself is stored (LNN_W_OIHW, or LNN_W_IOHW for the kernel of a transposed convolution; wp_layout NULL = all
 * LNN_W_OIHW).  The update stores every new value in the copy as well, so the copy stays valid across the optimizer
 * step and the next forward pass needs no permutation launch.  No counterpart in the reference
 * (Optimizer.py:117-147 updates tensor by tensor; conv2D_dI_gradfn re-transposes the kernel in every backward pass,
 * conv2D.py:48, conv2DTranspose swaps its channel axes in every pass, conv2DTranspose.py:33-47). */
int lnn_sgd_update_multi_wp_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g,
                                float* const* acc, float momentum, float lr, int nesterov, float* const* wp,
                                const int32_t* wp_c, const int32_t* wp_kk, const int32_t* wp_layout);
int lnn_adam_update_multi_wp_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g,
                                 float* const* m, float* const* v, float beta1, float beta2, float lr, float* const* wp,
                                 const int32_t* wp_c, const int32_t* wp_kk, const int32_t* wp_layout);

/* The same two multi-tensor updates with learning-rate dropout (Optimizer.py:186-203): inside each of the reference's
 * update kernels element gid of a tensor takes lr = 0 where hash_float_uint(gid + seed) <= lr_dropout, the seed a
 * fresh np.random.randint(2^31) per kernel launch (Optimizer.py:178-182), the hash the counter hash of the device
 * initialisers below.  seeds: SGD two per tensor - {accumulator kernel, value kernel} (SGD.py:42-74; the second
 * matters with nesterov only) - Adam one per tensor (Adam.py:61-72); lr_dropout == 0 ignores them (may be NULL).
 * wp .. wp_layout as above, all NULL for tensors without permuted copies. */
int lnn_sgd_update_multi_lrd_f32(int dev, int count, const uint64_t* n, float* const* v, const float* const* g,
                                 float* const* acc, float momentum, float lr, int nesterov, float lr_dropout,
                                 const uint32_t* seeds, float* const* wp, const int32_t* wp_c, const int32_t* wp_kk,
                                 const int32_t* wp_layout);
int lnn_adam_update_multi_lrd_f32(int dev, int count, const uint64_t* n, float* const* t, const float* const* g,
                                  float* const* m, float* const* v, float beta1, float beta2, float lr, float lr_dropout,
                                  const uint32_t* seeds, float* const* wp, const int32_t* wp_c, const int32_t* wp_kk,
                                  const int32_t* wp_layout);

/* On-device random initialisers: element i is drawn from a counter hash of (uint32)(i + seed), so a tensor
 * is filled in place without host staging (initializer/RandomUniform.py:13-27, RandomNormal.py:10-30; the PCG
 * hashes of CLKernelHelper.py:210-228).  The reference draws seed = np.random.randint(2^31) on the host.
 *   uniform: out[i] = u*(high-low) + low,           u = (float)hash(i+seed) * 2^-32   (can equal high)
 *   normal : out[i] = mean + stddev * sqrt(-2 ln u0) * cos(2 pi u1),  (u0,u1) = 2-D hash of (i+seed, 1) * 2^-32
 * Both affine maps are single precision, one fused multiply-add on (float)low, (float)high - (float)low resp.
 * (float)mean, (float)stddev: the reference compiles its kernels with -cl-single-precision-constant
 * (minicl/CLDevice.py:93), so the bounds it formats into the kernel text are float literals there.
 * He / Glorot initialisers are these two with derived bounds (initializer/He.py:18-33, Glorot.py:20-35). */
int lnn_random_uniform_f32(int dev, float* out, uint64_t n, uint32_t seed, double low, double high);
int lnn_random_normal_f32(int dev, float* out, uint64_t n, uint32_t seed, double mean, double stddev);

#ifdef __cplusplus
}
#endif
#endif /* LITENN_HIP_H */
