/* CPU restatement (fp32) of the reference's conv2D / matmul data flow.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests as a second checker (fp32, with the
 * reference's own summation order) and by the benchmark as the timed CPU
 * baseline.  Nothing in the shipped package links or loads this file.
 *
 * The reference runs every step below as an OpenCL kernel with one work-item
 * per output element (or per register tile); here each work-item is one
 * iteration of an OpenMP-parallel loop, which is how a CPU OpenCL driver
 * would execute it.  Citations are relative to the litenn source tree.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int ref_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* Tensor.py:236-237,264 + initializer/Scalar.py:11-12: every new tensor is
 * zero-filled when its buffer is first touched. */
static float* new_zero_tensor(size_t n) {
  float* p = (float*)malloc(n * sizeof(float) + 64);
  if (!p) return NULL;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < (int64_t)n; ++i) p[i] = 0.0f;
  return p;
}

/* op/unfold2D.py:93-110 (is_transpose = 0) and :121-137 (is_transpose = 1).
 * order 0 = 'CJI_NHW', order 1 = 'NHW_CJI'.  gid is decomposed last-axis
 * fastest (CLKernelHelper.py:91-132); the output index equals gid.
 * Argument names follow the kernel text: (H, W) is the *source* image size,
 * (OH, OW) the size the H/W output symbols run over. */
void ref_unfold2d(float* O, const float* I, int N, int C, int H, int W, int OH, int OW,
                  int KH, int KW, int PADL, int PADT, int DIL, int STRIDE,
                  int order, int is_transpose, int add) {
  const int64_t total = (int64_t)N * C * OH * OW * KH * KW;
#pragma omp parallel for schedule(static)
  for (int64_t gid = 0; gid < total; ++gid) {
    int64_t g = gid;
    int on, oc, oh, ow, oj, oi;
    if (order == 0) { /* C J I N H W */
      ow = (int)(g % OW); g /= OW;
      oh = (int)(g % OH); g /= OH;
      on = (int)(g % N);  g /= N;
      oi = (int)(g % KW); g /= KW;
      oj = (int)(g % KH); g /= KH;
      oc = (int)g;
    } else {          /* N H W C J I */
      oi = (int)(g % KW); g /= KW;
      oj = (int)(g % KH); g /= KH;
      oc = (int)(g % C);  g /= C;
      ow = (int)(g % OW); g /= OW;
      oh = (int)(g % OH); g /= OH;
      on = (int)g;
    }
    float value = 0.0f;
    if (!is_transpose) {
      int ih = -PADT + oj * DIL + oh * STRIDE;
      if (ih >= 0 && ih < H) {
        int iw = -PADL + oi * DIL + ow * STRIDE;
        if (iw >= 0 && iw < W) value = I[(((int64_t)on * C + oc) * H + ih) * W + iw];
      }
    } else {
      /* unsigned division in the kernel; a negative numerator there yields a
       * value that fails the range/equality tests, same as rejecting it here */
      int nh = PADT + oh - oj * DIL;
      if (nh >= 0) {
        int ih = nh / STRIDE;
        if (ih < H && oh == -PADT + oj * DIL + ih * STRIDE) {
          int nw = PADL + ow - oi * DIL;
          if (nw >= 0) {
            int iw = nw / STRIDE;
            if (iw < W && ow == -PADL + oi * DIL + iw * STRIDE)
              value = I[(((int64_t)on * C + oc) * H + ih) * W + iw];
          }
        }
      }
    }
    if (add) O[gid] += value; else O[gid] = value;
  }
}

/* op/transpose.py:97-103: O[perm(idx)] (+)= I[gid], rank <= 6. */
void ref_transpose(float* O, const float* I, int rank, const int* shape, const int* axes, int add) {
  int64_t total = 1, ostride_for_in_axis[6], oshape[6], ostrides[6];
  for (int a = 0; a < rank; ++a) total *= shape[a];
  for (int a = 0; a < rank; ++a) oshape[a] = shape[axes[a]];
  ostrides[rank - 1] = 1;
  for (int a = rank - 2; a >= 0; --a) ostrides[a] = ostrides[a + 1] * oshape[a + 1];
  for (int a = 0; a < rank; ++a) ostride_for_in_axis[axes[a]] = ostrides[a];
#pragma omp parallel for schedule(static)
  for (int64_t gid = 0; gid < total; ++gid) {
    int64_t g = gid, o = 0;
    for (int a = rank - 1; a >= 0; --a) {
      int64_t x = (a == 0) ? g : g % shape[a];
      g /= shape[a];
      o += x * ostride_for_in_axis[a];
    }
    if (add) O[o] += I[gid]; else O[o] = I[gid];
  }
}

/* op/matmul.py:127-164, column-major naming: A is [BATCH][K][M], B is
 * [BATCH][N][K], C is [BATCH][N][M].  One work-item = one NW x MW register
 * tile; accumulation order kt (outer), k, n, m (inner), fp32. */
#define GEMM_BODY(MW, KW)                                                                    \
  static void gemm_##MW##_##KW(const float* A, const float* B, float* C, int BATCH, int M,    \
                               int N, int K, int add) {                                       \
    enum { NW = KW };                                                                         \
    const int MT = M / MW, KT = K / KW, NT = N / NW;                                          \
    const int64_t items = (int64_t)MT * NT * BATCH;                                           \
    _Pragma("omp parallel for schedule(static)")                                              \
    for (int64_t it = 0; it < items; ++it) {                                                  \
      const int mt = (int)(it % MT);                                                          \
      const int nc = (int)((it / MT) % NT);                                                   \
      const int batch = (int)(it / ((int64_t)MT * NT));                                       \
      float AT[KW][MW], BT[NW][KW], CT[NW][MW];                                               \
      for (int i = 0; i < NW * MW; ++i) ((float*)CT)[i] = 0.0f;                               \
      for (int kt = 0; kt < KT; ++kt) {                                                       \
        for (int k = 0; k < KW; ++k)                                                          \
          memcpy(AT[k], A + ((int64_t)batch * K * MT + (int64_t)(kt * KW + k) * MT + mt) * MW, \
                 sizeof(float) * MW);                                                         \
        for (int n = 0; n < NW; ++n)                                                          \
          memcpy(BT[n], B + ((int64_t)batch * N * KT + (int64_t)(nc * NW + n) * KT + kt) * KW, \
                 sizeof(float) * KW);                                                         \
        for (int k = 0; k < KW; ++k)                                                          \
          for (int n = 0; n < NW; ++n)                                                        \
            for (int m = 0; m < MW; ++m) CT[n][m] += AT[k][m] * BT[n][k];                     \
      }                                                                                       \
      for (int n = 0; n < NW; ++n) {                                                          \
        float* c = C + ((int64_t)batch * N * MT + (int64_t)(nc * NW + n) * MT + mt) * MW;     \
        if (add) for (int m = 0; m < MW; ++m) c[m] += CT[n][m];                               \
        else     for (int m = 0; m < MW; ++m) c[m] = CT[n][m];                                \
      }                                                                                       \
    }                                                                                         \
  }

#define GEMM_FOR_MW(MW) GEMM_BODY(MW, 8) GEMM_BODY(MW, 4) GEMM_BODY(MW, 2) GEMM_BODY(MW, 1)
GEMM_FOR_MW(16) GEMM_FOR_MW(8) GEMM_FOR_MW(4) GEMM_FOR_MW(2) GEMM_FOR_MW(1)

typedef void (*gemm_fn)(const float*, const float*, float*, int, int, int, int, int);

/* Tile widths chosen exactly as op/matmul.py:106-113. */
void ref_gemm_tile_widths(int M, int N, int K, int* MW, int* KW) {
  static const int mws[] = {16, 8, 4, 2, 1}, kws[] = {8, 4, 2, 1};
  for (int i = 0; i < 5; ++i) if (M % mws[i] == 0) { *MW = mws[i]; break; }
  for (int i = 0; i < 4; ++i) if (N % kws[i] == 0 && K % kws[i] == 0) { *KW = kws[i]; break; }
}

void ref_gemmc(const float* A, const float* B, float* C, int BATCH, int M, int N, int K, int add) {
  static const gemm_fn table[5][4] = {
      {gemm_16_8, gemm_16_4, gemm_16_2, gemm_16_1}, {gemm_8_8, gemm_8_4, gemm_8_2, gemm_8_1},
      {gemm_4_8, gemm_4_4, gemm_4_2, gemm_4_1},     {gemm_2_8, gemm_2_4, gemm_2_2, gemm_2_1},
      {gemm_1_8, gemm_1_4, gemm_1_2, gemm_1_1}};
  int MW = 1, KW = 1;
  ref_gemm_tile_widths(M, N, K, &MW, &KW);
  int mi = MW == 16 ? 0 : MW == 8 ? 1 : MW == 4 ? 2 : MW == 2 ? 3 : 4;
  int ki = KW == 8 ? 0 : KW == 4 ? 1 : KW == 2 ? 2 : 3;
  table[mi][ki](A, B, C, BATCH, M, N, K, add);
}

/* Row-major user view, op/matmul.py:8-30: matmul(A_u[M,K], B_u[K,N]) runs the
 * column-major kernel with A := B_u, B := A_u. */
void ref_matmul(const float* A_u, const float* B_u, float* C_u, int BATCH, int M, int K, int N, int add) {
  ref_gemmc(B_u, A_u, C_u, BATCH, /*M=*/N, /*N=*/M, K, add);
}

/* op/matmul.py:64-72: each gradient first materialises a transposed operand
 * with the transpose kernel, then runs the GeMM with '+='. */
int ref_matmul_bwd(const float* A_u, const float* B_u, const float* dC, float* dA, float* dB,
                   int BATCH, int M, int K, int N) {
  int sh[3], ax[3] = {0, 2, 1};
  /* dB += A^T . dC : transpose user A [B,M,K] -> [B,K,M] */
  float* At = new_zero_tensor((size_t)BATCH * M * K);
  float* Bt = new_zero_tensor((size_t)BATCH * K * N);
  if (!At || !Bt) { free(At); free(Bt); return -1; }
  sh[0] = BATCH; sh[1] = M; sh[2] = K;
  ref_transpose(At, A_u, 3, sh, ax, 0);
  ref_matmul(At, dC, dB, BATCH, K, M, N, 1);
  /* dA += dC . B^T : transpose user B [B,K,N] -> [B,N,K] */
  sh[1] = K; sh[2] = N;
  ref_transpose(Bt, B_u, 3, sh, ax, 0);
  ref_matmul(dC, Bt, dA, BATCH, M, N, K, 1);
  free(At); free(Bt);
  return 0;
}

/* op/conv2D.py:39-42.  Y must hold N*O*OH*OW floats; it is overwritten. */
int ref_conv2d_fwd(const float* X, const float* W, float* Y, int N, int C, int IH, int IW, int O,
                   int KH, int KW, int OH, int OW, int PADL, int PADT, int STRIDE, int DIL) {
  const int64_t CKK = (int64_t)C * KH * KW, P = (int64_t)N * OH * OW;
  float* col = new_zero_tensor((size_t)(CKK * P));
  float* out = new_zero_tensor((size_t)((int64_t)O * P));
  if (!col || !out) { free(col); free(out); return -1; }
  ref_unfold2d(col, X, N, C, IH, IW, OH, OW, KH, KW, PADL, PADT, DIL, STRIDE, 0, 0, 0);
  ref_matmul(W, col, out, 1, O, (int)CKK, (int)P, 0);
  int sh[4] = {O, N, OH, OW}, ax[4] = {1, 0, 2, 3};
  ref_transpose(Y, out, 4, sh, ax, 0);
  free(col); free(out);
  return 0;
}

/* op/conv2D.py:46-50.  dX is accumulated into. */
int ref_conv2d_dx(const float* dY, const float* W, float* dX, int N, int C, int IH, int IW, int O,
                  int KH, int KW, int OH, int OW, int PADL, int PADT, int STRIDE, int DIL) {
  const int64_t OKK = (int64_t)O * KH * KW, Q = (int64_t)N * IH * IW;
  float* wt = new_zero_tensor((size_t)(OKK * C));
  float* rowT = new_zero_tensor((size_t)(Q * OKK));
  float* dI = new_zero_tensor((size_t)(Q * C));
  if (!wt || !rowT || !dI) { free(wt); free(rowT); free(dI); return -1; }
  int shw[4] = {O, C, KH, KW}, axw[4] = {0, 2, 3, 1};
  ref_transpose(wt, W, 4, shw, axw, 0);
  ref_unfold2d(rowT, dY, N, O, OH, OW, IH, IW, KH, KW, PADL, PADT, DIL, STRIDE, 1, 1, 0);
  ref_matmul(rowT, wt, dI, 1, (int)Q, (int)OKK, C, 0);
  int shi[4] = {N, IH, IW, C}, axi[4] = {0, 3, 1, 2};
  ref_transpose(dX, dI, 4, shi, axi, 1);
  free(wt); free(rowT); free(dI);
  return 0;
}

/* op/conv2D.py:52-54.  dW is accumulated into. */
int ref_conv2d_dw(const float* X, const float* dY, float* dW, int N, int C, int IH, int IW, int O,
                  int KH, int KW, int OH, int OW, int PADL, int PADT, int STRIDE, int DIL) {
  const int64_t CKK = (int64_t)C * KH * KW, P = (int64_t)N * OH * OW;
  float* dyt = new_zero_tensor((size_t)((int64_t)O * P));
  float* row = new_zero_tensor((size_t)(P * CKK));
  if (!dyt || !row) { free(dyt); free(row); return -1; }
  int sh[4] = {N, O, OH, OW}, ax[4] = {1, 0, 2, 3};
  ref_transpose(dyt, dY, 4, sh, ax, 0);
  ref_unfold2d(row, X, N, C, IH, IW, OH, OW, KH, KW, PADL, PADT, DIL, STRIDE, 1, 0, 0);
  ref_matmul(dyt, row, dW, 1, O, (int)P, (int)CKK, 1);
  free(dyt); free(row);
  return 0;
}
