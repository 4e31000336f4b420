// Plain tiled matrix product with 32-bit FMA accumulation, for every storage
// type pair.  out[n, o] = sum_k A[n, k] * W[o, k] (+ bias[o]) with an optional
// GELU-tanh or residual-add epilogue: y = x W^T + b as nn.Linear
// (reference: src/minigpt_infer/model.py:43-44,96-101).
//
// This is the kernel of the true 32-bit path: k runs 0..K-1 in order for every
// output element, so a row's result does not depend on which other rows share
// the launch.  The bfloat16 serving path uses it only for shapes the MFMA
// kernels refuse.
#include "common.h"
#include "launchers.h"

#define EPI_NONE 0
#define EPI_GELU 1
#define EPI_RESIDUAL 2  // out (float) += result

#define TILE 64
#define BK 16
#define PAD 4

template <typename AT, typename WT, typename OT, int EPI>
__global__ __launch_bounds__(256) void linear_generic_kernel(
    const AT* __restrict__ A, long lda, const WT* __restrict__ W, const float* __restrict__ bias,
    OT* __restrict__ out, long ldo, int n_rows, int n_out, int k_dim) {
  __shared__ float As[BK][TILE + PAD];
  __shared__ float Ws[BK][TILE + PAD];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int row0 = blockIdx.y * TILE, col0 = blockIdx.x * TILE;
  const int lrow = tid >> 2, lk = (tid & 3) * 4;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const int arow = row0 + lrow, wrow = col0 + lrow;
  const bool a_ok = arow < n_rows, w_ok = wrow < n_out;
  const AT* ap = A + (long)arow * lda + lk;
  const WT* wp = W + (long)wrow * k_dim + lk;

  for (int k0 = 0; k0 < k_dim; k0 += BK) {
    // an inner size that is no multiple of the stage ends in zeros: fma(0, 0, acc) leaves acc as it is
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool k_ok = k0 + lk + i < k_dim;
      As[lk + i][lrow] = (a_ok && k_ok) ? to_float<AT>(ap[k0 + i]) : 0.f;
      Ws[lk + i][lrow] = (w_ok && k_ok) ? to_float<WT>(wp[k0 + i]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int r = row0 + ty * 4 + i;
    if (r >= n_rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int c = col0 + tx * 4 + j;
      if (c >= n_out) continue;
      float v = acc[i][j];
      if (bias) v += bias[c];
      if (EPI == EPI_GELU) v = gelu_tanh(v);
      OT* dst = out + (long)r * ldo + c;
      if (EPI == EPI_RESIDUAL) {
        *dst = from_float<OT>(to_float<OT>(*dst) + v);
      } else {
        *dst = from_float<OT>(v);
      }
    }
  }
}

// The same product for few rows (a decode step on the 32-bit path): with 64 x 64 tiles a product of
// one row by 512 columns is eight workgroups that each walk the whole inner size.  Here a workgroup
// owns 16 rows x 16 columns, one output element a thread, so there are as many workgroups as the
// matrix has groups of 16 columns.  Every element is the same chain as above (acc = fma(a[k], w[k],
// acc) for k = 0..K-1 from zero, then the bias): the two kernels agree bit for bit, and a token's
// logits do not depend on which of them ran.
#define ROWS_TILE 16
#define ROWS_BK 64

template <typename AT, typename WT, typename OT, int EPI>
__global__ __launch_bounds__(256) void linear_generic_rows_kernel(
    const AT* __restrict__ A, long lda, const WT* __restrict__ W, const float* __restrict__ bias,
    OT* __restrict__ out, long ldo, int n_rows, int n_out, int k_dim) {
  __shared__ float As[ROWS_TILE][ROWS_BK + 1];
  __shared__ float Ws[ROWS_TILE][ROWS_BK + 1];
  const int tid = threadIdx.x;
  const int r = tid >> 4, c = tid & 15;        // the element this thread owns; also the row it stages
  const int sk = (tid & 15) * 4;               // ... and which four k of a stage
  const int row0 = blockIdx.y * ROWS_TILE, col0 = blockIdx.x * ROWS_TILE;
  const bool a_ok = row0 + r < n_rows, w_ok = col0 + r < n_out;
  const AT* ap = A + (long)(row0 + r) * lda + sk;
  const WT* wp = W + (long)(col0 + r) * k_dim + sk;
  float acc = 0.f;
  for (int k0 = 0; k0 < k_dim; k0 += ROWS_BK) {
    const int kmax = k_dim - k0 < ROWS_BK ? k_dim - k0 : ROWS_BK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool k_ok = sk + i < kmax;
      As[r][sk + i] = (a_ok && k_ok) ? to_float<AT>(ap[k0 + i]) : 0.f;
      Ws[r][sk + i] = (w_ok && k_ok) ? to_float<WT>(wp[k0 + i]) : 0.f;
    }
    __syncthreads();
    if (kmax == ROWS_BK) {
#pragma unroll
      for (int kk = 0; kk < ROWS_BK; ++kk) acc = fmaf(As[r][kk], Ws[c][kk], acc);
    } else {
      for (int kk = 0; kk < kmax; ++kk) acc = fmaf(As[r][kk], Ws[c][kk], acc);
    }
    __syncthreads();
  }
  const int row = row0 + r, col = col0 + c;
  if (row >= n_rows || col >= n_out) return;
  float v = acc;
  if (bias) v += bias[col];
  if (EPI == EPI_GELU) v = gelu_tanh(v);
  OT* dst = out + (long)row * ldo + col;
  if (EPI == EPI_RESIDUAL) {
    *dst = from_float<OT>(to_float<OT>(*dst) + v);
  } else {
    *dst = from_float<OT>(v);
  }
}

#define ROWS_KERNEL_MAX_ROWS 32   // more rows than this: the 64 x 64 tiles

template <typename AT, typename WT, typename OT>
static int launch_epi(const void* A, long lda, const void* W, const float* bias, void* out, long ldo,
                      int n_rows, int n_out, int k_dim, int epi, hipStream_t stream) {
  const bool few = n_rows <= ROWS_KERNEL_MAX_ROWS;
  dim3 grid((n_out + TILE - 1) / TILE, (n_rows + TILE - 1) / TILE), block(256);
  dim3 grid_rows((n_out + ROWS_TILE - 1) / ROWS_TILE, (n_rows + ROWS_TILE - 1) / ROWS_TILE);
#define LAUNCH(E)                                                                                      \
  if (few)                                                                                             \
    hipLaunchKernelGGL((linear_generic_rows_kernel<AT, WT, OT, E>), grid_rows, block, 0, stream,       \
                       (const AT*)A, lda, (const WT*)W, bias, (OT*)out, ldo, n_rows, n_out, k_dim);    \
  else                                                                                                 \
    hipLaunchKernelGGL((linear_generic_kernel<AT, WT, OT, E>), grid, block, 0, stream, (const AT*)A,   \
                       lda, (const WT*)W, bias, (OT*)out, ldo, n_rows, n_out, k_dim)
  if (epi == EPI_NONE) { LAUNCH(EPI_NONE); }
  else if (epi == EPI_GELU) { LAUNCH(EPI_GELU); }
  else if (epi == EPI_RESIDUAL) { LAUNCH(EPI_RESIDUAL); }
  else return MGPT_ERR_BAD_SHAPE;
#undef LAUNCH
  return mgpt_last_error();
}

template <typename AT, typename WT>
static int launch_out(const void* A, long lda, const void* W, const float* bias, void* out, long ldo,
                      int n_rows, int n_out, int k_dim, int epi, int out_dtype, hipStream_t stream) {
  if (out_dtype == MGPT_F32)
    return launch_epi<AT, WT, float>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epi, stream);
  if (out_dtype == MGPT_BF16) {
    if (epi == EPI_RESIDUAL) return MGPT_ERR_BAD_DTYPE;  // the residual stream is 32-bit
    return launch_epi<AT, WT, bf16_t>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epi, stream);
  }
  return MGPT_ERR_BAD_DTYPE;
}

// A: [n_rows, k_dim] with row stride lda; W: [n_out, k_dim] dense; out: [n_rows, n_out] with row
// stride ldo.  Any inner size.
extern "C" int mgpt_linear_generic(const void* A, int a_dtype, long lda, const void* W, int w_dtype,
                                   const float* bias, void* out, int out_dtype, long ldo, int n_rows,
                                   int n_out, int k_dim, int epilogue, hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!A || !W || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_out < 0 || k_dim <= 0 || lda < k_dim || ldo < n_out)
    return MGPT_ERR_BAD_SHAPE;
  if ((n_rows + TILE - 1) / TILE > 65535) return MGPT_ERR_TOO_LARGE;
  if (a_dtype == MGPT_F32 && w_dtype == MGPT_F32)
    return launch_out<float, float>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epilogue, out_dtype, stream);
  if (a_dtype == MGPT_BF16 && w_dtype == MGPT_BF16)
    return launch_out<bf16_t, bf16_t>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epilogue, out_dtype, stream);
  if (a_dtype == MGPT_BF16 && w_dtype == MGPT_F32)
    return launch_out<bf16_t, float>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epilogue, out_dtype, stream);
  if (a_dtype == MGPT_F32 && w_dtype == MGPT_BF16)
    return launch_out<float, bf16_t>(A, lda, W, bias, out, ldo, n_rows, n_out, k_dim, epilogue, out_dtype, stream);
  return MGPT_ERR_BAD_DTYPE;
}
