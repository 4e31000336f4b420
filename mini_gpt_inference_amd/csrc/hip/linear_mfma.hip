// Tiled bfloat16 matrix product on the MFMA units for many rows (prompt portions).
//
// out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]) with an optional GELU-tanh or
// residual-add epilogue: nn.Linear as in src/minigpt_infer/model.py:43-44,96-101.
//
// A workgroup of four waves owns a 128 x 128 tile of the output; each wave a
// 64 x 64 quarter, as 4 x 4 v_mfma_f32_16x16x32_bf16 accumulators.  Per step of
// 32 along k the workgroup stages a 128 x 32 slice of the activations and of W
// in LDS (rows padded by 16 bytes so the 16 rows a MFMA operand reads fall on
// distinct banks), with the next slice's global loads in flight while the
// current one is multiplied.  W is the first MFMA operand, so a lane ends up
// with four neighbouring output columns of one row and stores them as one
// vector.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define MM_EPI_NONE 0
#define MM_EPI_GELU 1
#define MM_EPI_RESIDUAL 2

#define MM_TILE 128
#define MM_BK 32
#define MM_LD (MM_BK + 8)  // LDS row stride in elements

template <int EPI, typename OT>
__global__ __launch_bounds__(256) void linear_mfma_kernel(
    const bf16_t* __restrict__ act, long lda, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, OT* __restrict__ out, long ldo, int n_rows, int n_out, int k_dim) {
  __shared__ __align__(16) bf16_t as[2][MM_TILE * MM_LD];
  __shared__ __align__(16) bf16_t ws[2][MM_TILE * MM_LD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row0 = blockIdx.y * MM_TILE, col0 = blockIdx.x * MM_TILE;
  const int wr = (wave >> 1) * 64, wc = (wave & 1) * 64;  // this wave's quarter
  const int lrow = lane & 15, lk = (lane >> 4) * 8;

  // staging: thread t copies 16 bytes of rows (t >> 2) and (t >> 2) + 64, k offset (t & 3) * 8
  const int srow = tid >> 2, sk = (tid & 3) * 8;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t ga[2], gw[2];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int r = srow + half * 64;
      const bool k_ok = k0 + sk + 8 <= k_dim;
      const int an = row0 + r, wo = col0 + r;
      ga[half] = (k_ok && an < n_rows) ? *reinterpret_cast<const bf16x8_t*>(act + (long)an * lda + k0 + sk) : zero8;
      gw[half] = (k_ok && wo < n_out) ? *reinterpret_cast<const bf16x8_t*>(w + (long)wo * k_dim + k0 + sk) : zero8;
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int r = srow + half * 64;
      *reinterpret_cast<bf16x8_t*>(&as[buf][r * MM_LD + sk]) = ga[half];
      *reinterpret_cast<bf16x8_t*>(&ws[buf][r * MM_LD + sk]) = gw[half];
    }
  };

  f32x4_t acc[4][4];  // [column tile of W][row tile of activations]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int k_steps = (k_dim + MM_BK - 1) / MM_BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int s = 0; s < k_steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < k_steps) load_global((s + 1) * MM_BK);
    bf16x8_t wf[4], af[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      wf[i] = *reinterpret_cast<const bf16x8_t*>(&ws[buf][(wc + i * 16 + lrow) * MM_LD + lk]);
      af[i] = *reinterpret_cast<const bf16x8_t*>(&as[buf][(wr + i * 16 + lrow) * MM_LD + lk]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
    if (s + 1 < k_steps) {
      store_lds(buf ^ 1);  // the other buffer: its readers finished before the last barrier
      __syncthreads();
    }
  }

  // lane holds out[row0 + wr + j*16 + (lane & 15)][col0 + wc + i*16 + (lane >> 4)*4 + e], e = 0..3
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = row0 + wr + j * 16 + lrow;
    if (n >= n_rows) continue;
    OT* orow = out + (long)n * ldo;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int oc = col0 + wc + i * 16 + (lane >> 4) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int o = oc + e;
        if (o >= n_out) continue;
        float v = acc[i][j][e];
        if (bias) v += bias[o];
        if (EPI == MM_EPI_GELU) v = gelu_tanh(v);
        if (EPI == MM_EPI_RESIDUAL) {
          orow[o] = from_float<OT>(to_float<OT>(orow[o]) + v);
        } else {
          orow[o] = from_float<OT>(v);
        }
      }
    }
  }
}

// act: [n_rows, k_dim] bfloat16 with row stride lda (a multiple of 8, 16-byte aligned base);
// w: [n_out, k_dim] dense bfloat16; out: [n_rows, n_out] with row stride ldo.  k_dim must be a
// multiple of 16.  Refuses other layouts with MGPT_ERR_BAD_SHAPE.
extern "C" int mgpt_linear_mfma(const void* act, long lda, const void* w, const float* bias, void* out,
                                int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue,
                                hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!act || !w || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_out < 0 || k_dim <= 0 || (k_dim % 16) != 0 || lda < k_dim || (lda % 8) != 0 ||
      ldo < n_out)
    return MGPT_ERR_BAD_SHAPE;
  dim3 grid((n_out + MM_TILE - 1) / MM_TILE, (n_rows + MM_TILE - 1) / MM_TILE), block(256);
  if (grid.y > 65535) return MGPT_ERR_TOO_LARGE;
#define MM_LAUNCH(E, OT)                                                                               \
  hipLaunchKernelGGL((linear_mfma_kernel<E, OT>), grid, block, 0, stream, (const bf16_t*)act, lda,     \
                     (const bf16_t*)w, bias, (OT*)out, ldo, n_rows, n_out, k_dim)
  if (epilogue == MM_EPI_NONE && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_NONE, bf16_t);
  else if (epilogue == MM_EPI_NONE && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_NONE, float);
  else if (epilogue == MM_EPI_GELU && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_GELU, bf16_t);
  else if (epilogue == MM_EPI_RESIDUAL && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_RESIDUAL, float);
  else return MGPT_ERR_BAD_DTYPE;
#undef MM_LAUNCH
  return mgpt_last_error();
}
