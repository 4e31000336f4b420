// Token embedding (+ learned position rows) into the 32-bit residual stream,
// and LayerNorm with 32-bit statistics.
//
// embedding: x0[t] = tok_emb[id_t] + pos_emb[pos_t]   (reference: src/minigpt_infer/model.py:183)
// LayerNorm: y = (x - mean) / sqrt(var_biased + eps) * w (+ b) over the last dim
//            (reference: nn.LayerNorm at src/minigpt_infer/model.py:107,109,127)
#include "common.h"
#include "launchers.h"

template <typename WT>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ pos,
                             const WT* __restrict__ tok, const WT* __restrict__ postab,
                             float* __restrict__ x, int n_tokens, int width) {
  int n = blockIdx.x;
  if (n >= n_tokens) return;
  long id = ids[n];
  const WT* trow = tok + id * (long)width;
  const WT* prow = postab ? postab + (long)pos[n] * width : nullptr;
  float* xr = x + (long)n * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = to_float<WT>(trow[c]);
    if (prow) v += to_float<WT>(prow[c]);
    xr[c] = v;
  }
}

extern "C" int mgpt_embed(const int* ids, const int* pos, const void* tok, const void* postab,
                          float* x, int n_tokens, int width, int table_dtype, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!ids || !tok || !x || (postab && !pos)) return MGPT_ERR_NULL;
  if (n_tokens < 0 || width <= 0) return MGPT_ERR_BAD_SHAPE;
  int threads = width >= 256 ? 256 : 64;
  if (table_dtype == MGPT_F32) {
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream, ids, pos,
                       (const float*)tok, (const float*)postab, x, n_tokens, width);
  } else if (table_dtype == MGPT_BF16) {
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream, ids, pos,
                       (const bf16_t*)tok, (const bf16_t*)postab, x, n_tokens, width);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
  return mgpt_last_error();
}

// One wave per row; four rows per workgroup.  A row of up to 64 * LN_CACHE values is read once
// and kept in registers.  First the mean; then, together, the centred sum of squares and what
// the mean lost to rounding (kept apart: the mean is a sum of two floats), so the variance is
// never a difference of large numbers and a row of nearly equal values far from zero stays exact.
// Wider rows take the same steps with the row re-read from cache.
#define LN_CACHE 16

template <typename OT>
__global__ void layernorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                 const float* __restrict__ b, OT* __restrict__ out,
                                 const int* __restrict__ rows, int n_rows, int width, float eps) {
  int lane = threadIdx.x & (MGPT_WAVE - 1);
  int row = blockIdx.x * (blockDim.x / MGPT_WAVE) + (threadIdx.x / MGPT_WAVE);
  if (row >= n_rows) return;
  long src = rows ? rows[row] : row;
  const float* xr = x + src * (long)width;
  OT* orow = out + (long)row * width;
  if (width <= MGPT_WAVE * LN_CACHE) {
    // the row, the gain and the bias are all asked for before anything is waited for
    float xv[LN_CACHE], gv[LN_CACHE], bv[LN_CACHE];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < LN_CACHE; ++i) {
      const int c = lane + i * MGPT_WAVE;
      const int cc = c < width ? c : 0;
      xv[i] = xr[cc];
      gv[i] = w[cc];
      bv[i] = b ? b[cc] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < LN_CACHE; ++i) {
      if (lane + i * MGPT_WAVE >= width) xv[i] = 0.f;
      s += xv[i];
    }
    const float mean = wave_sum(s) / (float)width;
    float e = 0.f, v2 = 0.f;
#pragma unroll
    for (int i = 0; i < LN_CACHE; ++i) {
      const float d = (lane + i * MGPT_WAVE < width) ? xv[i] - mean : 0.f;
      xv[i] = d;
      e += d;
      v2 = fmaf(d, d, v2);
    }
    const float corr = wave_sum(e) / (float)width;
    const float var = fmaxf(wave_sum(v2) / (float)width - corr * corr, 0.f);
    const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int i = 0; i < LN_CACHE; ++i) {
      const int c = lane + i * MGPT_WAVE;
      if (c < width) orow[c] = from_float<OT>((xv[i] - corr) * rstd * gv[i] + bv[i]);
    }
    return;
  }
  float s = 0.f;
  for (int c = lane; c < width; c += MGPT_WAVE) s += xr[c];
  const float mean = wave_sum(s) / (float)width;
  float e = 0.f, v2 = 0.f;
  for (int c = lane; c < width; c += MGPT_WAVE) {
    const float d = xr[c] - mean;
    e += d;
    v2 = fmaf(d, d, v2);
  }
  const float corr = wave_sum(e) / (float)width;
  const float var = fmaxf(wave_sum(v2) / (float)width - corr * corr, 0.f);
  const float rstd = 1.0f / sqrtf(var + eps);
  for (int c = lane; c < width; c += MGPT_WAVE) {
    float y = ((xr[c] - mean) - corr) * rstd * w[c];
    if (b) y += b[c];
    orow[c] = from_float<OT>(y);
  }
}

// The same for widths that are multiples of 4 up to 64 * 4 * LN_VEC with 16-byte aligned rows: every
// lane loads and stores vectors of four (a row of 512 is two loads per lane instead of eight).
// LN_VEC is the number of such vectors a lane holds: the row's width / 256, rounded up to one of
// 1, 2, 3, 4, 6, 8 (rows up to 2048 wide), so that a row of 512 costs two loads and not four.
template <typename OT, int LN_VEC>
__global__ void layernorm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                     const float* __restrict__ b, OT* __restrict__ out,
                                     const int* __restrict__ rows, int n_rows, int width, float eps) {
  const int lane = threadIdx.x & (MGPT_WAVE - 1);
  const int row = blockIdx.x * (blockDim.x / MGPT_WAVE) + (threadIdx.x / MGPT_WAVE);
  if (row >= n_rows) return;
  const long src = rows ? rows[row] : row;
  const float4* xr = reinterpret_cast<const float4*>(x + src * (long)width);
  const float4* w4 = reinterpret_cast<const float4*>(w);
  const float4* b4 = reinterpret_cast<const float4*>(b);
  const int n4 = width >> 2;
  float4 xv[LN_VEC], gv[LN_VEC], bv[LN_VEC];
#pragma unroll
  for (int i = 0; i < LN_VEC; ++i) {
    const int c = lane + i * MGPT_WAVE;
    const int cc = c < n4 ? c : 0;
    xv[i] = xr[cc];
    gv[i] = w4[cc];
    bv[i] = b ? b4[cc] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < LN_VEC; ++i) {
    if (lane + i * MGPT_WAVE >= n4) xv[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    s += (xv[i].x + xv[i].y) + (xv[i].z + xv[i].w);
  }
  const float mean = wave_sum(s) / (float)width;
  float e = 0.f, v2 = 0.f;
#pragma unroll
  for (int i = 0; i < LN_VEC; ++i) {
    const bool in = lane + i * MGPT_WAVE < n4;
    float* p = reinterpret_cast<float*>(&xv[i]);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float d = in ? p[k] - mean : 0.f;
      p[k] = d;
      e += d;
      v2 = fmaf(d, d, v2);
    }
  }
  const float corr = wave_sum(e) / (float)width;
  const float var = fmaxf(wave_sum(v2) / (float)width - corr * corr, 0.f);
  const float rstd = 1.0f / sqrtf(var + eps);
  OT* orow = out + (long)row * width;
#pragma unroll
  for (int i = 0; i < LN_VEC; ++i) {
    const int c = lane + i * MGPT_WAVE;
    if (c >= n4) continue;
    const float y0 = (xv[i].x - corr) * rstd * gv[i].x + bv[i].x, y1 = (xv[i].y - corr) * rstd * gv[i].y + bv[i].y;
    const float y2 = (xv[i].z - corr) * rstd * gv[i].z + bv[i].z, y3 = (xv[i].w - corr) * rstd * gv[i].w + bv[i].w;
    if (sizeof(OT) == 4) {
      reinterpret_cast<float4*>(orow)[c] = make_float4(y0, y1, y2, y3);
    } else {
      uint2 pk;
      pk.x = pack_bf16x2(y0, y1);
      pk.y = pack_bf16x2(y2, y3);
      reinterpret_cast<uint2*>(orow)[c] = pk;
    }
  }
}

// rows: optional gather list (n_rows entries) of source rows of x; out row i <- x row rows[i].
extern "C" int mgpt_layernorm(const float* x, const float* w, const float* b, void* out,
                              const int* rows, int n_rows, int width, float eps, int out_dtype,
                              hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!x || !w || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || width <= 0) return MGPT_ERR_BAD_SHAPE;
  const int rows_per_block = 4;
  dim3 grid((n_rows + rows_per_block - 1) / rows_per_block), block(rows_per_block * MGPT_WAVE);
  const bool vec = (width % 4) == 0 && width <= MGPT_WAVE * 4 * 8 &&
                   ((((size_t)x) | ((size_t)w) | ((size_t)b) | ((size_t)out)) & 15) == 0;
  const int need = (width / 4 + MGPT_WAVE - 1) / MGPT_WAVE;   // vectors of four per lane
#define LN_LAUNCH(OT, V) \
  hipLaunchKernelGGL((layernorm_vec_kernel<OT, V>), grid, block, 0, stream, x, w, b, (OT*)out, rows, n_rows, width, eps)
#define LN_PICK(OT)                    \
  if (need <= 1) LN_LAUNCH(OT, 1);     \
  else if (need <= 2) LN_LAUNCH(OT, 2); \
  else if (need <= 3) LN_LAUNCH(OT, 3); \
  else if (need <= 4) LN_LAUNCH(OT, 4); \
  else if (need <= 6) LN_LAUNCH(OT, 6); \
  else LN_LAUNCH(OT, 8)
  if (vec && out_dtype == MGPT_F32) {
    LN_PICK(float);
  } else if (vec && out_dtype == MGPT_BF16) {
    LN_PICK(bf16_t);
#undef LN_PICK
#undef LN_LAUNCH
  } else if (out_dtype == MGPT_F32) {
    hipLaunchKernelGGL(layernorm_kernel<float>, grid, block, 0, stream, x, w, b, (float*)out, rows,
                       n_rows, width, eps);
  } else if (out_dtype == MGPT_BF16) {
    hipLaunchKernelGGL(layernorm_kernel<bf16_t>, grid, block, 0, stream, x, w, b, (bf16_t*)out,
                       rows, n_rows, width, eps);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
  return mgpt_last_error();
}
