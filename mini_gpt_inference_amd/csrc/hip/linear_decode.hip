// Matrix product for the rows of a decode step (at most 16) in bfloat16 on the MFMA units, laid
// out for latency: out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]), nn.Linear as in
// src/minigpt_infer/model.py:43-44,96-101.
//
// A decode step is a chain of some forty dependent kernels that each read a megabyte or two,
// so what counts is how soon a kernel is over, and that is set by the bytes one compute unit
// has to pull through its own cache.  Hence: one workgroup of four waves per 16 output
// columns (as many workgroups, on as many compute units, as the matrix has column tiles), the
// waves split k four ways, every lane issues all its loads (W, activations, and what the
// epilogue will need: bias, column sums, the old residual values, the cache slot) before it
// waits for any, rows beyond n_rows are not loaded at all, one v_mfma_f32_16x16x32_bf16 per 32
// k, the four waves' sums are added through LDS in wave order, and the first wave stores.
//
// Folded LayerNorm, epilogues and the key/value scatter are those of linear_skinny.hip (the
// LayerNorm of src/minigpt_infer/model.py:113-114,186-187 folded into W by fold_norm.hip;
// scatter as src/minigpt_infer/cache/paged.py:125-137).
#include "linear_skinny.h"

// VEC: n_out is a multiple of 16 and bias, column sums and output rows are aligned for vectors of
// four; otherwise every access of the epilogue is a single element with its own bound check.
template <int SMAX, bool LN, int EPI, typename OT, bool VEC>
__global__ __launch_bounds__(256) void linear_decode_kernel(SkinnyArgs a) {
  __shared__ float red[3 * 6 * 64];  // waves 1..3: four sums and two statistics per lane
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes: branches on it are scalar
  const int lrow = lane & 15, g = lane >> 4;
  const int K = a.k_dim;
  const int steps_total = K >> 5;
  const int per = (steps_total + 3) >> 2;
  const int steps = max(0, min(per, steps_total - wave * per));  // the last waves of a short k may have none
  const int kb = steps > 0 ? wave * per * 32 : 0;
  const int o0 = blockIdx.x * 16;
  const int wo = min(o0 + lrow, a.n_out - 1);  // a column past the end reads the last row; never stored
  const bool row_ok = lrow < a.n_rows;
  const int oc = o0 + g * 4;  // this lane's four output columns, of row lrow

  // ---- every load this lane will need, issued before anything waits.  Loads are unconditional
  // within a row (a k step past this wave's range reads the range's first step again and is not
  // multiplied), so that nothing but the data stands between one load and the next.
  int src = lrow;
  if (LN && a.rows != nullptr && row_ok) src = a.rows[lrow];
  // the epilogue's inputs (first wave only)
  const bool writer = wave == 0 && row_ok && oc < a.n_out;
  float bias4[4] = {0.f, 0.f, 0.f, 0.f}, cs4[4] = {0.f, 0.f, 0.f, 0.f}, old4[4] = {0.f, 0.f, 0.f, 0.f};
  int slot = -1;
  OT* orow = reinterpret_cast<OT*>(a.out) + (long)lrow * a.ldo;
  if (writer) {
    if (VEC) {
      if (a.bias != nullptr) {
        const float4 b4 = *reinterpret_cast<const float4*>(a.bias + oc);
        bias4[0] = b4.x; bias4[1] = b4.y; bias4[2] = b4.z; bias4[3] = b4.w;
      }
      if (LN) {
        const float4 c4 = *reinterpret_cast<const float4*>(a.colsum + oc);
        cs4[0] = c4.x; cs4[1] = c4.y; cs4[2] = c4.z; cs4[3] = c4.w;
      }
      if (EPI == SK_EPI_RESIDUAL) {
        const float4 o4 = *reinterpret_cast<const float4*>(orow + oc);
        old4[0] = o4.x; old4[1] = o4.y; old4[2] = o4.z; old4[3] = o4.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = min(oc + i, a.n_out - 1);
        if (a.bias != nullptr) bias4[i] = a.bias[o];
        if (LN) cs4[i] = a.colsum[o];
        if (EPI == SK_EPI_RESIDUAL) old4[i] = to_float<OT>(orow[o]);
      }
    }
    if (EPI == SK_EPI_QKV) slot = a.slot_mapping[lrow];
  }

  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t wv[SMAX], av[SMAX];
  const bf16_t* wp = a.w + (long)wo * K + kb + g * 8;
#pragma unroll
  for (int i = 0; i < SMAX; ++i) wv[i] = *reinterpret_cast<const bf16x8_t*>(wp + (i < steps ? i : 0) * 32);
  float4 lo[LN ? SMAX : 1], hi[LN ? SMAX : 1];
  float x0 = 0.f;
  if (LN) {
#pragma unroll
    for (int i = 0; i < SMAX; ++i) lo[i] = hi[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row_ok) {
      const float* xr = a.x + (long)src * K;
#pragma unroll
      for (int i = 0; i < SMAX; ++i) {
        const float4* p = reinterpret_cast<const float4*>(xr + kb + g * 8 + (i < steps ? i : 0) * 32);
        lo[i] = p[0];
        hi[i] = p[1];
      }
      x0 = xr[0];
    }
  } else {
#pragma unroll
    for (int i = 0; i < SMAX; ++i) av[i] = zero8;
    if (row_ok) {
      const bf16_t* ap = a.act + (long)lrow * a.lda + kb + g * 8;
#pragma unroll
      for (int i = 0; i < SMAX; ++i) av[i] = *reinterpret_cast<const bf16x8_t*>(ap + (i < steps ? i : 0) * 32);
    }
  }
  // ---- multiply
  float sd = 0.f, sq = 0.f;  // sums of (x - x0) and (x - x0)^2 over what this lane loaded of its row
  if (LN) {
#pragma unroll
    for (int i = 0; i < SMAX; ++i) {
      const float f[8] = {lo[i].x, lo[i].y, lo[i].z, lo[i].w, hi[i].x, hi[i].y, hi[i].z, hi[i].w};
      typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;
      const u32x4_t pk = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                          pack_bf16x2(f[6], f[7])};
      av[i] = __builtin_bit_cast(bf16x8_t, pk);
      if (i < steps) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = f[e] - x0;
          sd += d;
          sq = fmaf(d, d, sq);
        }
      }
    }
  }
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < SMAX; ++i)
    if (i < steps) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], av[i], acc, 0, 0, 0);
  if (LN) {
    // the four lanes that share a row hold parts of its sums
    sd += __shfl_xor(sd, 16, 64);
    sd += __shfl_xor(sd, 32, 64);
    sq += __shfl_xor(sq, 16, 64);
    sq += __shfl_xor(sq, 32, 64);
  }

  // ---- the four waves' parts, added in wave order by the first
  if (wave > 0) {
    float* r = red + (wave - 1) * 6 * 64 + lane;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i * 64] = acc[i];
    if (LN) {
      r[4 * 64] = sd;
      r[5 * 64] = sq;
    }
  }
  __syncthreads();
  if (!writer) return;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    const float* r = red + s * 6 * 64 + lane;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] += r[i * 64];
    if (LN) {
      sd += r[4 * 64];
      sq += r[5 * 64];
    }
  }

  // ---- epilogue: lane holds out[lrow][oc + i], i = 0..3
  float v[4];
  float mean = 0.f, rstd = 1.f;
  if (LN) {
    const float inv_k = 1.0f / (float)K;
    const float md = sd * inv_k;  // mean of x - x0
    mean = x0 + md;
    rstd = 1.0f / sqrtf(fmaxf(sq * inv_k - md * md, 0.f) + a.eps);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] = acc[i];
    if (LN) v[i] = rstd * (v[i] - mean * cs4[i]);
    v[i] += bias4[i];
    if (EPI == SK_EPI_GELU) v[i] = gelu_tanh(v[i]);
    if (EPI == SK_EPI_RESIDUAL) v[i] += old4[i];
  }
  if (VEC && sizeof(OT) == 4) {
    *reinterpret_cast<float4*>(orow + oc) = make_float4(v[0], v[1], v[2], v[3]);
  } else if (VEC) {
    uint2 pk;
    pk.x = pack_bf16x2(v[0], v[1]);
    pk.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(orow + oc) = pk;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (oc + i < a.n_out) orow[oc + i] = from_float<OT>(v[i]);
  }
  if (EPI == SK_EPI_QKV) {
    if (slot >= 0 && oc >= a.q_width) {
      // the four columns lie in one head (head sizes and widths are multiples of 4): one 8-byte store
      const long page = slot / a.page_size;
      const int off = slot - (int)page * a.page_size;
      const int c = oc - a.q_width;  // column among keys then values
      const bool is_v = c >= a.kv_width;
      const int cc = is_v ? c - a.kv_width : c;
      const int h = cc / a.head_dim, d = cc - h * a.head_dim;
      const long dst = ((page * a.n_kv_head + h) * a.page_size + off) * (long)a.head_dim + d;
      uint2 pk;
      pk.x = pack_bf16x2(v[0], v[1]);
      pk.y = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<uint2*>((is_v ? a.vpool : a.kpool) + dst) = pk;
    }
  }
}

template <int SMAX, bool LN>
static int launch_decode(const SkinnyArgs& a, int epi, int out_dtype, dim3 grid, hipStream_t s) {
  const size_t align = sizeof(float) * 4 - 1;  // bfloat16 rows are stored 8 bytes at a time: covered as well
  const bool vec = (a.n_out % 16) == 0 && (a.ldo % 4) == 0 &&
                   ((((size_t)a.bias) | ((size_t)a.colsum) | ((size_t)a.out)) & align) == 0;
#define LD_LAUNCH(E, OT)                                                                                \
  do {                                                                                                  \
    if (vec) hipLaunchKernelGGL((linear_decode_kernel<SMAX, LN, E, OT, true>), grid, dim3(256), 0, s, a); \
    else hipLaunchKernelGGL((linear_decode_kernel<SMAX, LN, E, OT, false>), grid, dim3(256), 0, s, a);  \
  } while (0)
  if (epi == SK_EPI_NONE && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_NONE, bf16_t);
  else if (epi == SK_EPI_NONE && out_dtype == MGPT_F32) LD_LAUNCH(SK_EPI_NONE, float);
  else if (epi == SK_EPI_GELU && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_GELU, bf16_t);
  else if (epi == SK_EPI_RESIDUAL && out_dtype == MGPT_F32) LD_LAUNCH(SK_EPI_RESIDUAL, float);
  else if (epi == SK_EPI_QKV && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_QKV, bf16_t);
  else return MGPT_ERR_BAD_DTYPE;
#undef LD_LAUNCH
  return mgpt_last_error();
}

// The caller (mgpt_linear_skinny) has checked pointers, strides and the scatter's sizes.
int mgpt_launch_linear_decode(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  if (a.n_rows > 16 || (a.k_dim % 32) != 0 || a.k_dim > 2048) return MGPT_ERR_BAD_SHAPE;
  // the scatter stores four neighbouring columns of a head at once
  if (epilogue == SK_EPI_QKV && ((a.n_out % 16) != 0 || (a.ldo % 4) != 0 || (((size_t)a.out) & 15) != 0))
    return MGPT_ERR_BAD_SHAPE;
  const bool ln = a.x != nullptr;
  const int per = (a.k_dim / 32 + 3) / 4;  // k steps of the first waves
  dim3 grid((a.n_out + 15) / 16);
#define LD_PICK(S) \
  (ln ? launch_decode<S, true>(a, epilogue, out_dtype, grid, stream) : launch_decode<S, false>(a, epilogue, out_dtype, grid, stream))
  if (per <= 4) return LD_PICK(4);
  if (per <= 8) return LD_PICK(8);
  return LD_PICK(16);
#undef LD_PICK
}
