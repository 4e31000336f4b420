// The kernel of linear_decode.hip and linear_decode_rows.hip: a matrix product for the rows of a
// decode step in bfloat16 on the MFMA units, laid out for latency.
//
// out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]), nn.Linear as in
// src/minigpt_infer/model.py:43-44,96-101.
//
// A decode step is a chain of some forty dependent kernels that each read a megabyte or two,
// so what counts is how soon a kernel is over, and that is set by the bytes one compute unit
// has to pull through its own cache.  Hence: one workgroup of four waves per 16 output
// columns (as many workgroups, on as many compute units, as the matrix has column tiles), the
// waves split k four ways, every lane issues all its loads (W, activations, and what the
// epilogue will need: bias, column sums, the old residual values, the cache slot) before it
// waits for any, rows beyond n_rows are not loaded at all, one v_mfma_f32_16x16x32_bf16 per 32
// k and 16 rows, the four waves' sums are added through LDS in wave order, and the first wave
// stores.  NT tiles of 16 rows share the W a lane has loaded.  A wave's k range longer than SMAX
// steps of 32 takes several passes of loads.
//
// Folded LayerNorm, epilogues and the key/value scatter are those of linear_skinny.hip (the
// LayerNorm of src/minigpt_infer/model.py:113-114,186-187 folded into W by fold_norm.hip;
// scatter as src/minigpt_infer/cache/paged.py:125-137).
#pragma once
#include "linear_skinny.h"

// DPP row_shl:n: lane l of a row of 16 gets the value of lane l + n (0 from past the row's end)
template <int N>
__device__ __forceinline__ unsigned int ld_shl(unsigned int v) {
  return N == 0 ? v : (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0x100 + (N == 0 ? 1 : N), 0xf, 0xf, false);
}
__device__ __forceinline__ float ld_shl_f(float v, int n) {
  switch (n) {
    case 1: return __uint_as_float(ld_shl<1>(__float_as_uint(v)));
    case 2: return __uint_as_float(ld_shl<2>(__float_as_uint(v)));
    case 4: return __uint_as_float(ld_shl<4>(__float_as_uint(v)));
    default: return __uint_as_float(ld_shl<8>(__float_as_uint(v)));
  }
}
// the 8 rounded values of a k step, taken from the lane FEW * j further on in the row
template <int FEW>
__device__ __forceinline__ bf16x8_t ld_row_shl(bf16x8_t v, int j) {
  typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;
  const u32x4_t s = __builtin_bit_cast(u32x4_t, v);
  u32x4_t r = s;
#define LD_CASE(J)                                                                                   \
  case J:                                                                                            \
    if (FEW * J < 16)                                                                                \
      r = (u32x4_t){ld_shl<(FEW * J < 16 ? FEW * J : 0)>(s[0]), ld_shl<(FEW * J < 16 ? FEW * J : 0)>(s[1]), \
                    ld_shl<(FEW * J < 16 ? FEW * J : 0)>(s[2]), ld_shl<(FEW * J < 16 ? FEW * J : 0)>(s[3])}; \
    break;
  switch (j) {
    LD_CASE(1) LD_CASE(2) LD_CASE(3) LD_CASE(4) LD_CASE(5) LD_CASE(6) LD_CASE(7) LD_CASE(8)
    LD_CASE(9) LD_CASE(10) LD_CASE(11) LD_CASE(12) LD_CASE(13) LD_CASE(14) LD_CASE(15)
    default: break;
  }
#undef LD_CASE
  return __builtin_bit_cast(bf16x8_t, r);
}

// VEC: n_out is a multiple of 16 and bias, column sums and output rows are aligned for vectors of
// four; otherwise every access of the epilogue is a single element with its own bound check.
// SPLIT: k is also split over a.k_parts workgroups per column tile; each stores its raw sums to
// a.partials (no LayerNorm, no epilogue: linear_partials_epilogue_kernel finishes the job).
// FEW (with LN and one tile; 1, 2, 4 or 8, at least the rows of a group): the residual rows are
// loaded by all sixteen lanes of a lane row, not only by the FEW that hold a row: lane r + FEW j
// loads the j-th of 16 / FEW k steps of row r, rounds it and adds up its statistics, and the row's
// own lane takes the rounded values over with a DPP shift.  A load instruction costs the compute
// unit the same whether four of its lanes are live or all: at one row that is 2 instead of 26 of
// them for an inner size of 1600 ([6400 x 1600] at one row: 6.9 us with the LayerNorm against 6.9
// over rows that are normed already, where it was 2.2 us more; at 8 rows 9.9 against 7.9).  0: every
// lane loads what it multiplies.
template <int NT, int SMAX, bool LN, int EPI, typename OT, bool VEC, bool SPLIT = false, int FEW = 0>
__global__ __launch_bounds__(256) void linear_decode_kernel(SkinnyArgs a) {
  static_assert(FEW == 0 || (LN && NT == 1 && !SPLIT && (FEW == 1 || FEW == 2 || FEW == 4 || FEW == 8)),
                "rows packed into a load: one tile, with the LayerNorm, 1, 2, 4 or 8 rows");
  __shared__ float red[3 * NT * 6 * 64];  // waves 1..3: per row tile four sums and two statistics per lane
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes: branches on it are scalar
  const int lrow = lane & 15, g = lane >> 4;
  const int K = a.k_dim;
  const int part = SPLIT ? (int)(blockIdx.x % a.k_parts) : 0;
  const int steps_total = SPLIT ? (K >> 5) / a.k_parts : K >> 5;   // of this workgroup
  const int per = (steps_total + 3) >> 2;
  const int steps = max(0, min(per, steps_total - wave * per));  // the last waves of a short k may have none
  const int kb = (steps > 0 ? wave * per * 32 : 0) + part * steps_total * 32;
  const int o0 = (SPLIT ? (int)(blockIdx.x / a.k_parts) : (int)blockIdx.x) * 16;
  const int wo = min(o0 + lrow, a.n_out - 1);  // a column past the end reads the last row; never stored
  const int oc = o0 + g * 4;  // this lane's four output columns, of rows lrow + 16 t
  // rows of this workgroup: with gridDim.y > 1 the rows are dealt out in groups of NT * 16
  // (one tile a workgroup: the group may be smaller than the tile, a.rows_per_group of its 16 rows)
  const int rpg = NT == 1 ? a.rows_per_group : 16;
  const int r0 = (int)blockIdx.y * (NT == 1 ? rpg : NT * 16) + lrow;
  bool row_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) row_ok[t] = lrow < rpg && r0 + t * 16 < a.n_rows;

  // ---- every load this lane will need, issued before anything waits.  Loads are unconditional
  // within a row (a k step past this wave's range reads the range's first step again and is not
  // multiplied), so that nothing but the data stands between one load and the next.
  int src[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    src[t] = r0 + t * 16;
    if (LN && a.rows != nullptr && row_ok[t]) src[t] = a.rows[r0 + t * 16];
  }
  // the epilogue's inputs (first wave only)
  const bool col_writer = wave == 0 && oc < a.n_out;
  float bias4[4] = {0.f, 0.f, 0.f, 0.f}, cs4[4] = {0.f, 0.f, 0.f, 0.f};
  float old4[NT][4];
  int slot[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    slot[t] = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) old4[t][i] = 0.f;
  }
  OT* const out = reinterpret_cast<OT*>(a.out);
  if (col_writer && (!SPLIT || (a.bias_in_part0 && part == 0))) {
    if (VEC) {
      if (a.bias != nullptr) {
        const float4 b4 = *reinterpret_cast<const float4*>(a.bias + oc);
        bias4[0] = b4.x; bias4[1] = b4.y; bias4[2] = b4.z; bias4[3] = b4.w;
      }
      if (LN) {
        const float4 c4 = *reinterpret_cast<const float4*>(a.colsum + oc);
        cs4[0] = c4.x; cs4[1] = c4.y; cs4[2] = c4.z; cs4[3] = c4.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = min(oc + i, a.n_out - 1);
        if (a.bias != nullptr) bias4[i] = a.bias[o];
        if (LN) cs4[i] = a.colsum[o];
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!row_ok[t]) continue;
      const OT* orow = out + (long)(r0 + t * 16) * a.ldo;
      if (EPI == SK_EPI_RESIDUAL) {
        if (VEC) {
          const float4 o4 = *reinterpret_cast<const float4*>(orow + oc);
          old4[t][0] = o4.x; old4[t][1] = o4.y; old4[t][2] = o4.z; old4[t][3] = o4.w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) old4[t][i] = to_float<OT>(orow[min(oc + i, a.n_out - 1)]);
        }
      }
      if (EPI == SK_EPI_QKV) slot[t] = a.slot_mapping[r0 + t * 16];
    }
  }

  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  f32x4_t acc[NT];
  float x0[NT], sd[NT], sq[NT];  // sums of (x - x0) and (x - x0)^2 over what this lane loads of its rows
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    x0[t] = sd[t] = sq[t] = 0.f;
    // the shift of a row: the median of three of its values, so that one channel that stands far
    // out (residual streams have such) does not become the shift
    if (LN && FEW == 0 && row_ok[t]) {
      const float* xr = a.x + (long)src[t] * K;
      x0[t] = __builtin_amdgcn_fmed3f(xr[0], xr[K >> 1], xr[K - 1]);
    }
  }
  // FEW: the row this lane loads for (fr of the group) and which of a batch's k steps (fj)
  constexpr int FJ = FEW > 0 ? 16 / FEW : 1;
  const int fr = FEW > 0 ? (lrow & (FEW - 1)) : 0, fj = FEW > 0 ? lrow / (FEW > 0 ? FEW : 1) : 0;
  const float* frow_x = a.x;
  bool f_ok = false;
  if (FEW > 0) {
    const int frow = (int)blockIdx.y * rpg + fr;
    f_ok = fr < rpg && frow < a.n_rows;
    const int fsrc = f_ok ? (a.rows != nullptr ? a.rows[frow] : frow) : 0;
    frow_x = a.x + (long)fsrc * K;
    // (the lane that holds the row is its first loader: fj = 0, fr = lrow)
    if (f_ok) x0[0] = __builtin_amdgcn_fmed3f(frow_x[0], frow_x[K >> 1], frow_x[K - 1]);
  }
  // W as it is (a wave's load is sixteen rows' 64 bytes), or packed so that it is 1 KB in one piece
  const bf16_t* wp = a.w_packed ? a.w_packed + (((long)(o0 >> 4) * (K >> 5) + (kb >> 5)) * 64 + lane) * 8
                                : a.w + (long)wo * K + kb + g * 8;
  const int w_step = a.w_packed ? 512 : 32;
  for (int s0 = 0; s0 < steps; s0 += SMAX) {
    bf16x8_t wv[SMAX], av[NT][SMAX];
#pragma unroll
    for (int i = 0; i < SMAX; ++i)
      wv[i] = *reinterpret_cast<const bf16x8_t*>(wp + (s0 + i < steps ? s0 + i : 0) * w_step);
    if (LN && FEW > 0) {
      // a batch of FJ k steps per pair of loads: this lane loads step b * FJ + fj of the pass
      constexpr int NB = (SMAX + FJ - 1) / FJ;
      bf16x8_t packed[NB];
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const int st = s0 + b * FJ + fj;
        const bool live = f_ok && st < steps && b * FJ + fj < SMAX;
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        if (live) {
          const float4* p = reinterpret_cast<const float4*>(frow_x + kb + g * 8 + st * 32);
          lo = p[0];
          hi = p[1];
        }
        const float xs0 = x0[0];
        const float f[8] = {lo.x - xs0, lo.y - xs0, lo.z - xs0, lo.w - xs0, hi.x - xs0, hi.y - xs0, hi.z - xs0, hi.w - xs0};
        typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;
        u32x4_t pk = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
        if (!live) pk = (u32x4_t){0u, 0u, 0u, 0u};
        packed[b] = __builtin_bit_cast(bf16x8_t, pk);
        if (live) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            sd[0] += f[e];
            sq[0] = fmaf(f[e], f[e], sq[0]);
          }
        }
      }
      // the row's own lane (lrow < FEW) takes step i from the lane that loaded it
#pragma unroll
      for (int i = 0; i < SMAX; ++i) av[0][i] = ld_row_shl<FEW>(packed[i / FJ], i % FJ);
    } else if (LN) {
      float4 lo[NT][SMAX], hi[NT][SMAX];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int i = 0; i < SMAX; ++i) lo[t][i] = hi[t][i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row_ok[t]) {
          const float* xr = a.x + (long)src[t] * K + kb + g * 8;
#pragma unroll
          for (int i = 0; i < SMAX; ++i) {
            const float4* p = reinterpret_cast<const float4*>(xr + (s0 + i < steps ? s0 + i : 0) * 32);
            lo[t][i] = p[0];
            hi[t][i] = p[1];
          }
        }
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int i = 0; i < SMAX; ++i) {
          // what is rounded to bfloat16 is the distance from the row's first value: a row far from
          // zero loses nothing to its offset (the epilogue corrects with the mean of the distances);
          // a row that is not loaded has x0 = 0 and zeros
          const float f[8] = {lo[t][i].x - x0[t], lo[t][i].y - x0[t], lo[t][i].z - x0[t], lo[t][i].w - x0[t],
                              hi[t][i].x - x0[t], hi[t][i].y - x0[t], hi[t][i].z - x0[t], hi[t][i].w - x0[t]};
          typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;
          const u32x4_t pk = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                              pack_bf16x2(f[6], f[7])};
          av[t][i] = __builtin_bit_cast(bf16x8_t, pk);
          if (s0 + i < steps) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              sd[t] += f[e];
              sq[t] = fmaf(f[e], f[e], sq[t]);
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int i = 0; i < SMAX; ++i) av[t][i] = zero8;
        if (row_ok[t]) {
          const bf16_t* ap = a.act + (long)(r0 + t * 16) * a.lda + kb + g * 8;
#pragma unroll
          for (int i = 0; i < SMAX; ++i)
            av[t][i] = *reinterpret_cast<const bf16x8_t*>(ap + (s0 + i < steps ? s0 + i : 0) * 32);
        }
      }
    }
    // ---- multiply
#pragma unroll
    for (int i = 0; i < SMAX; ++i)
      if (s0 + i < steps) {
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], av[t][i], acc[t], 0, 0, 0);
      }
  }
  if (LN && FEW > 0) {
    // the loaders of a row lie FEW lanes apart: their sums meet in the row's own lane
#pragma unroll
    for (int n = FEW; n < 16; n <<= 1) {
      sd[0] += ld_shl_f(sd[0], n);
      sq[0] += ld_shl_f(sq[0], n);
    }
  }
  if (LN) {
    // the four lanes that share a row hold parts of its sums
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      sd[t] += __shfl_xor(sd[t], 16, 64);
      sd[t] += __shfl_xor(sd[t], 32, 64);
      sq[t] += __shfl_xor(sq[t], 16, 64);
      sq[t] += __shfl_xor(sq[t], 32, 64);
    }
  }

  // ---- the four waves' parts, added in wave order by the first
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float* r = red + ((wave - 1) * NT + t) * 6 * 64 + lane;
#pragma unroll
      for (int i = 0; i < 4; ++i) r[i * 64] = acc[t][i];
      if (LN) {
        r[4 * 64] = sd[t];
        r[5 * 64] = sq[t];
      }
    }
  }
  __syncthreads();
  if (!col_writer) return;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const float* r = red + (s * NT + t) * 6 * 64 + lane;
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t][i] += r[i * 64];
      if (LN) {
        sd[t] += r[4 * 64];
        sq[t] += r[5 * 64];
      }
    }
  }

  // ---- epilogue: lane holds out[r0 + t * 16][oc + i], i = 0..3
  if (SPLIT) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!row_ok[t]) continue;
      float* prow = a.partials + ((long)part * a.n_rows + r0 + t * 16) * a.n_out + oc;
      // (the bias is zero unless this part carries it)
      *reinterpret_cast<float4*>(prow) = make_float4(acc[t][0] + bias4[0], acc[t][1] + bias4[1], acc[t][2] + bias4[2],
                                                     acc[t][3] + bias4[3]);
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    if (!row_ok[t]) continue;
    OT* orow = out + (long)(r0 + t * 16) * a.ldo;
    float v[4];
    float md = 0.f, rstd = 1.f;
    if (LN) {
      const float inv_k = 1.0f / (float)K;
      md = sd[t] * inv_k;  // mean of x - x0, and the products were of x - x0 as well
      rstd = 1.0f / sqrtf(fmaxf(sq[t] * inv_k - md * md, 0.f) + a.eps);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = acc[t][i];
      if (LN) v[i] = rstd * (v[i] - md * cs4[i]);
      v[i] += bias4[i];
      if (EPI == SK_EPI_GELU) v[i] = gelu_tanh_fast(v[i]);
      if (EPI == SK_EPI_RESIDUAL) v[i] += old4[t][i];
    }
    if (VEC && sizeof(OT) == 4) {
      *reinterpret_cast<float4*>(orow + oc) = make_float4(v[0], v[1], v[2], v[3]);
      if (NT == 1 && EPI == SK_EPI_NONE && a.best_val != nullptr) {
        // the row's best of this tile: of this lane's four columns in rising order, then over the
        // four lanes that hold the row (all of them are here: VEC means whole tiles)
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (oc + i < a.best_limit && v[i] > bv) { bv = v[i]; bi = oc + i; }
#pragma unroll
        for (int m = 16; m <= 32; m <<= 1) {
          const float ov = __shfl_xor(bv, m, 64);
          const int oi = __shfl_xor(bi, m, 64);
          if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (g == 0) {
          const long at = (long)(r0 + t * 16) * (a.n_out >> 4) + (o0 >> 4);
          a.best_val[at] = bv;
          a.best_idx[at] = bi;
        }
      }
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
      if (slot[t] >= 0 && oc >= a.q_width) {
        // the four columns lie in one head (head sizes and widths are multiples of 4): one 8-byte store
        const long page = slot[t] / a.page_size;
        const int off = slot[t] - (int)page * a.page_size;
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
}

template <int NT, int SMAX, bool LN, bool VEC, int FEW = 0>
static int launch_decode_epi(const SkinnyArgs& a, int epi, int out_dtype, dim3 grid, hipStream_t s) {
#define LD_LAUNCH(E, OT) \
  hipLaunchKernelGGL((linear_decode_kernel<NT, SMAX, LN, E, OT, VEC, false, FEW>), grid, dim3(256), 0, s, a)
  if (epi == SK_EPI_NONE && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_NONE, bf16_t);
  else if (epi == SK_EPI_NONE && out_dtype == MGPT_F32) LD_LAUNCH(SK_EPI_NONE, float);
  else if (epi == SK_EPI_GELU && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_GELU, bf16_t);
  else if (epi == SK_EPI_RESIDUAL && out_dtype == MGPT_F32) LD_LAUNCH(SK_EPI_RESIDUAL, float);
  else if (epi == SK_EPI_QKV && out_dtype == MGPT_BF16) LD_LAUNCH(SK_EPI_QKV, bf16_t);
  else return MGPT_ERR_BAD_DTYPE;
#undef LD_LAUNCH
  return mgpt_last_error();
}

// whether the epilogue may use vectors of four (see VEC above)
static inline bool decode_vec_ok(const SkinnyArgs& a) {
  const size_t align = sizeof(float) * 4 - 1;  // bfloat16 rows are stored 8 bytes at a time: covered as well
  return (a.n_out % 16) == 0 && (a.ldo % 4) == 0 &&
         ((((size_t)a.bias) | ((size_t)a.colsum) | ((size_t)a.out)) & align) == 0;
}
