// Tiled bfloat16 matrix product on the MFMA units for many rows (prompt portions).
//
// out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]) with an optional GELU-tanh or
// residual-add epilogue: nn.Linear as in src/minigpt_infer/model.py:43-44,96-101.
//
// A workgroup of four waves owns a 128 x 128 (or, for small problems, 64 x 64)
// tile of the output; each wave a quarter of it, as 4 x 4 (2 x 2)
// v_mfma_f32_16x16x32_bf16 accumulators.  Per step of 32 along k the workgroup
// stages a slice (32 or 64 along k) of the activations and of W
// in LDS (rows padded by 16 bytes so the 16 rows a MFMA operand reads fall on
// distinct banks), with the global loads of the next two to four slices in
// flight while the current one is multiplied.  W is the first MFMA operand, so a lane ends up
// with four neighbouring output columns of one row and stores them as one
// vector.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define MM_EPI_NONE 0
#define MM_EPI_GELU 1
#define MM_EPI_RESIDUAL 2
#define MM_EPI_QKV 3   // store, and scatter the key and value columns into their cache pages

// where the key and value columns of a fused QKV product go (src/minigpt_infer/cache/paged.py:125-137)
struct MfmaScatter {
  bf16_t* kpool;
  bf16_t* vpool;
  const int* slot_mapping;  // per row: page * page_size + offset, or -1 for a padded row
  int q_width, kv_width, head_dim, n_kv_head, page_size;
};

// WT: 16-wide tiles per wave in each direction.  4 -> 128 x 128 per workgroup, 2 -> 64 x 64, 1 -> 32 x 32.
template <int WT, int EPI, typename OT>
__global__ __launch_bounds__(256) void linear_mfma_kernel(
    const bf16_t* __restrict__ act, long lda, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, OT* __restrict__ out, long ldo, int n_rows, int n_out, int k_dim,
    MfmaScatter sc) {
  constexpr int TILE = 2 * WT * 16;   // rows and columns of the workgroup's tile
  constexpr int MM_BK = WT == 4 ? 32 : 64;   // k per step: what fits LDS twice over
  constexpr int MM_LD = MM_BK + 8;           // LDS row stride in elements (16 bytes of padding)
  constexpr int TPR = MM_BK / 8;             // threads per staged row (16 bytes each)
  constexpr int RPP = 256 / TPR;             // rows per staging pass
  constexpr int PASSES = TILE / RPP;
  __shared__ __align__(16) bf16_t as[2][TILE * MM_LD];
  __shared__ __align__(16) bf16_t ws[2][TILE * MM_LD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // Workgroups go to the eight XCDs in turn by their id, and each XCD has an L2 of its own.  The ids
  // are therefore dealt out so that an XCD's workgroups are neighbours in tile order: they walk the
  // column tiles of the same few row tiles, whose activations then come from memory once instead
  // of once per XCD.
  int tile_id;
  {
    const int total = gridDim.x, pid = blockIdx.x;
    const int per_xcd = (total + 7) >> 3, tall = (total & 7) ? (total & 7) : 8;
    const int xcd = pid & 7, local = pid >> 3;
    tile_id = xcd < tall ? xcd * per_xcd + local : tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
  }
  const int col_tiles = (n_out + TILE - 1) / TILE;
  const int row0 = (tile_id / col_tiles) * TILE, col0 = (tile_id % col_tiles) * TILE;
  const int wr = (wave >> 1) * (WT * 16), wc = (wave & 1) * (WT * 16);  // this wave's quarter
  const int lrow = lane & 15, lk = (lane >> 4) * 8;

  // staging: thread t copies 16 bytes of rows (t / TPR) + RPP * pass, k offset (t % TPR) * 8
  const int srow = tid / TPR, sk = (tid % TPR) * 8;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // PD slices along k are on their way from memory at any time, each in registers of its own: with
  // few workgroups on a compute unit the latency of a load is what a step costs, and it is paid
  // once per PD - 1 steps
  constexpr int PD = WT == 4 ? 2 : 4;
  bf16x8_t ga[PD][PASSES], gw[PD][PASSES];

  // Rows past the end are read from the last row (their results are never stored), so that a
  // load's value is used only when the slice is multiplied: a select on it right after the load
  // would wait for it and leave nothing in flight.  Only a last, partial slice along k needs zeros.
  const bf16_t* ap[PASSES];
  const bf16_t* wp[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int r = srow + p * RPP;
    const int an = row0 + r < n_rows ? row0 + r : n_rows - 1;
    const int wo = col0 + r < n_out ? col0 + r : n_out - 1;
    ap[p] = act + (long)an * lda + sk;
    wp[p] = w + (long)wo * k_dim + sk;
  }
  auto load_global = [&](int set, int k0) {
    if (k0 + MM_BK <= k_dim) {
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        ga[set][p] = *reinterpret_cast<const bf16x8_t*>(ap[p] + k0);
        gw[set][p] = *reinterpret_cast<const bf16x8_t*>(wp[p] + k0);
      }
    } else {
      const bool k_ok = k0 + sk + 8 <= k_dim;
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        const bf16x8_t av = *reinterpret_cast<const bf16x8_t*>(ap[p] + (k_ok ? k0 : 0));
        const bf16x8_t wv = *reinterpret_cast<const bf16x8_t*>(wp[p] + (k_ok ? k0 : 0));
        ga[set][p] = k_ok ? av : zero8;
        gw[set][p] = k_ok ? wv : zero8;
      }
    }
  };
  auto store_lds = [&](int set, int buf) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int r = srow + p * RPP;
      *reinterpret_cast<bf16x8_t*>(&as[buf][r * MM_LD + sk]) = ga[set][p];
      *reinterpret_cast<bf16x8_t*>(&ws[buf][r * MM_LD + sk]) = gw[set][p];
    }
  };

  f32x4_t acc[WT][WT];  // [column tile of W][row tile of activations]
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int k_steps = (k_dim + MM_BK - 1) / MM_BK;
#pragma unroll
  for (int d = 0; d < PD; ++d)
    if (d < k_steps) load_global(d, d * MM_BK);
  store_lds(0, 0);
  __syncthreads();
  for (int s0 = 0; s0 < k_steps; s0 += PD) {
#pragma unroll
    for (int d = 0; d < PD; ++d) {
      const int s = s0 + d;  // this step's slice sat in register set d and is in LDS buffer s & 1 now
      if (s < k_steps) {
        const int buf = s & 1;
        if (s + PD < k_steps) load_global(d, (s + PD) * MM_BK);
#pragma unroll
        for (int kk = 0; kk < MM_BK; kk += 32) {
          bf16x8_t wf[WT], af[WT];
#pragma unroll
          for (int i = 0; i < WT; ++i) {
            wf[i] = *reinterpret_cast<const bf16x8_t*>(&ws[buf][(wc + i * 16 + lrow) * MM_LD + kk + lk]);
            af[i] = *reinterpret_cast<const bf16x8_t*>(&as[buf][(wr + i * 16 + lrow) * MM_LD + kk + lk]);
          }
#pragma unroll
          for (int i = 0; i < WT; ++i)
#pragma unroll
            for (int j = 0; j < WT; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < k_steps) {
          store_lds((d + 1) % PD, buf ^ 1);  // the other buffer: its readers finished before the last barrier
          __syncthreads();
        }
      }
    }
  }

  // lane holds out[row0 + wr + j*16 + (lane & 15)][col0 + wc + i*16 + (lane >> 4)*4 + e], e = 0..3
  const bool vec = (n_out & 3) == 0 && (ldo & 3) == 0 &&
                   (((size_t)out | (size_t)bias) & 15) == 0;  // the four columns as one aligned vector
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    const int oc = col0 + wc + i * 16 + (lane >> 4) * 4;
    if (oc >= n_out) continue;
    float b4[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
      if (vec) {
        const float4 t = *reinterpret_cast<const float4*>(bias + oc);
        b4[0] = t.x; b4[1] = t.y; b4[2] = t.z; b4[3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) b4[e] = oc + e < n_out ? bias[oc + e] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int n = row0 + wr + j * 16 + lrow;
      if (n >= n_rows) continue;
      OT* orow = out + (long)n * ldo;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = acc[i][j][e] + b4[e];
        if (EPI == MM_EPI_GELU) v[e] = gelu_tanh_fast(v[e]);
      }
      if (vec && sizeof(OT) == 4) {
        float4* dst = reinterpret_cast<float4*>(orow + oc);
        if (EPI == MM_EPI_RESIDUAL) {
          const float4 old = *dst;
          *dst = make_float4(old.x + v[0], old.y + v[1], old.z + v[2], old.w + v[3]);
        } else {
          *dst = make_float4(v[0], v[1], v[2], v[3]);
        }
      } else if (vec && EPI != MM_EPI_RESIDUAL) {
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>(orow + oc) = pk;
        if (EPI == MM_EPI_QKV && oc >= sc.q_width) {
          // the four columns lie in one head (the launcher checks that sizes are multiples of 4)
          const int slot = sc.slot_mapping[n];
          if (slot >= 0) {
            const long page = slot / sc.page_size;
            const int off = slot - (int)page * sc.page_size;
            const int c = oc - sc.q_width;  // column among keys then values
            const bool is_v = c >= sc.kv_width;
            const int cc = is_v ? c - sc.kv_width : c;
            const int h = cc / sc.head_dim, d = cc - h * sc.head_dim;
            const long dst = ((page * sc.n_kv_head + h) * sc.page_size + off) * (long)sc.head_dim + d;
            *reinterpret_cast<uint2*>((is_v ? sc.vpool : sc.kpool) + dst) = pk;
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int o = oc + e;
          if (o >= n_out) continue;
          if (EPI == MM_EPI_RESIDUAL) {
            orow[o] = from_float<OT>(to_float<OT>(orow[o]) + v[e]);
          } else {
            orow[o] = from_float<OT>(v[e]);
          }
        }
      }
    }
  }
}

template <int WT>
static int launch_tile(const void* act, long lda, const void* w, const float* bias, void* out, int out_dtype,
                       long ldo, int n_rows, int n_out, int k_dim, int epilogue, const MfmaScatter& sc,
                       hipStream_t stream) {
  constexpr int TILE = 2 * WT * 16;
  const long tiles = (long)((n_out + TILE - 1) / TILE) * ((n_rows + TILE - 1) / TILE);
  if (tiles > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  dim3 grid((unsigned int)tiles), block(256);
#define MM_LAUNCH(E, OT)                                                                               \
  hipLaunchKernelGGL((linear_mfma_kernel<WT, E, OT>), grid, block, 0, stream, (const bf16_t*)act, lda, \
                     (const bf16_t*)w, bias, (OT*)out, ldo, n_rows, n_out, k_dim, sc)
  if (epilogue == MM_EPI_NONE && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_NONE, bf16_t);
  else if (epilogue == MM_EPI_NONE && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_NONE, float);
  else if (epilogue == MM_EPI_GELU && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_GELU, bf16_t);
  else if (epilogue == MM_EPI_RESIDUAL && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_RESIDUAL, float);
  else if (epilogue == MM_EPI_QKV && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_QKV, bf16_t);
  else return MGPT_ERR_BAD_DTYPE;
#undef MM_LAUNCH
  return mgpt_last_error();
}

// act: [n_rows, k_dim] bfloat16 with row stride lda (a multiple of 8, 16-byte aligned base);
// w: [n_out, k_dim] dense bfloat16; out: [n_rows, n_out] with row stride ldo.  k_dim must be a
// multiple of 16.  Refuses other layouts with MGPT_ERR_BAD_SHAPE.
static int linear_mfma_any(const void* act, long lda, const void* w, const float* bias, void* out,
                           int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue,
                           const MfmaScatter& sc, hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!act || !w || !out) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_out < 0 || k_dim <= 0 || (k_dim % 16) != 0 || lda < k_dim || (lda % 8) != 0 ||
      ldo < n_out)
    return MGPT_ERR_BAD_SHAPE;
  // large tiles reuse operands better, small tiles fill the 256 compute units: take the large
  // ones only when they alone give every unit several workgroups
  const long big = (long)((n_out + 127) / 128) * ((n_rows + 127) / 128);
  if (big >= 384)
    return launch_tile<4>(act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue, sc, stream);
  // and tiles of 32 x 32 where the 64 x 64 ones would leave most of the units idle (a prompt
  // portion of a few hundred tokens)
  const long mid = (long)((n_out + 63) / 64) * ((n_rows + 63) / 64);
  if (mid < 192)
    return launch_tile<1>(act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue, sc, stream);
  return launch_tile<2>(act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue, sc, stream);
}

extern "C" int mgpt_linear_mfma(const void* act, long lda, const void* w, const float* bias, void* out,
                                int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue,
                                hipStream_t stream) {
  if (epilogue == MM_EPI_QKV) return MGPT_ERR_BAD_SHAPE;  // mgpt_linear_mfma_qkv brings the pools
  MfmaScatter sc = {};
  return linear_mfma_any(act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue, sc, stream);
}

// The fused QKV product of a step with prompt portions: out[n] = act[n] W^T + bias in bfloat16, and
// the key and value columns (after the first q_width) of every row with a slot also go into the
// cache pools [pages, n_kv_head, page_size, head_dim].  Refuses (MGPT_ERR_BAD_SHAPE) sizes that
// are no multiples of 4 and outputs that are not aligned for 8-byte stores.
extern "C" int mgpt_linear_mfma_qkv(const void* act, long lda, const void* w, const float* bias, void* out,
                                    long ldo, int n_rows, int n_out, int k_dim, void* kpool, void* vpool,
                                    const int* slot_mapping, int q_width, int kv_width, int head_dim,
                                    int n_kv_head, int page_size, hipStream_t stream) {
  if (!kpool || !vpool || !slot_mapping) return MGPT_ERR_NULL;
  if (head_dim <= 0 || (head_dim % 4) != 0 || (q_width % 4) != 0 || q_width + 2 * kv_width != n_out ||
      kv_width != n_kv_head * head_dim || page_size <= 0 || (n_out % 4) != 0 || (ldo % 4) != 0 ||
      (((size_t)out | (size_t)bias) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  MfmaScatter sc = {(bf16_t*)kpool, (bf16_t*)vpool, slot_mapping, q_width, kv_width, head_dim, n_kv_head, page_size};
  return linear_mfma_any(act, lda, w, bias, out, MGPT_BF16, ldo, n_rows, n_out, k_dim, MM_EPI_QKV, sc, stream);
}
