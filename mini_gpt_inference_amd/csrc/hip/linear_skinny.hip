// Matrix product for few rows (a decode step: 1..64 tokens) in bfloat16 on the MFMA units.
//
// out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]), nn.Linear as in
// src/minigpt_infer/model.py:43-44,96-101 of the reference.  With so few rows the
// work is streaming W once from HBM, so the kernel is laid out around that: a
// workgroup of four waves owns a strip of output columns, its waves split the
// strip and/or the k range, every lane keeps several 16-byte loads of W in
// flight, and one v_mfma_f32_16x16x32_bf16 per 32 k turns a 16-column tile of W
// and 16 rows of activations into float32 sums.  Waves that split k add their
// sums through LDS in a fixed order, so results do not depend on timing.
//
// Prologue (optional): LayerNorm of the float32 residual rows, statistics in
// float32, result in bfloat16 in LDS (src/minigpt_infer/model.py:113-114: every
// linear that reads the residual stream reads it through a LayerNorm), with an
// optional gather of rows (the logit rows of the output head).
// Epilogues: plain store (bfloat16 or float32), GELU-tanh, add into the float32
// residual stream, or store plus scatter of the key and value columns into
// their cache pages by slot_mapping (src/minigpt_infer/cache/paged.py:125-137).
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_EPI_NONE 0
#define SK_EPI_GELU 1
#define SK_EPI_RESIDUAL 2
#define SK_EPI_QKV 3

#define SK_WAVES 4        // waves of a workgroup without a prologue
#define SK_LN_WAVES 16    // waves of a workgroup with the LayerNorm prologue: one row each
#define SK_LN_MAX_PER_LANE 16  // a prologue row is held in registers: k_dim <= 64 * 32
#define SK_PAD 8  // bfloat16 elements of padding per LDS row: keeps the 16 rows a MFMA reads on distinct banks

struct SkinnyArgs {
  const bf16_t* act;  // [n_rows, k_dim] bfloat16, row stride lda (no prologue)
  long lda;
  const float* x;     // residual stream, float32, row stride k_dim (LayerNorm prologue)
  const int* rows;    // optional gather of residual rows
  const float* ln_w;
  const float* ln_b;
  float eps;
  const bf16_t* w;    // [n_out, k_dim]
  const float* bias;  // [n_out] or null
  void* out;          // [n_rows, n_out], row stride ldo
  long ldo;
  int n_rows, n_out, k_dim;
  int ksplit;         // waves of a workgroup that share a column tile: 1, 2 or 4
  // key/value scatter (SK_EPI_QKV)
  bf16_t* kpool;
  bf16_t* vpool;
  const int* slot_mapping;
  int q_width, kv_width, head_dim, n_kv_head, page_size;
};

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) {
  return *reinterpret_cast<const bf16x8_t*>(p);
}


template <int NT, bool LN, int WAVES, int EPI, typename OT>
__global__ __launch_bounds__(WAVES * 64) void linear_skinny_kernel(SkinnyArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int SK_BATCH = 4;  // k steps whose loads are issued together; the next batch is in flight meanwhile
  const int ks = a.ksplit, cw_per_wg = WAVES / ks;
  const int cw = wave / ks, kw = wave - cw * ks;
  const int K = a.k_dim;
  const int ldh = K + SK_PAD;
  bf16_t* hs = reinterpret_cast<bf16_t*>(smem);                       // [16][ldh] when LN
  float* red = reinterpret_cast<float*>(smem + (LN ? (size_t)16 * ldh * sizeof(bf16_t) : 0));

  // this wave's k range, in steps of 32
  const int k_per = ((K / ks + 31) / 32) * 32;
  const int k_begin = kw * k_per;
  const int k_end = (k_begin + k_per < K) ? k_begin + k_per : K;
  const int steps = (k_end - k_begin + 31) / 32;
  const int lrow = lane & 15, lk = (lane >> 4) * 8;
  const int tiles = (a.n_out + 15) / 16;
  const int n_groups = (tiles + cw_per_wg - 1) / cw_per_wg;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // Loads are unconditional (a lane that has nothing to load reads the start of its row and
  // discards it), so that a whole batch of them is in flight before the first is waited for.
  bf16x8_t wv[SK_BATCH], wn[SK_BATCH];
  bf16x8_t av[NT][SK_BATCH], an[NT][SK_BATCH];
  auto load_w = [&](bf16x8_t (&dst)[SK_BATCH], int o0, int sb) {
    const int wo = o0 + lrow;
    const bool w_ok = wo < a.n_out;
    const bf16_t* wp = a.w + (long)(w_ok ? wo : 0) * K;
#pragma unroll
    for (int i = 0; i < SK_BATCH; ++i) {
      const int k0 = k_begin + (sb + i) * 32 + lk;
      const bool ok = w_ok && (sb + i) < steps && k0 + 8 <= k_end;
      const bf16x8_t v = load8(wp + (ok ? k0 : 0));
      dst[i] = ok ? v : zero8;
    }
  };
  auto load_a = [&](bf16x8_t (&dst)[NT][SK_BATCH], int sb) {
    if (LN) return;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = t * 16 + lrow;
      const bool n_ok = n < a.n_rows;
      const bf16_t* ap = a.act + (long)(n_ok ? n : 0) * a.lda;
#pragma unroll
      for (int i = 0; i < SK_BATCH; ++i) {
        const int k0 = k_begin + (sb + i) * 32 + lk;
        const bool ok = n_ok && (sb + i) < steps && k0 + 8 <= k_end;
        const bf16x8_t v = load8(ap + (ok ? k0 : 0));
        dst[t][i] = ok ? v : zero8;
      }
    }
  };

  int group = blockIdx.x;
  // the first batch does not depend on the prologue: start it now
  load_w(wv, (group * cw_per_wg + cw) * 16, 0);
  load_a(av, 0);

  if (LN) {
    // LayerNorm of up to 16 rows, one wave per row, the row read once and kept in registers:
    // the mean, then together the centred sum of squares and what the mean lost to rounding.
    const int r = wave;
    bf16_t* hr = hs + (long)r * ldh;
    if (r < a.n_rows) {
      const float* xr = a.x + (long)(a.rows ? a.rows[r] : r) * K;
      float xv[SK_LN_MAX_PER_LANE], gw[SK_LN_MAX_PER_LANE], gb[SK_LN_MAX_PER_LANE];
#pragma unroll
      for (int i = 0; i < SK_LN_MAX_PER_LANE; ++i) {
        const int c = lane + i * 64;
        const bool ok = c < K;
        xv[i] = xr[ok ? c : 0];
        gw[i] = a.ln_w[ok ? c : 0];
        gb[i] = a.ln_b ? a.ln_b[ok ? c : 0] : 0.f;
      }
      float s0 = 0.f;
#pragma unroll
      for (int i = 0; i < SK_LN_MAX_PER_LANE; ++i) {
        if (lane + i * 64 >= K) xv[i] = 0.f;
        s0 += xv[i];
      }
      const float mean = wave_sum(s0) / (float)K;
      float e = 0.f, v2 = 0.f;
#pragma unroll
      for (int i = 0; i < SK_LN_MAX_PER_LANE; ++i) {
        const float d = (lane + i * 64 < K) ? xv[i] - mean : 0.f;
        xv[i] = d;
        e += d;
        v2 = fmaf(d, d, v2);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        e += __shfl_xor(e, off, 64);
        v2 += __shfl_xor(v2, off, 64);
      }
      const float corr = e / (float)K;  // what the mean lost to rounding, kept apart
      const float var = fmaxf(v2 / (float)K - corr * corr, 0.f);
      const float rstd = 1.0f / sqrtf(var + a.eps);
#pragma unroll
      for (int i = 0; i < SK_LN_MAX_PER_LANE; ++i) {
        const int c = lane + i * 64;
        if (c < K) hr[c] = float_to_bf16((xv[i] - corr) * rstd * gw[i] + gb[i]);
      }
    } else {
      for (int c = lane; c < K; c += 64) hr[c] = 0;
    }
    __syncthreads();
  }

  for (bool first = true; group < n_groups; group += gridDim.x, first = false) {
    const int o0 = (group * cw_per_wg + cw) * 16;
    f32x4_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    if (!first) {
      load_w(wv, o0, 0);
      load_a(av, 0);
    }
    for (int sb = 0; sb < steps; sb += SK_BATCH) {
      const bool more = sb + SK_BATCH < steps;
      if (more) {
        load_w(wn, o0, sb + SK_BATCH);
        load_a(an, sb + SK_BATCH);
      }
#pragma unroll
      for (int i = 0; i < SK_BATCH; ++i) {
        const int k0 = k_begin + (sb + i) * 32 + lk;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          bf16x8_t b;
          if (LN) {
            // rows of hs are readable up to K + SK_PAD; what lies past k_end meets zeros of W
            b = load8(hs + (long)(t * 16 + lrow) * ldh + ((sb + i) < steps && k0 + 8 <= k_end ? k0 : 0));
          } else {
            b = av[t][i];
          }
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], b, acc[t], 0, 0, 0);
        }
      }
      if (more) {
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i) {
          wv[i] = wn[i];
#pragma unroll
          for (int t = 0; t < NT; ++t) av[t][i] = an[t][i];
        }
      }
    }

    // waves that split k hand their sums to the first of them, which adds in wave order
    if (ks > 1) {
      if (!first) __syncthreads();  // the previous group's sums have been read
      if (kw > 0) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[((wave * NT + t) * 4 + i) * 64 + lane] = acc[t][i];
      }
      __syncthreads();
      if (kw == 0) {
        for (int s = 1; s < ks; ++s)
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][i] += red[(((wave + s) * NT + t) * 4 + i) * 64 + lane];
      }
    }
    if (kw != 0 || o0 >= a.n_out) continue;

    // lane holds out[n = t*16 + (lane & 15)][o0 + (lane >> 4) * 4 + i], i = 0..3
    const int oc = o0 + (lane >> 4) * 4;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = t * 16 + lrow;
      if (n >= a.n_rows) continue;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[t][i];
        if (a.bias && oc + i < a.n_out) v[i] += a.bias[oc + i];
        if (EPI == SK_EPI_GELU) v[i] = gelu_tanh(v[i]);
      }
      OT* orow = reinterpret_cast<OT*>(a.out) + (long)n * a.ldo;
      const bool whole = oc + 4 <= a.n_out && (a.ldo & 3) == 0;  // four columns, one aligned vector
      if (whole && sizeof(OT) == 4) {
        float4* dst = reinterpret_cast<float4*>(orow + oc);
        float4 r = make_float4(v[0], v[1], v[2], v[3]);
        if (EPI == SK_EPI_RESIDUAL) {
          const float4 old = *dst;
          r = make_float4(old.x + v[0], old.y + v[1], old.z + v[2], old.w + v[3]);
        }
        *dst = r;
      } else if (whole && EPI != SK_EPI_RESIDUAL) {
        uint2 pk;
        pk.x = (unsigned int)float_to_bf16(v[0]) | ((unsigned int)float_to_bf16(v[1]) << 16);
        pk.y = (unsigned int)float_to_bf16(v[2]) | ((unsigned int)float_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>(orow + oc) = pk;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (oc + i >= a.n_out) continue;
          if (EPI == SK_EPI_RESIDUAL) {
            orow[oc + i] = from_float<OT>(to_float<OT>(orow[oc + i]) + v[i]);
          } else {
            orow[oc + i] = from_float<OT>(v[i]);
          }
        }
      }
      if (EPI == SK_EPI_QKV) {
        const int slot = a.slot_mapping[n];
        if (slot >= 0 && oc >= a.q_width && oc < a.n_out) {
          // the four columns lie in one head (head sizes are multiples of 4): one 8-byte store
          const long page = slot / a.page_size;
          const int off = slot - (int)page * a.page_size;
          const int c = oc - a.q_width;  // column among keys then values
          const bool is_v = c >= a.kv_width;
          const int cc = is_v ? c - a.kv_width : c;
          const int h = cc / a.head_dim, d = cc - h * a.head_dim;
          const long dst = ((page * a.n_kv_head + h) * a.page_size + off) * (long)a.head_dim + d;
          uint2 pk;
          pk.x = (unsigned int)float_to_bf16(v[0]) | ((unsigned int)float_to_bf16(v[1]) << 16);
          pk.y = (unsigned int)float_to_bf16(v[2]) | ((unsigned int)float_to_bf16(v[3]) << 16);
          *reinterpret_cast<uint2*>((is_v ? a.vpool : a.kpool) + dst) = pk;
        }
      }
    }
  }
}

template <int NT, bool LN, int WAVES>
static int launch_nt(const SkinnyArgs& a, int epi, int out_dtype, dim3 grid, size_t smem, hipStream_t s) {
#define SK_LAUNCH(E, OT) \
  hipLaunchKernelGGL((linear_skinny_kernel<NT, LN, WAVES, E, OT>), grid, dim3(WAVES * 64), smem, s, a)
  if (epi == SK_EPI_NONE && out_dtype == MGPT_BF16) SK_LAUNCH(SK_EPI_NONE, bf16_t);
  else if (epi == SK_EPI_NONE && out_dtype == MGPT_F32) SK_LAUNCH(SK_EPI_NONE, float);
  else if (epi == SK_EPI_GELU && out_dtype == MGPT_BF16) SK_LAUNCH(SK_EPI_GELU, bf16_t);
  else if (epi == SK_EPI_RESIDUAL && out_dtype == MGPT_F32) SK_LAUNCH(SK_EPI_RESIDUAL, float);
  else if (epi == SK_EPI_QKV && out_dtype == MGPT_BF16) SK_LAUNCH(SK_EPI_QKV, bf16_t);
  else return MGPT_ERR_BAD_DTYPE;
#undef SK_LAUNCH
  return mgpt_last_error();
}

// LayerNorm prologue when x is given (then act is ignored), plain bfloat16 activations otherwise.
// Refuses (MGPT_ERR_BAD_SHAPE) more than 64 rows, k_dim that is no multiple of 16, and a LayerNorm
// prologue for more than 16 rows or rows that do not fit 64 KB of LDS; the caller then runs the
// LayerNorm by itself, or takes the general kernels.
extern "C" int mgpt_linear_skinny(const void* act, long lda, const float* x, const int* rows,
                                  const float* ln_w, const float* ln_b, float eps, const void* w,
                                  const float* bias, void* out, int out_dtype, long ldo, int n_rows,
                                  int n_out, int k_dim, int epilogue, void* kpool, void* vpool,
                                  const int* slot_mapping, int q_width, int kv_width, int head_dim,
                                  int n_kv_head, int page_size, hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!w || !out || (!act && !x)) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_rows > 64 || n_out < 0 || k_dim <= 0 || (k_dim % 16) != 0 || ldo < n_out)
    return MGPT_ERR_BAD_SHAPE;
  const bool ln = x != nullptr;
  if (ln && !ln_w) return MGPT_ERR_NULL;
  // the prologue normalises at most 16 rows (one per wave), each held in registers
  if (ln && (n_rows > 16 || k_dim > 64 * SK_LN_MAX_PER_LANE)) return MGPT_ERR_BAD_SHAPE;
  if (!ln && (lda < k_dim || (lda % 8) != 0)) return MGPT_ERR_BAD_SHAPE;
  if (epilogue == SK_EPI_QKV) {
    if (!kpool || !vpool || !slot_mapping) return MGPT_ERR_NULL;
    if (head_dim <= 0 || (head_dim % 4) != 0 || (q_width % 4) != 0 || q_width + 2 * kv_width != n_out ||
        kv_width != n_kv_head * head_dim || page_size <= 0)
      return MGPT_ERR_BAD_SHAPE;
  }
  const int nt = (n_rows + 15) / 16;
  // Sixteen waves with the prologue (one per row) and for long inner sizes, where splitting k
  // sixteen ways keeps every wave's loads to one batch; four otherwise.
  const int waves = (ln || (k_dim >= 1024 && nt <= 2)) ? SK_LN_WAVES : SK_WAVES;  // more row tiles need the registers
  // waves sharing a column tile: as many as keep every wave at least 128 k wide and the grid large
  int ks = 1;
  const int tiles = (n_out + 15) / 16;
  while (ks < waves && (k_dim % (64 * ks)) == 0 && k_dim / (ks * 2) >= 128 && tiles / (waves / ks) < 1024) ks *= 2;
  const size_t hs_bytes = ln ? (size_t)16 * (k_dim + SK_PAD) * sizeof(bf16_t) : 0;
  auto red_of = [&](int k) { return k > 1 ? (size_t)waves * nt * 4 * 64 * sizeof(float) : (size_t)0; };
  while (ks > 1 && hs_bytes + red_of(ks) > 64 * 1024) ks = 1;  // give up the k split before the kernel
  const size_t red_bytes = red_of(ks);
  if (hs_bytes + red_bytes > 64 * 1024) return MGPT_ERR_BAD_SHAPE;
  SkinnyArgs a;
  a.act = (const bf16_t*)act; a.lda = lda; a.x = x; a.rows = rows; a.ln_w = ln_w; a.ln_b = ln_b; a.eps = eps;
  a.w = (const bf16_t*)w; a.bias = bias; a.out = out; a.ldo = ldo; a.n_rows = n_rows; a.n_out = n_out;
  a.k_dim = k_dim; a.ksplit = ks; a.kpool = (bf16_t*)kpool; a.vpool = (bf16_t*)vpool;
  a.slot_mapping = slot_mapping; a.q_width = q_width; a.kv_width = kv_width; a.head_dim = head_dim;
  a.n_kv_head = n_kv_head; a.page_size = page_size;
  const int cw_per_wg = waves / ks;
  const int n_groups = (tiles + cw_per_wg - 1) / cw_per_wg;
  // with a prologue every workgroup repeats the LayerNorm, so few workgroups walk many column groups
  const int max_wg = ln ? 256 : 2048;
  dim3 grid(n_groups < max_wg ? n_groups : max_wg);
  const size_t smem = hs_bytes + red_bytes;
#define SK_NT(N)                                                                                   \
  (ln ? launch_nt<N, true, SK_LN_WAVES>(a, epilogue, out_dtype, grid, smem, stream)                \
      : (waves == SK_LN_WAVES ? launch_nt<N, false, SK_LN_WAVES>(a, epilogue, out_dtype, grid, smem, stream) \
                              : launch_nt<N, false, SK_WAVES>(a, epilogue, out_dtype, grid, smem, stream)))
  switch (nt) {
    case 1: return SK_NT(1);
    case 2: return SK_NT(2);
    case 3: return SK_NT(3);
    default: return SK_NT(4);
  }
#undef SK_NT
}
