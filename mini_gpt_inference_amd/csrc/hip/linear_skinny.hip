// Matrix product for few rows (a decode step: 1..64 tokens) in bfloat16 on the MFMA units: the
// general kernel, for every inner size that is a multiple of 16 and any alignment.  Shapes that
// linear_decode.hip takes (inner sizes that are multiples of 32) go there from this file's
// launcher.
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
// Reading the residual stream through a LayerNorm (src/minigpt_infer/model.py:113-114,186-187:
// every linear that reads the residual stream does): the LayerNorm's gain and bias are folded
// into W beforehand (fold_norm.hip), the kernel multiplies the raw float32 rows (rounded to
// bfloat16 on the way into the MFMA, with an optional gather of rows for the output head),
// gathers each row's sum and sum of squares from the very values it loads, and applies
// rstd * (acc - mean * S[o]) + b'[o] in the epilogue.  Nothing waits for the statistics.
// Epilogues: plain store (bfloat16 or float32), GELU-tanh, add into the float32
// residual stream, or store plus scatter of the key and value columns into
// their cache pages by slot_mapping (src/minigpt_infer/cache/paged.py:125-137).
#include "linear_skinny.h"

#include <mutex>
#include "launchers.h"

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
  float* red = reinterpret_cast<float*>(smem);   // [wave][NT][4 sums (+ 2 statistics)][64 lanes]
  constexpr int RED_PER = LN ? 6 : 4;

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
  // folded LayerNorm: sums of (x - x0) and (x - x0)^2 over what this lane loads of its rows
  float x0[NT], sd[NT], sq[NT];
  const float* xrow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    sd[t] = sq[t] = x0[t] = 0.f;
    xrow[t] = nullptr;
    if (LN) {
      const int n = t * 16 + lrow;
      const int src = n < a.n_rows ? (a.rows ? a.rows[n] : n) : 0;
      xrow[t] = a.x + (long)src * K;
      // the shift of a row: the median of three of its values, so that one channel that stands
      // far out (residual streams have such) does not become the shift
      x0[t] = __builtin_amdgcn_fmed3f(xrow[t][0], xrow[t][K >> 1], xrow[t][K - 1]);
    }
  }
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
  auto load_a = [&](bf16x8_t (&dst)[NT][SK_BATCH], int sb, bool stats) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = t * 16 + lrow;
      const bool n_ok = n < a.n_rows;
      if (LN) {
        float4 lo[SK_BATCH], hi[SK_BATCH];
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i) {
          const int k0 = k_begin + (sb + i) * 32 + lk;
          const bool ok = (sb + i) < steps && k0 + 8 <= k_end;
          const float4* p = reinterpret_cast<const float4*>(xrow[t] + (ok ? k0 : 0));
          lo[i] = p[0];
          hi[i] = p[1];
        }
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i) {
          const int k0 = k_begin + (sb + i) * 32 + lk;
          const bool ok = n_ok && (sb + i) < steps && k0 + 8 <= k_end;
          const float f[8] = {lo[i].x, lo[i].y, lo[i].z, lo[i].w, hi[i].x, hi[i].y, hi[i].z, hi[i].w};
          bf16x8_t v;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            // what is rounded to bfloat16 is the distance from the row's first value: a row far from
            // zero loses nothing to its offset (the epilogue corrects with the mean of the distances)
            v[e] = (short)float_to_bf16(f[e] - x0[t]);
            if (ok && stats) {
              const float d = f[e] - x0[t];
              sd[t] += d;
              sq[t] = fmaf(d, d, sq[t]);
            }
          }
          dst[t][i] = ok ? v : zero8;
        }
      } else {
        const bf16_t* ap = a.act + (long)(n_ok ? n : 0) * a.lda;
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i) {
          const int k0 = k_begin + (sb + i) * 32 + lk;
          const bool ok = n_ok && (sb + i) < steps && k0 + 8 <= k_end;
          const bf16x8_t v = load8(ap + (ok ? k0 : 0));
          dst[t][i] = ok ? v : zero8;
        }
      }
    }
  };

  int group = blockIdx.x;
  // When a wave's k range fits one batch its activations are loaded once and serve every column
  // group the workgroup walks; the next group's W is then in flight while this one is multiplied.
  const bool one_batch = steps <= SK_BATCH;
  if (group < n_groups) {
    load_w(wv, (group * cw_per_wg + cw) * 16, 0);
    load_a(av, 0, true);
  }
  for (bool first = true; group < n_groups; group += gridDim.x, first = false) {
    const int o0 = (group * cw_per_wg + cw) * 16;
    f32x4_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    if (one_batch) {
      const int next = group + gridDim.x;
      if (next < n_groups) load_w(wn, (next * cw_per_wg + cw) * 16, 0);
#pragma unroll
      for (int i = 0; i < SK_BATCH; ++i)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], av[t][i], acc[t], 0, 0, 0);
      if (next < n_groups) {
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i) wv[i] = wn[i];
      }
    } else {
      if (!first) {
        load_w(wv, o0, 0);
        load_a(av, 0, false);
      }
      for (int sb = 0; sb < steps; sb += SK_BATCH) {
        const bool more = sb + SK_BATCH < steps;
        if (more) {
          load_w(wn, o0, sb + SK_BATCH);
          load_a(an, sb + SK_BATCH, first);
        }
#pragma unroll
        for (int i = 0; i < SK_BATCH; ++i)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], av[t][i], acc[t], 0, 0, 0);
        if (more) {
#pragma unroll
          for (int i = 0; i < SK_BATCH; ++i) {
            wv[i] = wn[i];
#pragma unroll
            for (int t = 0; t < NT; ++t) av[t][i] = an[t][i];
          }
        }
      }
    }
    if (LN && first) {
      // the four lanes that share a row hold parts of its sums: add them
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        sd[t] += __shfl_xor(sd[t], 16, 64);
        sd[t] += __shfl_xor(sd[t], 32, 64);
        sq[t] += __shfl_xor(sq[t], 16, 64);
        sq[t] += __shfl_xor(sq[t], 32, 64);
      }
    }

    // waves that split k hand their sums to the first of them, which adds in wave order
    if (ks > 1) {
      if (!first) __syncthreads();  // the previous group's sums have been read
      if (kw > 0) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
#pragma unroll
          for (int i = 0; i < 4; ++i) red[((wave * NT + t) * RED_PER + i) * 64 + lane] = acc[t][i];
          if (LN && first) {
            red[((wave * NT + t) * RED_PER + 4) * 64 + lane] = sd[t];
            red[((wave * NT + t) * RED_PER + 5) * 64 + lane] = sq[t];
          }
        }
      }
      __syncthreads();
      if (kw == 0) {
        for (int s = 1; s < ks; ++s)
#pragma unroll
          for (int t = 0; t < NT; ++t) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][i] += red[(((wave + s) * NT + t) * RED_PER + i) * 64 + lane];
            if (LN && first) {
              sd[t] += red[(((wave + s) * NT + t) * RED_PER + 4) * 64 + lane];
              sq[t] += red[(((wave + s) * NT + t) * RED_PER + 5) * 64 + lane];
            }
          }
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
      float md = 0.f, rstd = 1.f;
      if (LN) {
        md = sd[t] / (float)K;   // mean of x - x0, and the products were of x - x0 as well
        rstd = 1.0f / sqrtf(fmaxf(sq[t] / (float)K - md * md, 0.f) + a.eps);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[t][i];
        if (LN && oc + i < a.n_out) v[i] = rstd * (v[i] - md * a.colsum[oc + i]);
        if (a.bias && oc + i < a.n_out) v[i] += a.bias[oc + i];
        if (EPI == SK_EPI_GELU) v[i] = gelu_tanh_fast(v[i]);
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
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
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
          pk.x = pack_bf16x2(v[0], v[1]);
          pk.y = pack_bf16x2(v[2], v[3]);
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

// With x given (then act is ignored) the rows are read from the float32 residual stream through
// a LayerNorm whose gain and bias were folded into w, bias and colsum (fold_norm.hip); otherwise
// act holds bfloat16 activations.  Refuses (MGPT_ERR_BAD_SHAPE) more than 64 rows and k_dim that
// is no multiple of 16; the caller then takes the general kernels.  mode: 0 = the launcher chooses;
// 1 keeps to this file's kernel also where linear_decode.hip would take the shape; SK_ROWS_SHARE_W
// and SK_ROWS_GROUPS say how linear_decode.hip treats more than 16 rows (see there); 16, 8, 4, 2 or 1 in
// the bits above the lowest eight fix the rows it gives a workgroup of one tile.  w_packed: optional, the
// same matrix in mgpt_pack_weight's layout (only linear_decode.hip reads it).  partials: optional scratch of
// mgpt_linear_skinny_partials(...) floats; with it a long inner size with many rows is split over
// workgroups (two launches).
static int linear_skinny_launch(const void* act, long lda, const float* x, const int* rows,
                                const float* colsum, float eps, const void* w, const void* w_packed,
                                const float* bias, void* out, int out_dtype, long ldo, int n_rows,
                                int n_out, int k_dim, int epilogue, void* kpool, void* vpool,
                                const int* slot_mapping, int q_width, int kv_width, int head_dim,
                                int n_kv_head, int page_size, int mode, float* partials,
                                long partials_floats, float* best_val, int* best_idx, int best_limit,
                                hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!w || !out || (!act && !x)) return MGPT_ERR_NULL;
  if (n_rows < 0 || n_rows > 64 || n_out < 0 || k_dim <= 0 || (k_dim % 16) != 0 || ldo < n_out)
    return MGPT_ERR_BAD_SHAPE;
  const bool ln = x != nullptr;
  if (ln && !colsum) return MGPT_ERR_NULL;
  if (!ln && (lda < k_dim || (lda % 8) != 0)) return MGPT_ERR_BAD_SHAPE;
  // rows and matrix are loaded 16 bytes at a time
  if (((((size_t)act) | ((size_t)x) | ((size_t)w) | ((size_t)w_packed)) & 15) != 0) return MGPT_ERR_BAD_SHAPE;
  if (epilogue == SK_EPI_QKV) {
    if (!kpool || !vpool || !slot_mapping) return MGPT_ERR_NULL;
    if (head_dim <= 0 || (head_dim % 4) != 0 || (q_width % 4) != 0 || q_width + 2 * kv_width != n_out ||
        kv_width != n_kv_head * head_dim || page_size <= 0)
      return MGPT_ERR_BAD_SHAPE;
  }
  const int nt = (n_rows + 15) / 16;
  // Sixteen waves for long inner sizes, where splitting k sixteen ways keeps every wave's loads
  // to one batch (only with one row tile of bfloat16 activations: more need the registers).
  const int waves = (k_dim >= 1024 && nt == 1 && !ln) ? SK_LN_WAVES : SK_WAVES;
  // waves sharing a column tile: as many as keep every wave at least 128 k wide
  int ks = 1;
  const int tiles = (n_out + 15) / 16;
  // (a very wide output has waves enough without a split, and then needs no reduction through LDS)
  while (tiles < 1024 && ks < waves && (k_dim % (64 * ks)) == 0 && k_dim / (ks * 2) >= 128) ks *= 2;
  const int red_per = ln ? 6 : 4;
  size_t red_bytes = ks > 1 ? (size_t)waves * nt * red_per * 64 * sizeof(float) : 0;
  if (red_bytes > 64 * 1024) {  // give up the k split before giving up the kernel
    ks = 1;
    red_bytes = 0;
  }
  SkinnyArgs a;
  a.act = (const bf16_t*)act; a.lda = lda; a.x = x; a.rows = rows; a.colsum = colsum; a.eps = eps;
  a.w = (const bf16_t*)w; a.w_packed = (const bf16_t*)w_packed; a.bias = bias; a.out = out; a.ldo = ldo; a.n_rows = n_rows; a.n_out = n_out;
  a.k_dim = k_dim; a.ksplit = ks; a.kpool = (bf16_t*)kpool; a.vpool = (bf16_t*)vpool;
  a.slot_mapping = slot_mapping; a.q_width = q_width; a.kv_width = kv_width; a.head_dim = head_dim;
  a.n_kv_head = n_kv_head; a.page_size = page_size;
  a.best_val = best_val; a.best_idx = best_idx; a.best_limit = best_limit;
  a.bias_in_part0 = 0;
  // room for the parts of a split over workgroups, if the caller brought enough of it
  a.k_parts = 1;
  a.rows_mode = ((mode & 0xFF) == SK_ROWS_SHARE_W || (mode & 0xFF) == SK_ROWS_GROUPS) ? (mode & 0xFF) : 0;
  a.rows_per_group = mode >> 8;
  a.partials = (partials && partials_floats >= mgpt_linear_decode_partials(n_rows, n_out, k_dim, ln, epilogue,
                                                                           a.rows_mode))
                   ? partials : nullptr;
  if (mode != 1) {
    // the rows of a decode step: the kernel laid out for latency, where it takes the shape
    const int rc = mgpt_launch_linear_decode(a, epilogue, out_dtype, stream);
    if (rc != MGPT_ERR_BAD_SHAPE || best_val) return rc;
  }
  const int cw_per_wg = waves / ks;
  const int n_groups = (tiles + cw_per_wg - 1) / cw_per_wg;
  // few enough workgroups that each walks several column groups and reuses its activations
  dim3 grid(n_groups < 1024 ? n_groups : 1024);
  const size_t smem = red_bytes;
#define SK_NT(N)                                                                       \
  (ln ? launch_nt<N, true, SK_WAVES>(a, epilogue, out_dtype, grid, smem, stream)       \
      : launch_nt<N, false, SK_WAVES>(a, epilogue, out_dtype, grid, smem, stream))
  switch (nt) {
    case 1:
      if (waves == SK_LN_WAVES)
        return launch_nt<1, false, SK_LN_WAVES>(a, epilogue, out_dtype, grid, smem, stream);
      return SK_NT(1);
    case 2: return SK_NT(2);
    case 3: return SK_NT(3);
    default: return SK_NT(4);
  }
#undef SK_NT
}

extern "C" int mgpt_linear_skinny(const void* act, long lda, const float* x, const int* rows,
                                  const float* colsum, float eps, const void* w, const void* w_packed,
                                  const float* bias, void* out, int out_dtype, long ldo, int n_rows,
                                  int n_out, int k_dim, int epilogue, void* kpool, void* vpool,
                                  const int* slot_mapping, int q_width, int kv_width, int head_dim,
                                  int n_kv_head, int page_size, int mode, float* partials,
                                  long partials_floats, hipStream_t stream) {
  return linear_skinny_launch(act, lda, x, rows, colsum, eps, w, w_packed, bias, out, out_dtype, ldo, n_rows, n_out,
                              k_dim, epilogue, kpool, vpool, slot_mapping, q_width, kv_width, head_dim, n_kv_head,
                              page_size, mode, partials, partials_floats, nullptr, nullptr, 0, stream);
}

// The output head of a decode step: float32 logits for at most 16 rows, and with them, per row and
// tile of 16 columns, the largest logit among the columns below best_limit and its column
// (best_val, best_idx: [n_rows][n_out / 16]), so that a greedy choice need not read the logits again
// (mgpt_sample's best_* arguments).  Takes what linear_decode.hip takes with whole tiles and aligned
// rows; MGPT_ERR_BAD_SHAPE otherwise, having launched nothing (mgpt_linear_skinny then does the product).
// The tied head of src/minigpt_infer/model.py:128-130,187 before the argmax of sampling.py:97-103.
extern "C" int mgpt_linear_head_best(const void* act, long lda, const float* x, const int* rows,
                                     const float* colsum, float eps, const void* w, const void* w_packed,
                                     const float* bias, float* out, long ldo, int n_rows, int n_out, int k_dim,
                                     float* best_val, int* best_idx, int best_limit, hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!best_val || !best_idx) return MGPT_ERR_NULL;
  if (n_rows > 16 || (k_dim % 32) != 0 || (n_out % 16) != 0 || (ldo % 4) != 0 || best_limit <= 0 ||
      ((((size_t)out) | ((size_t)bias) | ((size_t)colsum)) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  return linear_skinny_launch(act, lda, x, rows, colsum, eps, w, w_packed, bias, out, MGPT_F32, ldo, n_rows, n_out,
                              k_dim, SK_EPI_NONE, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, 0, nullptr, 0, best_val,
                              best_idx, best_limit, stream);
}

// floats of scratch with which mgpt_linear_skinny splits this shape's inner size over workgroups; 0: it would not
extern "C" long mgpt_linear_skinny_partials(int n_rows, int n_out, int k_dim, int has_ln, int epilogue) {
  return mgpt_linear_decode_partials(n_rows, n_out, k_dim, has_ln != 0, epilogue, 0);
}

// 1 if mgpt_linear_skinny, left to choose, deals the rows of this shape out in groups of 16 (then a
// folded LayerNorm costs a workgroup no more than at 16 rows)
extern "C" int mgpt_linear_skinny_row_groups(int n_rows, int n_out, int k_dim) {
  return mgpt_linear_decode_row_groups(n_rows, n_out, k_dim, 0) ? 1 : 0;
}

// ---- the variant that allocates nothing (declared in linear_skinny.h)
static __device__ __align__(256) float scratch[MGPT_STATIC_SCRATCH_FLOATS];

#define MGPT_MAX_DEVICES 64
static float* scratch_of_device[MGPT_MAX_DEVICES];  // the array's address on each GPU, asked for once
static std::mutex scratch_mutex;

// The device address of `scratch` on the current GPU.  In host code the array's name is only a
// handle for the runtime, not an address a kernel could use: the address comes from
// hipGetSymbolAddress, and every GPU has its own.
static int static_scratch(float** ptr) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  if (dev < 0 || dev >= MGPT_MAX_DEVICES) return MGPT_ERR_TOO_LARGE;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_of_device[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!p) return MGPT_ERR_NULL;
    scratch_of_device[dev] = (float*)p;
  }
  *ptr = scratch_of_device[dev];
  return MGPT_OK;
}

extern "C" long mgpt_linear_skinny_static_scratch_floats() { return MGPT_STATIC_SCRATCH_FLOATS; }

extern "C" int mgpt_linear_skinny_static_scratch_init() {
  float* p = nullptr;
  return static_scratch(&p);
}

extern "C" int mgpt_linear_skinny_static_scratch(
    const void* act, long lda, const float* x, const int* rows, const float* colsum, float eps, const void* w,
    const void* w_packed, const float* bias, void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim,
    int epilogue, void* kpool, void* vpool, const int* slot_mapping, int q_width, int kv_width, int head_dim,
    int n_kv_head, int page_size, int mode, hipStream_t stream) {
  if (n_rows < 0 || n_rows > 64 || n_out < 0 || k_dim <= 0) return MGPT_ERR_BAD_SHAPE;
  const int rows_mode = ((mode & 0xFF) == SK_ROWS_SHARE_W || (mode & 0xFF) == SK_ROWS_GROUPS) ? (mode & 0xFF) : 0;
  const long need = mode == 1 ? 0 : mgpt_linear_decode_partials(n_rows, n_out, k_dim, x != nullptr, epilogue, rows_mode);
  if (need > MGPT_STATIC_SCRATCH_FLOATS) return MGPT_ERR_SCRATCH;
  float* partials = nullptr;
  if (need > 0) {
    const int rc = static_scratch(&partials);
    if (rc != MGPT_OK) return rc;
  }
  return mgpt_linear_skinny(act, lda, x, rows, colsum, eps, w, w_packed, bias, out, out_dtype, ldo, n_rows, n_out,
                            k_dim, epilogue, kpool, vpool, slot_mapping, q_width, kv_width, head_dim, n_kv_head,
                            page_size, mode, partials, need, stream);
}
