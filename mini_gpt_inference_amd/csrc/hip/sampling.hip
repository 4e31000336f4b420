// Next-token choice from 32-bit logits: one workgroup per row.
//
// Order of operations as the reference (src/minigpt_infer/sampling.py:97-137,
// src/minigpt_infer/engine/engine.py:154-159): ids at or above real_vocab are
// never chosen; temperature <= 0 takes the argmax of the unscaled logits (the
// lowest index among equals); otherwise s = logits / max(T, 1e-6); top-k keeps
// the values >= the k-th largest (ties pass, sampling.py:39-52); top-p keeps a
// token iff the probability mass of the strictly larger ones is <= p, so the
// largest always stays (sampling.py:55-76); then a softmax over what is left.
//
// Where the reference draws with torch.multinomial from one shared generator,
// this draws by inverse CDF in vocabulary order with a uniform number that is a
// pure function of (engine seed, request seed, index of the output token), so a
// request's tokens do not depend on batching or preemption.
#include "common.h"
#include "launchers.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / MGPT_WAVE)
static_assert(SAMPLE_WAVES <= 16, "the greedy path reduces the waves' results within one row of 16 lanes");

__device__ __forceinline__ unsigned int float_key(float f) {
  unsigned int u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // monotone: larger float -> larger key
}

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}

// uniform in [0, 1) with 24 bits
__device__ __forceinline__ float sample_uniform(uint64_t engine_seed, uint64_t request_seed,
                                                uint64_t index) {
  uint64_t z = engine_seed * 0x9E3779B97F4A7C15ull + request_seed * 0xD1B54A32D192ED03ull +
               index * 0x8CB92BA72F3D8DD7ull + 0x2545F4914F6CDD1Dull;
  z = mix64(mix64(z));
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__device__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < SAMPLE_WAVES; ++i) t += red[i];  // fixed order
  return t;
}

__device__ int block_sum_int(int v, int* red) {
  v = wave_sum_int(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  int t = 0;
  for (int i = 0; i < SAMPLE_WAVES; ++i) t += red[i];
  return t;
}

__device__ float block_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = -INFINITY;
  for (int i = 0; i < SAMPLE_WAVES; ++i) t = fmaxf(t, red[i]);
  return t;
}

// DPP move within rows of 16 lanes
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }

// (value, index) of the largest value, the lowest index among equals, over each row of 16 lanes;
// every lane of the row gets it.  Four DPP exchanges: neighbours, pairs, halves of 8, halves of 16.
__device__ __forceinline__ void argmax_rows16(float& best, int& best_i) {
#define ARGMAX_STEP(CTRL)                                                         \
  {                                                                               \
    const float ov = __int_as_float(dpp_i<CTRL>(__float_as_int(best)));           \
    const int oi = dpp_i<CTRL>(best_i);                                           \
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }     \
  }
  ARGMAX_STEP(0xB1)   // quad_perm [1,0,3,2]
  ARGMAX_STEP(0x4E)   // quad_perm [2,3,0,1]
  ARGMAX_STEP(0x141)  // row_half_mirror
  ARGMAX_STEP(0x140)  // row_mirror
#undef ARGMAX_STEP
}

// Calls f(index, value) for every logit below nv, each thread taking indices 1024 apart.  When the
// row is 16-byte aligned the loads are four floats wide and eight of them are issued before any
// is used, so one pass over the vocabulary costs a few memory latencies, not one per element.
template <typename F>
__device__ __forceinline__ void scan_row(const float* __restrict__ lg, int nv, F f) {
  const int tid = threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(lg) & 15) == 0) {
    const int n4 = nv >> 2;
    const float4* lg4 = reinterpret_cast<const float4*>(lg);
    constexpr int U = 16;
    for (int base = tid; base < n4; base += SAMPLE_THREADS * U) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i4 = base + u * SAMPLE_THREADS;
        v[u] = lg4[i4 < n4 ? i4 : base];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i4 = base + u * SAMPLE_THREADS;
        if (i4 < n4) {
          f(4 * i4, v[u].x);
          f(4 * i4 + 1, v[u].y);
          f(4 * i4 + 2, v[u].z);
          f(4 * i4 + 3, v[u].w);
        }
      }
    }
    const int i = 4 * n4 + tid;
    if (i < nv) f(i, lg[i]);
  } else {
    for (int i = tid; i < nv; i += SAMPLE_THREADS) f(i, lg[i]);
  }
}

// After a decode-only step (token n is request n's one token and every row is sampled) the row's
// first thread can prepare the next step on the device: the sampled token becomes the next input,
// position, length and output index go up by one, the cache slot of the new position is looked up
// in the block tables (which already hold the pages of the steps planned ahead), and the token is
// also appended to the row's column of a history that the host reads once at the end.  Then
// several decode steps run back to back with no copy between them.  token_ids == nullptr: off.
struct AdvanceArgs {
  int* token_ids;
  int* positions;
  int* seq_lens;
  int* out_index;
  const int* q_req;         // -1: a padded row, left alone
  int* slot_mapping;        // [n_groups][n_stride]
  const int* block_tables;  // [n_groups][r_stride][max_blocks]
  const int* page_sizes;    // [n_groups]
  int n_groups, n_stride, r_stride, max_blocks;
  int* history;             // [history_rows][history_stride]
  int* history_pos;         // per row: how many tokens it has appended
  int history_rows, history_stride;
};

// What the row's first thread reads for that, asked for at the kernel's start: none of it depends on the
// token, and two of the loads depend on each other (the position, then the block table's entry), so
// behind the choice they would be two trips to memory more.
#define SAMPLE_ADV_GROUPS 4   // cache groups whose slots are looked up ahead; more are looked up at the end
struct AdvanceAhead {
  bool live;
  int pos, seq_len, out_index, history_pos;
  int slot[SAMPLE_ADV_GROUPS];
};

__device__ __forceinline__ int advance_slot(int row, int pos, int g, const AdvanceArgs& adv) {
  const int ps = adv.page_sizes[g];
  const int idx = pos / ps;
  const int page = idx < adv.max_blocks ? adv.block_tables[((long)g * adv.r_stride + row) * adv.max_blocks + idx] : -1;
  return page >= 0 ? page * ps + pos % ps : -1;
}

__device__ __forceinline__ AdvanceAhead look_ahead(int row, const AdvanceArgs& adv) {
  AdvanceAhead a;
  a.live = adv.token_ids != nullptr && adv.q_req[row] >= 0;
  a.pos = a.seq_len = a.out_index = a.history_pos = 0;
#pragma unroll
  for (int g = 0; g < SAMPLE_ADV_GROUPS; ++g) a.slot[g] = -1;
  if (!a.live) return a;
  a.pos = adv.positions[row] + 1;
  a.seq_len = adv.seq_lens[row] + 1;
  a.out_index = adv.out_index[row] + 1;
  a.history_pos = adv.history_pos[row];
#pragma unroll
  for (int g = 0; g < SAMPLE_ADV_GROUPS; ++g)
    if (g < adv.n_groups) a.slot[g] = advance_slot(row, a.pos, g, adv);
  return a;
}

__device__ __forceinline__ void finish_row(int row, int token, int* out_tokens, const AdvanceArgs& adv,
                                           const AdvanceAhead& ahead) {
  out_tokens[row] = token;
  if (!ahead.live) return;
  adv.token_ids[row] = token;
  adv.positions[row] = ahead.pos;
  adv.seq_lens[row] = ahead.seq_len;
  adv.out_index[row] = ahead.out_index;
#pragma unroll
  for (int g = 0; g < SAMPLE_ADV_GROUPS; ++g)
    if (g < adv.n_groups) adv.slot_mapping[(long)g * adv.n_stride + row] = ahead.slot[g];
  for (int g = SAMPLE_ADV_GROUPS; g < adv.n_groups; ++g)
    adv.slot_mapping[(long)g * adv.n_stride + row] = advance_slot(row, ahead.pos, g, adv);
  const int j = ahead.history_pos;
  if (j < adv.history_rows) adv.history[(long)j * adv.history_stride + row] = token;
  adv.history_pos[row] = j + 1;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, long ld, int vocab, int real_vocab,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const uint64_t* __restrict__ request_seed,
    const int* out_index, uint64_t engine_seed, int* out_tokens, AdvanceArgs adv,
    const float* __restrict__ tile_best, const int* __restrict__ tile_best_idx, int n_tiles) {
  __shared__ float red_f[SAMPLE_WAVES];
  __shared__ int red_i[SAMPLE_WAVES];
  __shared__ float part[SAMPLE_THREADS];
  __shared__ float wave_off[SAMPLE_WAVES + 1];
  __shared__ int chosen;

  const int row = blockIdx.x, tid = threadIdx.x;
  AdvanceAhead ahead;
  ahead.live = false;
  if (tid == 0) ahead = look_ahead(row, adv);
  const float* lg = logits + (long)row * ld;
  const int nv = real_vocab < vocab ? real_vocab : vocab;
  const float temp = temperature[row];

  if (temp <= 0.f) {
    // argmax, the lowest index among equals.  A thread meets its indices in rising order, so a
    // strictly larger value is all it has to look for; four logits are compared as their maximum.
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    if (tile_best != nullptr) {
      // the kernel that made the logits has left every tile's best (mgpt_linear_head_best, which
      // already kept to the columns below real_vocab): a few kilobytes to read instead of the row
      const float* tb = tile_best + (long)row * n_tiles;
      const int* ti = tile_best_idx + (long)row * n_tiles;
      constexpr int U = 4;
      for (int base = tid; base < n_tiles; base += SAMPLE_THREADS * U) {
        float v[U];
        int ix[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = base + u * SAMPLE_THREADS;
          v[u] = tb[i < n_tiles ? i : base];
          ix[u] = ti[i < n_tiles ? i : base];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (base + u * SAMPLE_THREADS < n_tiles && v[u] > best) { best = v[u]; best_i = ix[u]; }
      }
    } else if ((reinterpret_cast<uintptr_t>(lg) & 15) == 0) {
      const int n4 = nv >> 2;
      const float4* lg4 = reinterpret_cast<const float4*>(lg);
      constexpr int U = 16;  // loads in flight per thread: one pass covers 64 Ki logits
      for (int base = tid; base < n4; base += SAMPLE_THREADS * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i4 = base + u * SAMPLE_THREADS;
          v[u] = lg4[i4 < n4 ? i4 : base];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i4 = base + u * SAMPLE_THREADS;
          const float m = fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w));
          if (i4 < n4 && m > best) {
            best = m;
            best_i = 4 * i4 + (v[u].x == m ? 0 : (v[u].y == m ? 1 : (v[u].z == m ? 2 : 3)));
          }
        }
      }
      const int i = 4 * n4 + tid;  // the row's last one to three logits
      if (i < nv && lg[i] > best) { best = lg[i]; best_i = i; }
    } else {
      for (int i = tid; i < nv; i += SAMPLE_THREADS)
        if (lg[i] > best) { best = lg[i]; best_i = i; }
    }
    // NaN-free rows always have a candidate; a row of -inf falls back to index 0
    argmax_rows16(best, best_i);
    // lanes 0, 16, 32, 48 hold their rows' best: the wave's best through scalar registers
    {
      float wb = best;
      int wi = best_i;
#pragma unroll
      for (int r = 1; r < 4; ++r) {
        const float ov = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(best), 16 * r));
        const int oi = __builtin_amdgcn_readlane(best_i, 16 * r);
        if (ov > wb || (ov == wb && oi < wi)) { wb = ov; wi = oi; }
      }
      best = wb;  // right in lane 0 (and in every lane of the first row)
      best_i = wi;
    }
    if ((tid & 63) == 0) { red_f[tid >> 6] = best; red_i[tid >> 6] = best_i; }
    __syncthreads();
    if (tid < MGPT_WAVE) {
      // the sixteen waves' results, one per lane of the first row, reduced the same way
      best = tid < SAMPLE_WAVES ? red_f[tid] : -INFINITY;
      best_i = tid < SAMPLE_WAVES ? red_i[tid] : 0x7fffffff;
      argmax_rows16(best, best_i);
    }
    if (tid == 0) finish_row(row, best_i == 0x7fffffff ? 0 : best_i, out_tokens, adv, ahead);
    return;
  }

  const float t_safe = fmaxf(temp, 1e-6f);
  // largest scaled logit
  float mx = -INFINITY;
  scan_row(lg, nv, [&](int, float v) { mx = fmaxf(mx, v / t_safe); });
  mx = block_max(mx, red_f);

  // top-k: key of the k-th largest value, by bisection on the ordered bit pattern
  unsigned int key_floor = 0u;  // keep keys >= key_floor
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < nv) {
    unsigned int lo = 0u, hi = 0xffffffffu;  // invariant: count(key >= lo) >= k
    while (lo < hi) {
      unsigned int mid = lo + (unsigned int)(((uint64_t)hi - lo + 1) >> 1);
      int cnt = 0;
      scan_row(lg, nv, [&](int, float v) { cnt += float_key(v / t_safe) >= mid; });
      cnt = block_sum_int(cnt, red_i);
      if (cnt >= k) lo = mid; else hi = mid - 1;
    }
    key_floor = lo;
  }

  // top-p: smallest key kappa with mass(key > kappa) <= p * Z
  const float p = top_p ? top_p[row] : 1.0f;
  if (p < 1.0f) {
    float z = 0.f;
    scan_row(lg, nv, [&](int, float v) {
      const float s = v / t_safe;
      if (float_key(s) >= key_floor) z += expf(s - mx);
    });
    z = block_sum(z, red_f);
    const float budget = p * z;
    unsigned int lo = key_floor, hi = float_key(mx);  // G(hi) = 0 <= budget always
    while (lo < hi) {
      unsigned int mid = lo + ((hi - lo) >> 1);
      float g = 0.f;
      scan_row(lg, nv, [&](int, float v) {
        const float s = v / t_safe;
        const unsigned int key = float_key(s);
        if (key > mid && key >= key_floor) g += expf(s - mx);
      });
      g = block_sum(g, red_f);
      if (g <= budget) hi = mid; else lo = mid + 1;
    }
    key_floor = lo;
  }

  // inverse CDF in vocabulary order over what is kept
  const int per = (nv + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int i0 = tid * per, i1 = (i0 + per < nv) ? i0 + per : nv;
  float mine = 0.f;
  int last_kept = -1;
  for (int i = i0; i < i1; ++i) {
    float s = lg[i] / t_safe;
    if (float_key(s) >= key_floor) { mine += expf(s - mx); last_kept = i; }
  }
  part[tid] = mine;
  if (tid == 0) chosen = 0x7fffffff;
  __syncthreads();
  // serial scans keep the prefix sums monotone
  if ((tid & 63) == 0) {
    float run = 0.f;
    for (int i = 0; i < MGPT_WAVE; ++i) { run += part[tid + i]; part[tid + i] = run; }
  }
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    wave_off[0] = 0.f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) { run += part[w * MGPT_WAVE + MGPT_WAVE - 1]; wave_off[w + 1] = run; }
  }
  __syncthreads();
  const float total = wave_off[SAMPLE_WAVES];
  const float u = sample_uniform(engine_seed, request_seed ? request_seed[row] : 0ull,
                                 (uint64_t)(out_index ? out_index[row] : 0));
  const float target = u * total;
  const int w = tid >> 6;
  const float incl = wave_off[w] + part[tid];
  const float excl = (tid & 63) ? wave_off[w] + part[tid - 1] : wave_off[w];
  if (mine > 0.f && excl <= target && target < incl) {
    float run = excl;
    int pick = last_kept;
    for (int i = i0; i < i1; ++i) {
      float s = lg[i] / t_safe;
      if (float_key(s) >= key_floor) {
        run += expf(s - mx);
        if (run > target) { pick = i; break; }
      }
    }
    atomicMin(&chosen, pick);
  }
  // rounding can leave target >= total: then the last kept id stands
  int lk = last_kept;
  for (int off = 32; off > 0; off >>= 1) lk = max(lk, __shfl_xor(lk, off, MGPT_WAVE));
  __syncthreads();
  if ((tid & 63) == 0) red_i[tid >> 6] = lk;
  __syncthreads();
  if (tid == 0) {
    int c = chosen;
    if (c == 0x7fffffff) {
      c = 0;
      for (int i = 0; i < SAMPLE_WAVES; ++i) c = max(c, red_i[i]);
    }
    finish_row(row, c, out_tokens, adv, ahead);
  }
}

// logits: [n_rows, vocab] floats with row stride ld.  top_k (0 = off), top_p (1 = off),
// request_seed and out_index may be null.  tile_best, tile_best_idx [n_rows][n_tiles] (optional): what
// mgpt_linear_head_best left beside these logits with best_limit = real_vocab; greedy rows then read
// those instead of the logits.
static int launch_sample(const float* logits, long ld, int n_rows, int vocab, int real_vocab,
                         const float* temperature, const int* top_k, const float* top_p,
                         const uint64_t* request_seed, const int* out_index, uint64_t engine_seed,
                         int* out_tokens, const AdvanceArgs& adv, const float* tile_best,
                         const int* tile_best_idx, int n_tiles, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!logits || !temperature || !out_tokens) return MGPT_ERR_NULL;
  if (n_rows < 0 || vocab <= 0 || real_vocab <= 0 || ld < vocab) return MGPT_ERR_BAD_SHAPE;
  if (tile_best && (!tile_best_idx || n_tiles <= 0)) return MGPT_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, ld, vocab,
                     real_vocab, temperature, top_k, top_p, request_seed, out_index, engine_seed,
                     out_tokens, adv, tile_best, tile_best_idx, n_tiles);
  return mgpt_last_error();
}

extern "C" int mgpt_sample(const float* logits, long ld, int n_rows, int vocab, int real_vocab,
                           const float* temperature, const int* top_k, const float* top_p,
                           const uint64_t* request_seed, const int* out_index, uint64_t engine_seed,
                           int* out_tokens, const float* tile_best, const int* tile_best_idx, int n_tiles,
                           hipStream_t stream) {
  AdvanceArgs adv = {};
  return launch_sample(logits, ld, n_rows, vocab, real_vocab, temperature, top_k, top_p, request_seed,
                       out_index, engine_seed, out_tokens, adv, tile_best, tile_best_idx, n_tiles, stream);
}

// mgpt_sample, then each row prepares the next decode step on the device (AdvanceArgs above).
// Rows are requests: n_rows <= n_stride, r_stride.
extern "C" int mgpt_sample_advance(const float* logits, long ld, int n_rows, int vocab, int real_vocab,
                                   const float* temperature, const int* top_k, const float* top_p,
                                   const uint64_t* request_seed, int* out_index, uint64_t engine_seed,
                                   int* out_tokens, int* token_ids, int* positions, int* seq_lens,
                                   const int* q_req, int* slot_mapping, const int* block_tables,
                                   const int* page_sizes, int n_groups, int n_stride, int r_stride,
                                   int max_blocks, int* history, int* history_pos, int history_rows,
                                   int history_stride, const float* tile_best, const int* tile_best_idx,
                                   int n_tiles, hipStream_t stream) {
  if (!token_ids || !positions || !seq_lens || !out_index || !q_req || !slot_mapping || !block_tables ||
      !page_sizes || !history || !history_pos)
    return MGPT_ERR_NULL;
  if (n_groups <= 0 || n_rows > n_stride || n_rows > r_stride || max_blocks <= 0 || history_rows <= 0 ||
      history_stride < n_rows)
    return MGPT_ERR_BAD_SHAPE;
  AdvanceArgs adv = {token_ids, positions, seq_lens, out_index, q_req, slot_mapping, block_tables, page_sizes,
                     n_groups, n_stride, r_stride, max_blocks, history, history_pos, history_rows, history_stride};
  return launch_sample(logits, ld, n_rows, vocab, real_vocab, temperature, top_k, top_p, request_seed,
                       out_index, engine_seed, out_tokens, adv, tile_best, tile_best_idx, n_tiles, stream);
}
