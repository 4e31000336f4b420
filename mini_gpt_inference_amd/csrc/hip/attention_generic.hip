// Paged key/value store and the general paged causal attention kernel.
//
// A page pool of one cache slot holds keys (or values) as
//   [num_pages][n_kv_head][page_size][head_dim].
// New keys and values are stored after projection, unscaled, before attention
// reads them (reference: src/minigpt_infer/model.py:55-59,
// src/minigpt_infer/cache/paged.py:125-137).
//
// attention: S = q k^T * scale; a query at absolute position p sees the keys at
// positions max(0, p-window+1)..p of its own request (window 0 = all of them);
// softmax over keys in 32-bit; y = P v (reference: src/minigpt_infer/model.py:61-87,
// the rule col <= cache_len + row of src/minigpt_infer/batch.py:202-227).
//
// The general kernel runs one wave per (token, head).  Keys are reduced in
// chunks of 64 that start at absolute positions that are multiples of 64, so the
// order of the sums for a query depends only on its position, never on how the
// tokens were cut into steps or what else is in the batch.  Slots outside
// [begin, end) are never loaded.
#include "common.h"
#include "launchers.h"

template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ qkv, long ld, int k_off, int v_off,
                                T* __restrict__ kpool, T* __restrict__ vpool,
                                const int* __restrict__ slot_mapping, int n_tokens, int n_kv_head,
                                int head_dim, int page_size) {
  int n = blockIdx.x;
  if (n >= n_tokens) return;
  int slot = slot_mapping[n];
  if (slot < 0) return;  // padded row
  long page = slot / page_size;
  int off = slot - (int)page * page_size;
  const T* src = qkv + (long)n * ld;
  int width = n_kv_head * head_dim;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    int h = c / head_dim, d = c - h * head_dim;
    long dst = ((page * n_kv_head + h) * page_size + off) * (long)head_dim + d;
    kpool[dst] = src[k_off + c];
    vpool[dst] = src[v_off + c];
  }
}

extern "C" int mgpt_kv_write(const void* qkv, int dtype, long ld, int k_off, int v_off, void* kpool,
                             void* vpool, const int* slot_mapping, int n_tokens, int n_kv_head,
                             int head_dim, int page_size, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!qkv || !kpool || !vpool || !slot_mapping) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_kv_head <= 0 || head_dim <= 0 || page_size <= 0) return MGPT_ERR_BAD_SHAPE;
  int width = n_kv_head * head_dim;
  int threads = width >= 256 ? 256 : 64;
  if (dtype == MGPT_F32) {
    hipLaunchKernelGGL(kv_write_kernel<float>, dim3(n_tokens), dim3(threads), 0, stream,
                       (const float*)qkv, ld, k_off, v_off, (float*)kpool, (float*)vpool,
                       slot_mapping, n_tokens, n_kv_head, head_dim, page_size);
  } else if (dtype == MGPT_BF16) {
    hipLaunchKernelGGL(kv_write_kernel<bf16_t>, dim3(n_tokens), dim3(threads), 0, stream,
                       (const bf16_t*)qkv, ld, k_off, v_off, (bf16_t*)kpool, (bf16_t*)vpool,
                       slot_mapping, n_tokens, n_kv_head, head_dim, page_size);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
  return mgpt_last_error();
}

#define MAX_DPL 4  // head_dim <= 256

template <typename T, bool FAST_EXP>
__global__ __launch_bounds__(64) void paged_attention_generic_kernel(
    const T* __restrict__ q, long ldq, T* __restrict__ out, long ldo, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ cu_q, const int* __restrict__ seq_lens, const int* __restrict__ q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window) {
  __shared__ float q_s[MAX_DPL * MGPT_WAVE];
  __shared__ float p_s[MGPT_WAVE];
  __shared__ int page_s[MGPT_WAVE];

  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  if (n >= n_tokens) return;
  const int r = q_req[n];
  if (r < 0) return;  // padded token
  const int seq_len = seq_lens[r];
  const int q_start = cu_q[r], q_len = cu_q[r + 1] - q_start;
  const int qpos = seq_len - q_len + (n - q_start);
  const int kv_end = qpos + 1;
  const int kv_begin = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  const int hk = h / (n_head / n_kv_head);
  const int* bt = block_tables + (long)r * max_blocks;

  for (int d = lane; d < head_dim; d += MGPT_WAVE)
    q_s[d] = to_float<T>(q[(long)n * ldq + (long)h * head_dim + d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[MAX_DPL];
#pragma unroll
  for (int i = 0; i < MAX_DPL; ++i) acc[i] = 0.f;

  for (int c0 = (kv_begin / MGPT_WAVE) * MGPT_WAVE; c0 < kv_end; c0 += MGPT_WAVE) {
    const int j = c0 + lane;
    const bool valid = (j >= kv_begin) && (j < kv_end);
    float s = -INFINITY;
    int page = -1;
    if (valid) {
      page = bt[j / page_size];
      const int off = j % page_size;
      const T* kr = kpool + (((long)page * n_kv_head + hk) * page_size + off) * (long)head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(q_s[d], to_float<T>(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    float p = 0.f;
    if (valid) p = FAST_EXP ? __expf(s - m_new) : expf(s - m_new);
    const float alpha = (m == -INFINITY) ? 0.f : (FAST_EXP ? __expf(m - m_new) : expf(m - m_new));
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();  // previous chunk's readers of p_s / page_s are done
    p_s[lane] = p;
    page_s[lane] = page;
    __syncthreads();
    const int j_lo = (kv_begin > c0 ? kv_begin : c0) - c0;
    const int j_hi = (kv_end < c0 + MGPT_WAVE ? kv_end : c0 + MGPT_WAVE) - c0;
#pragma unroll
    for (int i = 0; i < MAX_DPL; ++i) {
      const int d = lane + i * MGPT_WAVE;
      if (d < head_dim) {
        float a = acc[i] * alpha;
        for (int jj = j_lo; jj < j_hi; ++jj) {
          const int off = (c0 + jj) % page_size;
          const T* vr = vpool + (((long)page_s[jj] * n_kv_head + hk) * page_size + off) * (long)head_dim;
          a = fmaf(p_s[jj], to_float<T>(vr[d]), a);
        }
        acc[i] = a;
      }
    }
  }
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAX_DPL; ++i) {
    const int d = lane + i * MGPT_WAVE;
    if (d < head_dim) out[(long)n * ldo + (long)h * head_dim + d] = from_float<T>(acc[i] * inv_l);
  }
}

// q: [n_tokens, n_head*head_dim] with row stride ldq; out likewise with ldo.
// q_req[t] = index of token t's request in this step (or -1 for a padded token),
// cu_q[r]..cu_q[r+1] = the tokens of request r, seq_lens[r] = its length after this step.
extern "C" int mgpt_paged_attention_generic(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int* q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    int dtype, int fast_exp, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !cu_q || !seq_lens || !q_req) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 || head_dim <= 0 ||
      head_dim > MAX_DPL * MGPT_WAVE || page_size <= 0 || max_blocks <= 0 || window < 0)
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid(n_tokens, n_head), block(MGPT_WAVE);
#define LAUNCH(T, F)                                                                              \
  hipLaunchKernelGGL((paged_attention_generic_kernel<T, F>), grid, block, 0, stream, (const T*)q, ldq, \
                     (T*)out, ldo, (const T*)kpool, (const T*)vpool, block_tables, max_blocks, cu_q,  \
                     seq_lens, q_req, n_tokens, n_head, n_kv_head, head_dim, page_size, scale, window)
  if (dtype == MGPT_F32) {
    if (fast_exp) LAUNCH(float, true); else LAUNCH(float, false);
  } else if (dtype == MGPT_BF16) {
    if (fast_exp) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false);
  } else {
    return MGPT_ERR_BAD_DTYPE;
  }
#undef LAUNCH
  return mgpt_last_error();
}
