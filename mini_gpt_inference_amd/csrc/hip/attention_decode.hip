// Paged attention for bfloat16 caches with the keys of one (token, head) split over the four
// waves of a workgroup, for any number of tokens per request: what steps use that neither
// attention_decode_wide.hip (one token per request) nor attention_prefill.hip (prompt portions)
// takes, such as padded steps with several tokens per request or other head sizes.  Same rule as
// the general kernel (a query at
// position p sees the keys max(0, p-window+1)..p of its own request; scores, softmax and the
// weighted sum in float32; reference: src/minigpt_infer/model.py:61-87 and the Triton decode
// kernel src/minigpt_infer/attention/triton_paged.py:44-123, which walks the whole context in
// one program).
//
// Wave w takes the 64-key chunks w, w+4, w+8, ... (chunks start at multiples of 64 of the
// absolute key position).  Inside a chunk each lane scores one key with 16-byte loads of its
// row; then the lanes turn to the head's channels and add the chunk's values.  The four
// partial results (max, sum, weighted values) are merged through LDS in wave order.
// Slots outside the visible range are never loaded.
#include "common.h"
#include "launchers.h"

#define AD_WAVES 4
#define AD_MAX_DPL 4  // head_dim <= 256

__global__ __launch_bounds__(256) void paged_attention_split_kernel(
    const bf16_t* __restrict__ q, long ldq, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, const int* __restrict__ q_req, int n_tokens, int n_head,
    int n_kv_head, int head_dim, int page_size, float scale, int window) {
  __shared__ float q_s[AD_MAX_DPL * 64];
  __shared__ float p_s[AD_WAVES][64];
  __shared__ int page_s[AD_WAVES][64];
  __shared__ float m_s[AD_WAVES], l_s[AD_WAVES];
  __shared__ float acc_s[AD_WAVES][AD_MAX_DPL * 64];

  const int n = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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

  for (int d = tid; d < head_dim; d += 256)
    q_s[d] = bf16_to_float(q[(long)n * ldq + (long)h * head_dim + d]) * scale;
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[AD_MAX_DPL];
#pragma unroll
  for (int i = 0; i < AD_MAX_DPL; ++i) acc[i] = 0.f;

  const int first_chunk = kv_begin / 64;
  for (int c0 = (first_chunk + wave) * 64; c0 < kv_end; c0 += 64 * AD_WAVES) {
    const int j = c0 + lane;
    const bool valid = (j >= kv_begin) && (j < kv_end);
    float s = -INFINITY;
    int page = -1;
    if (valid) {
      page = bt[j / page_size];
      const int off = j % page_size;
      const bf16_t* kr = kpool + (((long)page * n_kv_head + hk) * page_size + off) * (long)head_dim;
      float dot = 0.f;
      for (int d = 0; d < head_dim; d += 8) {
        const uint4 raw = *reinterpret_cast<const uint4*>(kr + d);
        const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          dot = fmaf(q_s[d + 2 * e], __uint_as_float(w[e] << 16), dot);
          dot = fmaf(q_s[d + 2 * e + 1], __uint_as_float(w[e] & 0xffff0000u), dot);
        }
      }
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? __expf(s - m_new) : 0.f;
    const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
    // p_s / page_s rows are private to the wave; a wave runs in lockstep, so no barrier is needed
    p_s[wave][lane] = p;
    page_s[wave][lane] = page;
    __builtin_amdgcn_wave_barrier();
    const int j_lo = (kv_begin > c0 ? kv_begin : c0) - c0;
    const int j_hi = (kv_end < c0 + 64 ? kv_end : c0 + 64) - c0;
#pragma unroll
    for (int i = 0; i < AD_MAX_DPL; ++i) {
      const int d = lane + i * 64;
      if (d < head_dim) {
        float a = acc[i] * alpha;
#pragma unroll 8
        for (int jj = j_lo; jj < j_hi; ++jj) {
          const int off = (c0 + jj) % page_size;
          const bf16_t* vr = vpool + (((long)page_s[wave][jj] * n_kv_head + hk) * page_size + off) * (long)head_dim;
          a = fmaf(p_s[wave][jj], bf16_to_float(vr[d]), a);
        }
        acc[i] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
#pragma unroll
  for (int i = 0; i < AD_MAX_DPL; ++i) {
    const int d = lane + i * 64;
    if (d < head_dim) acc_s[wave][d] = acc[i];
  }
  __syncthreads();
  if (wave == 0) {
    float mx = m_s[0];
    for (int w = 1; w < AD_WAVES; ++w) mx = fmaxf(mx, m_s[w]);
    float lt = 0.f;
    float f[AD_WAVES];
    for (int w = 0; w < AD_WAVES; ++w) {
      f[w] = (m_s[w] == -INFINITY) ? 0.f : __expf(m_s[w] - mx);
      lt += l_s[w] * f[w];
    }
    const float inv = 1.0f / lt;
#pragma unroll
    for (int i = 0; i < AD_MAX_DPL; ++i) {
      const int d = lane + i * 64;
      if (d < head_dim) {
        float a = 0.f;
        for (int w = 0; w < AD_WAVES; ++w) a += acc_s[w][d] * f[w];
        out[(long)n * ldo + (long)h * head_dim + d] = float_to_bf16(a * inv);
      }
    }
  }
}

extern "C" int mgpt_paged_attention_split_bf16(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int* q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !cu_q || !seq_lens || !q_req) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 || head_dim <= 0 ||
      head_dim > AD_MAX_DPL * 64 || (head_dim % 8) != 0 || page_size <= 0 || max_blocks <= 0 || window < 0)
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(paged_attention_split_kernel, dim3(n_tokens, n_head), dim3(256), 0, stream,
                     (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)kpool, (const bf16_t*)vpool,
                     block_tables, max_blocks, cu_q, seq_lens, q_req, n_tokens, n_head, n_kv_head, head_dim,
                     page_size, scale, window);
  return mgpt_last_error();
}

// ---------------------------------------------------------------------------------------------
// The same computation for head sizes 16, 32, 64 and 128 with every load 16 bytes wide and all
// loads of a chunk in flight at once.  D/8 lanes share a key: lane L of instruction i holds
// channels (L % (D/8))*8 .. +8 of key c0 + i*(512/D) + L/(D/8), for the key's score (a short
// cross-lane sum) and, with the same mapping, for its value row, so a key's weight never leaves
// the lanes that need it.  Partial sums over keys are combined across lanes once, at the end.
template <int D>
__global__ __launch_bounds__(256) void paged_attention_split_fast_kernel(
    const bf16_t* __restrict__ q, long ldq, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, const int* __restrict__ q_req, int n_tokens, int n_head,
    int n_kv_head, int page_size, float scale, int window) {
  constexpr int LPK = D / 8;     // lanes per key
  constexpr int KPI = 64 / LPK;  // keys per load instruction
  __shared__ float m_s[AD_WAVES], l_s[AD_WAVES];
  __shared__ float acc_s[AD_WAVES][D];

  const int n = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
  const int sub = lane / LPK, dg = lane % LPK;

  float qv[8];
  {
    const uint4 raw = *reinterpret_cast<const uint4*>(q + (long)n * ldq + (long)h * D + dg * 8);
    const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      qv[2 * e] = __uint_as_float(w[e] << 16) * scale;
      qv[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u) * scale;
    }
  }

  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;

  const int first_chunk = kv_begin / 64;
  for (int c0 = (first_chunk + wave) * 64; c0 < kv_end; c0 += 64 * AD_WAVES) {
    long base[LPK];
    bool valid[LPK];
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      const int j = c0 + i * KPI + sub;
      valid[i] = (j >= kv_begin) && (j < kv_end);
      base[i] = 0;
      if (valid[i]) {
        const int page = bt[j / page_size];
        base[i] = (((long)page * n_kv_head + hk) * page_size + (j % page_size)) * (long)D + dg * 8;
      }
    }
    uint4 kraw[LPK], vraw[LPK];
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      kraw[i] = valid[i] ? *reinterpret_cast<const uint4*>(kpool + base[i]) : make_uint4(0, 0, 0, 0);
      vraw[i] = valid[i] ? *reinterpret_cast<const uint4*>(vpool + base[i]) : make_uint4(0, 0, 0, 0);
    }
    float s[LPK];
    float cmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      const unsigned int w[4] = {kraw[i].x, kraw[i].y, kraw[i].z, kraw[i].w};
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        dot = fmaf(qv[2 * e], __uint_as_float(w[e] << 16), dot);
        dot = fmaf(qv[2 * e + 1], __uint_as_float(w[e] & 0xffff0000u), dot);
      }
#pragma unroll
      for (int off = 1; off < LPK; off <<= 1) dot += __shfl_xor(dot, off, 64);
      s[i] = valid[i] ? dot : -INFINITY;
      cmax = fmaxf(cmax, s[i]);
    }
    const float m_new = fmaxf(m, wave_max(cmax));
    const float alpha = (m == -INFINITY) ? 0.f : __expf(m - m_new);
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= alpha;
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      const float p = valid[i] ? __expf(s[i] - m_new) : 0.f;
      psum += p;
      const unsigned int w[4] = {vraw[i].x, vraw[i].y, vraw[i].z, vraw[i].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] = fmaf(p, __uint_as_float(w[e] << 16), acc[2 * e]);
        acc[2 * e + 1] = fmaf(p, __uint_as_float(w[e] & 0xffff0000u), acc[2 * e + 1]);
      }
    }
    // every key's weight sits on LPK lanes
    l = l * alpha + wave_sum(psum) * (1.0f / LPK);
    m = m_new;
  }

  // add the partial sums of the 64/LPK key subgroups: lanes with equal dg
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) acc[e] += __shfl_xor(acc[e], off, 64);
  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
  if (lane < LPK) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc_s[wave][lane * 8 + e] = acc[e];
  }
  __syncthreads();
  if (tid < D) {
    float mx = m_s[0];
    for (int w = 1; w < AD_WAVES; ++w) mx = fmaxf(mx, m_s[w]);
    float lt = 0.f, a = 0.f;
    for (int w = 0; w < AD_WAVES; ++w) {
      const float f = (m_s[w] == -INFINITY) ? 0.f : __expf(m_s[w] - mx);
      lt += l_s[w] * f;
      a += acc_s[w][tid] * f;
    }
    out[(long)n * ldo + (long)h * D + tid] = float_to_bf16(a / lt);
  }
}

extern "C" int mgpt_paged_attention_split_fast_bf16(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int* q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !cu_q || !seq_lens || !q_req) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 || page_size <= 0 ||
      max_blocks <= 0 || window < 0 || (ldq % 8) != 0)
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid(n_tokens, n_head), block(256);
#define AD_LAUNCH(DD)                                                                                   \
  hipLaunchKernelGGL(paged_attention_split_fast_kernel<DD>, grid, block, 0, stream, (const bf16_t*)q, ldq, \
                     (bf16_t*)out, ldo, (const bf16_t*)kpool, (const bf16_t*)vpool, block_tables,       \
                     max_blocks, cu_q, seq_lens, q_req, n_tokens, n_head, n_kv_head, page_size, scale, window)
  switch (head_dim) {
    case 16: AD_LAUNCH(16); break;
    case 32: AD_LAUNCH(32); break;
    case 64: AD_LAUNCH(64); break;
    case 128: AD_LAUNCH(128); break;
    default: return MGPT_ERR_BAD_SHAPE;  // other head sizes: the kernel above
  }
#undef AD_LAUNCH
  return mgpt_last_error();
}
