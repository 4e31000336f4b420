// Paged causal attention for prompt portions in bfloat16 on the MFMA units (flash style).
//
// Same rule as the general kernel: a query at absolute position p sees the keys
// max(0, p-window+1)..p of its own request, some of them written by earlier steps (a portion
// with ctx > 0 is the offset-causal case of src/minigpt_infer/batch.py:202-227), scores scaled,
// softmax and all sums in float32 (src/minigpt_infer/model.py:61-87).
//
// A workgroup of four waves takes 64 consecutive queries of one request and one head, 16 per
// wave.  It walks the keys in blocks of 128 (aligned to multiples of 128 of the key position):
// the block's key rows go to LDS as they are, its value rows transposed, gathered row by row
// through the block table, so any page size works and nothing outside [begin, end) is loaded;
// the next block is on its way from memory while the current one is multiplied.
// S = K Q^T uses the keys as the first MFMA operand, so a lane holds, for one query, four
// neighbouring keys of each 16-key tile; those are exactly the k-slots of the second MFMA
// (values^T times P) if the transposed values are read with the same interleaving, so the
// probabilities never leave their registers.  Running max, sum and rescaling per query are the
// usual online softmax.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define PF_QT 64   // queries per workgroup
#define PF_KT 128  // keys per block

template <int D>
__global__ __launch_bounds__(256) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, long ldq, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, int n_head, int n_kv_head, int page_size, float scale, int window) {
  constexpr int KLD = D + 8;       // key rows in LDS
  constexpr int VLD = PF_KT + 8;   // transposed value rows in LDS
  constexpr int KK = D / 32;       // MFMA k steps over the head size
  constexpr int DT = D / 16;       // 16-channel tiles of the output
  __shared__ __align__(16) bf16_t ks[PF_KT * KLD];
  __shared__ __align__(16) bf16_t vt[D * VLD];

  const int r = blockIdx.y, h = blockIdx.z;
  const int q_start = cu_q[r], q_len = cu_q[r + 1] - q_start;
  // later tiles see more keys: start them first
  const int q0 = (int)blockIdx.x * PF_QT;
  if (q0 >= q_len) return;
  const int seq_len = seq_lens[r];
  const int ctx = seq_len - q_len;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hk = h / (n_head / n_kv_head);
  const int* bt = block_tables + (long)r * max_blocks;
  const int qi = lane & 15, g = lane >> 4;

  // this lane's query (for masks and the final store) and the tile's key range
  const int my_q = q0 + wave * 16 + qi;
  const bool q_ok = my_q < q_len;
  const int my_pos = ctx + my_q;
  const int tile_q_hi = (q0 + PF_QT < q_len ? q0 + PF_QT : q_len) - 1;
  const int pos_lo = ctx + q0, pos_hi = ctx + tile_q_hi;
  const int kv_begin = (window > 0 && pos_lo - window + 1 > 0) ? pos_lo - window + 1 : 0;
  const int kv_end = pos_hi + 1;

  bf16x8_t qf[KK];
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int kk = 0; kk < KK; ++kk)
    qf[kk] = q_ok ? *reinterpret_cast<const bf16x8_t*>(q + (long)(q_start + my_q) * ldq + (long)h * D + kk * 32 + g * 8)
                  : zero8;

  float m = -INFINITY, l = 0.f;
  f32x4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // Staging: 256 / PF_KT threads per key row, each 16 bytes (8 channels) of the key row and of the
  // value row at a time; keys go to LDS as they are, values transposed.  The next block's rows
  // are fetched into registers while the current block is multiplied.
  constexpr int TPR = 256 / PF_KT;                 // threads per row
  constexpr int NC = (D / 8 + TPR - 1) / TPR;      // chunks per thread
  const int srow = tid / TPR, sc = tid % TPR;
  bf16x8_t kst[NC], vst[NC];
  bool st_ok[NC];  // whether the fetched chunk is a visible key's; decided at fetch, applied at deposit,
                   // so that nothing touches a loaded value while the current block is multiplied

  auto fetch = [&](int c0) {
    const int j = c0 + srow;
    const bool valid = (j >= kv_begin) && (j < kv_end);
    long base = 0;
    if (valid) {
      const int page = bt[j / page_size];
      base = (((long)page * n_kv_head + hk) * page_size + (j % page_size)) * (long)D;
    }
#pragma unroll
    for (int u = 0; u < NC; ++u) {
      const int c = sc + u * TPR;
      const bool ok = valid && c < D / 8;
      const bf16x8_t kv8 = *reinterpret_cast<const bf16x8_t*>(kpool + base + (ok ? c * 8 : 0));
      const bf16x8_t vv8 = *reinterpret_cast<const bf16x8_t*>(vpool + base + (ok ? c * 8 : 0));
      kst[u] = kv8;
      vst[u] = vv8;
      st_ok[u] = ok;
    }
  };
  auto deposit = [&]() {
#pragma unroll
    for (int u = 0; u < NC; ++u) {
      const int c = sc + u * TPR;
      if (c >= D / 8) continue;
      const bf16x8_t k8 = st_ok[u] ? kst[u] : zero8, v8 = st_ok[u] ? vst[u] : zero8;
      *reinterpret_cast<bf16x8_t*>(&ks[srow * KLD + c * 8]) = k8;
#pragma unroll
      for (int e = 0; e < 8; ++e) vt[(c * 8 + e) * VLD + srow] = (bf16_t)v8[e];
    }
  };

  const int c_first = (kv_begin / PF_KT) * PF_KT;
  fetch(c_first);
  for (int c0 = c_first; c0 < kv_end; c0 += PF_KT) {
    __syncthreads();  // the previous block's readers are done
    deposit();
    __syncthreads();
    if (c0 + PF_KT < kv_end) fetch(c0 + PF_KT);

    // scores of this wave's 16 queries against the block's 64 keys
    constexpr int NKT = PF_KT / 16;   // 16-key tiles per block
    f32x4_t s[NKT];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt) {
      s[kt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(&ks[(kt * 16 + qi) * KLD + kk * 32 + g * 8]);
        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[kk], s[kt], 0, 0, 0);
      }
    }
    // lane: query qi, keys c0 + kt*16 + g*4 + i.  Scores are kept in units of log2(e), so that
    // the exponential is one v_exp_f32.  A block that every query of this wave sees whole (the
    // common case away from the diagonal) needs no mask.
    const float sc2 = scale * 1.4426950408889634f;
    const int wave_pos_lo = ctx + q0 + wave * 16;   // first query position of this wave
    const bool whole = c0 + PF_KT - 1 <= wave_pos_lo && c0 >= kv_begin && wave_pos_lo + 15 < ctx + q_len &&
                       (window <= 0 || c0 > wave_pos_lo + 15 - window);
    float mx = -INFINITY;
    if (whole) {
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s[kt][i] *= sc2;
          mx = fmaxf(mx, s[kt][i]);
        }
    } else {
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = c0 + kt * 16 + g * 4 + i;
          const bool see = q_ok && key <= my_pos && key >= kv_begin && (window <= 0 || key > my_pos - window);
          const float v = see ? s[kt][i] * sc2 : -INFINITY;
          s[kt][i] = v;
          mx = fmaxf(mx, v);
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = (m == -INFINITY) ? ((m_new == -INFINITY) ? 1.f : 0.f) : __builtin_amdgcn_exp2f(m - m_new);
    const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;   // exp2(-inf - 0) = 0 for masked scores
    float rs = 0.f;
    bf16x8_t pf[NKT / 2];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(s[kt][i] - m_sub);
        rs += p;
        // p lies in [0, 1]: rounding to bfloat16 by adding half an ulp and truncating
        pf[kt >> 1][(kt & 1) * 4 + i] = (short)((__float_as_uint(p) + 0x8000u) >> 16);
      }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
#pragma unroll
      for (int b = 0; b < NKT / 2; ++b) {
        // k-slot (g, e): key b*32 + g*4 + e for e < 4, key b*32 + 16 + g*4 + (e - 4) otherwise
        const bf16_t* vrow = &vt[(dt * 16 + qi) * VLD + b * 32 + g * 4];
        const bf16x4_t lo = *reinterpret_cast<const bf16x4_t*>(vrow);
        const bf16x4_t hi = *reinterpret_cast<const bf16x4_t*>(vrow + 16);
        const bf16x8_t vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[b], o[dt], 0, 0, 0);
      }
    }
  }

  if (q_ok) {
    const float inv = 1.0f / l;
    bf16_t* orow = out + (long)(q_start + my_q) * ldo + (long)h * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) orow[dt * 16 + g * 4 + i] = float_to_bf16(o[dt][i] * inv);
  }
}

// One workgroup per (64-query tile, request, head); max_q_len sizes the grid and is the host's
// upper bound on the tokens any request brings.  Head sizes 32, 64, 96, 128; others are refused.
extern "C" int mgpt_prefill_attention_bf16(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, int n_req,
    int max_q_len, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    hipStream_t stream) {
  if (n_req == 0 || max_q_len == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !cu_q || !seq_lens) return MGPT_ERR_NULL;
  if (n_req < 0 || max_q_len < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 ||
      page_size <= 0 || max_blocks <= 0 || window < 0 || (ldq % 8) != 0)
    return MGPT_ERR_BAD_SHAPE;
  if (n_req > 65535 || n_head > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid((max_q_len + PF_QT - 1) / PF_QT, n_req, n_head), block(256);
#define PF_LAUNCH(DD)                                                                              \
  hipLaunchKernelGGL(prefill_attention_kernel<DD>, grid, block, 0, stream, (const bf16_t*)q, ldq,  \
                     (bf16_t*)out, ldo, (const bf16_t*)kpool, (const bf16_t*)vpool, block_tables,  \
                     max_blocks, cu_q, seq_lens, n_head, n_kv_head, page_size, scale, window)
  switch (head_dim) {
    case 32: PF_LAUNCH(32); break;
    case 64: PF_LAUNCH(64); break;
    case 96: PF_LAUNCH(96); break;
    case 128: PF_LAUNCH(128); break;
    default: return MGPT_ERR_BAD_SHAPE;
  }
#undef PF_LAUNCH
  return mgpt_last_error();
}
