// Paged attention for the single tokens of a decode step (bfloat16 cache, head sizes 16, 32, 64
// and 128), laid out for latency.  The rule is the general kernel's (a query at position p sees
// the keys max(0, p-window+1)..p of its own request; reference: src/minigpt_infer/model.py:61-87
// and the Triton decode kernel src/minigpt_infer/attention/triton_paged.py:44-123).
//
// A decode step is a chain of dependent kernels, and this one used to be the longest link: four
// memory round trips in a row (token -> request -> lengths -> block table -> keys) and
// cross-lane reductions through LDS for every 64 keys.  Here:
//  * a token's position comes from the step's position array and, when token n is request n (a
//    decode-only step), its block table row is read at once, before the position is known:
//    two round trips, block table then keys and values.  Block table entries that turn out to
//    lie beyond the sequence are never followed (their keys are masked before the load), and
//    an entry's page number is clamped to the pool so that a stale entry cannot send a load
//    outside it;
//  * eight waves, each with one 64-key chunk in flight (sixteen 16-byte loads per lane), so a
//    context of up to 512 keys is one pass;
//  * D/8 lanes share a key: scores with v_dot2_f32_bf16 on the packed rows as loaded, summed
//    over the D/8 lanes with DPP moves; one wave-wide maximum per chunk (DPP within rows of 16,
//    then the four rows' values through scalar registers); the weighted sum of values again with
//    v_dot2_f32_bf16, two keys at a time, the weights rounded to bfloat16 as the tile kernel
//    for prompts does;
//  * the waves' partial results (maximum, sum, weighted values per key subgroup) are merged
//    through LDS once, in a fixed order.
#include "common.h"
#include "launchers.h"

#define AW_WAVES 8

typedef __attribute__((ext_vector_type(2))) __bf16 aw_bf16x2_t;

template <int CTRL>
__device__ __forceinline__ float aw_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// sum over the LPK neighbouring lanes of an aligned group; every lane of the group gets it
template <int LPK>
__device__ __forceinline__ float aw_group_sum(float v) {
  v += aw_dpp<0xB1>(v);                 // quad_perm [1,0,3,2]
  if (LPK >= 4) v += aw_dpp<0x4E>(v);   // quad_perm [2,3,0,1]
  if (LPK >= 8) v += aw_dpp<0x141>(v);  // row_half_mirror: lane i of each 8 reads lane 7 - i
  if (LPK >= 16) v += aw_dpp<0x140>(v); // row_mirror: lane i of each 16 reads lane 15 - i
  return v;
}

// maximum over the 64 lanes, as a value that is the same in all of them
__device__ __forceinline__ float aw_wave_max(float v) {
  v = fmaxf(v, aw_dpp<0xB1>(v));
  v = fmaxf(v, aw_dpp<0x4E>(v));
  v = fmaxf(v, aw_dpp<0x141>(v));
  v = fmaxf(v, aw_dpp<0x140>(v));
  const int b = __float_as_int(v);
  const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
  const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
  const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
  const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

__device__ __forceinline__ float aw_dot2(unsigned int a, unsigned int b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(aw_bf16x2_t, a), __builtin_bit_cast(aw_bf16x2_t, b),
                                         c, false);
}

// IDENT: token n is request n (or padded), so its block table row is known before anything is loaded
template <int D, bool IDENT>
__global__ __launch_bounds__(AW_WAVES * 64) void paged_attention_decode_kernel(
    const bf16_t* __restrict__ q, long ldq, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ positions,
    const int* __restrict__ q_req, const int* __restrict__ cu_q, int n_head, int n_kv_head, int page_shift,
    int num_pages, unsigned int page_bytes, float scale_log2e, int window) {
  constexpr int LPK = D / 8;     // lanes per key
  constexpr int KPI = 64 / LPK;  // keys per load instruction
  constexpr int ROWS = AW_WAVES * KPI;      // partial results: one per (key subgroup, wave)
  constexpr int SUBSETS = AW_WAVES * 64 / D;  // groups of AW_WAVES partial rows, one thread per channel each
  __shared__ float m_s[AW_WAVES];
  __shared__ float l_s[ROWS];        // [sub][wave]
  __shared__ float acc_s[ROWS * D];  // [sub][wave][channel]
  __shared__ float part_s[SUBSETS * D];
  __shared__ float lpart_s[SUBSETS];

  const int n = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sub = lane / LPK, dg = lane % LPK;
  const int hk = h / (n_head / n_kv_head);

  // ---- first round trip: the token's request and position, its query, and (decode-only steps)
  // the block table entries of the first pass
  int qr = q_req[n];
  const int qpos = positions[n];
  uint4 qraw = *reinterpret_cast<const uint4*>(q + (long)n * ldq + (long)h * D + dg * 8);
  int r = n;
  if (!IDENT) {
    r = qr < 0 ? 0 : qr;  // waits for qr
    // a step that also holds prompt portions: their tokens are another kernel's, and count as padding here
    if (cu_q && cu_q[r + 1] - cu_q[r] != 1) qr = -1;
  }
  int first_chunk = 0;
  if (window > 0) first_chunk = (qpos - window + 1 > 0 ? qpos - window + 1 : 0) / 64;  // waits for qpos
  const int* bt = block_tables + (long)r * max_blocks;

  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;

  int c_base = first_chunk * 64;
  int kv_end = 0, kv_begin = 0;
  do {
    const int c0 = c_base + wave * 64;
    const int page_mask = (1 << page_shift) - 1;
    int page[LPK];
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      const int e = (c0 + i * KPI + sub) >> page_shift;
      page[i] = bt[e < max_blocks ? e : max_blocks - 1];
    }
    kv_end = qr < 0 ? 0 : qpos + 1;
    kv_begin = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
    c_base += 64 * AW_WAVES;
    // a chunk without a visible key costs its wave nothing more (the same decision in all lanes)
    if (__builtin_amdgcn_readfirstlane((c0 >= kv_end) | (c0 + 64 <= kv_begin))) continue;
    // ---- second round trip: keys and values of this wave's chunk.  Every lane loads (a masked
    // key reads the pool's first row instead and is zeroed afterwards), so that no branch stands
    // between the loads.  Offsets are 32-bit byte offsets from the pools' bases.
    uint4 kraw[LPK], vraw[LPK];
    bool valid[LPK];
    const unsigned int lane_off = ((unsigned int)(hk << page_shift) * D + dg * 8) * 2u;
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      const int j = c0 + i * KPI + sub;
      valid[i] = (j >= kv_begin) && (j < kv_end);
      const bool follow = valid[i] && (unsigned int)page[i] < (unsigned int)num_pages;
      const unsigned int row_off = ((unsigned int)page[i] * page_bytes) + (unsigned int)(j & page_mask) * (D * 2u);
      const unsigned int off = follow ? row_off + lane_off : 0u;
      kraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(kpool) + off);
      vraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(vpool) + off);
    }
#pragma unroll
    for (int i = 0; i < LPK; ++i)
      if (!valid[i]) vraw[i] = make_uint4(0, 0, 0, 0);  // its weight is 0, but 0 * NaN is not
    // ---- scores (in units of log2 e, so that exp2 serves)
    float s[LPK];
    float cmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < LPK; ++i) {
      float dot = aw_dot2(qraw.x, kraw[i].x, 0.f);
      dot = aw_dot2(qraw.y, kraw[i].y, dot);
      dot = aw_dot2(qraw.z, kraw[i].z, dot);
      dot = aw_dot2(qraw.w, kraw[i].w, dot);
      dot = aw_group_sum<LPK>(dot) * scale_log2e;
      s[i] = valid[i] ? dot : -INFINITY;
      cmax = fmaxf(cmax, s[i]);
    }
    const float m_new = fmaxf(m, aw_wave_max(cmax));
    if (m_new != -INFINITY) {  // the same in all lanes; false only while the wave has seen no key
      const float alpha = __builtin_amdgcn_exp2f(m - m_new);  // m = -inf: 0
      l *= alpha;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= alpha;
      m = m_new;
#pragma unroll
      for (int i = 0; i < LPK; i += 2) {
        const float pa = __builtin_amdgcn_exp2f(s[i] - m_new), pb = __builtin_amdgcn_exp2f(s[i + 1] - m_new);  // a masked key: exp2(-inf) = 0
        l += pa + pb;
        const unsigned int pp = pack_bf16x2(pa, pb);
        const unsigned int va[4] = {vraw[i].x, vraw[i].y, vraw[i].z, vraw[i].w};
        const unsigned int vb[4] = {vraw[i + 1].x, vraw[i + 1].y, vraw[i + 1].z, vraw[i + 1].w};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          // (va.low half, vb.low half) and (va.high half, vb.high half): channel 2w and 2w+1 of both keys
          const unsigned int lo = __builtin_amdgcn_perm(vb[w], va[w], 0x05040100u);
          const unsigned int hi = __builtin_amdgcn_perm(vb[w], va[w], 0x07060302u);
          acc[2 * w] = aw_dot2(pp, lo, acc[2 * w]);
          acc[2 * w + 1] = aw_dot2(pp, hi, acc[2 * w + 1]);
        }
      }
    }
  } while (c_base < kv_end);
  if (qr < 0) return;  // padded token (the whole workgroup)

  // ---- merge: partial rows [sub][wave] of D channels; every key's weight sits on LPK lanes, so
  // lane dg == 0 speaks for the group's sum
  if (lane == 0) m_s[wave] = m;
  if (dg == 0) l_s[sub * AW_WAVES + wave] = l;
  {
    float4* dst = reinterpret_cast<float4*>(acc_s + (sub * AW_WAVES + wave) * D + dg * 8);
    dst[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    dst[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
  __syncthreads();
  {
    float mx = m_s[0];
#pragma unroll
    for (int w = 1; w < AW_WAVES; ++w) mx = fmaxf(mx, m_s[w]);
    const int c = tid % D, sset = tid / D;  // this thread: channel c of the partial rows sset*AW_WAVES ..
    float a = 0.f, lt = 0.f;
#pragma unroll
    for (int w = 0; w < AW_WAVES; ++w) {
      const float f = __builtin_amdgcn_exp2f(m_s[w] - mx);  // a wave without keys: exp2(-inf) = 0, and its sums are 0
      a = fmaf(acc_s[(sset * AW_WAVES + w) * D + c], f, a);
      lt = fmaf(l_s[sset * AW_WAVES + w], f, lt);
    }
    part_s[sset * D + c] = a;
    if (c == 0) lpart_s[sset] = lt;
  }
  __syncthreads();
  if (tid < D) {
    float a = 0.f, lt = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < SUBSETS; ++s2) {
      a += part_s[s2 * D + tid];
      lt += lpart_s[s2];
    }
    out[(long)n * ldo + (long)h * D + tid] = float_to_bf16(a / lt);
  }
}

// positions[n]: absolute position of token n; q_req[n]: its request (block table row), -1 for a
// padded token.  identity != 0 promises q_req[n] is n or -1 (a decode-only step).  cu_q (optional,
// without identity): the requests' token offsets; tokens of requests that bring more than one token
// are then left to another kernel.  Refuses
// (MGPT_ERR_BAD_SHAPE) other head sizes than 16, 32, 64, 128, page sizes that are no power of two
// and pools of 4 GiB or more.
extern "C" int mgpt_paged_attention_decode_bf16(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* positions, const int* q_req, const int* cu_q,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, int num_pages, float scale, int window,
    int identity, hipStream_t stream) {
  if (n_tokens == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !positions || !q_req) return MGPT_ERR_NULL;
  if (n_tokens < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 || page_size <= 0 ||
      max_blocks <= 0 || num_pages <= 0 || window < 0 || (ldq % 8) != 0 || (identity && cu_q))
    return MGPT_ERR_BAD_SHAPE;
  if (n_head > 65535) return MGPT_ERR_TOO_LARGE;
  int page_shift = -1;
  for (int s = 0; s < 30; ++s)
    if ((1 << s) == page_size) page_shift = s;
  if (page_shift < 0) return MGPT_ERR_BAD_SHAPE;
  // the kernel addresses a pool by 32-bit byte offsets
  const long pool_bytes = (long)num_pages * n_kv_head * page_size * head_dim * 2;
  if (pool_bytes >= (1L << 32)) return MGPT_ERR_BAD_SHAPE;
  const unsigned int page_bytes = (unsigned int)(n_kv_head * page_size * head_dim * 2);
  const float scale_log2e = scale * 1.4426950408889634f;
  dim3 grid(n_tokens, n_head), block(AW_WAVES * 64);
#define AW_LAUNCH2(DD, ID)                                                                                 \
  hipLaunchKernelGGL((paged_attention_decode_kernel<DD, ID>), grid, block, 0, stream, (const bf16_t*)q, ldq, \
                     (bf16_t*)out, ldo, (const bf16_t*)kpool, (const bf16_t*)vpool, block_tables,          \
                     max_blocks, positions, q_req, cu_q, n_head, n_kv_head, page_shift, num_pages, page_bytes, \
                     scale_log2e, window)
#define AW_LAUNCH(DD)              \
  do {                             \
    if (identity) AW_LAUNCH2(DD, true); \
    else AW_LAUNCH2(DD, false);    \
  } while (0)
  switch (head_dim) {
    case 16: AW_LAUNCH(16); break;
    case 32: AW_LAUNCH(32); break;
    case 64: AW_LAUNCH(64); break;
    case 128: AW_LAUNCH(128); break;
    default: return MGPT_ERR_BAD_SHAPE;
  }
#undef AW_LAUNCH
#undef AW_LAUNCH2
  return mgpt_last_error();
}
