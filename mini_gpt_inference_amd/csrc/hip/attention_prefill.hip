// Paged causal attention for prompt portions in bfloat16 on the MFMA units (flash style).
//
// Same rule as the general kernel: a query at absolute position p sees the keys
// max(0, p-window+1)..p of its own request, some of them written by earlier steps (a portion
// with ctx > 0 is the offset-causal case of src/minigpt_infer/batch.py:202-227), scores scaled,
// softmax and all sums in float32 (src/minigpt_infer/model.py:61-87).
//
// A workgroup takes 64 consecutive queries of one request and one head, 16 per wave (four waves,
// or eight in two groups that share the keys between them, see the kernel).  It walks the keys in blocks of 128 (aligned to multiples of 128 of the key position):
// the block's key and value rows go to LDS as they are, gathered row by row through the block
// table, so any page size works and nothing outside [begin, end) is loaded.  LDS holds two
// blocks: while one is multiplied, the next (fetched from memory into registers a block earlier)
// is put beside it and the one after is sent for, with one barrier per block.
//
// S = K Q^T uses the keys as the first MFMA operand, so a lane holds, for one query, four
// neighbouring keys of each 16-key tile; those are exactly the k-slots of the second MFMA
// (values^T times P) if the values are read transposed with the same interleaving, so the
// probabilities never leave their registers.  The transposing LDS read of this chip
// (ds_read_b64_tr_b16) does that: the 16 lanes of a block point at 4 rows x 4 chunks of 4
// channels, row j / 4 and chunk j % 4 for lane j, and lane i comes back with channel i of the
// four rows.  Running max, sum and rescaling per query are the usual online softmax, kept short because at head size 64 it, not the MFMAs, is what a block
// costs: exp2(score * scale' - max) is one fused multiply-add and one v_exp_f32 (scale' holds
// log2 e), the maximum over the four lanes that share a query goes through two lane swaps
// instead of LDS, and the row sum stays split over those lanes until the end.
#include "common.h"
#include "launchers.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int u32x4_t;

#define PF_QT 64   // queries per workgroup
#define PF_KT 128  // keys per block

// max over the four lanes lane, lane ^ 16, lane ^ 32, lane ^ 48, the same in all four: each swap
// hands every lane the value of its partner in the other row (pair of rows).
__device__ __forceinline__ float pf_max_over_rows(float v) {
  const unsigned int u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned int ux = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane32_swap(ux, ux, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float pf_sum_over_rows(float v) {
  const unsigned int u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned int ux = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane32_swap(ux, ux, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// G: wave groups.  With G = 2 the workgroup has eight waves: both groups work on the same 64
// queries, group 0 on the first 128 keys of every stretch of 256 that is staged at a time and
// group 1 on the other 128, each with a running max, sum and output of its own that are put
// together at the end.  The longest tile's walk over the keys is half as many steps long, every
// thread stages as much per step as with one group, and on each SIMD a wave of one group has its
// softmax arithmetic while the other group's wave has its MFMAs.  Head sizes whose two stretches
// do not fit LDS run with one group.
template <int D, int G>
__global__ __launch_bounds__(256 * G) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, long ldq, bf16_t* __restrict__ out, long ldo,
    const bf16_t* __restrict__ kpool, const bf16_t* __restrict__ vpool,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q,
    const int* __restrict__ seq_lens, int n_head, int n_kv_head, int page_size, float scale, int window,
    int single_below) {
  constexpr int THREADS = 256 * G;
  constexpr int SB = PF_KT * G;    // keys staged per step
  // Key and value rows in LDS: as long as the head size where that is a power of two, the 16-byte
  // chunks of a row XORed with the row's low bits (then neither the operand reads, 16 rows x 4 chunks
  // an instruction, nor the transposing reads meet in a bank); padded by 16 bytes otherwise.
  constexpr bool SWZ = (D & (D - 1)) == 0;
  constexpr int KLD = SWZ ? D : D + 8;
  constexpr int KK = D / 32;       // MFMA k steps over the head size
  constexpr int DT = D / 16;       // 16-channel tiles of the output
  constexpr int KS_SIZE = SB * KLD;   // keys, and as much for values
  extern __shared__ __align__(16) bf16_t pf_lds[];   // [2][KS_SIZE] keys, then [2][KS_SIZE] values, then the row table
  // Where each key of a stretch lies in the pools, as a row index ((page * heads + head) * page_size +
  // offset; -1: not a key this tile sees), worked out three steps ahead by one thread per key: the
  // loads that fetch a stretch then wait for no block-table entry and divide nothing.
  int* const row_tab = reinterpret_cast<int*>(pf_lds + 4 * KS_SIZE);   // [4][SB]

  const int r = blockIdx.y, h = blockIdx.z;
  const int q_start = cu_q[r], q_len = cu_q[r + 1] - q_start;
  const int q0 = (int)blockIdx.x * PF_QT;
  if (q0 >= q_len || (q_len == 1 && q_start < single_below)) return;   // the same for the whole workgroup
  const int seq_len = seq_lens[r];
  const int ctx = seq_len - q_len;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int qwave = wave & 3, grp = wave >> 2;
  const int hk = h / (n_head / n_kv_head);
  const int* bt = block_tables + (long)r * max_blocks;
  const int qi = lane & 15, g = lane >> 4;

  // this lane's query (for masks and the final store) and the tile's key range
  const int my_q = q0 + qwave * 16 + qi;
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

  float m = -INFINITY, l = 0.f;   // m in units of log2 e; l: this lane's share of the row sum
  f32x4_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // Staging: the stretch's rows are dealt out 16 bytes (8 channels) at a time, a row's chunks to
  // neighbouring threads, so that one load instruction of a wave covers whole rows (64 lanes: 8 rows
  // of 128 bytes at head size 64) and the 64 chunks it later puts into LDS lie in as many places.
  constexpr int CH = D / 8;                      // chunks per row
  constexpr int NP = SB * CH / THREADS;          // chunks per thread (= D / 16)
  static_assert(SB * CH % THREADS == 0, "the stretch's chunks must divide among the threads");
  bf16x8_t kst[NP], vst[NP];
  bool k_ok[NP];   // whether the fetched row is a visible key's: decided at fetch, applied at deposit,
                   // so that nothing touches a loaded value while the current stretch is multiplied

  // the row index of key j, or -1; the block table entry is the only thing read from memory
  auto lookup = [&](int j) -> int {
    if (j < kv_begin || j >= kv_end) return -1;
    const int pg = j / page_size;
    return (bt[pg] * n_kv_head + hk) * page_size + (j - pg * page_size);
  };
  // where chunk c of LDS row `row` lies
  auto chunk_at = [](int row, int c) -> int {
    if (!SWZ) return c;
    return D == 32 ? c ^ ((row >> 1) & 3) : c ^ (row & 7);
  };
  auto fetch = [&](int step) {
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int idx = u * THREADS + tid;
      const int r = idx / CH, c = idx - r * CH;
      const int row = row_tab[(step & 3) * SB + r];
      k_ok[u] = row >= 0;
      const long base = (long)(k_ok[u] ? row : 0) * D + c * 8;
      kst[u] = *reinterpret_cast<const bf16x8_t*>(kpool + base);
      vst[u] = *reinterpret_cast<const bf16x8_t*>(vpool + base);
    }
  };
  auto deposit = [&](int buf) {
    bf16_t* ks = pf_lds + buf * KS_SIZE;
    bf16_t* vs = pf_lds + (2 + buf) * KS_SIZE;
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int idx = u * THREADS + tid;
      const int r = idx / CH, c = idx - r * CH;
      const int at = r * KLD + chunk_at(r, c) * 8;
      *reinterpret_cast<bf16x8_t*>(&ks[at]) = k_ok[u] ? kst[u] : zero8;
      *reinterpret_cast<bf16x8_t*>(&vs[at]) = k_ok[u] ? vst[u] : zero8;
    }
  };

  // scores are kept in units of log2(e), so that the exponential is one v_exp_f32 (scale > 0 here)
  const float sc2 = scale * 1.4426950408889634f;
  const int c_first = (kv_begin / SB) * SB;
  const int n_steps = (kv_end - c_first + SB - 1) / SB;
  // the rows of the first three stretches
  for (int t = tid; t < 3 * SB; t += THREADS) row_tab[t] = lookup(c_first + t);
  __syncthreads();
  fetch(0);
  deposit(0);
  if (n_steps > 1) fetch(1);
  __syncthreads();
  for (int b = 0; b < n_steps; ++b) {
    const int buf = b & 1;
    const int c0 = c_first + b * SB + grp * PF_KT;   // first key of this wave group's half
    int row_ahead = -1;
    if (b + 1 < n_steps) {
      deposit(buf ^ 1);   // its readers finished before the last barrier
      if (b + 2 < n_steps) fetch(b + 2);
      // asked for now, written to the table at the end of this step's work
      if (b + 3 < n_steps && tid < SB) row_ahead = lookup(c_first + (b + 3) * SB + tid);
    }
    // a half with no key that the tile sees (past the end, or before a window) is left out
    if (c0 < kv_end && c0 + PF_KT > kv_begin) {
      const bf16_t* ks = pf_lds + buf * KS_SIZE + grp * PF_KT * KLD;
      const bf16_t* vs = pf_lds + (2 + buf) * KS_SIZE + grp * PF_KT * KLD;

      // scores of this wave's 16 queries against the half's keys: all key operands are asked for
      // before the first MFMA, and MFMAs that add to the same scores lie NKT apart
      constexpr int NKT = PF_KT / 16;   // 16-key tiles
      f32x4_t s[NKT];
      {
        bf16x8_t kf[KK][NKT];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
          for (int kt = 0; kt < NKT; ++kt)
            kf[kk][kt] = *reinterpret_cast<const bf16x8_t*>(&ks[(kt * 16 + qi) * KLD + chunk_at(qi, kk * 4 + g) * 8]);
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) s[kt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
          for (int kt = 0; kt < NKT; ++kt)
            s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kk][kt], qf[kk], s[kt], 0, 0, 0);
      }
      // The value operands do not depend on the scores: asked for now, they arrive while the softmax
      // below keeps the wave busy.  k-slot (g, e) of operand (dt, bb): key bb*32 + g*4 + e for e < 4,
      // key bb*32 + 16 + g*4 + (e - 4) otherwise; this lane points at row g*4 + qi/4 of those, chunk qi%4.
      bf16x4_t vlo[DT][NKT / 2], vhi[DT][NKT / 2];
      typedef bf16x4_t __attribute__((address_space(3))) * lds_b64_t;
      // row g*4 + qi/4 of each 16; its 8 bytes are half (qi & 1) of the 16-byte chunk dt*2 + (qi & 3)/2
      const int vrow = g * 4 + (qi >> 2);
      const bf16_t* vlane = vs + vrow * KLD + (qi & 1) * 4;
#pragma unroll
      for (int bb = 0; bb < NKT / 2; ++bb)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const int off = chunk_at(vrow, dt * 2 + ((qi & 3) >> 1)) * 8;   // rows 16 and 32 apart swizzle alike
          vlo[dt][bb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_b64_t)(vlane + (bb * 32) * KLD + off));
          vhi[dt][bb] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_b64_t)(vlane + (bb * 32 + 16) * KLD + off));
        }
      __builtin_amdgcn_sched_barrier(0);   // or the compiler moves each read down to its use

      // lane: query qi, keys c0 + kt*16 + g*4 + i.  A half that every query of this wave sees whole
      // (the common case away from the diagonal) needs no mask.
      const int wave_pos_lo = ctx + q0 + qwave * 16;   // first query position of this wave
      const bool whole = c0 + PF_KT - 1 <= wave_pos_lo && c0 >= kv_begin && wave_pos_lo + 15 < ctx + q_len &&
                         (window <= 0 || c0 > wave_pos_lo + 15 - window);
      float mx = -INFINITY;
      if (whole) {
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kt][i]);
      } else {
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = c0 + kt * 16 + g * 4 + i;
            const bool see = q_ok && key <= my_pos && key >= kv_begin && (window <= 0 || key > my_pos - window);
            const float v = see ? s[kt][i] : -INFINITY;
            s[kt][i] = v;
            mx = fmaxf(mx, v);
          }
      }
      mx = pf_max_over_rows(mx) * sc2;   // -inf stays -inf
      const float m_new = fmaxf(m, mx);
      const float alpha = (m == -INFINITY) ? ((m_new == -INFINITY) ? 1.f : 0.f) : __builtin_amdgcn_exp2f(m - m_new);
      const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;   // exp2(-inf - 0) = 0 for masked scores
      float rs = 0.f;
      bf16x8_t pf[NKT / 2];
#pragma unroll
      for (int kt = 0; kt < NKT; kt += 2) {
        float p[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt + (i >> 2)][i & 3], sc2, -m_sub));
          rs += p[i];
        }
        const u32x4_t packed = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                                pack_bf16x2(p[6], p[7])};
        pf[kt >> 1] = __builtin_bit_cast(bf16x8_t, packed);
      }
      l = l * alpha + rs;
      m = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[dt][i] *= alpha;
#pragma unroll
      for (int bb = 0; bb < NKT / 2; ++bb)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16x8_t vf = {vlo[dt][bb][0], vlo[dt][bb][1], vlo[dt][bb][2], vlo[dt][bb][3],
                               vhi[dt][bb][0], vhi[dt][bb][1], vhi[dt][bb][2], vhi[dt][bb][3]};
          o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[bb], o[dt], 0, 0, 0);
        }
    }
    if (b + 1 < n_steps) {
      if (tid < SB) row_tab[((b + 3) & 3) * SB + tid] = row_ahead;   // that slot's stretch was fetched long ago
      __syncthreads();
    }
  }

  if (G > 1) {
    // group 1 hands its max, sum and output to group 0 through LDS (the staged keys are done with)
    __syncthreads();
    float* xch = reinterpret_cast<float*>(pf_lds) + (qwave * 64 + lane) * (DT * 4 + 2);
    if (grp == 1) {
      xch[0] = m;
      xch[1] = l;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) xch[2 + dt * 4 + i] = o[dt][i];
    }
    __syncthreads();
    if (grp == 1) return;
    const float m1 = xch[0], l1 = xch[1];
    const float m_all = fmaxf(m, m1);
    // a group that saw no key has max -inf and nothing to add
    const float a0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - m_all);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - m_all);
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[dt][i] = o[dt][i] * a0 + xch[2 + dt * 4 + i] * a1;
  }

  l = pf_sum_over_rows(l);
  if (q_ok) {
    const float inv = 1.0f / l;
    bf16_t* orow = out + (long)(q_start + my_q) * ldo + (long)h * D;
    // a lane's four neighbouring channels of a tile are one 8-byte store (the launcher has checked
    // that rows start 8 bytes aligned)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint2 pk;
      pk.x = pack_bf16x2(o[dt][0] * inv, o[dt][1] * inv);
      pk.y = pack_bf16x2(o[dt][2] * inv, o[dt][3] * inv);
      *reinterpret_cast<uint2*>(orow + dt * 16 + g * 4) = pk;
    }
  }
}

// One workgroup per (64-query tile, request, head); max_q_len sizes the grid and is the host's
// upper bound on the tokens any request brings (a request may bring none: its workgroups leave at
// once).  single_below: requests that bring exactly one token, and that as one of the step's first
// single_below tokens, are left to another kernel.  Head
// sizes 32, 64, 96, 128 and a positive scale; others are refused.
extern "C" int mgpt_prefill_attention_bf16(
    const void* q, long ldq, void* out, long ldo, const void* kpool, const void* vpool,
    const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, int n_req,
    int max_q_len, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    int single_below, hipStream_t stream) {
  if (n_req == 0 || max_q_len == 0) return MGPT_OK;
  if (!q || !out || !kpool || !vpool || !block_tables || !cu_q || !seq_lens) return MGPT_ERR_NULL;
  if (n_req < 0 || max_q_len < 0 || n_head <= 0 || n_kv_head <= 0 || (n_head % n_kv_head) != 0 ||
      page_size <= 0 || max_blocks <= 0 || window < 0 || (ldq % 8) != 0 || (ldo % 4) != 0 ||
      (((size_t)out) & 7) != 0 || !(scale > 0.f))
    return MGPT_ERR_BAD_SHAPE;
  if (n_req > 65535 || n_head > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid((max_q_len + PF_QT - 1) / PF_QT, n_req, n_head);
#define PF_LAUNCH(DD, GG)                                                                                       \
  {                                                                                                             \
    constexpr int sb = PF_KT * GG;                                                                              \
    constexpr int kld = (DD & (DD - 1)) == 0 ? DD : DD + 8;                                                     \
    constexpr int lds_bytes = 4 * sb * kld * (int)sizeof(bf16_t) + 4 * sb * 4;                                  \
    static bool allowed = false; /* more LDS than a kernel gets without asking */                               \
    if (!allowed) {                                                                                             \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_attention_kernel<DD, GG>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);         \
      if (e != hipSuccess) return (int)e;                                                                       \
      allowed = true;                                                                                           \
    }                                                                                                           \
    hipLaunchKernelGGL((prefill_attention_kernel<DD, GG>), grid, dim3(256 * GG), lds_bytes, stream,             \
                       (const bf16_t*)q, ldq, (bf16_t*)out, ldo, (const bf16_t*)kpool, (const bf16_t*)vpool,    \
                       block_tables, max_blocks, cu_q, seq_lens, n_head, n_kv_head, page_size, scale, window,   \
                       single_below);                                                                          \
  }
  // Two wave groups halve the walk of a tile over its keys; one group leaves LDS for a second
  // workgroup on the compute unit.  The first serves a step with few tiles, the second one with many.
  const long tiles = (long)grid.x * grid.y * grid.z;
  const bool two = tiles <= 320;
  switch (head_dim) {
    case 32: if (two) PF_LAUNCH(32, 2) else PF_LAUNCH(32, 1) break;
    case 64: if (two) PF_LAUNCH(64, 2) else PF_LAUNCH(64, 1) break;
    case 96: PF_LAUNCH(96, 1); break;
    case 128: PF_LAUNCH(128, 1); break;
    default: return MGPT_ERR_BAD_SHAPE;
  }
#undef PF_LAUNCH
  return mgpt_last_error();
}
