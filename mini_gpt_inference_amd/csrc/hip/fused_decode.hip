// The fused kernels of a decode step with few rows (bfloat16): two kernels a layer.
//
//  * fused_attention_decode_kernel, one workgroup per head and token (or two or four neighbouring
//    tokens, in steps of many rows): adds up the residual row that
//    the kernels before it left as a sum (fused_decode.h), LayerNorm, this head's query, key and
//    value (src/minigpt_infer/model.py:43,49-53), the key and value into their page
//    (src/minigpt_infer/cache/paged.py:125-137), attention over the request's pages and the new
//    key (model.py:61-87; the Triton decode kernel src/minigpt_infer/attention/triton_paged.py:44-123),
//    and this head's share of the output projection (model.py:89-90), left as one of n_head partial
//    sums of the residual.
//  * fused_mlp_decode_kernel, one workgroup per 64 hidden units (and group of rows): adds up the
//    residual rows, LayerNorm, its slice of the first product with bias and GELU-tanh, and that
//    slice's share of the second product (model.py:96-101), left as one of hidden/64 partial sums.
//  * residual_layernorm_kernel and residual_settle_kernel: the LayerNorm of rows that are still such
//    a sum (the final norm, model.py:186), and the sum itself for whoever needs plain rows.
//
// A decode step at a few rows is a chain of dependent kernels that each wait for one memory round
// trip; every load whose address does not depend on the step's data (weights, block table) is
// issued first, the sums of the residual and the LayerNorm happen while they are on their way.
// Sums are added in a fixed order, so results do not depend on timing.
#include "fused_decode.h"
#include "launchers.h"

typedef __attribute__((ext_vector_type(2))) __bf16 fd_bf16x2_t;

// A barrier between the waves of a workgroup that waits for this wave's LDS traffic only.
// __syncthreads() also waits for every global load in flight, and here the loads of the weights
// (and of keys and values) are meant to stay in flight across the barriers of the work that does
// not need them yet.  Only LDS is exchanged across these barriers, never global memory.
__device__ __forceinline__ void fd_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}


template <int CTRL>
__device__ __forceinline__ float fd_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// sum over the LPK neighbouring lanes of an aligned group; every lane of the group gets it
template <int LPK>
__device__ __forceinline__ float fd_group_sum(float v) {
  v += fd_dpp<MGPT_DPP_XOR1>(v);
  if (LPK >= 4) v += fd_dpp<MGPT_DPP_XOR2>(v);
  if (LPK >= 8) v += fd_dpp<MGPT_DPP_HALF_MIRROR>(v);
  if (LPK >= 16) v += fd_dpp<MGPT_DPP_MIRROR>(v);
  return v;
}

// sum over the lanes that hold the same channels of different keys (lane = key group * LPK + channel
// group): rotations within the rows of 16 lanes, then the four rows; no trip through LDS
template <int LPK>
__device__ __forceinline__ float fd_sum_over_keys(float v) {
  if (LPK <= 8) v += fd_dpp<0x128>(v);  // row_ror:8
  if (LPK <= 4) v += fd_dpp<0x124>(v);  // row_ror:4
  if (LPK <= 2) v += fd_dpp<0x122>(v);  // row_ror:2
  const unsigned int u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned int ux = __float_as_uint(x);
  const auto b = __builtin_amdgcn_permlane32_swap(ux, ux, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

__device__ __forceinline__ float fd_dot2(unsigned int a, unsigned int b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(fd_bf16x2_t, a), __builtin_bit_cast(fd_bf16x2_t, b),
                                         c, false);
}

__device__ __forceinline__ float4 fd_add4(float4 a, float4 b) {
  return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}

__device__ __forceinline__ float4 fd_keep4(bool keep, float4 v) {
  return make_float4(keep ? v.x : 0.f, keep ? v.y : 0.f, keep ? v.z : 0.f, keep ? v.w : 0.f);
}

__device__ __forceinline__ float4 fd_bf16x4(uint2 t) {
  return make_float4(__uint_as_float(t.x << 16), __uint_as_float(t.x & 0xffff0000u), __uint_as_float(t.y << 16),
                     __uint_as_float(t.y & 0xffff0000u));
}

__device__ __forceinline__ float fd_sum4(float4 v) { return (v.x + v.y) + (v.z + v.w); }

// the block (row tile, k step) of a packed matrix (fold_norm.hip: pack_weight_kernel), this lane's 8 values
__device__ __forceinline__ bf16x8_t fd_packed(const bf16_t* w, long tile, int k_steps, int s, int lane) {
  return *reinterpret_cast<const bf16x8_t*>(w + ((tile * k_steps + s) * 64 + lane) * 8);
}

// ---- A residual row added up by a whole workgroup.  The row has V = width / 4 vectors of four; the
// workgroup's threads form G = FUSED_THREADS / V groups of V, and group q loads the parts q, q + G,
// q + 2 G, q + 3 G (group 0 also the base): FUSED_GROUP_PARTS * G parts at most.  The loads are
// issued by fd_row_issue and used by fd_row_sum, so that the caller can issue other loads between
// the two; there is no branch between a load and the next (a load past the parts reads part 0
// again and is dropped), because the compiler waits for every load in flight where control flow
// joins.
struct FdRowLoads {
  float4 base;
  float4 part[FUSED_GROUP_PARTS];
};

// TABLES: the row is the token's and the position's table rows (no base, no parts)
template <bool TABLES>
__device__ __forceinline__ void fd_row_issue(const FusedResidual& r, long row, int id, int pos, int V, int G,
                                             FdRowLoads& L) {
  const int tid = threadIdx.x;
  const int gq = tid / V, vq = tid - gq * V;
  const int gc = gq < G ? gq : 0;
  if (TABLES) {
    const bool has_pos = r.pos_table != nullptr;
    const uint2 t = reinterpret_cast<const uint2*>(r.tok_table)[(long)id * V + vq];
    const uint2 q = reinterpret_cast<const uint2*>(has_pos ? r.pos_table : r.tok_table)[(long)(has_pos ? pos : id) * V + vq];
    L.base = fd_add4(fd_bf16x4(t), fd_keep4(has_pos, fd_bf16x4(q)));
  } else {
    L.base = reinterpret_cast<const float4*>(r.base)[row * V + vq];
    const float* parts = r.n_parts > 0 ? r.partials : r.base;  // no parts: every load below reads the base again
#pragma unroll
    for (int u = 0; u < FUSED_GROUP_PARTS; ++u) {
      const int p = gc + u * G;
      L.part[u] = reinterpret_cast<const float4*>(parts + (p < r.n_parts ? p * r.part_stride : 0))[row * V + vq];
    }
  }
}

// Returns, in the threads tid < V, the row's vector tid; xs: LDS for G * V vectors.  One barrier inside.
template <bool TABLES>
__device__ __forceinline__ float4 fd_row_sum(const FusedResidual& r, int V, int G, const FdRowLoads& L, float* xs) {
  const int tid = threadIdx.x;
  const int gq = tid / V, vq = tid - gq * V;
  float4 s = fd_keep4(gq == 0, L.base);
  if (!TABLES) {
#pragma unroll
    for (int u = 0; u < FUSED_GROUP_PARTS; ++u) s = fd_add4(s, fd_keep4(gq + u * G < r.n_parts, L.part[u]));
  }
  if (gq < G) reinterpret_cast<float4*>(xs)[gq * V + vq] = s;
  fd_barrier();
  float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (tid < V) {
    // groups beyond the parts hold zeros: only the groups that had something are read
    const int used = TABLES ? 1 : min(G, max(r.n_parts, 1));
    xv = reinterpret_cast<const float4*>(xs)[tid];
#pragma unroll 8
    for (int q = 1; q < used; ++q) xv = fd_add4(xv, reinterpret_cast<const float4*>(xs)[q * V + tid]);
  }
  return xv;
}

// LayerNorm of the row that the threads tid < V hold (xv), through two barriers: returns the normed
// values of this thread's vector (gain and beta applied) in the threads tid < V.
__device__ __forceinline__ float4 fd_row_norm(float4 xv, int V, int C, float eps, float4 gain4, float4 beta4,
                                              float* mean_s, float* var_s) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int waves_used = (V + 63) >> 6;  // the waves that hold the row
  const float ws = wave_sum(fd_sum4(xv));
  if (lane == 0) mean_s[wave] = ws;
  fd_barrier();
  float mean = 0.f;
  for (int w = 0; w < waves_used; ++w) mean += mean_s[w];
  mean /= (float)C;
  float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
  if (tid < V) d = make_float4(xv.x - mean, xv.y - mean, xv.z - mean, xv.w - mean);
  const float wq = wave_sum((d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w));
  if (lane == 0) var_s[wave] = wq;
  fd_barrier();
  float var = 0.f;
  for (int w = 0; w < waves_used; ++w) var += var_s[w];
  const float rstd = 1.0f / sqrtf(var / (float)C + eps);
  return make_float4(d.x * rstd * gain4.x + beta4.x, d.y * rstd * gain4.y + beta4.y, d.z * rstd * gain4.z + beta4.z,
                     d.w * rstd * gain4.w + beta4.w);
}

struct FusedAttnArgs {
  FusedResidual res;
  const float* gain;
  const float* beta;  // or null
  float eps;
  const bf16_t* wqkv;  // packed [3 * n_head * D rows, width]
  const float* bqkv;   // or null
  const bf16_t* wproj;  // packed [width rows, n_head * D]
  const float* bproj;   // or null
  const bf16_t* normed; // NORMED kernels: the rows after their LayerNorm, [rows][width]; the residual is not read
  float* out_partials;  // [n_head][part_rows][width]
  long out_part_stride;
  bf16_t* kpool;
  bf16_t* vpool;
  const int* slot_mapping;
  const int* block_tables;
  int max_blocks;
  const int* positions;
  const int* q_req;
  int n_rows, width, n_head, page_shift, num_pages;
  unsigned int page_bytes;
  float scale_log2e;
};

// Sixteen waves a workgroup: a compute unit issues a wave's 16-byte-a-lane load about every 6 ns
// (170 KB a microsecond) when sixteen waves each have up to sixteen of them in flight, and half of
// that with eight waves that have twice as many each.  A wave therefore holds few loads at a time,
// and a lane at most 128 registers.
// TK: tokens of a workgroup (the same head of TK neighbouring tokens).  The projections of all of
// them come out of the same matrix loads (a token a column of the MFMA's output), and the waves are
// dealt out to the tokens for attention.  More tokens a workgroup pay where the step has more
// (token, head) pairs than the machine has compute units.
// NORMED: the rows come normed, in bfloat16 (a.normed): every head's workgroup adding up the same
// pending parts of its tokens is, at many rows, more traffic between the XCDs than everything else
// the kernel reads (32 parts of 2 KB a token, eight heads: the first barrier passed after 12 us at
// 128 rows), so a LayerNorm kernel before this one adds them up once.
template <int D, bool TABLES, int TK = 1, bool NORMED = false>
__global__ __launch_bounds__(FUSED_THREADS) void fused_attention_decode_kernel(FusedAttnArgs a) {
  static_assert(!(NORMED && TABLES), "normed rows are no table rows");
  constexpr int T = 3 * D / 16;                  // row tiles of this head's q, k and v
  constexpr int TG = T < 12 ? T : 12;            // of them in flight together
  constexpr int NG = T / TG;
  constexpr int SMAX = 12 / TG;                  // k steps whose loads are in flight together
  constexpr int LPK = D / 8, KPI = 64 / LPK;     // lanes per key, keys per load instruction
  constexpr int NI = LPK / 2 < 2 ? 2 : LPK / 2;  // load instructions of a wave's keys in one pass
  constexpr int CHUNK = NI * KPI;                // keys of a wave in one pass
  constexpr int NK2 = D <= 32 ? 1 : D / 32;      // k steps of the projection that hold this head's columns
  constexpr int TP2 = 4 / NK2 > 0 ? 4 / NK2 : 1; // its row tiles per wave whose loads are in flight together
  // one pool for what is never alive together: the rows' partial sums, then the waves' sums of
  // q, k, v, then attention's partial results; a stretch of it per token
  constexpr int POOL_ONE = FUSED_WAVES * T * 16 > 4096 ? FUSED_WAVES * T * 16 : 4096;
  static_assert(FUSED_WAVES * T * 16 <= POOL_ONE, "the pool holds the waves' sums of q, k, v");
  static_assert(FUSED_WAVES * D <= POOL_ONE, "the pool holds the waves' sums of attention");
  static_assert(TK >= 1 && TK <= 4 && 3 * D * TK <= FUSED_THREADS, "a thread per value of q, k, v of every token");
  __shared__ __align__(16) float pool[POOL_ONE * TK];
  __shared__ __align__(16) bf16_t act_s[TK * FUSED_MAX_WIDTH];
  __shared__ __align__(16) float gain_s[FUSED_MAX_WIDTH], beta_s[FUSED_MAX_WIDTH];
  __shared__ __align__(16) float bproj_s[FUSED_MAX_WIDTH];  // the projection's bias (first head only)
  __shared__ __align__(16) bf16_t q_s[TK * D];
  __shared__ __align__(16) bf16_t k_s[TK * D];
  __shared__ __align__(16) bf16_t v_s[TK * D];
  __shared__ __align__(16) bf16_t y_s[TK * D];
  __shared__ float m_s[FUSED_WAVES];
  __shared__ float l_s[FUSED_WAVES];
  float* const red_s = pool;
  float* const acc_s = pool;

  const int h = blockIdx.x, n0 = blockIdx.y * TK;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 15, g = lane >> 4;
  const int sub = lane / LPK, dg = lane % LPK;
  const int C = a.width, KS = C >> 5, V = C >> 2;
  const int ltok = TK == 1 ? 0 : lrow % TK;  // the token whose column of an MFMA this lane holds

  // ---- The prologue.  A compute unit issues a wave's 16-byte loads at about a kilobyte every
  // twelve clocks, and a barrier lets a wave pass only when every other wave has issued what
  // stands before it: only a quarter of the weights' loads stand before the barrier at which the
  // row's partial sums meet (the row's loads of the last waves would otherwise wait behind all the
  // weights of the first: measured, 1.6 us a layer slower); the rest, and the keys and values, are
  // sent for behind it, while the first waves norm a row each.  A wave's loads come back in order:
  // the step's numbers and the rows first, keys and values last.
  // (a token beyond the step's rows repeats the workgroup's first and stores nothing, like a token of
  // the padding; a decode-only step: token n is request n)
  int tokn[TK], qpos[TK], slot[TK];
  bool ok[TK];
  const int* bt[TK];
  bool any = false;
#pragma unroll
  for (int t = 0; t < TK; ++t) {
    const bool in = n0 + t < a.n_rows;
    tokn[t] = in ? n0 + t : n0;
    ok[t] = in && a.q_req[tokn[t]] >= 0;
    any = any || ok[t];
    qpos[t] = a.positions[tokn[t]];
    slot[t] = a.slot_mapping[tokn[t]];
    bt[t] = a.block_tables + (long)tokn[t] * a.max_blocks;
  }
  // attention: the waves are dealt out to the tokens, WPT neighbouring waves each
  constexpr int WPT = FUSED_WAVES / TK;
  const int wt = wave / WPT, ww = wave - wt * WPT;  // this wave's token, and its place among the token's waves
  int my_qpos = qpos[0];
  bool my_ok = ok[0];
  const int* my_bt = bt[0];
#pragma unroll
  for (int t = 1; t < TK; ++t)
    if (wt == t) {
      my_qpos = qpos[t];
      my_ok = ok[t];
      my_bt = bt[t];
    }
  const int c00 = ww * CHUNK;
  int page0[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int e = (c00 + i * KPI + sub) >> a.page_shift;
    page0[i] = my_bt[e < a.max_blocks ? e : a.max_blocks - 1];
  }
  // a row: V vectors of four; the threads form G groups of V, group q adds up the parts q, q + G, ...
  // (group 0 the base as well)
  const int G = FUSED_THREADS / V;
  const int gq = tid / V, vq = tid - gq * V;
  float4 piece[TK];
  float4 part[TK][FUSED_GROUP_PARTS];
  uint2 normed4 = make_uint2(0u, 0u);  // NORMED: group t of the threads brings token t's row
  if (NORMED) {
#pragma unroll
    for (int t = 0; t < TK; ++t)
      if (gq == t) normed4 = reinterpret_cast<const uint2*>(a.normed)[(long)tokn[t] * V + vq];
  }
#pragma unroll
  for (int t = 0; t < TK; ++t) {
    piece[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (NORMED) continue;
    if (TABLES) {
      if (gq == 0) {
        const uint2 tr = reinterpret_cast<const uint2*>(a.res.tok_table)[(long)a.res.ids[tokn[t]] * V + vq];
        piece[t] = fd_bf16x4(tr);
        if (a.res.pos_table)
          piece[t] = fd_add4(piece[t], fd_bf16x4(reinterpret_cast<const uint2*>(
                                           a.res.pos_table)[(long)a.res.positions[tokn[t]] * V + vq]));
      }
    } else {
      if (gq == 0) piece[t] = reinterpret_cast<const float4*>(a.res.base)[(long)tokn[t] * V + vq];
#pragma unroll
      for (int u = 0; u < FUSED_GROUP_PARTS; ++u) {
        part[t][u] = make_float4(0.f, 0.f, 0.f, 0.f);
        const int p = gq + u * G;
        if (gq < G && p < a.res.n_parts)
          part[t][u] = reinterpret_cast<const float4*>(a.res.partials + p * a.res.part_stride)[(long)tokn[t] * V + vq];
      }
    }
  }
  // the LayerNorm's gain and bias go through LDS to the waves that will norm the rows, and so does
  // what the last epilogue adds (first head: the projection's bias); a group of threads each
  const bool proj_bias = h == 0 && a.bproj != nullptr;
  float4 gb4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (gq == 0 && !NORMED) gb4 = reinterpret_cast<const float4*>(a.gain)[vq];
  else if (gq == 1 && !NORMED && a.beta) gb4 = reinterpret_cast<const float4*>(a.beta)[vq];
  else if (gq == 2 && proj_bias) gb4 = reinterpret_cast<const float4*>(a.bproj)[vq];
  // what the epilogue of q, k, v adds: this thread's bias
  const int qt = tid / (3 * D), qi = tid - qt * (3 * D);  // this thread's token and value among its q, k, v
  float qkv_bias = 0.f;
  if (qt < TK && a.bqkv) qkv_bias = a.bqkv[(qi / D) * a.n_head * D + h * D + qi % D];
  const int n_tiles2 = C >> 4;
  const int per = (KS + FUSED_WAVES - 1) / FUSED_WAVES;  // k steps of a wave
  const int ks0 = wave * per;
  const int nks = max(0, min(per, KS - ks0));
  const int tiles_per_part = a.n_head * (D / 16);
  constexpr int NW = TG * SMAX;  // loads of the weights' first pass: a quarter before the first barrier, the rest behind it
  static_assert(NW % 4 == 0, "four pieces");
  bf16x8_t wv[TG][SMAX];
#define FA_LOAD_W(piece_no)                                                                                 \
  _Pragma("unroll") for (int q_ = 0; q_ < NW / 4; ++q_) {                                                  \
    const int idx_ = (piece_no) * (NW / 4) + q_, tt_ = idx_ / SMAX, i_ = idx_ % SMAX;                       \
    const long tile_ = (long)(tt_ / (D / 16)) * tiles_per_part + h * (D / 16) + (tt_ % (D / 16));           \
    wv[tt_][i_] = fd_packed(a.wqkv, tile_, KS, i_ < nks ? ks0 + i_ : 0, lane);                              \
  }
  // keys and values of a token's first pass: their addresses need the block table and the position only
  // (kv_end: the keys before the token's own)
  const int page_mask = (1 << a.page_shift) - 1;
  const unsigned int lane_off = ((unsigned int)(h << a.page_shift) * D + dg * 8) * 2u;
  uint4 kraw[NI], vraw[NI];
  const int kv_end = my_qpos;
#define FA_LOAD_KV                                                                                                    \
  if (my_ok && c00 < kv_end) { /* the same in all lanes of a wave */                                                 \
    _Pragma("unroll") for (int i = 0; i < NI; ++i) {                                                                 \
      const int j_ = c00 + i * KPI + sub;                                                                            \
      const bool follow_ = j_ < kv_end && (unsigned int)page0[i] < (unsigned int)a.num_pages;                        \
      const unsigned int row_off_ = ((unsigned int)page0[i] * a.page_bytes) + (unsigned int)(j_ & page_mask) * (D * 2u); \
      const unsigned int off_ = follow_ ? row_off_ + lane_off : 0u;                                                  \
      kraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.kpool) + off_);                      \
      vraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.vpool) + off_);                      \
    }                                                                                                                \
  }
  FA_LOAD_W(0)
  if (!any) return;  // tokens of the padding only (the whole workgroup)
  if (NORMED) {
    // all of the weights are sent for at once; the rows go to LDS as they are.  The keys and values
    // wait for the block table's entries: they are sent for behind the barrier, which then does not.
    FA_LOAD_W(1)
    FA_LOAD_W(2)
    FA_LOAD_W(3)
    if (gq < TK) reinterpret_cast<uint2*>(act_s + gq * FUSED_MAX_WIDTH)[vq] = normed4;
    if (gq == 2 && proj_bias) reinterpret_cast<float4*>(bproj_s)[vq] = gb4;
  } else {

    // ---- the residual rows' sums: every group of threads its parts, then a wave per row all groups
#pragma unroll
    for (int t = 0; t < TK; ++t) {
      if (!TABLES) {
#pragma unroll
        for (int u = 0; u < FUSED_GROUP_PARTS; ++u) piece[t] = fd_add4(piece[t], part[t][u]);
      }
      if (gq < G) reinterpret_cast<float4*>(pool + t * POOL_ONE)[gq * V + vq] = piece[t];
    }
    if (gq < 3) reinterpret_cast<float4*>(gq == 0 ? gain_s : gq == 1 ? beta_s : bproj_s)[vq] = gb4;
    fd_barrier();
    // every wave sends for the rest of its weights and for its keys and values; then the first waves
    // norm a row each (LDS and arithmetic only) while the others wait at the next barrier
    FA_LOAD_W(1)
    FA_LOAD_W(2)
    FA_LOAD_W(3)
    FA_LOAD_KV
    if (wave < TK) {
      const float* xs = pool + wave * POOL_ONE;
      int row = tokn[0];
      bool row_ok = ok[0];
#pragma unroll
      for (int t = 1; t < TK; ++t)
        if (wave == t) {
          row = tokn[t];
          row_ok = ok[t];
        }
      float4 xv[2];
      xv[0] = xv[1] = make_float4(0.f, 0.f, 0.f, 0.f);
      // ---- LayerNorm, within one wave: no barrier between the sums
      // groups beyond the parts hold zeros: only the groups that had something are read
      const int used = TABLES ? 1 : min(G, max(a.res.n_parts, 1));
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int v = lane + 64 * u;
        if (v < V) {
          xv[u] = reinterpret_cast<const float4*>(xs)[v];
#pragma unroll 8
          for (int q = 1; q < used; ++q) xv[u] = fd_add4(xv[u], reinterpret_cast<const float4*>(xs)[q * V + v]);
          // the row as it stands, stored by the first head's workgroup for the kernels behind this one
          if (h == 0 && row_ok && a.res.settled) reinterpret_cast<float4*>(a.res.settled + (long)row * C)[v] = xv[u];
        }
      }
      const float mean = wave_sum(fd_sum4(xv[0]) + fd_sum4(xv[1])) / (float)C;
      float4 dv[2];
      float sq = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const bool in = lane + 64 * u < V;
        dv[u] = in ? make_float4(xv[u].x - mean, xv[u].y - mean, xv[u].z - mean, xv[u].w - mean)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
        sq += (dv[u].x * dv[u].x + dv[u].y * dv[u].y) + (dv[u].z * dv[u].z + dv[u].w * dv[u].w);
      }
      const float rstd = 1.0f / sqrtf(wave_sum(sq) / (float)C + a.eps);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int v = lane + 64 * u;
        if (v < V) {
          const float4 gn = reinterpret_cast<const float4*>(gain_s)[v], bt4 = reinterpret_cast<const float4*>(beta_s)[v];
          uint2 pk;
          pk.x = pack_bf16x2(dv[u].x * rstd * gn.x + bt4.x, dv[u].y * rstd * gn.y + bt4.y);
          pk.y = pack_bf16x2(dv[u].z * rstd * gn.z + bt4.z, dv[u].w * rstd * gn.w + bt4.w);
          reinterpret_cast<uint2*>(act_s + wave * FUSED_MAX_WIDTH)[v] = pk;
        }
      }
    }
  }
  fd_barrier();  // also: the rows' partial sums are read, their place takes the waves' sums now
  if (NORMED) FA_LOAD_KV
#undef FA_LOAD_W
#undef FA_LOAD_KV

  // ---- q, k, v of this head: every wave a stretch of k over all the row tiles; the waves' sums
  // meet in LDS (column c of the MFMA's output holds token c mod TK: the lanes of the first TK columns speak)
  for (int s0 = 0, first = 1;; first = 0) {
#pragma unroll
    for (int grp = 0; grp < NG; ++grp) {
      if (grp > 0 || !first) {
#pragma unroll
        for (int tt = 0; tt < TG; ++tt) {
          const int t2 = grp * TG + tt;
          const long tile = (long)(t2 / (D / 16)) * tiles_per_part + h * (D / 16) + (t2 % (D / 16));
#pragma unroll
          for (int i = 0; i < SMAX; ++i) wv[tt][i] = fd_packed(a.wqkv, tile, KS, s0 + i < nks ? ks0 + s0 + i : 0, lane);
        }
      }
      bf16x8_t b[SMAX];
#pragma unroll
      for (int i = 0; i < SMAX; ++i)
        b[i] = *reinterpret_cast<const bf16x8_t*>(act_s + ltok * FUSED_MAX_WIDTH +
                                                  (s0 + i < nks ? ks0 + s0 + i : 0) * 32 + g * 8);
#pragma unroll
      for (int tt = 0; tt < TG; ++tt) {
        f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < SMAX; ++i)
          if (s0 + i < nks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[tt][i], b[i], acc, 0, 0, 0);
        if (lrow < TK) {
          float4* r = reinterpret_cast<float4*>(red_s + ((lrow * FUSED_WAVES + wave) * T + grp * TG + tt) * 16 + g * 4);
          float4 v = make_float4(acc[0], acc[1], acc[2], acc[3]);
          if (s0 > 0) v = fd_add4(v, *r);
          *r = v;
        }
      }
    }
    s0 += SMAX;
    if (s0 >= per) break;
  }
  // the output projection's matrix for this head: asked for now, used after attention
  const int ks_b = (h * D) >> 5;
  const int KS2 = (a.n_head * D) >> 5;
  bf16x8_t w2[TP2][NK2];
#pragma unroll
  for (int j = 0; j < TP2; ++j) {
    const int tile = wave + FUSED_WAVES * j;
#pragma unroll
    for (int i = 0; i < NK2; ++i) w2[j][i] = fd_packed(a.wproj, tile < n_tiles2 ? tile : 0, KS2, ks_b + i, lane);
  }
  fd_barrier();
  if (qt < TK) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < FUSED_WAVES; ++w) v += red_s[(qt * FUSED_WAVES + w) * T * 16 + qi];
    const int part = qi / D, d = qi - part * D;
    const bf16_t b = float_to_bf16(v + qkv_bias);
    if (part == 0) {
      q_s[qt * D + d] = b;
    } else {
      (part == 1 ? k_s : v_s)[qt * D + d] = b;
      int my_slot = -1;
#pragma unroll
      for (int t = 0; t < TK; ++t)
        if (qt == t && ok[t]) my_slot = slot[t];
      if (my_slot >= 0) {
        const long page = my_slot >> a.page_shift;
        const int off = my_slot & page_mask;
        const long dst = ((((page * a.n_head + h) << a.page_shift) + off) * (long)D) + d;
        (part == 1 ? a.kpool : a.vpool)[dst] = b;
      }
    }
  }
  fd_barrier();  // also: the waves' sums are read, their place takes attention's partial results

  // ---- attention: each token's waves over the keys before the token's own (from the pages); the
  // token's first wave its own as well (from LDS)
  float m = -INFINITY, l = 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (my_ok) {
    const uint4 qraw = *reinterpret_cast<const uint4*>(q_s + wt * D + dg * 8);
    for (int c_base = 0; c_base < kv_end; c_base += CHUNK * WPT) {
      const int c0 = c_base + c00;
      if (c_base > 0 && c0 < kv_end) {
        int page[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int e = (c0 + i * KPI + sub) >> a.page_shift;
          page[i] = my_bt[e < a.max_blocks ? e : a.max_blocks - 1];
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int j = c0 + i * KPI + sub;
          const bool follow = j < kv_end && (unsigned int)page[i] < (unsigned int)a.num_pages;
          const unsigned int row_off = ((unsigned int)page[i] * a.page_bytes) + (unsigned int)(j & page_mask) * (D * 2u);
          const unsigned int off = follow ? row_off + lane_off : 0u;
          kraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.kpool) + off);
          vraw[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(a.vpool) + off);
        }
      }
      if (__builtin_amdgcn_readfirstlane(c0 >= kv_end)) continue;
      bool valid[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        valid[i] = c0 + i * KPI + sub < kv_end;
        if (!valid[i]) vraw[i] = make_uint4(0, 0, 0, 0);  // its weight is 0, but 0 * NaN is not
      }
      float s[NI];
      float cmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        float dot = fd_dot2(qraw.x, kraw[i].x, 0.f);
        dot = fd_dot2(qraw.y, kraw[i].y, dot);
        dot = fd_dot2(qraw.z, kraw[i].z, dot);
        dot = fd_dot2(qraw.w, kraw[i].w, dot);
        dot = fd_group_sum<LPK>(dot) * a.scale_log2e;
        s[i] = valid[i] ? dot : -INFINITY;
        cmax = fmaxf(cmax, s[i]);
      }
      const float m_new = fmaxf(m, wave_max(cmax));
      if (m_new != -INFINITY) {  // the same in all lanes; false only while the wave has seen no key
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);  // m = -inf: 0
        l *= alpha;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] *= alpha;
        m = m_new;
#pragma unroll
        for (int i = 0; i < NI; i += 2) {
          const float pa = __builtin_amdgcn_exp2f(s[i] - m_new), pb = __builtin_amdgcn_exp2f(s[i + 1] - m_new);
          l += pa + pb;
          const unsigned int pp = pack_bf16x2(pa, pb);
          const unsigned int va[4] = {vraw[i].x, vraw[i].y, vraw[i].z, vraw[i].w};
          const unsigned int vb[4] = {vraw[i + 1].x, vraw[i + 1].y, vraw[i + 1].z, vraw[i + 1].w};
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            // (va.low half, vb.low half) and (va.high half, vb.high half): channel 2w and 2w+1 of both keys
            const unsigned int lo = __builtin_amdgcn_perm(vb[w], va[w], 0x05040100u);
            const unsigned int hi = __builtin_amdgcn_perm(vb[w], va[w], 0x07060302u);
            acc[2 * w] = fd_dot2(pp, lo, acc[2 * w]);
            acc[2 * w + 1] = fd_dot2(pp, hi, acc[2 * w + 1]);
          }
        }
      }
    }
    if (ww == 0) {
      // the token's own key and value: its first wave takes them in, that wave's first key group holds the weight
      const uint4 kk = *reinterpret_cast<const uint4*>(k_s + wt * D + dg * 8);
      const uint4 vv = *reinterpret_cast<const uint4*>(v_s + wt * D + dg * 8);
      float dot = fd_dot2(qraw.x, kk.x, 0.f);
      dot = fd_dot2(qraw.y, kk.y, dot);
      dot = fd_dot2(qraw.z, kk.z, dot);
      dot = fd_dot2(qraw.w, kk.w, dot);
      dot = fd_group_sum<LPK>(dot) * a.scale_log2e;
      const float m_new = fmaxf(m, dot);
      const float alpha = __builtin_amdgcn_exp2f(m - m_new);
      l *= alpha;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= alpha;
      m = m_new;
      const float p = __builtin_amdgcn_exp2f(dot - m_new);
      if (sub == 0) {
        l += p;
        const unsigned int pp = pack_bf16x2(p, 0.f);
        const unsigned int vw[4] = {vv.x, vv.y, vv.z, vv.w};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          acc[2 * w] = fd_dot2(pp, vw[w] & 0xffffu, acc[2 * w]);
          acc[2 * w + 1] = fd_dot2(pp, vw[w] >> 16, acc[2 * w + 1]);
        }
      }
    }
  }

  // ---- merge: first across the key groups of a wave (lanes that differ above the LPK lanes of a
  // key: the maximum is the wave's already, so the sums simply add), then across a token's waves in LDS
  // (the waves of a token that stores nothing leave zeros)
  l = fd_sum_over_keys<LPK>(l);
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = fd_sum_over_keys<LPK>(acc[e]);
  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
  if (lane < LPK) {
    float4* dst = reinterpret_cast<float4*>(acc_s + wave * D + dg * 8);
    dst[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    dst[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
  fd_barrier();
  if (tid < D * TK) {
    const int t = tid / D, d = tid - t * D;
    const int w0 = t * WPT;
    float mx = m_s[w0];
#pragma unroll
    for (int w = 1; w < WPT; ++w) mx = fmaxf(mx, m_s[w0 + w]);
    float av = 0.f, lt = 0.f;
#pragma unroll
    for (int w = 0; w < WPT; ++w) {
      const float f = __builtin_amdgcn_exp2f(m_s[w0 + w] - mx);  // a wave without keys: exp2(-inf) = 0, and its sums are 0
      av = fmaf(acc_s[(w0 + w) * D + d], f, av);
      lt = fmaf(l_s[w0 + w], f, lt);
    }
    y_s[tid] = float_to_bf16(av / lt);
  }
  fd_barrier();

  // ---- this head's share of the output projection: row tiles dealt out to the waves
  {
    const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t yb[NK2];
#pragma unroll
    for (int i = 0; i < NK2; ++i) {
      const int idx0 = (ks_b + i) * 32 + g * 8 - h * D;  // where this lane's 8 values of k lie in the head
      yb[i] = (idx0 >= 0 && idx0 < D) ? *reinterpret_cast<const bf16x8_t*>(y_s + ltok * D + idx0) : zero8;
    }
    bool store = false;
#pragma unroll
    for (int t = 0; t < TK; ++t)
      if (lrow == t) store = ok[t];
    float* orow = a.out_partials + h * a.out_part_stride + (long)(n0 + (lrow < TK ? lrow : 0)) * C;
    for (int pass = 0;; ++pass) {
#pragma unroll
      for (int j = 0; j < TP2; ++j) {
        const int tile = wave + FUSED_WAVES * (pass * TP2 + j);
        if (tile < n_tiles2) {
          f32x4_t o = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NK2; ++i) o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2[j][i], yb[i], o, 0, 0, 0);
          if (store) {
            const int oc = tile * 16 + g * 4;
            float4 v = make_float4(o[0], o[1], o[2], o[3]);
            if (proj_bias) v = fd_add4(v, *reinterpret_cast<const float4*>(bproj_s + oc));
            *reinterpret_cast<float4*>(orow + oc) = v;
          }
        }
      }
      if (FUSED_WAVES * (pass + 1) * TP2 >= n_tiles2) break;
#pragma unroll
      for (int j = 0; j < TP2; ++j) {
        const int tile = wave + FUSED_WAVES * ((pass + 1) * TP2 + j);
#pragma unroll
        for (int i = 0; i < NK2; ++i) w2[j][i] = fd_packed(a.wproj, tile < n_tiles2 ? tile : 0, KS2, ks_b + i, lane);
      }
    }
  }
}

struct FusedMlpArgs {
  FusedResidual res;
  const float* gain;
  const float* beta;  // or null
  float eps;
  const bf16_t* wfc;    // packed [hidden rows, width]
  const float* bfc;     // or null
  const bf16_t* wproj;  // packed [width rows, hidden]
  const float* bproj;   // or null
  float* out_partials;  // [hidden / FUSED_MLP_SLICE][part_rows][width]
  long out_part_stride;
  int n_rows, width, hidden, rows_per_wg;
};

#define FM_TS (FUSED_MLP_SLICE / 16)   // row tiles of a workgroup's slice of the first product
#define FM_KQ (FUSED_WAVES / FM_TS)    // waves that share a row tile, each a stretch of k
#define FM_SMAX 4                      // k steps of it whose loads are in flight together
#define FM_NK2 (FUSED_MLP_SLICE / 32)  // k steps of the second product that the slice covers
#define FM_TP2 2                       // row tiles of the second product per wave in flight together
#define FM_GS (FUSED_MLP_SLICE + 8)    // row stride of the slice's activations in LDS
#define FM_RED_BYTES (FM_KQ * FM_TS * 64 * 4 * 4)
#define FM_WAVE_PARTS 8                // parts of a residual row that one wave adds up

// VU: vectors of four that a lane holds of a row (width <= 256 VU).  The workgroup has rows_per_wg
// rows (a power of two up to 16); a row belongs to 16 / rows_per_wg waves, of which each adds up
// every (16 / rows_per_wg)-th part of it (FM_WAVE_PARTS at most), and the first the base as well.
template <int VU>
__global__ __launch_bounds__(FUSED_THREADS) void fused_mlp_decode_kernel(FusedMlpArgs a) {
  // the waves' sums of their rows [16][width] (later: of the first product), then the normed rows
  // [rows_per_wg][width + 8]
  extern __shared__ __align__(16) char smem[];
  __shared__ __align__(16) bf16_t g_s[16 * FM_GS];
  const int j = blockIdx.x, r0 = blockIdx.y * a.rows_per_wg;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 15, g = lane >> 4;
  const int C = a.width, KS = C >> 5, V = C >> 2;
  const int RW = a.rows_per_wg;
  const int lda = C + 8;
  float* xs = reinterpret_cast<float*>(smem);
  float* red = reinterpret_cast<float*>(smem);
  const int xs_bytes = FUSED_WAVES * C * 4 > FM_RED_BYTES ? FUSED_WAVES * C * 4 : FM_RED_BYTES;
  bf16_t* act_s = reinterpret_cast<bf16_t*>(smem + xs_bytes);

  // ---- loads in the order in which their data is needed: this wave's share of a residual row,
  // then the weights of both products (the second product's behind the barrier that the rows'
  // sums need: a wave passes a barrier only when all others have issued what stands before it)
  // Few parts (at most FM_WAVE_PARTS: what an attention kernel of eight heads leaves): a row's first
  // wave sends for all of them itself and adds them in its registers; nothing of the row goes through
  // LDS before the LayerNorm, no wave waits for another's loads, and the other waves have only their
  // weights to send for (a decode step of the 50.9M model: 0.146 -> 0.137 ms at batch 8).
  const bool alone = a.res.n_parts <= FM_WAVE_PARTS && RW <= 4;   // (with two waves a row the shares stay: 0.256 against 0.258 ms at 64 rows)
  const int wpr = FUSED_WAVES / RW;           // waves of a row
  const int lr = wave / wpr, sw = wave - lr * wpr;
  const int row = r0 + lr;
  const bool has_row = row < a.n_rows && (!alone || sw == 0);   // the same in all lanes, like everything that decides a load here
  float4 xs4[VU], gv[VU], bv[VU];
#pragma unroll
  for (int u = 0; u < VU; ++u) xs4[u] = gv[u] = bv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (has_row) {
    float4 xp[VU][FM_WAVE_PARTS];
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int c4 = lane + 64 * u;
      const int cc = c4 < V ? c4 : 0;
      if (sw == 0) {
        xs4[u] = reinterpret_cast<const float4*>(a.res.base)[(long)row * V + cc];
        gv[u] = reinterpret_cast<const float4*>(a.gain)[cc];
        if (a.beta) bv[u] = reinterpret_cast<const float4*>(a.beta)[cc];
      }
#pragma unroll
      for (int k = 0; k < FM_WAVE_PARTS; ++k) {
        xp[u][k] = make_float4(0.f, 0.f, 0.f, 0.f);
        const int p = alone ? k : sw + k * wpr;
        if (p < a.res.n_parts)
          xp[u][k] = reinterpret_cast<const float4*>(a.res.partials + p * a.res.part_stride)[(long)row * V + cc];
      }
    }
#pragma unroll
    for (int u = 0; u < VU; ++u)
#pragma unroll
      for (int k = 0; k < FM_WAVE_PARTS; ++k) xs4[u] = fd_add4(xs4[u], xp[u][k]);
  }
  // what the epilogues add: this thread's bias of the first product, and (first slice) the second's
  float fc_bias = 0.f;
  if (a.bfc) fc_bias = a.bfc[j * FUSED_MLP_SLICE + (tid >> 8) * 16 + (((tid >> 2) & 63) >> 4) * 4 + (tid & 3)];
  float4 proj_bias[FM_TP2];
#pragma unroll
  for (int q = 0; q < FM_TP2; ++q) {
    proj_bias[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    const int tile = wave + FUSED_WAVES * q;
    if (j == 0 && a.bproj && tile < (C >> 4)) proj_bias[q] = *reinterpret_cast<const float4*>(a.bproj + tile * 16 + g * 4);
  }
  const int tt = wave & (FM_TS - 1), kq = wave / FM_TS;  // this wave's row tile and stretch of k
  const int per = (KS + FM_KQ - 1) / FM_KQ;
  const int ks0 = kq * per;
  const int nks = max(0, min(per, KS - ks0));
  bf16x8_t wv[FM_SMAX];
#pragma unroll
  for (int i = 0; i < FM_SMAX; ++i) wv[i] = fd_packed(a.wfc, (long)j * FM_TS + tt, KS, i < nks ? ks0 + i : 0, lane);

  // ---- the waves' shares of the rows meet in LDS; a row's first wave adds them, LayerNorm, bfloat16
  if (!alone) {   // (the same for the whole workgroup)
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int c4 = lane + 64 * u;
      if (c4 < V) reinterpret_cast<float4*>(xs + wave * C)[c4] = xs4[u];
    }
  } else {
    // nothing is exchanged, but the barrier stays: the waves that gather reach it when their rows have
    // arrived, and it holds the second product's loads of all the others back behind those (without it
    // the step is slower, 0.1393 against 0.1369 ms at batch 8: the rows wait in the queue behind the weights)
    asm volatile("" ::"v"(xs4[0].x) : "memory");
  }
  fd_barrier();
  const int KS2 = a.hidden >> 5;
  const int n_tiles2 = C >> 4;
  bf16x8_t w2[FM_TP2][FM_NK2];
#pragma unroll
  for (int q = 0; q < FM_TP2; ++q) {
    const int tile = wave + FUSED_WAVES * q;
#pragma unroll
    for (int i = 0; i < FM_NK2; ++i) w2[q][i] = fd_packed(a.wproj, tile < n_tiles2 ? tile : 0, KS2, j * FM_NK2 + i, lane);
  }
  if (sw == 0 && has_row) {
    const int used = alone ? 1 : min(wpr, max(a.res.n_parts, 1));  // waves beyond the parts hold zeros
    float4 xv[VU];
    float s1 = 0.f;
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int c4 = lane + 64 * u;
      xv[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c4 < V) {
        xv[u] = xs4[u];
        for (int q = 1; q < used; ++q) xv[u] = fd_add4(xv[u], reinterpret_cast<const float4*>(xs + (wave + q) * C)[c4]);
        if (j == 0 && a.res.settled) reinterpret_cast<float4*>(a.res.settled + (long)row * C)[c4] = xv[u];
        s1 += fd_sum4(xv[u]);
      }
    }
    const float mean = wave_sum(s1) / (float)C;
    float sq = 0.f;
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const bool in = lane + 64 * u < V;
      xv[u] = in ? make_float4(xv[u].x - mean, xv[u].y - mean, xv[u].z - mean, xv[u].w - mean)
                 : make_float4(0.f, 0.f, 0.f, 0.f);
      sq += (xv[u].x * xv[u].x + xv[u].y * xv[u].y) + (xv[u].z * xv[u].z + xv[u].w * xv[u].w);
    }
    const float rstd = 1.0f / sqrtf(wave_sum(sq) / (float)C + a.eps);
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int c4 = lane + 64 * u;
      if (c4 < V) {
        uint2 pk;
        pk.x = pack_bf16x2(xv[u].x * rstd * gv[u].x + bv[u].x, xv[u].y * rstd * gv[u].y + bv[u].y);
        pk.y = pack_bf16x2(xv[u].z * rstd * gv[u].z + bv[u].z, xv[u].w * rstd * gv[u].w + bv[u].w);
        *reinterpret_cast<uint2*>(act_s + lr * lda + c4 * 4) = pk;
      }
    }
  }
  fd_barrier();

  // ---- first product: a wave one row tile of the slice over its stretch of k
  // (a column of the MFMA beyond the workgroup's rows repeats its first row and is never stored)
  const int arow = (lrow < RW && r0 + lrow < a.n_rows) ? lrow : 0;
  f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0;;) {
#pragma unroll
    for (int i = 0; i < FM_SMAX; ++i)
      if (s0 + i < nks) {
        const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(act_s + arow * lda + (ks0 + s0 + i) * 32 + g * 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[i], b, acc, 0, 0, 0);
      }
    s0 += FM_SMAX;
    if (s0 >= per) break;
#pragma unroll
    for (int i = 0; i < FM_SMAX; ++i)
      wv[i] = fd_packed(a.wfc, (long)j * FM_TS + tt, KS, s0 + i < nks ? ks0 + s0 + i : 0, lane);
  }
  // (the rows' sums were read before the last barrier: their place takes the waves' sums of the product)
  *reinterpret_cast<float4*>(red + ((kq * FM_TS + tt) * 64 + lane) * 4) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  fd_barrier();
  {
    // a thread one hidden unit of one row: the waves' sums in the order of k, bias, GELU
    const int t2 = tid >> 8, ln = (tid >> 2) & 63, i4 = tid & 3;
    float v = 0.f;
#pragma unroll
    for (int q = 0; q < FM_KQ; ++q) v += red[((q * FM_TS + t2) * 64 + ln) * 4 + i4];
    const int o = t2 * 16 + (ln >> 4) * 4 + i4;  // hidden unit within the slice
    g_s[(ln & 15) * FM_GS + o] = float_to_bf16(gelu_tanh_fast(v + fc_bias));
  }
  fd_barrier();

  // ---- the slice's share of the second product: row tiles dealt out to the waves
  bf16x8_t yb[FM_NK2];
#pragma unroll
  for (int i = 0; i < FM_NK2; ++i) yb[i] = *reinterpret_cast<const bf16x8_t*>(g_s + lrow * FM_GS + i * 32 + g * 8);
  const bool store = lrow < RW && r0 + lrow < a.n_rows;
  float* orow = a.out_partials + j * a.out_part_stride + (long)(r0 + lrow) * C;
  for (int pass = 0;; ++pass) {
#pragma unroll
    for (int q = 0; q < FM_TP2; ++q) {
      const int tile = wave + FUSED_WAVES * (pass * FM_TP2 + q);
      if (tile < n_tiles2) {
        f32x4_t o = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < FM_NK2; ++i) o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2[q][i], yb[i], o, 0, 0, 0);
        if (store) {
          const int oc = tile * 16 + g * 4;
          float4 v = make_float4(o[0], o[1], o[2], o[3]);
          if (pass == 0) v = fd_add4(v, proj_bias[q]);
          else if (j == 0 && a.bproj) v = fd_add4(v, *reinterpret_cast<const float4*>(a.bproj + oc));
          *reinterpret_cast<float4*>(orow + oc) = v;
        }
      }
    }
    if (FUSED_WAVES * (pass + 1) * FM_TP2 >= n_tiles2) break;
#pragma unroll
    for (int q = 0; q < FM_TP2; ++q) {
      const int tile = wave + FUSED_WAVES * ((pass + 1) * FM_TP2 + q);
#pragma unroll
      for (int i = 0; i < FM_NK2; ++i) w2[q][i] = fd_packed(a.wproj, tile < n_tiles2 ? tile : 0, KS2, j * FM_NK2 + i, lane);
    }
  }
}

// out[i] = LayerNorm(row rows[i] (or i) of a residual that is still a sum); a workgroup a row
template <typename OT>
__global__ __launch_bounds__(FUSED_THREADS) void residual_layernorm_kernel(FusedResidual res, const float* __restrict__ gain,
                                                                           const float* __restrict__ beta, float eps,
                                                                           const int* __restrict__ rows,
                                                                           OT* __restrict__ out, int width) {
  __shared__ __align__(16) float xs[4 * FUSED_THREADS];
  __shared__ float mean_s[FUSED_WAVES], var_s[FUSED_WAVES];
  const int i = blockIdx.x, tid = threadIdx.x;
  const int V = width >> 2, G = FUSED_THREADS / V;
  const long row = rows ? rows[i] : i;
  FdRowLoads L;
  fd_row_issue<false>(res, row, 0, 0, V, G, L);
  const int vc = tid < V ? tid : 0;
  const float4 gain4 = reinterpret_cast<const float4*>(gain)[vc];
  const float4 beta4 = fd_keep4(beta != nullptr, reinterpret_cast<const float4*>(beta ? beta : gain)[vc]);
  const float4 xv = fd_row_sum<false>(res, V, G, L, xs);
  // (this workgroup is the row's only reader in this launch: the sum may go where the base was)
  if (res.settled && tid < V) reinterpret_cast<float4*>(res.settled + row * width)[tid] = xv;
  const float4 y = fd_row_norm(xv, V, width, eps, gain4, beta4, mean_s, var_s);
  if (tid < V) {
    OT* orow = out + (long)i * width;
    if (sizeof(OT) == 4) {
      reinterpret_cast<float4*>(orow)[tid] = y;
    } else {
      uint2 pk;
      pk.x = pack_bf16x2(y.x, y.y);
      pk.y = pack_bf16x2(y.z, y.w);
      reinterpret_cast<uint2*>(orow)[tid] = pk;
    }
  }
}

// settled[row] = the row's sum; a thread four values (settled may be the base itself).  Not on
// the path of a decode step: for parts that need plain rows.
__global__ __launch_bounds__(256) void residual_settle_kernel(FusedResidual res, int n_rows, int width) {
  const int V = width >> 2;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_rows * V) return;
  const long row = idx / V;
  const int c4 = (int)(idx - row * V);
  float4 s = reinterpret_cast<const float4*>(res.base)[row * V + c4];
  // eight parts on their way at a time, added in the order of the parts (a part beyond the last reads the
  // last one again and is dropped)
  for (int p0 = 0; p0 < res.n_parts; p0 += 8) {
    float4 t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int p = p0 + u < res.n_parts ? p0 + u : res.n_parts - 1;
      t[u] = reinterpret_cast<const float4*>(res.partials + p * res.part_stride)[row * V + c4];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) s = fd_add4(s, fd_keep4(p0 + u < res.n_parts, t[u]));
  }
  reinterpret_cast<float4*>(res.settled)[row * V + c4] = s;
}

// What every launcher checks of a residual that is still a sum.  tables_ok: the kernel can look the
// rows up in the token and position tables itself.
static int check_residual(const FusedResidual& r, int width, bool tables_ok, int max_width = FUSED_MAX_WIDTH) {
  if (width <= 0 || (width % 32) != 0 || width > max_width) return MGPT_ERR_BAD_SHAPE;
  if (!r.base) {
    if (!tables_ok || r.n_parts != 0) return MGPT_ERR_BAD_SHAPE;
    if (!r.tok_table || !r.ids || (r.pos_table && !r.positions)) return MGPT_ERR_NULL;
  }
  if (r.n_parts < 0 || (r.n_parts > 0 && !r.partials)) return MGPT_ERR_NULL;
  if (r.n_parts > 0 && r.part_stride < width) return MGPT_ERR_BAD_SHAPE;
  const size_t align = (size_t)r.base | (size_t)r.partials | (size_t)r.settled | (size_t)(r.part_stride * 4);
  if ((align & 15) != 0 || (((size_t)r.tok_table | (size_t)r.pos_table) & 7) != 0) return MGPT_ERR_BAD_SHAPE;
  return MGPT_OK;
}

// parts that a workgroup of FUSED_THREADS threads adds up of one row (fd_row_issue)
static int group_parts_limit(int width) { return FUSED_GROUP_PARTS * (FUSED_THREADS / (width / 4)); }

static FusedResidual make_residual(const float* base, const float* partials, int n_parts, long part_stride,
                                   const void* tok_table, const void* pos_table, const int* ids,
                                   const int* positions, float* settled) {
  FusedResidual r;
  r.base = base; r.partials = n_parts > 0 ? partials : nullptr; r.n_parts = n_parts; r.part_stride = part_stride;
  r.tok_table = (const bf16_t*)tok_table; r.pos_table = (const bf16_t*)pos_table; r.ids = ids;
  r.positions = positions; r.settled = settled;
  return r;
}

// Most parts of a pending residual of this width that mgpt_residual_layernorm takes (0: the width is not taken).
extern "C" int mgpt_residual_parts_limit(int width) {
  if (width <= 0 || (width % 32) != 0 || width > RESIDUAL_MAX_WIDTH) return 0;
  return group_parts_limit(width);
}

// Most parts of a pending residual of this width that the fused kernels take (0: the width is not taken).
extern "C" int mgpt_fused_parts_limit(int width) {
  if (width <= 0 || (width % 32) != 0 || width > FUSED_MAX_WIDTH) return 0;
  const int a = group_parts_limit(width), b = FM_WAVE_PARTS * FUSED_WAVES;
  return a < b ? a : b;
}

// Tokens that a workgroup of the attention kernel takes in a step of n_rows rows: two from where one
// a workgroup would be more workgroups than compute units, four from where two would (heads of 128
// keep to two: four tokens' q, k, v are more values than the workgroup has threads).  0: more rows
// than the kernel takes (more workgroups than compute units even so: the kernels that share a matrix
// among all rows are faster there).
extern "C" int mgpt_fused_attention_tokens(int n_rows, int n_head, int head_dim) {
  const long pairs = (long)n_rows * n_head;
  const int most = head_dim > 64 ? 2 : 4;
  if (pairs > (long)most * FUSED_ATTN_ONE_TOKEN_WGS) return 0;
  return pairs > 2 * FUSED_ATTN_ONE_TOKEN_WGS ? 4 : pairs > FUSED_ATTN_ONE_TOKEN_WGS ? 2 : 1;
}

// The attention half of a layer for the single tokens of a decode-only step (token n is request n or,
// with q_req[n] < 0, padding).  Refuses (MGPT_ERR_BAD_SHAPE) head sizes other than 16, 32, 64, 128,
// widths beyond FUSED_MAX_WIDTH or no multiple of 32, n_head * head_dim no multiple of 32, pages that
// are no power of two, pools of 4 GiB or more, more parts than mgpt_fused_parts_limit.
// out_partials gets n_head parts.
// Where mgpt_fused_attention_tokens(...) is more than one and the rows are no table rows, the rows
// must come normed as well (normed: bfloat16 [rows][width], the LayerNorm of base; base then has no
// parts, and nothing is stored to settled); with one token a workgroup normed is not read.
extern "C" int mgpt_fused_attention_decode(
    const float* base, const float* partials, int n_parts, long part_stride, const void* tok_table,
    const void* pos_table, const int* ids, const int* token_positions, float* settled, const void* normed,
    const float* gain,
    const float* beta, float eps, const void* wqkv_packed, const float* bqkv, const void* wproj_packed,
    const float* bproj, float* out_partials, long out_part_stride, void* kpool, void* vpool,
    const int* slot_mapping, const int* block_tables, int max_blocks, const int* positions, const int* q_req,
    int n_rows, int width, int n_head, int head_dim, int page_size, int num_pages, float scale,
    hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!gain || !wqkv_packed || !wproj_packed || !out_partials || !kpool || !vpool || !slot_mapping ||
      !block_tables || !positions || !q_req)
    return MGPT_ERR_NULL;
  FusedAttnArgs a;
  a.res = make_residual(base, partials, n_parts, part_stride, tok_table, pos_table, ids, token_positions, settled);
  int rc = check_residual(a.res, width, true);
  if (rc != MGPT_OK) return rc;
  if (n_rows < 0 || n_head <= 0 || max_blocks <= 0 || num_pages <= 0 || ((n_head * head_dim) % 32) != 0 ||
      n_parts > group_parts_limit(width) || out_part_stride < (long)n_rows * width || ((out_part_stride * 4) & 15) != 0 ||
      (((size_t)out_partials | (size_t)gain | (size_t)beta | (size_t)bproj) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  if (n_rows > 65535) return MGPT_ERR_TOO_LARGE;
  int page_shift = -1;
  for (int s = 0; s < 30; ++s)
    if ((1 << s) == page_size) page_shift = s;
  if (page_shift < 0) return MGPT_ERR_BAD_SHAPE;
  const long pool_bytes = (long)num_pages * n_head * page_size * head_dim * 2;
  if (pool_bytes >= (1L << 32)) return MGPT_ERR_BAD_SHAPE;
  const int tk = mgpt_fused_attention_tokens(n_rows, n_head, head_dim);
  if (tk == 0) return MGPT_ERR_BAD_SHAPE;
  if (tk > 1 && base && (!normed || n_parts != 0 || (((size_t)normed) & 7) != 0)) return MGPT_ERR_BAD_SHAPE;
  a.gain = gain; a.beta = beta; a.eps = eps;
  a.wqkv = (const bf16_t*)wqkv_packed; a.bqkv = bqkv; a.wproj = (const bf16_t*)wproj_packed; a.bproj = bproj;
  a.normed = (const bf16_t*)normed;
  a.out_partials = out_partials; a.out_part_stride = out_part_stride;
  a.kpool = (bf16_t*)kpool; a.vpool = (bf16_t*)vpool; a.slot_mapping = slot_mapping;
  a.block_tables = block_tables; a.max_blocks = max_blocks; a.positions = positions; a.q_req = q_req;
  a.n_rows = n_rows; a.width = width; a.n_head = n_head; a.page_shift = page_shift; a.num_pages = num_pages;
  a.page_bytes = (unsigned int)(n_head * page_size * head_dim * 2);
  a.scale_log2e = scale * 1.4426950408889634f;
  // the head is the fast index: the workgroups of a head then land on the same XCD when the number
  // of heads is a multiple of 8, and share its copy of the head's weights
  dim3 grid(n_head, (n_rows + tk - 1) / tk), block(FUSED_THREADS);
#define FA_LAUNCH(DD)                                                                                           \
  do {                                                                                                          \
    constexpr int D4 = DD > 64 ? 64 : DD; /* (heads of 128 never come with four tokens) */                      \
    if (tk == 4) {                                                                                              \
      if (base) hipLaunchKernelGGL((fused_attention_decode_kernel<D4, false, 4, true>), grid, block, 0, stream, a); \
      else hipLaunchKernelGGL((fused_attention_decode_kernel<D4, true, 4>), grid, block, 0, stream, a);         \
    } else if (tk == 2) {                                                                                       \
      if (base) hipLaunchKernelGGL((fused_attention_decode_kernel<DD, false, 2, true>), grid, block, 0, stream, a); \
      else hipLaunchKernelGGL((fused_attention_decode_kernel<DD, true, 2>), grid, block, 0, stream, a);         \
    } else {                                                                                                    \
      if (base) hipLaunchKernelGGL((fused_attention_decode_kernel<DD, false, 1>), grid, block, 0, stream, a);   \
      else hipLaunchKernelGGL((fused_attention_decode_kernel<DD, true, 1>), grid, block, 0, stream, a);         \
    }                                                                                                           \
  } while (0)
  switch (head_dim) {
    case 16: FA_LAUNCH(16); break;
    case 32: FA_LAUNCH(32); break;
    case 64: FA_LAUNCH(64); break;
    case 128: FA_LAUNCH(128); break;
    default: return MGPT_ERR_BAD_SHAPE;
  }
#undef FA_LAUNCH
  return mgpt_last_error();
}

// rows of a workgroup of the feed-forward kernel, a power of two: as few as keep the workgroups
// within 256, and no more than leave every row the waves that its parts need
static int mlp_rows_per_wg(int n_rows, int hidden, int n_parts) {
  const int slices = hidden / FUSED_MLP_SLICE;
  int most = FUSED_WAVES;  // a row needs a wave per FM_WAVE_PARTS parts
  while (most > 1 && (FUSED_WAVES / most) * FM_WAVE_PARTS < n_parts) most >>= 1;
  int rw = 1;
  while (rw < most && (long)slices * ((n_rows + rw - 1) / rw) > 256) rw <<= 1;
  return rw;
}

// The feed-forward half of a layer.  hidden must be a multiple of FUSED_MLP_SLICE; the residual must
// have a base (no table rows); out_partials gets hidden / FUSED_MLP_SLICE parts.
extern "C" int mgpt_fused_mlp_decode(const float* base, const float* partials, int n_parts, long part_stride,
                                     const void* tok_table, const void* pos_table, const int* ids,
                                     const int* token_positions, float* settled, const float* gain,
                                     const float* beta, float eps, const void* wfc_packed, const float* bfc,
                                     const void* wproj_packed, const float* bproj, float* out_partials,
                                     long out_part_stride, int n_rows, int width, int hidden, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!gain || !wfc_packed || !wproj_packed || !out_partials) return MGPT_ERR_NULL;
  FusedMlpArgs a;
  a.res = make_residual(base, partials, n_parts, part_stride, tok_table, pos_table, ids, token_positions, settled);
  int rc = check_residual(a.res, width, false);
  if (rc != MGPT_OK) return rc;
  if (n_rows < 0 || hidden <= 0 || (hidden % FUSED_MLP_SLICE) != 0 || n_parts > FM_WAVE_PARTS * FUSED_WAVES ||
      out_part_stride < (long)n_rows * width || ((out_part_stride * 4) & 15) != 0 ||
      (((size_t)out_partials | (size_t)gain | (size_t)beta | (size_t)bproj) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  a.gain = gain; a.beta = beta; a.eps = eps;
  a.wfc = (const bf16_t*)wfc_packed; a.bfc = bfc; a.wproj = (const bf16_t*)wproj_packed; a.bproj = bproj;
  a.out_partials = out_partials; a.out_part_stride = out_part_stride;
  a.n_rows = n_rows; a.width = width; a.hidden = hidden;
  a.rows_per_wg = mlp_rows_per_wg(n_rows, hidden, n_parts);
  const int groups = (n_rows + a.rows_per_wg - 1) / a.rows_per_wg;
  if (groups > 65535) return MGPT_ERR_TOO_LARGE;
  dim3 grid(hidden / FUSED_MLP_SLICE, groups), block(FUSED_THREADS);
  size_t smem = (size_t)FUSED_WAVES * width * 4;
  if (smem < FM_RED_BYTES) smem = FM_RED_BYTES;
  smem += (size_t)a.rows_per_wg * (width + 8) * 2;
  if (width <= 256) hipLaunchKernelGGL(fused_mlp_decode_kernel<1>, grid, block, smem, stream, a);
  else hipLaunchKernelGGL(fused_mlp_decode_kernel<2>, grid, block, smem, stream, a);
  return mgpt_last_error();
}

extern "C" int mgpt_fused_mlp_parts(int hidden) {
  return (hidden > 0 && (hidden % FUSED_MLP_SLICE) == 0) ? hidden / FUSED_MLP_SLICE : 0;
}

// out[i] = LayerNorm of row rows[i] (or i) of a residual that is still a sum (with a base); out float32 or
// bfloat16.  settled (optional; may be the base): the rows' sums are stored there as well, row by row
// as named by rows[].  Widths up to RESIDUAL_MAX_WIDTH, at most mgpt_residual_parts_limit(width) parts.
extern "C" int mgpt_residual_layernorm(const float* base, const float* partials, int n_parts, long part_stride,
                                       const void* tok_table, const void* pos_table, const int* ids,
                                       const int* token_positions, const float* gain, const float* beta,
                                       float eps, const int* rows, void* out, int out_dtype, int n_rows, int width,
                                       float* settled, hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!gain || !out) return MGPT_ERR_NULL;
  const FusedResidual r = make_residual(base, partials, n_parts, part_stride, tok_table, pos_table, ids,
                                        token_positions, settled);
  int rc = check_residual(r, width, false, RESIDUAL_MAX_WIDTH);
  if (rc != MGPT_OK) return rc;
  if (n_rows < 0 || n_parts > group_parts_limit(width) || (((size_t)out | (size_t)gain | (size_t)beta) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  dim3 grid(n_rows), block(FUSED_THREADS);
  if (out_dtype == MGPT_F32)
    hipLaunchKernelGGL(residual_layernorm_kernel<float>, grid, block, 0, stream, r, gain, beta, eps, rows, (float*)out, width);
  else if (out_dtype == MGPT_BF16)
    hipLaunchKernelGGL(residual_layernorm_kernel<bf16_t>, grid, block, 0, stream, r, gain, beta, eps, rows, (bf16_t*)out, width);
  else
    return MGPT_ERR_BAD_DTYPE;
  return mgpt_last_error();
}

// settled[row] = base[row] + the parts; settled may be base
extern "C" int mgpt_residual_settle(const float* base, const float* partials, int n_parts, long part_stride,
                                    const void* tok_table, const void* pos_table, const int* ids,
                                    const int* token_positions, float* settled, int n_rows, int width,
                                    hipStream_t stream) {
  if (n_rows == 0) return MGPT_OK;
  if (!settled) return MGPT_ERR_NULL;
  const FusedResidual r = make_residual(base, partials, n_parts, part_stride, tok_table, pos_table, ids,
                                        token_positions, settled);
  int rc = check_residual(r, width, false, RESIDUAL_MAX_WIDTH);
  if (rc != MGPT_OK) return rc;
  if (n_rows < 0) return MGPT_ERR_BAD_SHAPE;
  const long total = (long)n_rows * (width / 4);
  hipLaunchKernelGGL(residual_settle_kernel, dim3((unsigned int)((total + 255) / 256)), dim3(256), 0, stream, r,
                     n_rows, width);
  return mgpt_last_error();
}
