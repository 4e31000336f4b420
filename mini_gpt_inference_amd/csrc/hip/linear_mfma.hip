// Tiled bfloat16 matrix product on the MFMA units for many rows (prompt portions):
// out[n, o] = sum_k act[n, k] * W[o, k] (+ bias[o]) with an optional GELU-tanh or residual-add
// epilogue, or one that also stores new keys and values into their cache pages (nn.Linear as in
// src/minigpt_infer/model.py:43-44,96-101; the cache write of src/minigpt_infer/cache/paged.py:125-137).
//
// One kernel template, five tile shapes.  What bounds a tile kernel on this machine is the traffic
// between LDS and the MFMA units: a wave that owns R x C outputs reads (R + C) * 32 operand values
// from LDS for R * C * 32 multiply-adds, so a wave's tile is as large as the problem allows while
// it still gives every compute unit work: 256 x 256 outputs per workgroup (eight waves of
// 128 x 64) for large problems, down to 32 x 32 (four waves of 16 x 16) for a prompt portion of a
// hundred tokens.  A step along k is 64 long.
//
// The workgroup stages its slice of the activations and of W in LDS twice over.  A row of a slice
// is 128 bytes, eight chunks of 16; chunk c of row r lies at position c ^ (r & 7) of its row.  With
// that, the 16 rows x 4 chunks that an MFMA operand read (ds_read_b128) touches are served at the
// full 256 bytes per clock; rows padded by 16 bytes, the usual remedy, take twice as long on this
// LDS (measured with SQ_LDS_BANK_CONFLICT), and unpadded rows four times.
//
// Two steps' worth of loads are in flight: while step s is multiplied, the chunks of step s + 1
// (loaded during step s - 1) go into the other LDS buffer and those of step s + 2 are sent for,
// both spread between the MFMAs, because LDS takes writes at half the rate of reads and all at
// once they would hold every wave up.  MFMA operands are read from LDS two groups of MFMAs ahead
// of their use.  W is the first MFMA operand, so a lane ends up with four neighbouring output
// columns of one row and stores them as one vector.
//
// Tiles are numbered so that the workgroups that run at the same time on an XCD (which has an L2
// of its own) form a block of a few row tiles by a few column tiles, whose operands that L2 holds.
//
// Five further variants (DIRECT) send the slices from memory straight into LDS
// (global_load_lds_dwordx4) instead of through registers: three or four stages for a long inner
// size, 128 x 192 tiles for wide outputs under many rows, and four or six stages of 32 x 32 tiles for
// the rows of a decode step under a large matrix; see the kernel, choose_direct and launch_any.
#include "common.h"
#include <type_traits>
#include "launchers.h"

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

// The bias of the four neighbouring output columns oc..oc+3 a lane holds.
__device__ __forceinline__ void mfma_bias4(const float* __restrict__ bias, int oc, int n_out, bool vec, float b4[4]) {
  b4[0] = b4[1] = b4[2] = b4[3] = 0.f;
  if (!bias) return;
  if (vec) {
    const float4 t = *reinterpret_cast<const float4*>(bias + oc);
    b4[0] = t.x; b4[1] = t.y; b4[2] = t.z; b4[3] = t.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) b4[e] = oc + e < n_out ? bias[oc + e] : 0.f;
  }
}

// Stores the four columns oc..oc+3 of row n: bias, activation, then a plain store, an add into
// the residual stream, or a store that also puts the four values at cache_dst (a key's or value's
// place in its cache page; null for query columns and rows without a slot).
// `vec`: the four columns can go as one aligned vector.
template <int EPI, typename OT>
__device__ __forceinline__ void mfma_store4(const f32x4_t& a, const float b4[4], OT* __restrict__ out, long ldo,
                                            int n, int oc, int n_out, bool vec, bf16_t* cache_dst) {
  OT* orow = out + (long)n * ldo;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] = a[e] + b4[e];
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
    // the four columns lie in one head (the launcher checks that sizes are multiples of 4)
    if (EPI == MM_EPI_QKV && cache_dst) *reinterpret_cast<uint2*>(cache_dst) = pk;
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

// Deals the workgroup ids out so that an XCD's workgroups (ids that agree modulo 8 go to the same
// XCD, which has an L2 of its own) are neighbours in tile order.
__device__ __forceinline__ int mfma_xcd_tile_id(int pid, int total) {
  const int per_xcd = (total + 7) >> 3, tall = (total & 7) ? (total & 7) : 8;
  const int xcd = pid & 7, local = pid >> 3;
  return xcd < tall ? xcd * per_xcd + local : tall * per_xcd + (xcd - tall) * (per_xcd - 1) + local;
}

namespace {

constexpr int MM_BK = 64;
constexpr int MM_LD = MM_BK;       // LDS row stride in elements: 128 bytes, eight 16-byte chunks
constexpr int MM_GROUP = 4;         // row tiles per block of tiles

// WTM x WTN: 16-wide tiles per wave along the rows of the activations and along the rows of W;
// WVM x WVN: waves in a workgroup along the same.
// AHEAD: steps whose chunks are on their way from memory beyond the one that is being put into LDS
// (1: the schedule described above).  With few tiles of few rows over a large matrix that has to
// come from memory, a step's MFMAs are over long before the chunks of the step after next arrive
// (a 64 x 64 tile: 8 MFMAs a wave and step against a microsecond or more), and the product takes
// a memory round trip every two steps; more steps in flight, each in registers of its own, take that
// wait apart.
// KG: wave groups that share a tile (1 or 2).  With 2, the workgroup has twice the waves: group 0
// multiplies the first half (32) of every step along k and group 1 the second, each wave over the same
// part of the tile as its twin in the other group, and the twins' sums meet in LDS once, after the last
// step (float32 outputs only: the epilogue that stores them has no barrier, so group 1 is done then).
// For few tiles of 64 x 64 under a long inner size: a compute unit that has one such tile has four
// waves, too few to cover each other's waits for LDS and the barrier.
template <int WTM, int WTN, int WVM, int WVN, int EPI, typename OT, int AHEAD = 1, int KG = 1, int DIRECT = 0>
__global__ __launch_bounds__(64 * WVM * WVN * KG) void linear_mfma_kernel(
    const bf16_t* __restrict__ act, long lda, const bf16_t* __restrict__ w,
    const float* __restrict__ bias, OT* __restrict__ out, long ldo, int n_rows, int n_out, int k_dim,
    int k_parts, long part_stride, MfmaScatter sc) {
  static_assert(KG == 1 || (KG == 2 && sizeof(OT) == 4 && AHEAD == 1), "two wave groups: float32 outputs");
  static_assert(DIRECT == 0 || (DIRECT >= 2 && AHEAD == 1 && KG == 1), "slices straight into LDS: two stages or more");
  constexpr int T = 64 * WVM * WVN * KG;
  constexpr int STAGES = DIRECT > 0 ? DIRECT : 2;   // slices of a step that LDS holds
  constexpr int HALVES = (MM_BK / 32) / KG;   // halves of a step along k that a wave multiplies
  constexpr int BM = WVM * WTM * 16, BN = WVN * WTN * 16;
  constexpr int TPR = MM_BK / 8;  // threads per staged row (16 bytes each)
  constexpr int RPP = T / TPR;      // rows per staging pass
  constexpr int PA = BM / RPP, PW = BN / RPP;
  static_assert(DIRECT > 0 || (BM % RPP == 0 && BN % RPP == 0), "tile rows must be whole staging passes");
  static_assert(RPP % 8 == 0 && MM_BK == 64 && BM % 8 == 0 && BN % 8 == 0, "rows of eight chunks, swizzled in eights");
  extern __shared__ __align__(16) bf16_t lds[];
  bf16_t* const as_base = lds;                           // [STAGES][BM * MM_LD]
  bf16_t* const ws_base = lds + STAGES * BM * MM_LD;   // [STAGES][BN * MM_LD]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kg = KG == 1 ? 0 : wave_all / (WVM * WVN);     // this wave's group: which half of a step it multiplies
  const int wave = KG == 1 ? wave_all : wave_all - kg * (WVM * WVN);
  const int row_tiles = (n_rows + BM - 1) / BM, col_tiles = (n_out + BN - 1) / BN;
  int row_tile, col_tile, part;
  {
    // with the inner size split into k_parts, part p of every tile comes before part p + 1 of any
    const int tiles = row_tiles * col_tiles;
    const int wid = mfma_xcd_tile_id(blockIdx.x, gridDim.x);
    part = wid / tiles;
    const int id = wid - part * tiles;
    const int per_group = MM_GROUP * col_tiles;
    const int group = id / per_group, in_group = id - group * per_group;
    const int first = group * MM_GROUP;
    const int rows_here = row_tiles - first < MM_GROUP ? row_tiles - first : MM_GROUP;
    row_tile = first + in_group % rows_here;
    col_tile = in_group / rows_here;
  }
  const int row0 = row_tile * BM, col0 = col_tile * BN;
  // this workgroup's stretch of the inner size (all of it unless the product is split), in whole steps
  const int k_per = (((k_dim + MM_BK - 1) / MM_BK + k_parts - 1) / k_parts) * MM_BK;
  const int k_begin = part * k_per;
  const int k_len = k_dim - k_begin < k_per ? k_dim - k_begin : k_per;
  out += part * part_stride;
  if (part != 0) bias = nullptr;  // of a product split along k, the first stretch's sums carry the bias (if any is given)
  const int wr = (wave / WVN) * (WTM * 16), wc = (wave % WVN) * (WTN * 16);
  const int lrow = lane & 15;

  const int srow = tid / TPR, sk = (tid % TPR) * 8;
  const int s_lds = srow * MM_LD + (((tid % TPR) ^ (srow & 7)) * 8);  // where this thread's chunk goes (RPP % 8 == 0)
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // What a thread stages per step: PA chunks of the activations' slice and PW of W's, each 16 bytes.
  constexpr int ITEMS = PA + PW;
  bf16x8_t gv[AHEAD][ITEMS];
  // rows past the end are read from the last row: their results are never stored
  const bf16_t* gp[ITEMS];
#pragma unroll
  for (int p = 0; p < PA; ++p) {
    const int r = row0 + srow + p * RPP;
    gp[p] = act + (long)(r < n_rows ? r : n_rows - 1) * lda + k_begin + sk;
  }
#pragma unroll
  for (int p = 0; p < PW; ++p) {
    const int r = col0 + srow + p * RPP;
    gp[PA + p] = w + (long)(r < n_out ? r : n_out - 1) * k_dim + k_begin + sk;
  }
  // A chunk that lies beyond the stretch's end (in its last, partial step) is read from the stretch's start instead
  // and counts as zero when it is stored: the select then waits for no load.
  // (set: which of the AHEAD sets of registers; a constant wherever these are called)
  auto load_item = [&](int p, int step, int set = 0) {
    const int k0 = step * MM_BK;
    gv[set][p] = *reinterpret_cast<const bf16x8_t*>(gp[p] + (k0 + sk + 8 <= k_len ? k0 : -sk));
  };
  auto store_item = [&](int p, int step, int buf, int set = 0) {
    bf16_t* dst = p < PA ? as_base + buf * (BM * MM_LD) + p * RPP * MM_LD
                         : ws_base + buf * (BN * MM_LD) + (p - PA) * RPP * MM_LD;
    *reinterpret_cast<bf16x8_t*>(dst + s_lds) = step * MM_BK + sk + 8 <= k_len ? gv[set][p] : zero8;
  };

  f32x4_t acc[WTN][WTM];  // [column tile of W][row tile of activations]
#pragma unroll
  for (int i = 0; i < WTN; ++i)
#pragma unroll
    for (int j = 0; j < WTM; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int k_steps = (k_len + MM_BK - 1) / MM_BK;
  const int c0 = ((lane >> 4) ^ (lrow & 7)) * 8;  // this lane's chunk of an operand row, first half of a step

  // One step along k.  Its 2 * WTM groups of MFMAs (one row tile of the activations against the
  // wave's WTN column tiles, for one half of the step) read their operands from LDS two groups
  // ahead of their use, so that a read's latency hides behind the MFMAs of the groups before it.
  // Spread between the groups, the thread puts the next step's chunks (loaded during the step
  // before this one) into the other LDS buffer and sends for those of the step after: LDS takes
  // writes at half the rate of reads, and all at once they would hold every wave up.
  // store_next / load_after: a compile-time yes or no; set: the registers that hold step s + 1 and
  // take step s + 1 + AHEAD
  auto k_step = [&](int s, auto store_next, auto load_after, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    const int buf = DIRECT > 0 ? s % STAGES : s & 1;
    const bf16_t* as = as_base + buf * (BM * MM_LD) + (wr + lrow) * MM_LD;
    const bf16_t* ws = ws_base + buf * (BN * MM_LD) + (wc + lrow) * MM_LD;
    constexpr int GROUPS = HALVES * WTM;
    bf16x8_t wf[HALVES][WTN], af[3];
    // the second half's chunk is 4 further, which the swizzle turns into a flip of bit 5 of the offset
    // (with two wave groups a wave has one half only: its group's)
    const int h0 = kg * 32;
    auto read_a = [&](int g) {
      return *reinterpret_cast<const bf16x8_t*>(as + (g % WTM) * 16 * MM_LD + (c0 ^ (KG == 1 ? (g / WTM) * 32 : h0)));
    };
#pragma unroll
    for (int i = 0; i < WTN; ++i) wf[0][i] = *reinterpret_cast<const bf16x8_t*>(ws + i * 16 * MM_LD + (c0 ^ h0));
    if (WTM == 1 && HALVES == 2) {  // the second half's groups start at once
#pragma unroll
      for (int i = 0; i < WTN; ++i) wf[1][i] = *reinterpret_cast<const bf16x8_t*>(ws + i * 16 * MM_LD + (c0 ^ 32));
    }
    af[0] = read_a(0);
    af[1] = read_a(1);
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      if (g + 2 < GROUPS) af[(g + 2) % 3] = read_a(g + 2);
      if (WTM >= 2 && g % WTM == WTM - 2 && g / WTM + 1 < HALVES) {
#pragma unroll
        for (int i = 0; i < WTN; ++i)
          wf[g / WTM + 1][i] = *reinterpret_cast<const bf16x8_t*>(ws + i * 16 * MM_LD + (c0 ^ ((g / WTM + 1) * 32)));
      }
#pragma unroll
      for (int p = g * ITEMS / GROUPS; p < (g + 1) * ITEMS / GROUPS; ++p) {
        if (decltype(store_next)::value) store_item(p, s + 1, buf ^ 1, set);
        if (decltype(load_after)::value) load_item(p, s + 1 + AHEAD, set);
      }
      // the compiler's scheduler would move each read down to its use again
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < WTN; ++i)
        acc[i][g % WTM] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g / WTM][i], af[g % 3], acc[i][g % WTM], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (decltype(store_next)::value) __syncthreads();  // the other buffer's readers finished before the last barrier
  };
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  using set0 = std::integral_constant<int, 0>;

  if constexpr (DIRECT > 0) {
    // The slices go from memory straight into LDS (global_load_lds_dwordx4: a wave's load puts its 64 lanes'
    // 16 bytes side by side, 1 KB, which is 8 rows of a slice).  The lane that fills position p of row r
    // fetches the chunk that belongs there, p ^ (r & 7).  No registers hold operands on their way and no
    // wave spends instructions on LDS stores; a compute unit also takes in more bytes a microsecond this
    // way than through registers.  STAGES slices of a step in LDS, STAGES - 1 steps on their way; a
    // step's loads are issued behind the barrier that says every wave has read the stage they overwrite.
    // The inner size is whole steps here (the launcher sees to it): nothing can be zeroed on its way.
    constexpr int WAVES = T / 64;
    constexpr int GROUPS_A = BM / 8, GROUPS = (BM + BN) / 8;
    // loads per wave and step: the same for every wave (each counts its own on their way)
    static_assert(GROUPS % WAVES == 0, "the groups of eight rows go round among the waves");
    constexpr int LPW = GROUPS / WAVES;
    constexpr int D = STAGES - 1;
    static_assert((D - 1) * LPW < 64, "the counter of loads in flight");
    typedef __attribute__((address_space(1))) const void* global_ptr_t;
    typedef __attribute__((address_space(3))) void* lds_ptr_t;
    const int lr = lane >> 3, lc = ((lane & 7) ^ lr) * 8;
    const bf16_t* dp[LPW];
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int g = wave_all + i * WAVES;   // 8 rows of the activations' slice, or of W's
      if (g < GROUPS_A) {
        const int r = row0 + g * 8 + lr;
        dp[i] = act + (long)(r < n_rows ? r : n_rows - 1) * lda + k_begin + lc;
      } else {
        const int r = col0 + (g - GROUPS_A) * 8 + lr;
        dp[i] = w + (long)(r < n_out ? r : n_out - 1) * k_dim + k_begin + lc;
      }
    }
    auto issue = [&](int step) {
      const int st = step % STAGES;
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        const int g = wave_all + i * WAVES;
        bf16_t* dst = g < GROUPS_A ? as_base + st * (BM * MM_LD) + g * (8 * MM_LD)
                                   : ws_base + st * (BN * MM_LD) + (g - GROUPS_A) * (8 * MM_LD);
        __builtin_amdgcn_global_load_lds((global_ptr_t)(dp[i] + step * MM_BK), (lds_ptr_t)dst, 16, 0, 0);
      }
    };
    // waits until at most `steps_behind` steps' loads of this wave are still on their way, then for every wave
    auto arrive = [&](int steps_behind) {
#define MM_WAIT_CASE(N) \
  case N: asm volatile("s_waitcnt vmcnt(%0)" ::"n"((N < D ? N : 0) * LPW) : "memory"); break;
      switch (steps_behind) {
        MM_WAIT_CASE(0) MM_WAIT_CASE(1) MM_WAIT_CASE(2) MM_WAIT_CASE(3) MM_WAIT_CASE(4) MM_WAIT_CASE(5) MM_WAIT_CASE(6)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
      }
#undef MM_WAIT_CASE
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    static_assert(D <= 7, "arrive() knows up to six steps behind the one waited for");
#pragma unroll
    for (int j = 0; j < D; ++j)
      if (j < k_steps) issue(j);
    int s = 0;
    for (; s + D < k_steps; ++s) {
      arrive(D - 1);
      issue(s + D);
      k_step(s, no{}, no{}, set0{});
    }
    for (; s < k_steps; ++s) {   // the last steps: nothing more to send for
      arrive(k_steps - 1 - s);
      k_step(s, no{}, no{}, set0{});
    }
  } else {
    // The first two steps' chunks are sent for together, the first step's into registers of their own
    // (free before the loop needs them for MFMA operands): one trip to memory before the first MFMA
    // instead of two, which is a fifth of the whole kernel when the inner size is a few steps long.
    {
      bf16x8_t first[ITEMS];
  #pragma unroll
      for (int p = 0; p < ITEMS; ++p) first[p] = *reinterpret_cast<const bf16x8_t*>(gp[p] + (sk + 8 <= k_len ? 0 : -sk));
      if (AHEAD > 1 || k_steps > 1) {
  #pragma unroll
        for (int j = 1; j <= AHEAD; ++j)
  #pragma unroll
          for (int p = 0; p < ITEMS; ++p) load_item(p, j, j - 1);
      }
  #pragma unroll
      for (int p = 0; p < ITEMS; ++p) {
        bf16_t* dst = p < PA ? as_base + p * RPP * MM_LD : ws_base + (p - PA) * RPP * MM_LD;
        *reinterpret_cast<bf16x8_t*>(dst + s_lds) = sk + 8 <= k_len ? first[p] : zero8;
      }
    }
    __syncthreads();
    int s = 0;
    if constexpr (AHEAD == 1) {
      for (; s + 2 < k_steps; ++s) k_step(s, yes{}, yes{}, set0{});
      if (s + 1 < k_steps) k_step(s++, yes{}, no{}, set0{});
      k_step(s, no{}, no{}, set0{});
    } else {
      // Step s + 1 lies in set s mod AHEAD: the sets take turns, AHEAD steps a round, in whole rounds
      // and without a branch (where control flow joins the compiler waits for every load in flight):
      // a step beyond the last multiplies the zeros that stand in for chunks beyond the stretch's
      // end, and its loads read the stretch's start.
      auto round = [&](auto... set_c) { ((k_step(s, yes{}, yes{}, set_c), ++s), ...); };
      while (s < k_steps) {
        if constexpr (AHEAD == 2) round(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        else if constexpr (AHEAD == 3) round(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{},
                                             std::integral_constant<int, 2>{});
        else round(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{},
                   std::integral_constant<int, 3>{});
      }
    }
  }

  if constexpr (KG == 2) {
    // the two groups' sums of the same part of the tile meet: group 1 hands its over through LDS (the
    // staged operands are done with) and is finished; group 0 adds them, first half of k first
    static_assert(WVM * WVN * WTN * WTM * 64 * 16 <= 2 * (BM + BN) * MM_LD * (int)sizeof(bf16_t), "the sums fit the LDS");
    f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);
    __syncthreads();
    if (kg == 1) {
#pragma unroll
      for (int i = 0; i < WTN; ++i)
#pragma unroll
        for (int j = 0; j < WTM; ++j) red[((wave * WTN + i) * WTM + j) * 64 + lane] = acc[i][j];
    }
    __syncthreads();
    if (kg == 1) return;
#pragma unroll
    for (int i = 0; i < WTN; ++i)
#pragma unroll
      for (int j = 0; j < WTM; ++j) {
        const f32x4_t t = red[((wave * WTN + i) * WTM + j) * 64 + lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][j][e] += t[e];
      }
  }

  // lane holds out[row0 + wr + j*16 + (lane & 15)][col0 + wc + i*16 + (lane >> 4)*4 + e], e = 0..3
  const bool vec = (n_out & 3) == 0 && (ldo & 3) == 0 && (((size_t)out | (size_t)bias) & 15) == 0;
  // bfloat16 outputs go through LDS (the staged operands are done with): a lane's four columns of
  // sixteen different rows would be sixteen 8-byte pieces per store; from LDS a thread stores 16
  // bytes and a row's threads a whole stretch of the row, and a key's or value's eight channels
  // go to their cache page the same way.
  constexpr int LDT = BN + 8;   // row stride of the tile in LDS
  constexpr int LDS_ELEMS = STAGES * (BM + BN) * MM_LD;
  // the whole tile at once if it fits, else the rows of one row of waves at a time
  constexpr int STAGE_ROWS = BM * LDT <= LDS_ELEMS ? BM : BM / WVM;
  constexpr bool CAN_STAGE = sizeof(OT) == 2 && STAGE_ROWS * LDT <= LDS_ELEMS;
  if (CAN_STAGE && EPI != MM_EPI_RESIDUAL && (n_out & 7) == 0 && (ldo & 7) == 0 && (((size_t)out) & 15) == 0 &&
      (EPI != MM_EPI_QKV || ((sc.q_width | sc.kv_width | sc.head_dim) & 7) == 0)) {
    bf16_t* tile = lds;
    for (int part = 0; part < BM / STAGE_ROWS; ++part) {
      __syncthreads();   // the staged operands, or the part before this one, are done with
      if (wr / STAGE_ROWS == part) {
#pragma unroll
        for (int i = 0; i < WTN; ++i) {
          const int tc = wc + i * 16 + (lane >> 4) * 4, oc = col0 + tc;
          float b4[4];
          mfma_bias4(bias, oc < n_out ? oc : 0, n_out, (((size_t)bias) & 15) == 0, b4);
#pragma unroll
          for (int j = 0; j < WTM; ++j) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              v[e] = acc[i][j][e] + b4[e];
              if (EPI == MM_EPI_GELU) v[e] = gelu_tanh_fast(v[e]);
            }
            uint2 pk;
            pk.x = pack_bf16x2(v[0], v[1]);
            pk.y = pack_bf16x2(v[2], v[3]);
            *reinterpret_cast<uint2*>(&tile[(wr - part * STAGE_ROWS + j * 16 + lrow) * LDT + tc]) = pk;
          }
        }
      }
      __syncthreads();
      constexpr int CPR = BN / 8;   // 16-byte chunks per tile row
      for (int c = tid; c < STAGE_ROWS * CPR; c += T) {
        const int row = c / CPR, tc = (c % CPR) * 8;
        const int n = row0 + part * STAGE_ROWS + row, oc = col0 + tc;
        if (n >= n_rows || oc >= n_out) continue;
        const uint4 v8 = *reinterpret_cast<const uint4*>(&tile[row * LDT + tc]);
        *reinterpret_cast<uint4*>(reinterpret_cast<bf16_t*>(out) + (long)n * ldo + oc) = v8;
        if (EPI == MM_EPI_QKV && oc >= sc.q_width) {
          // the chunk's eight columns lie in one head
          const int slot = sc.slot_mapping[n];
          if (slot >= 0) {
            const int page = slot / sc.page_size, off = slot - page * sc.page_size;
            const int cq = oc - sc.q_width;  // column among keys then values
            const bool is_v = cq >= sc.kv_width;
            const int cc = is_v ? cq - sc.kv_width : cq;
            const int hh = cc / sc.head_dim, d = cc - hh * sc.head_dim;
            const long dst = (((long)page * sc.n_kv_head + hh) * sc.page_size + off) * sc.head_dim + d;
            *reinterpret_cast<uint4*>((is_v ? sc.vpool : sc.kpool) + dst) = v8;
          }
        }
      }
    }
    return;
  }
  // A key or value at (row n, column c of head hh, channel d) goes to
  // ((page * n_kv_head + hh) * page_size + offset) * head_dim + d of its pool, page and offset from
  // the row's slot: the row's part and the column's part of that are worked out once each.
  long cache_row[WTM];
  if (EPI == MM_EPI_QKV) {
#pragma unroll
    for (int j = 0; j < WTM; ++j) {
      const int n = row0 + wr + j * 16 + lrow;
      const int slot = n < n_rows ? sc.slot_mapping[n] : -1;
      const int page = slot / sc.page_size, off = slot - page * sc.page_size;
      cache_row[j] = slot < 0 ? -1 : ((long)page * sc.n_kv_head * sc.page_size + off) * sc.head_dim;
    }
  }
#pragma unroll
  for (int i = 0; i < WTN; ++i) {
    const int oc = col0 + wc + i * 16 + (lane >> 4) * 4;
    if (oc >= n_out) continue;
    float b4[4];
    mfma_bias4(bias, oc, n_out, vec, b4);
    bf16_t* cache_col = nullptr;
    if (EPI == MM_EPI_QKV && oc >= sc.q_width) {
      const int c = oc - sc.q_width;  // column among keys then values
      const bool is_v = c >= sc.kv_width;
      const int cc = is_v ? c - sc.kv_width : c;
      const int hh = cc / sc.head_dim, d = cc - hh * sc.head_dim;
      cache_col = (is_v ? sc.vpool : sc.kpool) + (long)hh * sc.page_size * sc.head_dim + d;
    }
#pragma unroll
    for (int j = 0; j < WTM; ++j) {
      const int n = row0 + wr + j * 16 + lrow;
      if (n >= n_rows) continue;
      bf16_t* cache_dst = nullptr;
      if (EPI == MM_EPI_QKV && cache_col && cache_row[j] >= 0) cache_dst = cache_col + cache_row[j];
      mfma_store4<EPI, OT>(acc[i][j], b4, out, ldo, n, oc, n_out, vec, cache_dst);
    }
  }
}

template <int WTM, int WTN, int WVM, int WVN, int EPI, typename OT, int AHEAD, int KG = 1, int DIRECT = 0>
int launch_one(const void* act, long lda, const void* w, const float* bias, void* out, long ldo, int n_rows,
               int n_out, int k_dim, int k_parts, long part_stride, const MfmaScatter& sc, hipStream_t stream) {
  static_assert(AHEAD >= 1 && AHEAD <= 4, "sets of staging registers");
  constexpr int BM = WVM * WTM * 16, BN = WVN * WTN * 16;
  constexpr size_t lds_bytes = (DIRECT > 0 ? DIRECT : 2ul) * (BM + BN) * MM_LD * sizeof(bf16_t);
  static_assert(lds_bytes <= 160 * 1024, "a workgroup's LDS");
  auto kernel = linear_mfma_kernel<WTM, WTN, WVM, WVN, EPI, OT, AHEAD, KG, DIRECT>;
  static bool allowed = false;  // more LDS than a kernel gets without asking
  if (!allowed) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    allowed = true;
  }
  const long tiles = (long)((n_rows + BM - 1) / BM) * ((n_out + BN - 1) / BN) * k_parts;
  if (tiles > 0x7fffffffL) return MGPT_ERR_TOO_LARGE;
  hipLaunchKernelGGL(kernel, dim3((unsigned int)tiles), dim3(64 * WVM * WVN * KG), lds_bytes, stream,
                     (const bf16_t*)act, lda, (const bf16_t*)w, bias, (OT*)out, ldo, n_rows, n_out, k_dim, k_parts,
                     part_stride, sc);
  return mgpt_last_error();
}

template <int WTM, int WTN, int WVM, int WVN, int AHEAD = 1, int DIRECT = 0>
int launch_shape(const void* act, long lda, const void* w, const float* bias, void* out, int out_dtype, long ldo,
                 int n_rows, int n_out, int k_dim, int epilogue, int k_parts, long part_stride,
                 const MfmaScatter& sc, hipStream_t stream) {
#define MM_LAUNCH(E, OT)                                                                                            \
  return launch_one<WTM, WTN, WVM, WVN, E, OT, AHEAD, 1, DIRECT>(act, lda, w, bias, out, ldo, n_rows, n_out, k_dim, \
                                                                 k_parts, part_stride, sc, stream)
  if (epilogue == MM_EPI_NONE && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_NONE, bf16_t);
  if (epilogue == MM_EPI_NONE && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_NONE, float);
  if (epilogue == MM_EPI_GELU && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_GELU, bf16_t);
  if (epilogue == MM_EPI_RESIDUAL && out_dtype == MGPT_F32) MM_LAUNCH(MM_EPI_RESIDUAL, float);
  if (epilogue == MM_EPI_QKV && out_dtype == MGPT_BF16) MM_LAUNCH(MM_EPI_QKV, bf16_t);
#undef MM_LAUNCH
  return MGPT_ERR_BAD_DTYPE;
}

// The 64 x 64 tile with two wave groups (float32 outputs: plain, or added into the residual stream).
int launch_two_groups(const void* act, long lda, const void* w, const float* bias, void* out, int out_dtype, long ldo,
                      int n_rows, int n_out, int k_dim, int epilogue, int k_parts, long part_stride,
                      const MfmaScatter& sc, hipStream_t stream) {
  if (out_dtype != MGPT_F32) return MGPT_ERR_BAD_DTYPE;
  if (epilogue == MM_EPI_NONE)
    return launch_one<2, 2, 2, 2, MM_EPI_NONE, float, 1, 2>(act, lda, w, bias, out, ldo, n_rows, n_out, k_dim, k_parts,
                                                          part_stride, sc, stream);
  if (epilogue == MM_EPI_RESIDUAL)
    return launch_one<2, 2, 2, 2, MM_EPI_RESIDUAL, float, 1, 2>(act, lda, w, bias, out, ldo, n_rows, n_out, k_dim,
                                                              k_parts, part_stride, sc, stream);
  return MGPT_ERR_BAD_DTYPE;
}

// Tile shapes, largest first: rows x columns of a workgroup's tile.
constexpr int MM_SHAPES = 5;
constexpr int MM_TILE_ROWS[MM_SHAPES] = {256, 128, 128, 64, 32};
constexpr int MM_TILE_COLS[MM_SHAPES] = {256, 256, 64, 64, 32};
constexpr int MM_MAX_PARTS = 8;
constexpr int MM_AHEAD = 4;  // steps on their way from memory in the variant for few tiles over a large matrix
// Shape ids from MM_DIRECT_FIRST on: the variants whose slices go from memory straight into LDS, by tile
// (rows x columns), waves and stages: 32 x 32 (four waves of 16 x 16) and 64 x 64 (four of 32 x 32) with four
// stages, 128 x 64 (eight of 32 x 32) with three, 128 x 192 (eight of 64 x 48) with two, 32 x 32 with six.
constexpr int MM_DIRECT_FIRST = MM_SHAPES + 3;
constexpr int MM_DIRECT_VARIANTS = 5;
constexpr int MM_DIRECT_ROWS[MM_DIRECT_VARIANTS] = {32, 64, 128, 128, 32};
constexpr int MM_DIRECT_COLS[MM_DIRECT_VARIANTS] = {32, 64, 64, 192, 32};
constexpr int MM_SHAPE_IDS = MM_DIRECT_FIRST + MM_DIRECT_VARIANTS;

long tiles_of(int shape, int n_rows, int n_out) {
  return (long)((n_rows + MM_TILE_ROWS[shape] - 1) / MM_TILE_ROWS[shape]) *
         ((n_out + MM_TILE_COLS[shape] - 1) / MM_TILE_COLS[shape]);
}

// The largest tile that still fills the machine's 256 compute units.  The two largest shapes run
// one workgroup per unit, so what counts for them is also how full their last round is.
int choose_shape(int n_rows, int n_out) {
  // Few rows under a wide output (the head of a decode step, 50k columns): the product is a pass over
  // the matrix, and a tile taller than the rows only makes each workgroup's share of that pass
  // larger.  Measured at 50304 x 512 (and alike at inner sizes 768 and 1600): 32 rows take 11.4 us
  // with 32 x 32 tiles and 17.9 with 256 x 256, 64 rows 13.9 with 64 x 64 and 19.3, 128 rows 17.5
  // with 128 x 256 and 22.4; from 256 rows on the largest tile is the fastest again.
  if (n_rows <= 32 && tiles_of(4, n_rows, n_out) >= 256) return 4;
  if (n_rows <= 64 && tiles_of(3, n_rows, n_out) >= 256) return 3;
  if (n_rows <= 128 && tiles_of(1, n_rows, n_out) >= 160) return 1;
  for (int shape = 0; shape < 2; ++shape) {
    const long t = tiles_of(shape, n_rows, n_out);
    const long rounds = (t + 255) / 256;
    if (t >= (shape == 0 ? 160 : 140) && 10 * t >= 7 * rounds * 256) return shape;
  }
  // 128 x 64 tiles only where their last round of 256 is well filled: 384 of them (2,048 rows under 1,536
  // columns) leave half the compute units with two tiles and half with one, and 768 tiles of 64 x 64
  // take 8.4 us where they take 9.2; 512 (under 2,048 columns) take 10.3 against 10.6
  {
    const long t = tiles_of(2, n_rows, n_out);
    if (t >= 300 && 100 * t >= 85 * ((t + 255) / 256) * 256) return 2;
  }
  if (tiles_of(3, n_rows, n_out) >= 192) return 3;
  return 4;
}

// Whether the inner size is split into stretches, and then with which tile shape and into how many
// (parts == 1: not at all, and the shape is the one chosen by the tiles alone).  A long inner size
// with few tiles leaves most compute units idle for a long time: then several workgroups share a
// tile, each writes the sum over its stretch to the caller's buffer, and a second kernel adds the
// sums in the order of k (so the result does not depend on which workgroup ran when) and applies
// the epilogue.  That costs a pass over parts x the output, so it is done only for an inner size of
// at least 32 steps whose unsplit product would not fill the compute units; every stretch is at
// least 8 steps long; 64 x 64 tiles if they and the stretches together fill the units, else 32 x 32.
// The QKV epilogue is never split.
void choose_split(int n_rows, int n_out, int k_dim, int epilogue, int* shape, int* parts) {
  *shape = choose_shape(n_rows, n_out);
  *parts = 1;
  const int steps = (k_dim + MM_BK - 1) / MM_BK;
  // "would not fill the units": counted in 64 x 64 tiles for a very long inner size, where the many
  // 32 x 32 tiles that would fill them take far longer than 64 x 64 tiles with stretches
  if (epilogue == MM_EPI_QKV || (n_out & 3) != 0 || steps < 32 || tiles_of(steps >= 64 ? 3 : 4, n_rows, n_out) >= 256)
    return;
  for (int sh = 3; sh <= 4; ++sh) {
    const long t = tiles_of(sh, n_rows, n_out);
    int p = 1;
    while (p < MM_MAX_PARTS && t * p * 2 <= 640 && steps / (p * 2) >= 8) p *= 2;
    if (p > 1 && (t * p >= 256 || sh == 4)) {
      *shape = sh;
      *parts = p;
      return;
    }
  }
}

// drops stretches that would be empty (the stretch length is rounded up to whole steps)
int used_parts(int k_dim, int parts) {
  const int steps = (k_dim + MM_BK - 1) / MM_BK;
  const int per = (steps + parts - 1) / parts;
  return (steps + per - 1) / per;
}

// out[n, o] = sum over the stretches' sums, in their order, + bias, with the epilogue
template <int EPI, typename OT>
__global__ __launch_bounds__(256) void linear_mfma_join_kernel(const float* __restrict__ partials, int k_parts,
                                                               const float* __restrict__ bias, OT* __restrict__ out,
                                                               long ldo, int n_rows, int n_out) {
  const int quads = n_out >> 2;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_rows * quads) return;
  const int row = (int)(idx / quads), oc = (int)(idx - (long)row * quads) * 4;
  const float* p = partials + (long)row * n_out + oc;
  const long part_stride = (long)n_rows * n_out;
  float4 v = *reinterpret_cast<const float4*>(p);
  for (int s = 1; s < k_parts; ++s) {
    const float4 t = *reinterpret_cast<const float4*>(p + s * part_stride);
    v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
  }
  if (bias) {
    const bool al = (((size_t)bias) & 15) == 0;
    if (al) {
      const float4 b4 = *reinterpret_cast<const float4*>(bias + oc);
      v.x += b4.x; v.y += b4.y; v.z += b4.z; v.w += b4.w;
    } else {
      v.x += bias[oc]; v.y += bias[oc + 1]; v.z += bias[oc + 2]; v.w += bias[oc + 3];
    }
  }
  if (EPI == MM_EPI_GELU) {
    v.x = gelu_tanh_fast(v.x); v.y = gelu_tanh_fast(v.y); v.z = gelu_tanh_fast(v.z); v.w = gelu_tanh_fast(v.w);
  }
  OT* orow = out + (long)row * ldo + oc;
  const float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (EPI == MM_EPI_RESIDUAL) orow[e] = from_float<OT>(to_float<OT>(orow[e]) + r[e]);
    else orow[e] = from_float<OT>(r[e]);
  }
}

int launch_join(const float* partials, int k_parts, const float* bias, void* out, int out_dtype, long ldo,
                int n_rows, int n_out, int epilogue, hipStream_t stream) {
  const long work = (long)n_rows * (n_out >> 2);
  dim3 grid((unsigned int)((work + 255) / 256));
#define MM_JOIN(E, OT)                                                                                  \
  hipLaunchKernelGGL((linear_mfma_join_kernel<E, OT>), grid, dim3(256), 0, stream, partials, k_parts, \
                     bias, (OT*)out, ldo, n_rows, n_out)
  if (epilogue == MM_EPI_NONE && out_dtype == MGPT_BF16) MM_JOIN(MM_EPI_NONE, bf16_t);
  else if (epilogue == MM_EPI_NONE && out_dtype == MGPT_F32) MM_JOIN(MM_EPI_NONE, float);
  else if (epilogue == MM_EPI_GELU && out_dtype == MGPT_BF16) MM_JOIN(MM_EPI_GELU, bf16_t);
  else if (epilogue == MM_EPI_RESIDUAL && out_dtype == MGPT_F32) MM_JOIN(MM_EPI_RESIDUAL, float);
  else return MGPT_ERR_BAD_DTYPE;
#undef MM_JOIN
  return mgpt_last_error();
}

bool shapes_ok(const void* act, long lda, const void* w, const void* out, long ldo, int n_rows, int n_out, int k_dim) {
  return act && w && out && n_rows >= 0 && n_out >= 0 && k_dim > 0 && (k_dim % 16) == 0 && lda >= k_dim &&
         (lda % 8) == 0 && ldo >= n_out;
}

// whole steps along k, and operands aligned for 16-byte loads: what the variants that load straight into LDS need
bool direct_ok(const void* act, const void* w, int k_dim) {
  return (k_dim % MM_BK) == 0 && ((((size_t)act) | ((size_t)w)) & 15) == 0;
}

long direct_tiles(int variant, int n_rows, int n_out) {
  return (long)((n_rows + MM_DIRECT_ROWS[variant] - 1) / MM_DIRECT_ROWS[variant]) *
         ((n_out + MM_DIRECT_COLS[variant] - 1) / MM_DIRECT_COLS[variant]);
}

// The shape id for a product of a prompt portion (128 rows and more) whose slices can go straight into
// LDS and that gains by it, or -1: the rules further down decide.  Which products gain was measured inside
// the prefill step, one product of the layer changed at a time (alone in a graph of its own, with its
// operands in the L2 from the launch before, every such variant is 10-20 % ahead of the register path, and
// most of that is not there in the step):
// - a long inner size (32 steps and more: the second feed-forward product).  Through registers two steps are
//   on their way, or the inner size is split over workgroups and a second kernel adds the parts; here three
//   or four stages hold as many steps, with no registers spent on them.  Prefill steps of 256 to 2,048
//   tokens: width 512 -3 %, width 768 -1 to -10 %, width 1600 at 2,048 tokens -7 %.
// - a wide output under many rows: tiles of 128 x 192 where a round of them costs less than a round of
//   256 x 256 (qkv and first feed-forward product at 8,192 tokens, widths 512 to 1600: -2 to -5 % of the step).
int choose_direct(int n_rows, int n_out, int k_dim) {
  if (n_rows < 128 || (k_dim % MM_BK) != 0) return -1;
  if (k_dim / MM_BK >= 32) {
    const long t128 = direct_tiles(2, n_rows, n_out), t64 = direct_tiles(1, n_rows, n_out);
    if (t128 > 520) return -1;
    if (t128 >= 190) return MM_DIRECT_FIRST + 2;
    return MM_DIRECT_FIRST + (t64 >= 190 ? 1 : 0);
  }
  // (measured from 1,536 columns up; under 512 columns at 8,192 rows those tiles lose 2 % of the step)
  const long wide = direct_tiles(3, n_rows, n_out), largest = tiles_of(0, n_rows, n_out);
  if (n_out < 1536 || wide < 190) return -1;
  // a tile's cost: its outputs, times a factor that falls with its size, times the rounds of 256 tiles
  const double cost_wide = (double)((wide + 255) / 256) * 128 * 192 * 0.78;
  const double cost_largest = (double)((largest + 255) / 256) * 256 * 256 * 0.72;
  if (largest >= 160 && cost_largest <= cost_wide) return -1;
  return MM_DIRECT_FIRST + 3;
}

// shape < 0: chosen by the size.  k_parts: 0 = chosen by the size, together with the shape, if
// `partials` holds enough floats (else unsplit; with a given shape unsplit too), 1 = unsplit,
// more = that many stretches (refused if the buffer is too small).
// leave_parts: the stretches' sums stay in `partials` ([parts][n_rows][n_out], the first with the
// bias), no second kernel joins them; *leave_parts gets the number of parts, 0 if the product is not split.
int launch_any(int shape, int k_parts, const void* act, long lda, const void* w, const float* bias, void* out,
               int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue, float* partials,
               long partials_floats, const MfmaScatter& sc, hipStream_t stream, int* leave_parts = nullptr) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!act || !w || !out) return MGPT_ERR_NULL;
  if (!shapes_ok(act, lda, w, out, ldo, n_rows, n_out, k_dim)) return MGPT_ERR_BAD_SHAPE;
  // shapes MM_SHAPES and MM_SHAPES + 1: the two smallest tiles with more steps on their way from memory
  int ahead = 0;  // 0: chosen below
  bool two_groups = false;  // the 64 x 64 tile with two wave groups (shape MM_SHAPES + 2)
  int direct = -1;  // which of the variants whose slices go straight into LDS (-1: through registers)
  if (shape < 0 && k_parts <= 1 && !leave_parts) {
    const int chosen = direct_ok(act, w, k_dim) ? choose_direct(n_rows, n_out, k_dim) : -1;
    if (chosen >= 0) shape = chosen, k_parts = 1;
  }
  if (shape >= MM_DIRECT_FIRST) {
    if (shape >= MM_SHAPE_IDS || !direct_ok(act, w, k_dim)) return MGPT_ERR_BAD_SHAPE;
    direct = shape - MM_DIRECT_FIRST;
    shape = 3;   // (the rules below for the other variants do not apply)
    ahead = 1;
  } else if (shape == MM_SHAPES + 2) {
    shape = 3;
    ahead = 1;
    two_groups = true;
  } else if (shape >= MM_SHAPES && shape < MM_SHAPES + 2) {
    shape -= 2;
    ahead = MM_AHEAD;
  } else if (shape >= 0) {
    ahead = 1;
  }
  const bool forced = k_parts > 1;
  if (shape < 0 && k_parts == 0 && partials) {
    choose_split(n_rows, n_out, k_dim, epilogue, &shape, &k_parts);
    if (k_parts > 1 && (long)used_parts(k_dim, k_parts) * n_rows * n_out > partials_floats) shape = -1, k_parts = 1;
  }
  if (shape < 0) shape = choose_shape(n_rows, n_out);
  if (shape >= MM_SHAPES) return MGPT_ERR_BAD_SHAPE;
  if (k_parts == 0) k_parts = 1;
  if (ahead == 0) {
    // Few small tiles over a long enough stretch: the workgroups are too few to hide a trip to
    // memory behind one another.  Measured over matrices that come from memory, 32 x 32 tiles, 40-64
    // rows: [4800 x 1600] 9.8-10.0 us against 10.8, [6400 x 1600] 10.7-11.9 against 15.6, [1600 x 1600]
    // 8.4 against 10.3 (and 8.6 / 10.5 at 136 rows, 250 tiles), [4096 x 1024] 6.3 against 7.6; with more
    // than two such workgroups a compute unit nothing is gained ([4800 x 1600] at 136 rows, 750 tiles:
    // 12.8 against 11.7).
    const int steps = (k_dim + MM_BK - 1) / MM_BK;
    ahead = (shape == 4 && steps / k_parts >= 12 && tiles_of(4, n_rows, n_out) * k_parts <= 512) ? MM_AHEAD : 1;
    // The same with the slices straight into LDS, where the operands allow it: the steps on their way need no
    // registers, so there can be more of them (six stages while a compute unit has one such workgroup, four
    // with more).  Decode steps of 12 layers of width 1600, in turns with the variant above on one box: 24 rows
    // 0.774 -> 0.740 ms, 32 rows 0.795 -> 0.762, 64 rows 1.000 -> 0.949 (with six stages there 0.970).
    if (ahead == MM_AHEAD && direct_ok(act, w, k_dim)) {
      direct = tiles_of(4, n_rows, n_out) * k_parts <= 256 ? 4 : 0;
      ahead = 1;
    }
  }
  if (k_parts > 1) {
    k_parts = used_parts(k_dim, k_parts > MM_MAX_PARTS ? MM_MAX_PARTS : k_parts);
    const bool fits = partials && (long)k_parts * n_rows * n_out <= partials_floats &&
                      (((size_t)partials) & 15) == 0 && (n_out & 3) == 0 && epilogue != MM_EPI_QKV;
    if (!fits) {
      if (forced) return MGPT_ERR_BAD_SHAPE;
      k_parts = 1;
    }
  }
  const bool split = k_parts > 1;
  if (two_groups) {
    // forced: what this kernel stores must be float32, plain or added into the residual stream (the sums of
    // a split product are)
    const int dt_here = split ? MGPT_F32 : out_dtype, epi_here = split ? MM_EPI_NONE : epilogue;
    if (dt_here != MGPT_F32 || (epi_here != MM_EPI_NONE && epi_here != MM_EPI_RESIDUAL)) return MGPT_ERR_BAD_SHAPE;
  } else if (shape == 3 && ahead == 1 && direct < 0) {
    // 64 x 64 tiles under a long inner size (16 steps and more a workgroup), float32 out: two wave groups
    // a tile.  [2048 x 2048 -> 512] 12.9 us against 14.4, [1024 x 2048 -> 512] 12.2 / 13.4, [2048 x 3072 ->
    // 768] 24.2 / 25.5, [8192 x 2048 -> 512] 33.9 / 35.3; at 8 steps ([2048 x 512 -> 512]) nothing.
    const int steps_here = ((k_dim + MM_BK - 1) / MM_BK + k_parts - 1) / k_parts;
    const int dt_here = split ? MGPT_F32 : out_dtype, epi_here = split ? MM_EPI_NONE : epilogue;
    // (alone in a graph the variant is ahead at 256 tiles too, 12.9 us against 14.4; inside the 2,048-token
    // prefill step it is not, 0.599-0.607 ms against 0.596-0.602 in turns on one box: more than a tile a unit)
    two_groups = steps_here >= 16 && dt_here == MGPT_F32 && (epi_here == MM_EPI_NONE || epi_here == MM_EPI_RESIDUAL) &&
                 tiles_of(3, n_rows, n_out) * k_parts > 256;
  }
  if (leave_parts) {
    *leave_parts = split ? k_parts : 0;
    if (!split) return MGPT_OK;  // nothing launched: the caller takes another way
  }
  void* dst = split ? (void*)partials : out;
  const float* b = (split && !leave_parts) ? nullptr : bias;
  const int dt = split ? MGPT_F32 : out_dtype, epi = split ? MM_EPI_NONE : epilogue;
  const long ld = split ? n_out : ldo, stride = split ? (long)n_rows * n_out : 0;
#define MM_ARGS act, lda, w, b, dst, dt, ld, n_rows, n_out, k_dim, epi, k_parts, stride, sc, stream
  int rc = MGPT_ERR_BAD_SHAPE;
  if (direct >= 0) {
    switch (direct) {
      case 0: rc = launch_shape<1, 1, 2, 2, 1, 4>(MM_ARGS); break;
      case 1: rc = launch_shape<2, 2, 2, 2, 1, 4>(MM_ARGS); break;
      case 2: rc = launch_shape<2, 2, 4, 2, 1, 3>(MM_ARGS); break;
      case 3: rc = launch_shape<4, 3, 2, 4, 1, 2>(MM_ARGS); break;
      case 4: rc = launch_shape<1, 1, 2, 2, 1, 6>(MM_ARGS); break;
      default: break;
    }
  } else
  switch (shape) {
    case 0: rc = launch_shape<8, 4, 2, 4>(MM_ARGS); break;  // 256 x 256, eight waves of 128 x 64
    case 1: rc = launch_shape<4, 4, 2, 4>(MM_ARGS); break;  // 128 x 256, eight waves of 64 x 64
    case 2: rc = launch_shape<4, 2, 2, 2>(MM_ARGS); break;  // 128 x 64, four waves of 64 x 32
    case 3:  // 64 x 64, four waves of 32 x 32 (or eight, in two groups)
      rc = two_groups ? launch_two_groups(MM_ARGS)
                      : ahead > 1 ? launch_shape<2, 2, 2, 2, MM_AHEAD>(MM_ARGS) : launch_shape<2, 2, 2, 2>(MM_ARGS);
      break;
    case 4:  // 32 x 32, four waves of 16 x 16
      rc = ahead > 1 ? launch_shape<1, 1, 2, 2, MM_AHEAD>(MM_ARGS) : launch_shape<1, 1, 2, 2>(MM_ARGS);
      break;
  }
#undef MM_ARGS
  if (rc != MGPT_OK || !split || leave_parts) return rc;
  return launch_join(partials, k_parts, bias, out, out_dtype, ldo, n_rows, n_out, epilogue, stream);
}

}  // namespace

// How many floats of scratch the product would use if it were split along its inner size (0: it
// would not be split).  The caller brings that buffer to mgpt_linear_mfma.
extern "C" long mgpt_linear_mfma_partials(int n_rows, int n_out, int k_dim, int epilogue) {
  if (n_rows <= 0 || n_out <= 0 || k_dim <= 0) return 0;
  int shape, parts;
  choose_split(n_rows, n_out, k_dim, epilogue, &shape, &parts);
  return parts > 1 ? (long)used_parts(k_dim, parts) * n_rows * n_out : 0;
}

// The first half of a split product alone: partials[p][n][o] = the sum over stretch p of the inner
// size (+ bias[o] in p = 0), p < mgpt_linear_mfma_partials(n_rows, n_out, k_dim, residual epilogue) /
// (n_rows * n_out), for a caller that adds the parts up itself (a pending residual: fused_decode.h).
// MGPT_ERR_BAD_SHAPE, with nothing launched, if the product would not be split or the buffer is too small.
extern "C" int mgpt_linear_mfma_parts(const void* act, long lda, const void* w, const float* bias, float* partials,
                                      long partials_floats, int n_rows, int n_out, int k_dim, hipStream_t stream) {
  if (!partials) return MGPT_ERR_NULL;
  MfmaScatter sc = {};
  int parts = 0;
  const int rc = launch_any(-1, 0, act, lda, w, bias, partials, MGPT_F32, n_out, n_rows, n_out, k_dim, MM_EPI_RESIDUAL,
                            partials, partials_floats, sc, stream, &parts);
  if (rc != MGPT_OK) return rc;
  return parts > 1 ? MGPT_OK : MGPT_ERR_BAD_SHAPE;
}

// act: [n_rows, k_dim] bfloat16 with row stride lda (a multiple of 8, 16-byte aligned base);
// w: [n_out, k_dim] dense bfloat16; out: [n_rows, n_out] with row stride ldo.  k_dim must be a
// multiple of 16.  partials: scratch of partials_floats floats (16-byte aligned) or null; with it
// a long inner size over few tiles is split (mgpt_linear_mfma_partials says how much that needs).
// Refuses other layouts with MGPT_ERR_BAD_SHAPE.
extern "C" int mgpt_linear_mfma(const void* act, long lda, const void* w, const float* bias, void* out,
                                int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue,
                                float* partials, long partials_floats, hipStream_t stream) {
  if (epilogue == MM_EPI_QKV) return MGPT_ERR_BAD_SHAPE;  // mgpt_linear_mfma_qkv brings the pools
  MfmaScatter sc = {};
  return launch_any(-1, 0, act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue, partials,
                    partials_floats, sc, stream);
}

// The same product with the tile shape given (0 = 256 x 256, 1 = 128 x 256, 2 = 128 x 64,
// 3 = 64 x 64, 4 = 32 x 32, 5 and 6 = 64 x 64 and 32 x 32 with four steps on their way from memory,
// 7 = 64 x 64 with two wave groups a tile (float32 outputs), 8 to 12 = the slices straight into LDS: 32 x 32 and
// 64 x 64 with four stages, 128 x 64 with three, 128 x 192 with two, 32 x 32 with six (an inner size of whole steps of 64 and operands
// aligned to 16 bytes, else refused); negative: chosen) and the number of stretches of the inner size given
// (k_parts as for launch_any above), instead of chosen by the size: for tests and measurements.
extern "C" int mgpt_linear_mfma_shape(int shape, int k_parts, const void* act, long lda, const void* w,
                                      const float* bias, void* out, int out_dtype, long ldo, int n_rows,
                                      int n_out, int k_dim, int epilogue, float* partials, long partials_floats,
                                      hipStream_t stream) {
  if (epilogue == MM_EPI_QKV || shape >= MM_SHAPE_IDS || k_parts < 0) return MGPT_ERR_BAD_SHAPE;
  MfmaScatter sc = {};
  return launch_any(shape, k_parts, act, lda, w, bias, out, out_dtype, ldo, n_rows, n_out, k_dim, epilogue,
                    partials, partials_floats, sc, stream);
}

// The fused QKV product of a step with prompt portions: out[n] = act[n] W^T + bias in bfloat16, and
// the key and value columns (after the first q_width) of every row with a slot also go into the
// cache pools [pages, n_kv_head, page_size, head_dim].  Refuses (MGPT_ERR_BAD_SHAPE) sizes that
// are no multiples of 4 and outputs that are not aligned for 8-byte stores.  shape: as for
// mgpt_linear_mfma_shape, or negative to have it chosen.
extern "C" int mgpt_linear_mfma_qkv(const void* act, long lda, const void* w, const float* bias, void* out,
                                    long ldo, int n_rows, int n_out, int k_dim, void* kpool, void* vpool,
                                    const int* slot_mapping, int q_width, int kv_width, int head_dim,
                                    int n_kv_head, int page_size, int shape, hipStream_t stream) {
  if (!kpool || !vpool || !slot_mapping) return MGPT_ERR_NULL;
  if (head_dim <= 0 || (head_dim % 4) != 0 || (q_width % 4) != 0 || q_width + 2 * kv_width != n_out ||
      kv_width != n_kv_head * head_dim || page_size <= 0 || (n_out % 4) != 0 || (ldo % 4) != 0 ||
      (((size_t)out | (size_t)bias) & 15) != 0 || (shape >= MM_SHAPES + 2 && shape < MM_DIRECT_FIRST) ||
      shape >= MM_SHAPE_IDS)
    return MGPT_ERR_BAD_SHAPE;
  MfmaScatter sc = {(bf16_t*)kpool, (bf16_t*)vpool, slot_mapping, q_width, kv_width, head_dim, n_kv_head, page_size};
  return launch_any(shape, 1, act, lda, w, bias, out, MGPT_BF16, ldo, n_rows, n_out, k_dim, MM_EPI_QKV, nullptr, 0, sc,
                    stream);
}
