// linear_decode.h's kernel for 17 to 64 rows: two to four tiles of 16 rows share the W a lane loads.
#include "linear_decode.h"
#include "launchers.h"

template <int NT>
static int launch_tiles(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t s) {
  const bool ln = a.x != nullptr;
  const int per = (a.k_dim / 32 + 3) / 4;
  dim3 grid((a.n_out + 15) / 16);
  if (per <= 4)
    return ln ? launch_decode_epi<NT, 4, true, true>(a, epilogue, out_dtype, grid, s)
              : launch_decode_epi<NT, 4, false, true>(a, epilogue, out_dtype, grid, s);
  return ln ? launch_decode_epi<NT, 8, true, true>(a, epilogue, out_dtype, grid, s)
            : launch_decode_epi<NT, 8, false, true>(a, epilogue, out_dtype, grid, s);
}

// The output head over a vocabulary that is no multiple of 16 (GPT-2's 50257): float32 logits, no
// epilogue, every store a single element.
template <int NT>
static int launch_tiles_unaligned_head(const SkinnyArgs& a, hipStream_t s) {
  const bool ln = a.x != nullptr;
  const int per = (a.k_dim / 32 + 3) / 4;
  dim3 grid((a.n_out + 15) / 16);
#define LDR_LAUNCH(SMAX, LN) \
  hipLaunchKernelGGL((linear_decode_kernel<NT, SMAX, LN, SK_EPI_NONE, float, false>), grid, dim3(256), 0, s, a)
  if (per <= 4) {
    if (ln) LDR_LAUNCH(4, true); else LDR_LAUNCH(4, false);
  } else {
    if (ln) LDR_LAUNCH(8, true); else LDR_LAUNCH(8, false);
  }
#undef LDR_LAUNCH
  return mgpt_last_error();
}

// ---- k split over workgroups, for a long k and few column tiles: with 64 rows a workgroup that owns
// 16 columns pulls all the activations (256 KB for k = 2048) through one compute unit; four
// workgroups per tile pull a quarter each, write their sums, and a second kernel adds the parts in
// order and applies bias, GELU or the residual add.
#define LDR_PARTS 4

// Up to 16 rows are split as well when the inner size is long and the column tiles are few: a tile's
// workgroup then streams 16 x k_dim of the matrix through one compute unit (205 KB for k = 6400),
// and fewer workgroups than compute units do ([1600 x 6400] at one row: 11.5 us as 100 workgroups).
// Below 3072 the second kernel costs more than the split saves (64 KB a workgroup at k = 2048).
#define LDR_FEW_ROWS_MIN_K 3072
long mgpt_linear_decode_partials(int n_rows, int n_out, int k_dim, bool ln, int epilogue, int rows_mode) {
  if (ln || epilogue == SK_EPI_QKV || n_rows <= 0 || n_rows > 64) return 0;
  if ((k_dim % (32 * LDR_PARTS)) != 0 || (n_out % 16) != 0 || n_out / 16 >= 128) return 0;
  if (n_rows <= 16) return k_dim >= LDR_FEW_ROWS_MIN_K ? (long)LDR_PARTS * n_rows * n_out : 0;
  if (mgpt_linear_decode_row_groups(n_rows, n_out, k_dim, rows_mode)) return 0;
  if (k_dim < 1024) return 0;
  return (long)LDR_PARTS * n_rows * n_out;
}

template <int EPI, typename OT>
__global__ __launch_bounds__(256) void linear_partials_epilogue_kernel(
    const float* __restrict__ partials, const float* __restrict__ bias, OT* __restrict__ out, long ldo,
    int n_rows, int n_out) {
  const int quads = n_out >> 2;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= n_rows * quads) return;
  const int row = idx / quads, oc = (idx - row * quads) * 4;
  float4 p[LDR_PARTS];
#pragma unroll
  for (int s = 0; s < LDR_PARTS; ++s)
    p[s] = *reinterpret_cast<const float4*>(partials + ((long)s * n_rows + row) * n_out + oc);
  float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) b4 = *reinterpret_cast<const float4*>(bias + oc);
  OT* orow = out + (long)row * ldo + oc;
  float4 old = make_float4(0.f, 0.f, 0.f, 0.f);
  if (EPI == SK_EPI_RESIDUAL) old = *reinterpret_cast<const float4*>(orow);
  float v[4] = {p[0].x, p[0].y, p[0].z, p[0].w};
#pragma unroll
  for (int s = 1; s < LDR_PARTS; ++s) {  // in the order of k, whatever order the parts were written in
    v[0] += p[s].x; v[1] += p[s].y; v[2] += p[s].z; v[3] += p[s].w;
  }
  const float b[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] += b[i];
    if (EPI == SK_EPI_GELU) v[i] = gelu_tanh_fast(v[i]);
  }
  if (sizeof(OT) == 4) {
    *reinterpret_cast<float4*>(orow) = make_float4(v[0] + old.x, v[1] + old.y, v[2] + old.z, v[3] + old.w);
  } else {
    uint2 pk;
    pk.x = pack_bf16x2(v[0], v[1]);
    pk.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(orow) = pk;
  }
}

// the first of the split's two kernels: every workgroup's sums to a.partials
template <int NT>
static int launch_split_parts(const SkinnyArgs& a, hipStream_t s) {
  const int per = (a.k_dim / 32 / LDR_PARTS + 3) / 4;
  dim3 grid((a.n_out / 16) * LDR_PARTS);
  if (per <= 4) hipLaunchKernelGGL((linear_decode_kernel<NT, 4, false, SK_EPI_NONE, float, true, true>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((linear_decode_kernel<NT, 8, false, SK_EPI_NONE, float, true, true>), grid, dim3(256), 0, s, a);
  return mgpt_last_error();
}

template <int NT>
static int launch_split(const SkinnyArgs& a0, int epilogue, int out_dtype, hipStream_t s) {
  SkinnyArgs a = a0;
  a.k_parts = LDR_PARTS;
  a.bias_in_part0 = 0;
  int rc = launch_split_parts<NT>(a, s);
  if (rc != MGPT_OK) return rc;
  dim3 egrid((a.n_rows * (a.n_out / 4) + 255) / 256);
#define LDR_EPI(E, OT) \
  hipLaunchKernelGGL((linear_partials_epilogue_kernel<E, OT>), egrid, dim3(256), 0, s, a.partials, a.bias, (OT*)a.out, a.ldo, a.n_rows, a.n_out)
  if (epilogue == SK_EPI_NONE && out_dtype == MGPT_BF16) LDR_EPI(SK_EPI_NONE, bf16_t);
  else if (epilogue == SK_EPI_NONE && out_dtype == MGPT_F32) LDR_EPI(SK_EPI_NONE, float);
  else if (epilogue == SK_EPI_GELU && out_dtype == MGPT_BF16) LDR_EPI(SK_EPI_GELU, bf16_t);
  else if (epilogue == SK_EPI_RESIDUAL && out_dtype == MGPT_F32) LDR_EPI(SK_EPI_RESIDUAL, float);
  else return MGPT_ERR_BAD_DTYPE;
#undef LDR_EPI
  return mgpt_last_error();
}

// The split's first kernel alone: partials[p][row][column], p < mgpt_linear_decode_parts_count(), are
// the sums over the p-th quarter of the inner size, the first with the bias added, and nobody adds
// them up here: the caller leaves them to whoever reads the sum next (a residual stream kept as
// base + parts, fused_decode.h).  Takes what mgpt_linear_decode_partials(..., SK_EPI_RESIDUAL) splits
// (bfloat16 rows, up to 64 of them); partials must hold that many floats.  MGPT_ERR_BAD_SHAPE otherwise.
extern "C" int mgpt_linear_decode_parts(const void* act, long lda, const void* w, const void* w_packed,
                                        const float* bias, float* partials, int n_rows, int n_out, int k_dim,
                                        hipStream_t stream) {
  if (n_rows == 0 || n_out == 0) return MGPT_OK;
  if (!act || !w || !partials) return MGPT_ERR_NULL;
  if (n_rows < 0 || lda < k_dim || (lda % 8) != 0 ||
      ((((size_t)act) | ((size_t)w) | ((size_t)w_packed) | ((size_t)bias) | ((size_t)partials)) & 15) != 0 ||
      mgpt_linear_decode_partials(n_rows, n_out, k_dim, false, SK_EPI_RESIDUAL, 0) <= 0)
    return MGPT_ERR_BAD_SHAPE;
  SkinnyArgs a = {};
  a.act = (const bf16_t*)act; a.lda = lda; a.w = (const bf16_t*)w; a.w_packed = (const bf16_t*)w_packed;
  a.bias = bias; a.out = partials; a.ldo = n_out; a.n_rows = n_rows; a.n_out = n_out; a.k_dim = k_dim;
  a.ksplit = 1; a.partials = partials; a.k_parts = LDR_PARTS; a.bias_in_part0 = 1; a.rows_per_group = 16;
  switch ((n_rows + 15) / 16) {
    case 1: return launch_split_parts<1>(a, stream);
    case 2: return launch_split_parts<2>(a, stream);
    case 3: return launch_split_parts<3>(a, stream);
    case 4: return launch_split_parts<4>(a, stream);
    default: return MGPT_ERR_BAD_SHAPE;
  }
}

extern "C" int mgpt_linear_decode_parts_count() { return LDR_PARTS; }

int mgpt_launch_linear_decode_rows(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  const int nt = (a.n_rows + 15) / 16;
  if (a.partials != nullptr && decode_vec_ok(a) &&
      mgpt_linear_decode_partials(a.n_rows, a.n_out, a.k_dim, a.x != nullptr, epilogue, a.rows_mode) > 0) {
    switch (nt) {
      case 1: return launch_split<1>(a, epilogue, out_dtype, stream);
      case 2: return launch_split<2>(a, epilogue, out_dtype, stream);
      case 3: return launch_split<3>(a, epilogue, out_dtype, stream);
      case 4: return launch_split<4>(a, epilogue, out_dtype, stream);
      default: return MGPT_ERR_BAD_SHAPE;
    }
  }
  if (!decode_vec_ok(a)) {
    // odd widths with many rows: only the head's case here, the general kernel for the rest
    if (epilogue != SK_EPI_NONE || out_dtype != MGPT_F32) return MGPT_ERR_BAD_SHAPE;
    switch (nt) {
      case 2: return launch_tiles_unaligned_head<2>(a, stream);
      case 3: return launch_tiles_unaligned_head<3>(a, stream);
      case 4: return launch_tiles_unaligned_head<4>(a, stream);
      default: return MGPT_ERR_BAD_SHAPE;
    }
  }
  switch (nt) {
    case 2: return launch_tiles<2>(a, epilogue, out_dtype, stream);
    case 3: return launch_tiles<3>(a, epilogue, out_dtype, stream);
    case 4: return launch_tiles<4>(a, epilogue, out_dtype, stream);
    default: return MGPT_ERR_BAD_SHAPE;
  }
}
