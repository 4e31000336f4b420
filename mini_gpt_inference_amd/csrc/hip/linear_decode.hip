// linear_decode.h's kernel for up to 16 rows.
#include "linear_decode.h"

int mgpt_launch_linear_decode_rows(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream);

#define SK_ROW_GROUPS_MAX_BYTES (6L << 20)
#define SK_ROW_GROUPS_MAX_K 2048
#define SK_ROW_GROUPS_LONG_K_MAX_BYTES (8L << 20)

template <int SMAX>
static int launch_one_tile(const SkinnyArgs& a, int epilogue, int out_dtype, dim3 grid, hipStream_t s) {
  const bool ln = a.x != nullptr;
  if (decode_vec_ok(a)) {
    if (ln) {
      // few rows to a workgroup: the residual rows loaded by all lanes of a lane row (FEW in linear_decode.h)
      const int rows = a.rows_per_group < a.n_rows ? a.rows_per_group : a.n_rows;
      if (rows <= 1) return launch_decode_epi<1, SMAX, true, true, 1>(a, epilogue, out_dtype, grid, s);
      if (rows <= 2) return launch_decode_epi<1, SMAX, true, true, 2>(a, epilogue, out_dtype, grid, s);
      if (rows <= 4) return launch_decode_epi<1, SMAX, true, true, 4>(a, epilogue, out_dtype, grid, s);
      if (rows <= 8) return launch_decode_epi<1, SMAX, true, true, 8>(a, epilogue, out_dtype, grid, s);
    }
    return ln ? launch_decode_epi<1, SMAX, true, true>(a, epilogue, out_dtype, grid, s)
              : launch_decode_epi<1, SMAX, false, true>(a, epilogue, out_dtype, grid, s);
  }
  return ln ? launch_decode_epi<1, SMAX, true, false>(a, epilogue, out_dtype, grid, s)
            : launch_decode_epi<1, SMAX, false, false>(a, epilogue, out_dtype, grid, s);
}

// More than 16 rows: the rows either share the W that a workgroup loads (two to four tiles of 16
// rows per workgroup, linear_decode_rows.hip), or are dealt out in groups of 16 to workgroups of
// their own, which then are the 16-row kernel at its own pace: the matrix is read once per group,
// and a small matrix comes out of the L2 (the groups of a column tile run on one XCD when the number
// of column tiles is a multiple of 8).  The second is faster while the matrix is small and its
// inner size not long (measured on layer matrices of 0.5 to 19 MB at 17 to 64 rows: at 64 rows
// [1536 x 512] takes 4.6 us against 6.9 with the LayerNorm kernel that the first way needs,
// [512 x 2048] 4.6 against 6.3 with its split, [768 x 3072] at 17 rows 6.8 against 5.5,
// [6400 x 1600] at 64 rows 31.7 against 22.2).
bool mgpt_linear_decode_row_groups(int n_rows, int n_out, int k_dim, int rows_mode) {
  if (n_rows <= 16 || n_rows > 64 || (k_dim % 32) != 0) return false;
  if (rows_mode == SK_ROWS_GROUPS) return true;
  if (rows_mode == SK_ROWS_SHARE_W) return false;
  const long bytes = (long)n_out * k_dim * (long)sizeof(bf16_t);
  if (k_dim <= SK_ROW_GROUPS_MAX_K) return bytes <= SK_ROW_GROUPS_MAX_BYTES;
  // a longer inner size: the other way splits it over workgroups and adds the parts in a second
  // kernel, which from 33 rows on costs more than reading the matrix once per group
  // ([768 x 3072] at 64 rows: 7.0 us against 8.3, at 17 rows 6.8 against 5.5)
  return n_rows > 32 && bytes <= SK_ROW_GROUPS_LONG_K_MAX_BYTES;
}

// The caller (mgpt_linear_skinny) has checked pointers, strides and the scatter's sizes.  Takes up
// to 64 rows and any k_dim that is a multiple of 32; more than 16 rows only with an epilogue that
// can use vectors of four.
int mgpt_launch_linear_decode(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  if (a.n_rows > 64 || (a.k_dim % 32) != 0) return MGPT_ERR_BAD_SHAPE;
  // the scatter stores four neighbouring columns of a head at once
  if (epilogue == SK_EPI_QKV && ((a.n_out % 16) != 0 || (a.ldo % 4) != 0 || (((size_t)a.out) & 15) != 0))
    return MGPT_ERR_BAD_SHAPE;
  if (a.n_rows <= 16 && a.partials != nullptr && a.rows_per_group == 0 && decode_vec_ok(a) &&
      mgpt_linear_decode_partials(a.n_rows, a.n_out, a.k_dim, a.x != nullptr, epilogue, a.rows_mode) > 0) {
    // few rows under a long inner size and few column tiles: the inner size split over workgroups
    SkinnyArgs b = a;
    b.rows_per_group = 16;
    return mgpt_launch_linear_decode_rows(b, epilogue, out_dtype, stream);
  }
  if (a.n_rows > 16 && !mgpt_linear_decode_row_groups(a.n_rows, a.n_out, a.k_dim, a.rows_mode))
  {
    SkinnyArgs b = a;
    b.rows_per_group = 16;
    return mgpt_launch_linear_decode_rows(b, epilogue, out_dtype, stream);
  }
  const int per = (a.k_dim / 32 + 3) / 4;  // k steps of the first waves
  // Rows of a group: 16 fill the MFMA's tile, but while the workgroups are few, fewer rows to a
  // workgroup (the tile's other rows stay zero and are never loaded) make a workgroup's share of the
  // activations smaller and the workgroups more: the fewest rows of 1, 2, 4, 8 with which there are
  // no more than 256 workgroups, and only for a matrix small enough that reading it once more per
  // group costs nothing ([512 x 2048] at 16 rows: 3.4 us with groups of 2, 3.6 with groups of 4,
  // 4.4 with one of 16, and 4.2 with groups of 1, which are 512 workgroups; [1600 x 6400] at 8 rows:
  // 11.5 with groups of 4 against 8.7).  The sums are the same whatever the groups.  (rows_per_group forced: by the
  // caller's wish.)
  SkinnyArgs b = a;
  if (b.rows_per_group != 1 && b.rows_per_group != 2 && b.rows_per_group != 4 && b.rows_per_group != 8 &&
      b.rows_per_group != 16) {
    b.rows_per_group = 16;
    const long tiles = (a.n_out + 15) / 16;
    if ((long)a.n_out * a.k_dim * (long)sizeof(bf16_t) <= SK_ROW_GROUPS_MAX_BYTES) {
      for (int rpg = 1; rpg < 16; rpg *= 2)
        if (a.n_rows > rpg && tiles * ((a.n_rows + rpg - 1) / rpg) <= 256) {
          b.rows_per_group = rpg;
          break;
        }
    }
  }
  dim3 grid((a.n_out + 15) / 16, (a.n_rows + b.rows_per_group - 1) / b.rows_per_group);
  if (per <= 4) return launch_one_tile<4>(b, epilogue, out_dtype, grid, stream);
  if (per <= 8) return launch_one_tile<8>(b, epilogue, out_dtype, grid, stream);
  return launch_one_tile<16>(b, epilogue, out_dtype, grid, stream);  // longer ranges: several passes
}
