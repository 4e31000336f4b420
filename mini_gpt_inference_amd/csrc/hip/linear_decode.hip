// linear_decode.h's kernel for up to 16 rows.
#include "linear_decode.h"

int mgpt_launch_linear_decode_rows(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream);

template <int SMAX>
static int launch_one_tile(const SkinnyArgs& a, int epilogue, int out_dtype, dim3 grid, hipStream_t s) {
  const bool ln = a.x != nullptr;
  if (decode_vec_ok(a))
    return ln ? launch_decode_epi<1, SMAX, true, true>(a, epilogue, out_dtype, grid, s)
              : launch_decode_epi<1, SMAX, false, true>(a, epilogue, out_dtype, grid, s);
  return ln ? launch_decode_epi<1, SMAX, true, false>(a, epilogue, out_dtype, grid, s)
            : launch_decode_epi<1, SMAX, false, false>(a, epilogue, out_dtype, grid, s);
}

// The caller (mgpt_linear_skinny) has checked pointers, strides and the scatter's sizes.  Takes up
// to 64 rows and any k_dim that is a multiple of 32; more than 16 rows only with an epilogue that
// can use vectors of four.
int mgpt_launch_linear_decode(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  if (a.n_rows > 64 || (a.k_dim % 32) != 0) return MGPT_ERR_BAD_SHAPE;
  // the scatter stores four neighbouring columns of a head at once
  if (epilogue == SK_EPI_QKV && ((a.n_out % 16) != 0 || (a.ldo % 4) != 0 || (((size_t)a.out) & 15) != 0))
    return MGPT_ERR_BAD_SHAPE;
  if (a.n_rows > 16) return mgpt_launch_linear_decode_rows(a, epilogue, out_dtype, stream);
  const int per = (a.k_dim / 32 + 3) / 4;  // k steps of the first waves
  dim3 grid((a.n_out + 15) / 16);
  if (per <= 4) return launch_one_tile<4>(a, epilogue, out_dtype, grid, stream);
  if (per <= 8) return launch_one_tile<8>(a, epilogue, out_dtype, grid, stream);
  return launch_one_tile<16>(a, epilogue, out_dtype, grid, stream);  // longer ranges: several passes
}
