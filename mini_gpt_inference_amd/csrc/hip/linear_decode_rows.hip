// linear_decode.h's kernel for 17 to 64 rows: two to four tiles of 16 rows share the W a lane loads.
#include "linear_decode.h"

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

int mgpt_launch_linear_decode_rows(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  if (!decode_vec_ok(a)) return MGPT_ERR_BAD_SHAPE;  // odd widths with many rows: the general kernel
  switch ((a.n_rows + 15) / 16) {
    case 2: return launch_tiles<2>(a, epilogue, out_dtype, stream);
    case 3: return launch_tiles<3>(a, epilogue, out_dtype, stream);
    case 4: return launch_tiles<4>(a, epilogue, out_dtype, stream);
    default: return MGPT_ERR_BAD_SHAPE;
  }
}
