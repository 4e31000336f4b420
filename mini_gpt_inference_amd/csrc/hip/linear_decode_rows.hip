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

int mgpt_launch_linear_decode_rows(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream) {
  const int nt = (a.n_rows + 15) / 16;
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
