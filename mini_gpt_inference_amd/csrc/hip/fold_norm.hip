// Folds a LayerNorm's gain and bias into the linear layer that reads it, once, when the pair is
// first used:  LN(x) W^T + b  =  rstd * (x W'^T - mean * S) + b'
//   W'[o, k] = W[o, k] * gain[k]          (rounded to bfloat16)
//   S[o]     = sum_k W'[o, k]             (float32, of the rounded values)
//   b'[o]    = b[o] + sum_k beta[k] * W[o, k]
// so that a decode step can multiply the raw residual rows and correct with the row's mean
// and rstd afterwards, instead of waiting for the statistics before the product can start.
// LayerNorm as in src/minigpt_infer/model.py:107,109,127; the linear layers that read it:
// model.py:43,96,128.
#include "common.h"
#include "launchers.h"

__global__ void fold_layernorm_kernel(const bf16_t* __restrict__ w, const float* __restrict__ gain,
                                      const float* __restrict__ beta, const float* __restrict__ bias,
                                      bf16_t* __restrict__ w_out, float* __restrict__ colsum,
                                      float* __restrict__ bias_out, int n_out, int k_dim) {
  const int lane = threadIdx.x & 63;
  const int o = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (o >= n_out) return;
  const bf16_t* wr = w + (long)o * k_dim;
  bf16_t* wo = w_out + (long)o * k_dim;
  float s = 0.f, bb = 0.f;
  for (int k = lane; k < k_dim; k += 64) {
    const float wv = bf16_to_float(wr[k]);
    const bf16_t folded = float_to_bf16(wv * gain[k]);
    wo[k] = folded;
    s += bf16_to_float(folded);
    if (beta) bb = fmaf(beta[k], wv, bb);
  }
  s = wave_sum(s);
  bb = wave_sum(bb);
  if (lane == 0) {
    colsum[o] = s;
    bias_out[o] = bb + (bias ? bias[o] : 0.f);
  }
}

extern "C" int mgpt_fold_layernorm(const void* w, const float* gain, const float* beta, const float* bias,
                                   void* w_out, float* colsum, float* bias_out, int n_out, int k_dim,
                                   hipStream_t stream) {
  if (n_out == 0) return MGPT_OK;
  if (!w || !gain || !w_out || !colsum || !bias_out) return MGPT_ERR_NULL;
  if (n_out < 0 || k_dim <= 0) return MGPT_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(fold_layernorm_kernel, dim3((n_out + 3) / 4), dim3(256), 0, stream, (const bf16_t*)w,
                     gain, beta, bias, (bf16_t*)w_out, colsum, bias_out, n_out, k_dim);
  return mgpt_last_error();
}

// The layout the decode step's product reads fastest: for every 16 rows of W and every 32 along k
// one block of 1 KB, in which lane l of a wave finds its MFMA operand, the 8 values
// W[16 t + (l & 15)][32 s + (l >> 4) * 8 ..], at offset 16 l.  A wave's load is then 1 KB in one piece
// instead of sixteen pieces of 64 bytes.  Rows past n_out are zeros.  Made once per matrix.
__global__ void pack_weight_kernel(const bf16_t* __restrict__ w, bf16_t* __restrict__ packed, int n_out,
                                   int k_dim, long blocks) {
  const long b = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);  // block (t, s), one wave each
  if (b >= blocks) return;
  const int lane = threadIdx.x & 63;
  const int steps = k_dim >> 5;
  const long t = b / steps;
  const int s = (int)(b - t * steps);
  const long row = t * 16 + (lane & 15);
  uint4 v = make_uint4(0, 0, 0, 0);
  if (row < n_out) v = *reinterpret_cast<const uint4*>(w + row * k_dim + s * 32 + (lane >> 4) * 8);
  *reinterpret_cast<uint4*>(packed + (b * 64 + lane) * 8) = v;
}

// packed: ceil(n_out / 16) * 16 * k_dim elements.  k_dim must be a multiple of 32.
extern "C" int mgpt_pack_weight(const void* w, void* packed, int n_out, int k_dim, hipStream_t stream) {
  if (n_out == 0) return MGPT_OK;
  if (!w || !packed) return MGPT_ERR_NULL;
  if (n_out < 0 || k_dim <= 0 || (k_dim % 32) != 0 || ((((size_t)w) | ((size_t)packed)) & 15) != 0)
    return MGPT_ERR_BAD_SHAPE;
  const long blocks = (long)((n_out + 15) / 16) * (k_dim / 32);
  hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned int)((blocks + 3) / 4)), dim3(256), 0, stream,
                     (const bf16_t*)w, (bf16_t*)packed, n_out, k_dim, blocks);
  return mgpt_last_error();
}
