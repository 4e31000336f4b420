// Shared device helpers for the gfx950 kernels: storage-type conversion,
// wave-wide (64 lanes) reductions and the C return codes of the launchers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Return codes of every extern "C" launcher: 0 = launched, >0 = a hipError_t,
// <0 = the arguments were refused before anything was launched.
#define MGPT_OK 0
#define MGPT_ERR_BAD_DTYPE (-1)
#define MGPT_ERR_BAD_SHAPE (-2)
#define MGPT_ERR_TOO_LARGE (-3)
#define MGPT_ERR_NULL (-4)

// dtype codes shared with the Python bindings
#define MGPT_F32 0
#define MGPT_BF16 1

#define MGPT_WAVE 64

typedef unsigned short bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(((unsigned int)v) << 16);
}

// round-to-nearest-even, NaN kept quiet: gfx950 converts in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}

// two floats to two bfloat16 in one register, `lo` in the low half
__device__ __forceinline__ unsigned int pack_bf16x2(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  const f32x2_t f = {lo, hi};
  const bf16x2_t b = __builtin_convertvector(f, bf16x2_t);
  return __builtin_bit_cast(unsigned int, b);
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// Reductions over the 64 lanes of a wave, for waves whose lanes are all active.  Within each row
// of 16 lanes by DPP moves (neighbours, pairs, halves of 8, halves of 16), then the four rows'
// results through scalar registers: no trip through LDS, and the result is the same in all lanes.
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
#define MGPT_DPP_XOR1 0xB1          // quad_perm [1,0,3,2]
#define MGPT_DPP_XOR2 0x4E          // quad_perm [2,3,0,1]
#define MGPT_DPP_HALF_MIRROR 0x141  // lane i of each 8 reads lane 7 - i
#define MGPT_DPP_MIRROR 0x140       // lane i of each 16 reads lane 15 - i

__device__ __forceinline__ float wave_sum(float v) {
  v += __int_as_float(dpp_move<MGPT_DPP_XOR1>(__float_as_int(v)));
  v += __int_as_float(dpp_move<MGPT_DPP_XOR2>(__float_as_int(v)));
  v += __int_as_float(dpp_move<MGPT_DPP_HALF_MIRROR>(__float_as_int(v)));
  v += __int_as_float(dpp_move<MGPT_DPP_MIRROR>(__float_as_int(v)));
  const int b = __float_as_int(v);
  return (__int_as_float(__builtin_amdgcn_readlane(b, 0)) + __int_as_float(__builtin_amdgcn_readlane(b, 16))) +
         (__int_as_float(__builtin_amdgcn_readlane(b, 32)) + __int_as_float(__builtin_amdgcn_readlane(b, 48)));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, __int_as_float(dpp_move<MGPT_DPP_XOR1>(__float_as_int(v))));
  v = fmaxf(v, __int_as_float(dpp_move<MGPT_DPP_XOR2>(__float_as_int(v))));
  v = fmaxf(v, __int_as_float(dpp_move<MGPT_DPP_HALF_MIRROR>(__float_as_int(v))));
  v = fmaxf(v, __int_as_float(dpp_move<MGPT_DPP_MIRROR>(__float_as_int(v))));
  const int b = __float_as_int(v);
  return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 0)), __int_as_float(__builtin_amdgcn_readlane(b, 16))),
               fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 32)), __int_as_float(__builtin_amdgcn_readlane(b, 48))));
}

__device__ __forceinline__ int wave_sum_int(int v) {
  v += dpp_move<MGPT_DPP_XOR1>(v);
  v += dpp_move<MGPT_DPP_XOR2>(v);
  v += dpp_move<MGPT_DPP_HALF_MIRROR>(v);
  v += dpp_move<MGPT_DPP_MIRROR>(v);
  return (__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16)) +
         (__builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}

// GELU with the tanh approximation, as F.gelu(approximate="tanh"):
// 0.5*u*(1 + tanh(sqrt(2/pi)*(u + 0.044715*u^3)))
__device__ __forceinline__ float gelu_tanh(float u) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  float inner = k * (u + 0.044715f * u * u * u);
  return 0.5f * u * (1.0f + tanhf(inner));
}

// The same with tanh(z) = 1 - 2 / (exp(2z) + 1) on the hardware's exp2 and reciprocal (a few ulp
// of float32): for the kernels whose results are rounded to bfloat16 anyway.
__device__ __forceinline__ float gelu_tanh_fast(float u) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  const float inner = k * (u + 0.044715f * u * u * u);
  const float e = __builtin_amdgcn_exp2f(inner * 2.8853900817779268f);  // exp(2 inner); inf and 0 at the ends are right
  const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
  return 0.5f * u * (1.0f + t);
}

static inline int mgpt_last_error() { return (int)hipGetLastError(); }
