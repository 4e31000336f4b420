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

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, MGPT_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MGPT_WAVE));
  return v;
}

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, MGPT_WAVE);
  return v;
}

// GELU with the tanh approximation, as F.gelu(approximate="tanh"):
// 0.5*u*(1 + tanh(sqrt(2/pi)*(u + 0.044715*u^3)))
__device__ __forceinline__ float gelu_tanh(float u) {
  const float k = 0.7978845608028654f;  // sqrt(2/pi)
  float inner = k * (u + 0.044715f * u * u * u);
  return 0.5f * u * (1.0f + tanhf(inner));
}

static inline int mgpt_last_error() { return (int)hipGetLastError(); }
