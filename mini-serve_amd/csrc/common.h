// Shared device helpers for the gfx950 kernels: element types, conversions, wave and block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16;

#define WAVE 64

// Error codes returned by every extern "C" entry point (0 = launched).
#define MS_OK 0
#define MS_BAD_ARG 1
#define MS_UNSUPPORTED 2
#define MS_LAUNCH_FAILED 3

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16 x) { return static_cast<float>(x); }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float x) { return static_cast<bf16>(x); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (one element of each 16-lane row), the
// same bits in all four: v_permlane16_swap and v_permlane32_swap hand a lane its partner's value
// without a trip through LDS. The sum is (row 0 + row 1) + (row 2 + row 3) for every lane.
__device__ __forceinline__ float rows4_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float rows4_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024). `red` holds NT / 64 floats.
// Every thread receives the total; the order of additions is fixed by NT alone.
template <int NT> __device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < NT / WAVE; ++i) total += red[i];
  return total;
}

// Sum of `splits` floats spaced `stride` apart, added in ascending order. Loads are issued eight at a
// time so that they overlap; absent splits contribute an exact zero.
__device__ __forceinline__ float sum_splits(const float* __restrict__ p, int splits, size_t stride) {
  float acc = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = (s0 + u < splits) ? p[(size_t)(s0 + u) * stride] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  return acc;
}

// Which elements of a head make pair j of a rotary position encoding: (j, j + rot/2) or (2j, 2j + 1).
#define MS_ROPE_HALVES 0
#define MS_ROPE_ADJACENT 1

// Activations of the gated feed-forward, by the number the host passes: out = act(gate) * up, in float32.
#define MS_ACT_SILU 0
#define MS_ACT_GELU_TANH 1
#define MS_ACT_COUNT 2
__device__ __forceinline__ float activate(float x, int act) {
  if (act == MS_ACT_GELU_TANH) return 0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
  return x / (1.f + expf(-x));
}

static inline int launch_status() { return hipGetLastError() == hipSuccess ? MS_OK : MS_LAUNCH_FAILED; }
