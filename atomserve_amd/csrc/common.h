// Shared device helpers for the gfx950 kernels: element types, conversions and
// wave/block reductions.  A wavefront is 64 lanes wide everywhere in this code.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16;

#define WAVE 64

// Every entry point returns 0 on success and a negative code when it refuses its
// arguments (the Python wrapper turns the code into an exception).
#define AS_OK 0
#define AS_BAD_DTYPE -1
#define AS_BAD_SHAPE -2
#define AS_LAUNCH_FAILED -3

#define DT_F32 0
#define DT_BF16 1

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }  // round to nearest even

// What the cache pools may hold: a value that is not finite (a model that overflowed) is stored
// as zero.  Kernels multiply keys and values of masked places by a weight of zero, which is only
// harmless while every stored value is finite; pages are used again by other requests.
__device__ __forceinline__ float finite_or_zero(float v) {
  return (__float_as_uint(v) & 0x7f800000u) == 0x7f800000u ? 0.f : v;
}
__device__ __forceinline__ bf16 finite_or_zero(bf16 v) {
  return (__builtin_bit_cast(unsigned short, v) & 0x7f80u) == 0x7f80u ? (bf16)0.f : v;
}

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

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` is a
// __shared__ float[17].  The order of additions is fixed, so the result is reproducible.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (WAVE - 1), wid = threadIdx.x / WAVE;
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  __syncthreads();  // protects `red` against a previous use
  if (lane == 0) red[wid] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    red[16] = s;
  }
  __syncthreads();
  return red[16];
}

static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? AS_OK : AS_LAUNCH_FAILED;
}

// Compute units of the current device (asked once per device).
static inline int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
