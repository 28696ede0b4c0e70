// Shared device helpers for the gfx950 kernels: bfloat16 <-> float, wave (64 lanes) and
// block reductions, element loads templated on the storage type.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define ZF_WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits

// bits << 16 (src/tensor/formats/bfloat16.zig:3-6 of the reference)
__device__ __forceinline__ float bf16_to_float(bf16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// round to nearest even, (bits + 0x7fff + lsb) >> 16 (bfloat16.zig:8-13), a NaN stays a NaN:
// gfx950 has an instruction for it (v_cvt_pk_bf16_f32), which the cast below becomes; it
// gives the same 16 bits as the formula for every one of the 2^32 inputs
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  const __bf16 b = (__bf16)f;
  return *(const bf16_t*)&b;
}
// two values in one register, `lo` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2_native __attribute__((ext_vector_type(2)));
  typedef float floatx2_native __attribute__((ext_vector_type(2)));
  const bf16x2_native v = __builtin_convertvector(floatx2_native{lo, hi}, bf16x2_native);
  return *(const uint32_t*)&v;
}

template <typename T> __device__ __forceinline__ float load_as_float(const T* p);
template <> __device__ __forceinline__ float load_as_float<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_as_float<bf16_t>(const bf16_t* p) {
  return bf16_to_float(*p);
}
template <typename T> __device__ __forceinline__ void store_from_float(T* p, float v);
template <> __device__ __forceinline__ void store_from_float<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_from_float<bf16_t>(bf16_t* p, float v) {
  *p = float_to_bf16(v);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = ZF_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, ZF_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = ZF_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, ZF_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` is LDS for
// at least 16 floats.  The order of the additions depends only on the block size.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int nwaves = (blockDim.x + ZF_WAVE - 1) / ZF_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += red[w];
  return total;
}

// dtype codes shared with the Python side
#define ZF_F32 0
#define ZF_BF16 1

#define ZF_CHECK_LAUNCH() return (int)hipGetLastError()
