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

// RMSNorm over a head and rotation of its pairs (i, i + hd / 2) for the 8 elements a lane
// holds: x0 = elements 4 li .. 4 li + 3 of the head, x1 = those hd / 2 further on; LPH lanes
// side by side hold the head (src/kernel/norm/basic.zig:5-22 and src/kernel/rope/basic.zig:5-30
// of the reference: x / sqrt(mean(x^2) + eps) * gain, then (x0 c - x1 s, x1 c + x0 s) with the
// angle of (position, pair)).  Every lane of the LPH calls it (the sum goes over all of them);
// a lane that is not `active` holds zeros and keeps them.  The gains and the angles' cosines
// and sines of the lane's elements are loaded apart (a null table: none), so that a kernel
// can ask for them early.  One function for the kernel that writes the cache and for the
// decode attention that does the same work itself, so that both round alike.
struct HeadCoef {
  float g0[4], g1[4], c[4], sn[4];
  bool has_gain, has_rotation;
};
__device__ __forceinline__ void load_head_coef(HeadCoef& cf, int li, int hd,
                                               const float* __restrict__ gain,
                                               const float* __restrict__ cos_t,
                                               const float* __restrict__ sin_t, int pos) {
  // hd % 8 == 0 and 4 li < hd / 2: each group of four is one 16-byte load (as four 4-byte
  // loads they were two thirds of the load instructions of the kernels that call this)
  const int half = hd / 2;
  cf.has_gain = gain != nullptr;
  cf.has_rotation = cos_t != nullptr;
  float4 g0 = float4{1.f, 1.f, 1.f, 1.f}, g1 = g0, c = g0, sn = float4{0.f, 0.f, 0.f, 0.f};
  if (cf.has_gain) {
    g0 = *(const float4*)(gain + 4 * li);
    g1 = *(const float4*)(gain + half + 4 * li);
  }
  if (cf.has_rotation) {
    c = *(const float4*)(cos_t + (size_t)pos * half + 4 * li);
    sn = *(const float4*)(sin_t + (size_t)pos * half + 4 * li);
  }
  cf.g0[0] = g0.x; cf.g0[1] = g0.y; cf.g0[2] = g0.z; cf.g0[3] = g0.w;
  cf.g1[0] = g1.x; cf.g1[1] = g1.y; cf.g1[2] = g1.z; cf.g1[3] = g1.w;
  cf.c[0] = c.x; cf.c[1] = c.y; cf.c[2] = c.z; cf.c[3] = c.w;
  cf.sn[0] = sn.x; cf.sn[1] = sn.y; cf.sn[2] = sn.z; cf.sn[3] = sn.w;
}
// the same head at another position: the gains stay, cosines and sines are loaded anew
__device__ __forceinline__ void load_head_rotation(HeadCoef& cf, int li, int hd,
                                                   const float* __restrict__ cos_t,
                                                   const float* __restrict__ sin_t, int pos) {
  if (!cf.has_rotation) return;
  const int half = hd / 2;
  const float4 c = *(const float4*)(cos_t + (size_t)pos * half + 4 * li);
  const float4 sn = *(const float4*)(sin_t + (size_t)pos * half + 4 * li);
  cf.c[0] = c.x; cf.c[1] = c.y; cf.c[2] = c.z; cf.c[3] = c.w;
  cf.sn[0] = sn.x; cf.sn[1] = sn.y; cf.sn[2] = sn.z; cf.sn[3] = sn.w;
}
template <int LPH>
__device__ __forceinline__ void head_norm_rotate(float (&x0)[4], float (&x1)[4], int hd,
                                                 bool active, float eps, const HeadCoef& cf) {
  // every product and sum below is rounded on its own: fused multiply-adds, formed or not as
  // the code around a call happens to be scheduled, would let two kernels that call this
  // disagree in the last bit
#pragma clang fp contract(off)
  if (cf.has_gain) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += x0[e] * x0[e] + x1[e] * x1[e];
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
    if (active) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x0[e] = x0[e] * inv * cf.g0[e];
        x1[e] = x1[e] * inv * cf.g1[e];
      }
    }
  }
  if (active && cf.has_rotation) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float r0 = x0[e] * cf.c[e] - x1[e] * cf.sn[e];
      const float r1 = x1[e] * cf.c[e] + x0[e] * cf.sn[e];
      x0[e] = r0;
      x1[e] = r1;
    }
  }
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
