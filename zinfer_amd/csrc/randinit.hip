// The random-weights mode's counter-based draw on the device.  The value of an element depends
// on (key, element index) alone; zinfer_amd/weights/counter_rng.py is the same arithmetic in
// numpy and gives the same bits.  Everything below is integer arithmetic or IEEE 754 +, -, *,
// /, sqrt in 64-bit floats, each rounded on its own: no fused multiply-add may be formed, and
// the logarithm and cosine are the short series written out here, not a library's.
#include "zf_common.h"
#pragma clang fp contract(off)

#define RI_NORMAL 0
#define RI_GAIN 1
#define RI_ZEROS 2

__device__ __forceinline__ uint64_t ri_mix(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// ln m = 2 f (1 + f^2/3 + f^4/5 + ...) with f = (m - 1) / (m + 1)
__device__ __forceinline__ double ri_log_unit(uint32_t k1) {
  int e;
  double m = frexp((double)k1 + 1.0, &e);      // exact, m in [0.5, 1)
  if (m < 0.7071067811865476) {
    m = m * 2.0;
    e -= 1;
  }
  const double f = (m - 1.0) / (m + 1.0);
  const double s = f * f;
  double acc = 1.0 / 23.0;
#pragma unroll
  for (int k = 10; k >= 0; --k) acc = acc * s + 1.0 / (double)(2 * k + 1);
  return (double)(e - 32) * 0.6931471805599453 + 2.0 * f * acc;
}

__device__ __forceinline__ double ri_cos_turn(uint32_t k2) {
  const uint32_t octant = k2 >> 29, frac = k2 & ((1u << 29) - 1u);
  const uint32_t t = (octant & 1u) ? (1u << 29) - frac : frac;
  const double x = (double)t * (6.283185307179586 / 4294967296.0);
  const double s = x * x;
  double c;
  if ((octant + 1u) & 2u) {
    double acc = 1.0 / 355687428096000.0;
    acc = acc * s + -1.0 / 1307674368000.0;
    acc = acc * s + 1.0 / 6227020800.0;
    acc = acc * s + -1.0 / 39916800.0;
    acc = acc * s + 1.0 / 362880.0;
    acc = acc * s + -1.0 / 5040.0;
    acc = acc * s + 1.0 / 120.0;
    acc = acc * s + -1.0 / 6.0;
    acc = acc * s + 1.0;
    c = x * acc;
  } else {
    double acc = 1.0 / 20922789888000.0;
    acc = acc * s + -1.0 / 87178291200.0;
    acc = acc * s + 1.0 / 479001600.0;
    acc = acc * s + -1.0 / 3628800.0;
    acc = acc * s + 1.0 / 40320.0;
    acc = acc * s + -1.0 / 720.0;
    acc = acc * s + 1.0 / 24.0;
    acc = acc * s + -1.0 / 2.0;
    acc = acc * s + 1.0;
    c = acc;
  }
  return ((octant + 2u) & 4u) ? -c : c;
}

template <typename T>
__global__ __launch_bounds__(256) void randinit_kernel(T* __restrict__ out, uint64_t key,
                                                       uint64_t start, uint64_t count, int kind,
                                                       double std) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    const uint64_t z = ri_mix(key + (start + i + 1ull) * 0x9E3779B97F4A7C15ull);
    const uint32_t k1 = (uint32_t)(z >> 32), k2 = (uint32_t)z;
    float v;
    if (kind == RI_ZEROS) {
      v = 0.f;
    } else if (kind == RI_GAIN) {
      const double u = (double)k1 * (1.0 / 4294967296.0);
      v = (float)(1.0 + (u * 0.2 - 0.1));
    } else {
      const double r = sqrt(-2.0 * ri_log_unit(k1));
      v = (float)(r * ri_cos_turn(k2) * std);
    }
    store_from_float<T>(out + i, v);
  }
}

// out[i] = element start + i of the tensor with `key`, i in [0, count); dtype ZF_F32 or ZF_BF16
extern "C" int zf_randinit(void* out, int dtype, unsigned long long key, unsigned long long start,
                           unsigned long long count, int kind, double std, hipStream_t stream) {
  if (count == 0) return 0;
  if (kind < 0 || kind > 2 || (dtype != ZF_F32 && dtype != ZF_BF16)) return 1;
  unsigned long long blocks = (count + 256ull * 8ull - 1ull) / (256ull * 8ull);
  if (blocks > 65536ull) blocks = 65536ull;
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(randinit_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (float*)out, (uint64_t)key, (uint64_t)start, (uint64_t)count, kind, std);
  else
    hipLaunchKernelGGL(randinit_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (bf16_t*)out, (uint64_t)key, (uint64_t)start, (uint64_t)count, kind, std);
  ZF_CHECK_LAUNCH();
}
