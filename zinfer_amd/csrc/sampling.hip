// Sampling on the device with the reference's order of operations
// (src/sampling/sampler.zig:18-91): penalties on seen tokens, the k largest adjusted logits
// in descending order (lower id first among equals), exp((l / T) - max) in 32-bit with
// 64-bit sums, the min-p prefix, the top-p prefix on the renormalised kept set, then the
// draw u * kept_sum walked down the candidates.  One workgroup per row; k <= 1024.
#include "zf_common.h"

#define SMP_THREADS 1024
#define SMP_MAX_K 1024

// order-preserving map float -> uint32 (larger float, larger key)
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// ---------------------------------------------------------------- penalties, in place
// For every (row, token, count) triple: repetition (negative logits multiplied, others
// divided), presence, frequency, in this order (sampler.zig:186-201).
__global__ void apply_penalties_kernel(float* __restrict__ logits, const int* __restrict__ rows,
                                       const int* __restrict__ tokens,
                                       const int* __restrict__ counts,
                                       const float* __restrict__ params, int n, int V) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int row = rows[i];
  const float rep = params[row * 3 + 0], pres = params[row * 3 + 1], freq = params[row * 3 + 2];
  float* p = logits + (size_t)row * V + tokens[i];
  float a = *p;
  if (rep > 0.f && rep != 1.f) a = a < 0.f ? a * rep : a / rep;
  a -= pres;
  a -= (float)counts[i] * freq;
  *p = a;
}

extern "C" int zf_apply_penalties(float* logits, const int* rows, const int* tokens,
                                  const int* counts, const float* params, int n, int V,
                                  hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(apply_penalties_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, logits,
                     rows, tokens, counts, params, n, V);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- top-k sampling
// params per row: temperature, top_p, min_p (float), top_k (int), u (double, in [0, 1)).
struct SampleRow {
  float temperature, top_p, min_p;
  int top_k;
  double u;
};

__global__ __launch_bounds__(SMP_THREADS) void sample_topk_kernel(
    const float* __restrict__ logits, const SampleRow* __restrict__ params,
    int* __restrict__ out, int V) {
  __shared__ unsigned hist[256];
  __shared__ unsigned s_prefix, s_remaining;
  __shared__ float cval[SMP_MAX_K];
  __shared__ int cidx[SMP_MAX_K];
  __shared__ unsigned scan[SMP_THREADS];
  __shared__ unsigned s_count;
  const float* row = logits + (size_t)blockIdx.x * V;
  const SampleRow prm = params[blockIdx.x];
  const int tid = threadIdx.x;
  int k = prm.top_k <= 0 || prm.top_k > V ? V : prm.top_k;
  if (k > SMP_MAX_K) k = SMP_MAX_K;     // the host refuses such rows before launching

  // 1. radix select: the key of the k-th largest element, 8 bits a pass from the top
  if (tid == 0) {
    s_prefix = 0;
    s_remaining = (unsigned)k;
  }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const unsigned prefix = s_prefix;
    const unsigned mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    for (int i = tid; i < V; i += SMP_THREADS) {
      const uint32_t key = float_key(row[i]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 0xff], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      unsigned rem = s_remaining;
      int b = 255;
      for (; b > 0; --b) {
        if (hist[b] >= rem) break;
        rem -= hist[b];
      }
      s_prefix = prefix | ((unsigned)b << shift);
      s_remaining = rem;     // how many elements equal to the final key are still wanted
    }
    __syncthreads();
  }
  const uint32_t kth = s_prefix;
  const unsigned want_equal = s_remaining;

  // 2. gather: everything above the k-th key, then the lowest ids among those equal to it.
  //    Threads own contiguous index ranges so that the block-wide scans are in id order.
  const int per = (V + SMP_THREADS - 1) / SMP_THREADS;
  const int lo = tid * per, hi = min(V, lo + per);
  unsigned n_gt = 0, n_eq = 0;
  for (int i = lo; i < hi; ++i) {
    const uint32_t key = float_key(row[i]);
    n_gt += key > kth;
    n_eq += key == kth;
  }
  // exclusive scans of n_gt and n_eq over the threads
  unsigned off_gt, off_eq, total_gt;
  scan[tid] = n_gt;
  __syncthreads();
  for (int d = 1; d < SMP_THREADS; d <<= 1) {
    const unsigned v = tid >= d ? scan[tid - d] : 0;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  off_gt = scan[tid] - n_gt;
  total_gt = scan[SMP_THREADS - 1];
  __syncthreads();
  scan[tid] = n_eq;
  __syncthreads();
  for (int d = 1; d < SMP_THREADS; d <<= 1) {
    const unsigned v = tid >= d ? scan[tid - d] : 0;
    __syncthreads();
    scan[tid] += v;
    __syncthreads();
  }
  off_eq = scan[tid] - n_eq;
  __syncthreads();
  for (int i = lo; i < hi; ++i) {
    const float v = row[i];
    const uint32_t key = float_key(v);
    if (key > kth) {
      cval[off_gt] = v;
      cidx[off_gt] = i;
      ++off_gt;
    } else if (key == kth) {
      if (off_eq < want_equal) {
        cval[total_gt + off_eq] = v;
        cidx[total_gt + off_eq] = i;
      }
      ++off_eq;
    }
  }
  if (tid == 0) s_count = total_gt + want_equal;      // == k
  __syncthreads();
  const int n = (int)s_count;

  // 3. sort descending by value, ascending id among equals (bitonic over 1024 slots)
  for (int i = tid; i < SMP_MAX_K; i += SMP_THREADS)
    if (i >= n) {
      cval[i] = -INFINITY;
      cidx[i] = 0x7fffffff;
    }
  __syncthreads();
  for (int size = 2; size <= SMP_MAX_K; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const int i = tid;
      const int jj = i ^ stride;
      if (jj > i) {
        const bool up = (i & size) == 0;      // this half ends up in "before" order
        const float vi = cval[i], vj = cval[jj];
        const int ii = cidx[i], ij = cidx[jj];
        const bool i_before_j = vi > vj || (vi == vj && ii < ij);
        if (i_before_j != up) {
          cval[i] = vj;
          cval[jj] = vi;
          cidx[i] = ij;
          cidx[jj] = ii;
        }
      }
      __syncthreads();
    }
  }

  // 4. the reference's walk, by one thread: 32-bit exponentials, 64-bit sums
  if (tid == 0) {
    const float T = prm.temperature;
    const float max_scaled = cval[0] / T;
    double sum = 0.0;
    for (int i = 0; i < n; ++i) {
      const float p = expf(cval[i] / T - max_scaled);
      cval[i] = p;
      sum += (double)p;
    }
    int result = cidx[0];
    if (sum > 0.0) {
      int keep = n;
      const float min_p = fminf(fmaxf(prm.min_p, 0.f), 1.f);
      if (min_p > 0.f) {
        const float thr = cval[0] * min_p;
        keep = 0;
        while (keep < n && cval[keep] >= thr) ++keep;
        if (keep < 1) keep = 1;
        sum = 0.0;
        for (int i = 0; i < keep; ++i) sum += (double)cval[i];
      }
      const float top_p = fminf(fmaxf(prm.top_p, 0.f), 1.f);
      if (top_p < 1.f) {
        double cum = 0.0;
        int np = 0;
        while (np < keep) {
          cum += (double)cval[np] / sum;
          ++np;
          if (cum >= (double)top_p) break;
        }
        if (np < 1) np = 1;
        if (np < keep) keep = np;
      }
      double kept = 0.0;
      for (int i = 0; i < keep; ++i) kept += (double)cval[i];
      if (kept > 0.0) {
        double thr = prm.u * kept;
        result = cidx[keep - 1];
        for (int i = 0; i < keep; ++i) {
          thr -= (double)cval[i];
          if (thr <= 0.0) {
            result = cidx[i];
            break;
          }
        }
      }
    }
    out[blockIdx.x] = result;
  }
}

extern "C" int zf_sample_topk(const float* logits, const void* params, int* out, int n, int V,
                              hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(sample_topk_kernel, dim3(n), dim3(SMP_THREADS), 0, stream, logits,
                     (const SampleRow*)params, out, V);
  ZF_CHECK_LAUNCH();
}
