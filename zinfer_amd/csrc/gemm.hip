// Matrix products C[M,N] = A[M,K] * W[N,K]^T (the weight is [out, in], as in the reference:
// y[r] = sum_c W[r,c] x[c], src/tensor/storage/store.zig:286-319).
//
//  * gemm_fma: 32-bit FMA, any storage types, any sizes.  Every output element is the sum of
//    its products in ascending k, whatever M is and wherever the row lies in the batch, so a
//    token's result does not depend on how the batch was cut.  This is the true 32-bit path.
#include "zf_common.h"

#define GF_BM 64
#define GF_BN 64
#define GF_BK 16

template <typename TA, typename TW, typename TO, bool ACC>
__global__ __launch_bounds__(256) void gemm_fma_kernel(const TA* __restrict__ A,
                                                       const TW* __restrict__ W,
                                                       TO* __restrict__ C, int M, int N, int K) {
  __shared__ float As[GF_BK][GF_BM + 4];
  __shared__ float Ws[GF_BK][GF_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;       // 16 x 16 threads, each 4 x 4 outputs
  const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // each thread loads 4 elements of A and 4 of W per k-tile: row = tid / 4, k = (tid % 4) * 4..
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += GF_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + lk + i;
      const int am = m0 + lr, wn = n0 + lr;
      As[lk + i][lr] = (am < M && k < K) ? load_as_float<TA>(A + (size_t)am * K + k) : 0.f;
      Ws[lk + i][lr] = (wn < N && k < K) ? load_as_float<TW>(W + (size_t)wn * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GF_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      TO* c = C + (size_t)m * N + n;
      if (ACC)
        store_from_float<TO>(c, load_as_float<TO>(c) + acc[i][j]);
      else
        store_from_float<TO>(c, acc[i][j]);
    }
  }
}

template <typename TA, typename TW, typename TO>
static void launch_fma(const void* A, const void* W, void* C, int M, int N, int K, int accumulate,
                       hipStream_t stream) {
  dim3 grid((N + GF_BN - 1) / GF_BN, (M + GF_BM - 1) / GF_BM);
  if (accumulate)
    hipLaunchKernelGGL((gemm_fma_kernel<TA, TW, TO, true>), grid, dim3(256), 0, stream,
                       (const TA*)A, (const TW*)W, (TO*)C, M, N, K);
  else
    hipLaunchKernelGGL((gemm_fma_kernel<TA, TW, TO, false>), grid, dim3(256), 0, stream,
                       (const TA*)A, (const TW*)W, (TO*)C, M, N, K);
}

// dtypes: ZF_F32 / ZF_BF16 for a, w, out.  accumulate: out += (else out =).
extern "C" int zf_gemm_fma(const void* A, int a_dtype, const void* W, int w_dtype, void* C,
                           int c_dtype, int M, int N, int K, int accumulate,
                           hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (key) {
    case 0: launch_fma<float, float, float>(A, W, C, M, N, K, accumulate, stream); break;
    case 1: launch_fma<float, float, bf16_t>(A, W, C, M, N, K, accumulate, stream); break;
    case 2: launch_fma<float, bf16_t, float>(A, W, C, M, N, K, accumulate, stream); break;
    case 3: launch_fma<float, bf16_t, bf16_t>(A, W, C, M, N, K, accumulate, stream); break;
    case 4: launch_fma<bf16_t, float, float>(A, W, C, M, N, K, accumulate, stream); break;
    case 5: launch_fma<bf16_t, float, bf16_t>(A, W, C, M, N, K, accumulate, stream); break;
    case 6: launch_fma<bf16_t, bf16_t, float>(A, W, C, M, N, K, accumulate, stream); break;
    case 7: launch_fma<bf16_t, bf16_t, bf16_t>(A, W, C, M, N, K, accumulate, stream); break;
    default: return -1;
  }
  ZF_CHECK_LAUNCH();
}
