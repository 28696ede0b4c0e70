// Matrix products C[M,N] = A[M,K] * W[N,K]^T (the weight is [out, in], as in the reference:
// y[r] = sum_c W[r,c] x[c], src/tensor/storage/store.zig:286-319).
//
//  * gemm_fma: 32-bit FMA, any storage types, any sizes.  Every output element is the sum of
//    its products in ascending k, whatever M is and wherever the row lies in the batch, so a
//    token's result does not depend on how the batch was cut.  This is the true 32-bit path.
#include <type_traits>

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

// =====================================================================================
//  bfloat16 MFMA kernels (gfx950): v_mfma_f32_32x32x16_bf16 and v_mfma_f32_16x16x32_bf16,
//  fp32 accumulation.  A is [M, K] bfloat16, W is [N, K] bfloat16, both with K contiguous,
//  which is the operand order the instruction wants: every lane feeds 8 consecutive k of
//  one row of A and of one row of W.
// =====================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

#define EPI_STORE_BF16 0
#define EPI_STORE_F32 1
#define EPI_ACC_F32 2
// SwiGLU fused into the product: the rows of W alternate in groups of 16 between the gate
// and the up projection (gate 0..15, up 0..15, gate 16..31, ...); the output is
// silu(gate) * up as bfloat16 [M, N / 2]  (a_j = g_j / (1 + exp(-g_j)) * u_j, cpu.zig:130-147)
#define EPI_SWIGLU 3

__device__ __forceinline__ float swiglu_f(float g, float u) { return g / (1.0f + expf(-g)) * u; }

// ---------------------------------------------------------------- large M: LDS-tiled
// Block tile BM x BN x 64, waves laid out (BM/WM) x (BN/WN), each wave WM x WN through
// 32x32x16 MFMAs.  Tiles are staged through LDS with rows padded to 72 elements (144 bytes)
// so that the 16-byte operand reads of 8 neighbouring rows fall on distinct banks; the next
// tile's global loads are in flight while the current one is multiplied.
#define TK 64
#define LDS_ROW 72

// Pre-tiled weights (WT): W is stored as [N / 16][K / 64][2][64][8]: the 16 rows x 64 k of a
// tile lie together (2 KB) in the order in which the lanes of a 16x16x32 MFMA pair consume
// them (chunk c of lane l = 16 g + r holds row r, k = 16 g + 8 c .. + 8), so that one wave
// load of the weight-streaming kernel is 1 KB of consecutive memory.  This kernel reads the
// same layout 16 bytes at a time.
__device__ __forceinline__ size_t tiled_offset(int n, int k, int K) {
  const int kk = k % 64;
  return ((size_t)(n / 16) * (K / 64) + k / 64) * 1024 + ((kk % 16) / 8) * 512 +
         ((kk / 16) * 16 + n % 16) * 8 + kk % 8;
}

// XCD-aware tile order.  Consecutive workgroups go to different XCDs (8 of them, each with its
// own L2), so workgroup b takes place (b % 8) * per_xcd + b / 8 of the tile order: one XCD
// then walks neighbouring tiles.  The order runs through groups of at most GROUP tile rows,
// down the rows of a group first, so that the tiles an XCD walks share W tiles in its L2.  The
// rows are dealt evenly over the groups (9 rows in groups of 8: 5 + 4, not 8 + 1): a group of
// one row would send an XCD through every W tile on its own.
template <int GROUP>
__device__ __forceinline__ void tile_of_workgroup(int b, int tiles_m, int tiles_n, int& tm,
                                                  int& tn) {
  const int nblocks = tiles_m * tiles_n;
  {
    const int base = nblocks / 8, rem = nblocks % 8;
    const int xcd = b % 8, idx = b / 8;
    b = xcd * base + min(xcd, rem) + idx;   // XCD x owns base (+1 if x < rem) tiles in a row
  }
  const int ngroups = (tiles_m + GROUP - 1) / GROUP;
  const int rows = tiles_m / ngroups, longer = tiles_m % ngroups;   // the first groups: rows + 1
  const int in_longer = (rows + 1) * tiles_n;
  int first_m, gsize, at;
  if (b < longer * in_longer) {
    gsize = rows + 1;
    first_m = (b / in_longer) * gsize;
    at = b % in_longer;
  } else {
    const int bb = b - longer * in_longer, in_group = rows * tiles_n;
    gsize = rows;
    first_m = longer * (rows + 1) + (bb / in_group) * rows;
    at = bb % in_group;
  }
  tm = first_m + at % gsize;
  tn = at / gsize;
}

template <int BM, int BN, int WM, int WN, int EPI, bool WT>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void gemm_bf16_tile_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ Cv, int M,
    int N, int K, int tiles_m, int tiles_n) {
  constexpr int NWM = BM / WM, NWN = BN / WN;
  constexpr int NT = NWM * NWN * 64;
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int A_CHUNKS = BM * 8 / NT;   // 16-byte chunks per thread per tile
  constexpr int B_CHUNKS = BN * 8 / NT;
  static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile does not divide over the threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t* lds = (bf16_t*)lds_raw;
  // stage s: A at s*(BM+BN)*LDS_ROW, W after it
  constexpr int STAGE = (BM + BN) * LDS_ROW;

  int tm, tn;
  tile_of_workgroup<(BM >= 128 ? 8 : 1024 / BM)>(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int wm = wave / NWN, wn = wave % NWN;

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  u32x4_t areg[A_CHUNKS], breg[B_CHUNKS];

  // which 16 bytes of the W tile a thread moves: (row of the tile, k offset).  Plain layout:
  // 8 consecutive threads take the 8 chunks of a row.  Pre-tiled: 128 consecutive threads
  // take the 128 chunks of a 16-row group in the order they lie in memory (chunk p = 64 c +
  // 16 g + r holds row r, k = 16 g + 8 c), so their loads are consecutive 16-byte pieces.
  auto b_chunk = [&](int chunk, int& row, int& kc) {
    if (WT) {
      const int p = chunk % 128;
      row = (chunk / 128) * 16 + p % 16;
      kc = ((p % 64) / 16) * 16 + (p / 64) * 8;
    } else {
      row = chunk / 8;
      kc = (chunk % 8) * 8;
    }
  };

  auto gload = [&](int k0) {
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * NT;
      const int row = chunk / 8, kc = (chunk % 8) * 8;
      const int m = min(m0 + row, M - 1);
      if (k0 + kc < K)
        areg[c] = *(const u32x4_t*)(A + (size_t)m * K + k0 + kc);
      else
        areg[c] = u32x4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int c = 0; c < B_CHUNKS; ++c) {
      int row, kc;
      b_chunk(tid + c * NT, row, kc);
      const int n = min(n0 + row, N - 1);
      if (k0 + kc < K)
        breg[c] = *(const u32x4_t*)(W + (WT ? tiled_offset(n, k0 + kc, K)
                                            : (size_t)n * K + k0 + kc));
      else
        breg[c] = u32x4_t{0, 0, 0, 0};
    }
  };
  auto lstore = [&](int stage) {
    bf16_t* a_s = lds + stage * STAGE;
    bf16_t* b_s = a_s + BM * LDS_ROW;
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * NT;
      const int row = chunk / 8, kc = (chunk % 8) * 8;
      *(u32x4_t*)(a_s + row * LDS_ROW + kc) = areg[c];
    }
#pragma unroll
    for (int c = 0; c < B_CHUNKS; ++c) {
      int row, kc;
      b_chunk(tid + c * NT, row, kc);
      *(u32x4_t*)(b_s + row * LDS_ROW + kc) = breg[c];
    }
  };

  const int ktiles = (K + TK - 1) / TK;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const int stage = kt & 1;
    if (kt + 1 < ktiles) gload((kt + 1) * TK);
    const bf16_t* a_s = lds + stage * STAGE + (wm * WM) * LDS_ROW;
    const bf16_t* b_s = lds + stage * STAGE + BM * LDS_ROW + (wn * WN) * LDS_ROW;
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) {
      bf16x8_t af[FM], bfr[FN];
      const int koff = ks * 16 + (lane / 32) * 8;
#pragma unroll
      for (int i = 0; i < FM; ++i)
        af[i] = *(const bf16x8_t*)(a_s + (i * 32 + lane % 32) * LDS_ROW + koff);
#pragma unroll
      for (int j = 0; j < FN; ++j)
        bfr[j] = *(const bf16x8_t*)(b_s + (j * 32 + lane % 32) * LDS_ROW + koff);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ktiles) lstore(stage ^ 1);
    __syncthreads();
  }

  // D[i][j] of a 32x32 block: j = lane % 32, i = 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int n = n0 + wn * WN + j * 32 + lane % 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (EPI == EPI_SWIGLU) {
          // columns 0..15 of the 32-wide block are gate, 16..31 the matching up columns
          const float other = __shfl_xor(acc[i][j][r], 16, 64);
          if (lane % 32 < 16 && m < M && n < N)
            ((bf16_t*)Cv)[(size_t)m * (N / 2) + (n / 32) * 16 + n % 16] =
                float_to_bf16(swiglu_f(acc[i][j][r], other));
          continue;
        }
        if (m < M && n < N) {
          const size_t off = (size_t)m * N + n;
          if (EPI == EPI_STORE_BF16)
            ((bf16_t*)Cv)[off] = float_to_bf16(acc[i][j][r]);
          else if (EPI == EPI_STORE_F32)
            ((float*)Cv)[off] = acc[i][j][r];
          else
            ((float*)Cv)[off] += acc[i][j][r];
        }
      }
    }
}

// Epilogue through LDS of the kernels whose waves hold 32-row x 32-column MFMA results: a
// 32x32 result has a lane's 16 values in 16 different rows, so direct stores would be 2 or 4
// bytes wide in runs of 64 bytes.  Each wave lays 32 rows of WN columns of its tile (the FN
// column blocks from J0 on, at rows mw.., columns nw..) down in its own slab (32 rows of
// WN + 4 floats) and reads them back along the rows, 16 bytes per lane.  All waves of the
// workgroup call it together.
template <int FM, int FN, int WN, int EPI, int J0 = 0, int FNALL = FN>
__device__ __forceinline__ void store_through_slab(f32x16_t (&acc)[FM][FNALL], float* slab, int mw,
                                                   int nw, int M, int N, void* Cv, int lane) {
  static_assert(WN == 32 * FN && J0 + FN <= FNALL, "column blocks");
  constexpr int SLAB_ROW = WN + 4;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        slab[(8 * (r / 4) + 4 * (lane / 32) + r % 4) * SLAB_ROW + j * 32 + lane % 32] = acc[i][J0 + j][r];
    __syncthreads();
    if (EPI == EPI_SWIGLU) {
      // 16 gate columns, then the 16 up columns that belong to them: 8 outputs per lane
      constexpr int LPR = WN / 16;                  // lanes per row
#pragma unroll
      for (int it = 0; it < 32 * LPR / 64; ++it) {
        const int row = it * (64 / LPR) + lane / LPR, q = lane % LPR;
        const int m = mw + i * 32 + row;
        const int c = (q / 2) * 32 + (q % 2) * 8;   // first gate column inside the wave's tile
        const int n = nw + c;
        if (m < M && n < N) {
          const float* src = slab + row * SLAB_ROW + c;
          const float4 g0 = *(const float4*)src, g1 = *(const float4*)(src + 4);
          const float4 u0 = *(const float4*)(src + 16), u1 = *(const float4*)(src + 20);
          const u32x4_t v = u32x4_t{
              pack_bf16x2(swiglu_f(g0.x, u0.x), swiglu_f(g0.y, u0.y)),
              pack_bf16x2(swiglu_f(g0.z, u0.z), swiglu_f(g0.w, u0.w)),
              pack_bf16x2(swiglu_f(g1.x, u1.x), swiglu_f(g1.y, u1.y)),
              pack_bf16x2(swiglu_f(g1.z, u1.z), swiglu_f(g1.w, u1.w))};
          *(u32x4_t*)((bf16_t*)Cv + (size_t)m * (N / 2) + (n / 32) * 16 + (n % 32)) = v;
        }
      }
    } else if (EPI == EPI_STORE_BF16) {
      constexpr int LPR = WN / 8;
#pragma unroll
      for (int it = 0; it < 32 * LPR / 64; ++it) {
        const int row = it * (64 / LPR) + lane / LPR, c = (lane % LPR) * 8;
        const int m = mw + i * 32 + row, n = nw + c;
        if (m < M && n < N) {
          const float* src = slab + row * SLAB_ROW + c;
          const float4 x0 = *(const float4*)src, x1 = *(const float4*)(src + 4);
          const u32x4_t v = u32x4_t{pack_bf16x2(x0.x, x0.y), pack_bf16x2(x0.z, x0.w),
                                    pack_bf16x2(x1.x, x1.y), pack_bf16x2(x1.z, x1.w)};
          *(u32x4_t*)((bf16_t*)Cv + (size_t)m * N + n) = v;
        }
      }
    } else {
      constexpr int LPR = WN / 4;
#pragma unroll
      for (int it = 0; it < 32 * LPR / 64; ++it) {
        const int row = it * (64 / LPR) + lane / LPR, c = (lane % LPR) * 4;
        const int m = mw + i * 32 + row, n = nw + c;
        if (m < M && n < N) {
          float4 x = *(const float4*)(slab + row * SLAB_ROW + c);
          float4* dst = (float4*)((float*)Cv + (size_t)m * N + n);
          if (EPI == EPI_ACC_F32) {
            const float4 old = *dst;
            x = float4{old.x + x.x, old.y + x.y, old.z + x.z, old.w + x.w};
          }
          *dst = x;
        }
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------- large M, pre-tiled W: W not staged
// Tiles of BM tokens x BN outputs, k-tiles of TKM.  Only the tokens go through LDS; every wave
// takes its W operands straight from the pre-tiled matrix (16-byte pieces that lie in runs of
// 256 bytes), one k-tile ahead in registers.  That halves the LDS traffic per MFMA against
// the kernel above, whose LDS is as busy as its MFMAs.  With the waves side by side along the
// outputs (WM == BM) no two of them load the same part of W.
// ADMA: the tokens' k-tiles go from memory into LDS by direct-to-LDS loads (a wave instruction
// copies 64 x 16 bytes to one LDS address + 16 bytes a lane), not through registers: no
// registers hold them on the way, and the stores into LDS and their waits are gone (1 to 2 %
// at 2048 and 8192 tokens).  Such a copy lands as consecutive bytes, so instead of padded rows
// the 16-byte pieces of a row are permuted (piece c of row r lies at place c ^ ((r >> 1) & 7)
// of its 128 bytes): the 16 rows a quarter wave reads then fall into 16 different groups of
// banks.  Two stages in two arrays, so that the compiler knows which reads wait for which
// copies; the barrier is a bare s_barrier behind a wait that lets the W loads issued since
// (younger than the copies) stay in flight.
// TAIL: the tiles beyond the last whole round of the chip (the tile order's last `tail` ones)
// are shared by tail_split workgroups each, along K: workgroups [whole, whole + tail *
// tail_split) of the grid, which leave float32 partials [tail][tail_split][BM][BN] in tail_ws
// for tile_tail_reduce_kernel; a short last round then takes 1 / tail_split of a tile's time
// instead of a whole one.
// KG == 2: two groups of waves in one workgroup, each the whole tile over half of the
// workgroup's k-tiles (its own stages in LDS, its own W), for products whose tiles are so few
// that a CU holds one workgroup: twice the waves to hide a load behind, and no more traffic
// than one group has.  At the end each group hands one of its two column blocks to the other
// through LDS (half the tile's rows at a time), adds what it is handed (first half of K plus
// second half, whichever group adds) and stores the block it kept.
template <int BM, int BN, int WM, int WN, int EPI, int TKM = TK, bool W2 = false,
          bool ADMA = false, bool TAIL = false, int KG = 1>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64 * KG) void gemm_bf16_tile_wdirect_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ Cv, int M,
    int N, int K, int tiles_m, int tiles_n, int whole, int tail_split,
    float* __restrict__ tail_ws) {
  // (the host pass, which only needs the launch stub, does not know the buffer descriptor type)
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NWN = BN / WN, NT = (BM / WM) * NWN * 64;       // (NT: the threads of a group)
  constexpr int FM = WM / 32, FN = WN / 32;
  constexpr int LROW = TKM + 8, KCH = TKM / 8;      // LDS row in elements; 16-byte chunks per row
  static_assert(BM * KCH % NT == 0 && TKM % 64 == 0, "tile does not divide over the threads");
  static_assert(KG == 1 || (KG == 2 && ADMA && !TAIL && FN == 2 && FM % 2 == 0),
                "two groups: tokens copied straight into LDS, two column blocks a wave");
  constexpr int A_CHUNKS = BM * KCH / NT;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16_t* lds = (bf16_t*)lds_raw;       // two stages of BM rows of LROW elements

  // which tile, and which of how many parts of its k-tiles
  int tile = blockIdx.x, kpart = blockIdx.y, kparts = gridDim.y;
  bool in_tail = false;
  if constexpr (TAIL) {
    if ((int)blockIdx.x >= whole) {
      in_tail = true;
      tile = whole + ((int)blockIdx.x - whole) / tail_split;
      kpart = ((int)blockIdx.x - whole) % tail_split;
      kparts = tail_split;
    }
  }
  int tm, tn;
  tile_of_workgroup<(BM >= 128 ? 8 : 1024 / BM)>(tile, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // (a group's threads count from 0: what follows is one group's view)
  const int kgrp = KG > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x / NT) : 0;
  const int tid = KG > 1 ? (int)threadIdx.x % NT : (int)threadIdx.x;
  if (KG > 1) {
    kpart = kpart * KG + kgrp;
    kparts *= KG;
  }
  const int wave = tid / 64, lane = tid % 64;
  const int wm = wave / NWN, wn = wave % NWN;

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // W operand of MFMA (j, ks): column n = n0 + wn * WN + 32 j + lane % 32, k = 16 ks +
  // 8 (lane / 32) .. + 8 of the k-tile: piece 64 (lane / 32) + 16 ks + n % 16 of the 16-row
  // group n / 16.  Groups beyond N are clamped (their columns are never stored).
  // (loaded through a buffer descriptor on the tile's first group: a 32-bit offset per lane
  // and one all lanes share instead of a 64-bit address per lane, which issues faster and
  // needs no address arithmetic)
  const int grp0 = min(n0 / 16, N / 16 - 1);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(W + (size_t)grp0 * (K / 64) * 1024), 0, 0x7fffffff, 0x00020000);
  uint32_t wbase[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) {
    const int n = n0 + wn * WN + j * 32 + lane % 32;
    const int grp = min(n / 16, N / 16 - 1) - grp0;
    wbase[j] = ((uint32_t)grp * (uint32_t)(K / 64) * 1024 + ((lane / 32) * 64 + n % 16) * 8) * 2;
  }
  u32x4_t wreg[W2 ? 2 : 1][TKM / 16][FN];
  auto gload_w = [&](auto BUF, int kt, int ks) {
    constexpr int B = decltype(BUF)::value;
    const uint32_t at = ((uint32_t)kt * (TKM / 64) + ks / 4) * 2048 + (ks % 4) * 256;
#pragma unroll
    for (int j = 0; j < FN; ++j)
      wreg[B][ks][j] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wbase[j], at, 0);
  };
  // gridDim.y workgroups share a tile's k-tiles (split-K for products with few tiles); each
  // then leaves a float32 partial [gridDim.y, M, N] in Cv for skinny_reduce_kernel
  const int kt_all = K / TKM;
  const int kt0 = (int)((long long)kpart * kt_all / kparts);
  const int ktiles = (int)((long long)(kpart + 1) * kt_all / kparts);
  if (gridDim.y > 1) Cv = (float*)Cv + (size_t)blockIdx.y * M * N;
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;

  if constexpr (ADMA) {
    static_assert(TKM == 64, "direct-to-LDS tokens: k-tiles of 64 (rows of 8 pieces)");
    __shared__ u32x4_t a_stages0[KG * BM * 8];
    __shared__ u32x4_t a_stages1[KG * BM * 8];
    u32x4_t* const a_stage0 = a_stages0 + kgrp * (BM * 8);
    u32x4_t* const a_stage1 = a_stages1 + kgrp * (BM * 8);
    // the places this thread fills: place p = tid + c NT is row p / 8, slot p % 8, and takes
    // piece slot ^ ((row >> 1) & 7) of the row's 128 bytes (rows beyond M: the last row)
    uint32_t asrc[A_CHUNKS];
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int p = tid + c * NT, row = p / 8, piece = (p % 8) ^ ((row >> 1) & 7);
      asrc[c] = (uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)K + piece * 8;
    }
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(A + (size_t)m0 * K), 0, 0x7fffffff, 0x00020000);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);      // the LDS address is a scalar
    auto dma_a = [&](int k0, u32x4_t* stage) {
#pragma unroll
      for (int c = 0; c < A_CHUNKS; ++c)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            a_rsrc, (__attribute__((address_space(3))) void*)(stage + (wave_u * 64 + c * NT)), 16,
            asrc[c] * 2, (uint32_t)k0 * 2, 0, 0);
    };
    // the operand of MFMA row block i, k-step ks: row 32 i + lane % 32, piece 2 ks + lane / 32
    int a_at[TKM / 16];
#pragma unroll
    for (int ks = 0; ks < TKM / 16; ++ks)
      a_at[ks] = (wm * WM + lane % 32) * 8 + ((2 * ks + lane / 32) ^ (((lane % 32) >> 1) & 7));
    // (in this order, kept by the scheduling barriers: the first step's wait counts on it)
    dma_a(kt0 * TKM, a_stage0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < TKM / 16; ++ks) gload_w(Buf0{}, kt0, ks);
    __builtin_amdgcn_sched_barrier(0);
    if (W2) {
#pragma unroll
      for (int ks = 0; ks < TKM / 16; ++ks) gload_w(Buf1{}, min(kt0 + 1, ktiles - 1), ks);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Before a step: its tokens' copies have landed (the last of them is older than the 6 W
    // loads of the step before that were issued behind it, which may stay in flight), then
    // all waves meet: every wave has also read its last operands out of the other stage.
    static_assert(FN == 2 && TKM == 64 && A_CHUNKS == 4, "the wait counts the loads behind the last copy");
    auto meet = [&]() {
      __builtin_amdgcn_s_waitcnt(0x0f76);     // vmcnt(6)
      __builtin_amdgcn_s_barrier();
    };
    // A k-step's MFMAs run output block by output block, so that a W register is free after
    // the first FM of them.  What else a wave issues follows single MFMAs: the next k-step's
    // FM operand reads behind the first FM MFMAs, then (k-steps 0 and 1) two of the next
    // tile's four copies, then the two W loads that refill this k-step's registers, the
    // second behind the last MFMA.  (All copies in one place hold the wave, and with it its
    // MFMAs, while the CU's one path to memory takes them one by one.)
    auto step = [&](int kt, const u32x4_t* cur, u32x4_t* other, auto BUF) {
      constexpr int B = decltype(BUF)::value;
      meet();
      const int wnxt = min(kt + (W2 ? 2 : 1), ktiles - 1);
      const uint32_t next_k0 = (uint32_t)min(kt + 1, ktiles - 1) * TKM * 2;
      __builtin_amdgcn_sched_barrier(0);
      u32x4_t af[2][FM];
#pragma unroll
      for (int i = 0; i < FM; ++i) af[0][i] = cur[a_at[0] + i * 256];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint32_t w_at = ((uint32_t)wnxt * (TKM / 64) + ks / 4) * 2048 + (ks % 4) * 256;
#pragma unroll
        for (int m = 0; m < 2 * FM; ++m) {
          const int j = m / FM, i = m % FM;
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              *(const bf16x8_t*)&af[ks % 2][i], *(const bf16x8_t*)&wreg[B][ks][j], acc[i][j],
              0, 0, 0);
          if (m < FM && ks < 3) af[(ks + 1) % 2][m] = cur[a_at[ks + 1] + m * 256];
          // copies 2 ks and 2 ks + 1 of the four: behind the first two MFMAs of the second block
          if (ks < 2 && (m == FM || (FM > 2 && m == FM + 1))) {
            const int c0 = 2 * ks + (FM == 2 ? 0 : m - FM), c1 = FM == 2 ? c0 + 2 : c0 + 1;
#pragma unroll
            for (int c = c0; c < c1; ++c)
              __builtin_amdgcn_raw_ptr_buffer_load_lds(
                  a_rsrc, (__attribute__((address_space(3))) void*)(other + (wave_u * 64 + c * NT)),
                  16, asrc[c] * 2, next_k0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);      // (older than the W loads that follow)
          }
          if (m == 2 * FM - 2) wreg[B][ks][0] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wbase[0], w_at, 0);
          if (m == 2 * FM - 1) wreg[B][ks][1] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, wbase[1], w_at, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    if (W2) {       // an even number of k-tiles (the launch sees to it)
      for (int kt = kt0; kt < ktiles; kt += 2) {
        step(kt, a_stage0, a_stage1, Buf0{});
        step(kt + 1, a_stage1, a_stage0, Buf1{});
      }
    } else {
      int kt = kt0;
      for (; kt + 1 < ktiles; kt += 2) {
        step(kt, a_stage0, a_stage1, Buf0{});
        step(kt + 1, a_stage1, a_stage0, Buf0{});
      }
      if (kt < ktiles) step(kt, a_stage0, a_stage1, Buf0{});
    }
    // the last step copied its own tile once more: nothing may still be on its way into LDS
    // when the workgroup ends
    __builtin_amdgcn_s_waitcnt(0x0f70);       // vmcnt(0)
  } else {
  u32x4_t areg[A_CHUNKS];
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(A + (size_t)m0 * K), 0, 0x7fffffff, 0x00020000);
  uint32_t a_from[A_CHUNKS];
#pragma unroll
  for (int c = 0; c < A_CHUNKS; ++c) {
    const int chunk = tid + c * NT;
    const int row = chunk / KCH, kc = (chunk % KCH) * 8;
    a_from[c] = ((uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)K + kc) * 2;
  }
  auto gload_a = [&](int k0) {
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c)
      areg[c] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_from[c], (uint32_t)k0 * 2, 0);
  };
  auto lstore = [&](int stage) {
    bf16_t* a_s = lds + stage * BM * LROW;
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * NT;
      const int row = chunk / KCH, kc = (chunk % KCH) * 8;
      *(u32x4_t*)(a_s + row * LROW + kc) = areg[c];
    }
  };

  gload_a(kt0 * TKM);
#pragma unroll
  for (int ks = 0; ks < TKM / 16; ++ks) gload_w(Buf0{}, kt0, ks);
  if (W2) {
#pragma unroll
    for (int ks = 0; ks < TKM / 16; ++ks) gload_w(Buf1{}, min(kt0 + 1, ktiles - 1), ks);
  }
  lstore(0);
  __syncthreads();
  // One k-tile per step: MFMAs on LDS stage `stage`; meanwhile the tokens of tile kt + 1
  // travel through registers into the other stage, and every k-step's W registers are
  // refilled right after their last use with their part of tile kt + 1 (W2: of tile kt + 2,
  // from the other of two register sets, so that a miss in L2 has two k-tiles to arrive).
  // No branches around the loads (the last steps load their own tile once more), so the
  // compiler can count the loads in flight and waits for no younger one; the scheduling
  // barriers keep it from sinking the loads down to their first use, which would expose
  // their whole latency.
  auto step = [&](int kt, int stage, auto BUF) {
    constexpr int B = decltype(BUF)::value;
    const int nxt = min(kt + 1, ktiles - 1);
    const int wnxt = W2 ? min(kt + 2, ktiles - 1) : nxt;
    gload_a(nxt * TKM);
    __builtin_amdgcn_sched_barrier(0);
    const bf16_t* a_s = lds + stage * BM * LROW + (wm * WM) * LROW;
    // the token operands of k-step ks + 1 are read from LDS while the MFMAs of ks run
    bf16x8_t af[2][FM];
#pragma unroll
    for (int i = 0; i < FM; ++i)
      af[0][i] = *(const bf16x8_t*)(a_s + (i * 32 + lane % 32) * LROW + (lane / 32) * 8);
#pragma unroll
    for (int ks = 0; ks < TKM / 16; ++ks) {
      if (ks + 1 < TKM / 16) {
        const int koff = (ks + 1) * 16 + (lane / 32) * 8;
#pragma unroll
        for (int i = 0; i < FM; ++i)
          af[(ks + 1) % 2][i] = *(const bf16x8_t*)(a_s + (i * 32 + lane % 32) * LROW + koff);
      }
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              af[ks % 2][i], *(const bf16x8_t*)&wreg[B][ks][j], acc[i][j], 0, 0, 0);
      gload_w(BUF, wnxt, ks);
      __builtin_amdgcn_sched_barrier(0);
    }
    lstore(stage ^ 1);
    __syncthreads();
  };
  if (W2) {       // an even number of k-tiles (the launch sees to it)
    for (int kt = kt0; kt < ktiles; kt += 2) {
      step(kt, 0, Buf0{});
      step(kt + 1, 1, Buf1{});
    }
  } else {
    for (int kt = kt0; kt < ktiles; ++kt) step(kt, (kt - kt0) & 1, Buf0{});
  }
  }

  // (the main loop's last barrier has freed the token stages; the launch sizes the LDS for
  // stages and slabs)
  if constexpr (KG == 2) {
    // Half the tile's rows at a time: every wave lays down the column block it gives away
    // (group 0 its second, group 1 its first) where its partner in the other group finds it.
    constexpr int HALF = FM / 2, PER_WAVE = HALF * 16 * 64;
    float* const xch = (float*)lds_raw;
    float* const mine = xch + (size_t)(kgrp * (NT / 64) + wave) * PER_WAVE;
    const float* const theirs = xch + (size_t)((1 - kgrp) * (NT / 64) + wave) * PER_WAVE;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      __syncthreads();          // (the round before has been read)
#pragma unroll
      for (int ii = 0; ii < HALF; ++ii)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = half * HALF + ii;
          mine[(ii * 16 + r) * 64 + lane] = kgrp == 0 ? acc[i][1][r] : acc[i][0][r];
        }
      __syncthreads();
#pragma unroll
      for (int ii = 0; ii < HALF; ++ii)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = half * HALF + ii;
          const float v = theirs[(ii * 16 + r) * 64 + lane];
          // kept block = first half of K + second half of K, in either group
          const float mine0 = acc[i][0][r], mine1 = acc[i][1][r];
          acc[i][0][r] = kgrp == 0 ? mine0 + v : mine0;
          acc[i][1][r] = kgrp == 0 ? mine1 : v + mine1;
        }
    }
    __syncthreads();            // the slabs lie where the blocks were handed over
    f32x16_t kept[FM][1];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) kept[i][0][r] = kgrp == 0 ? acc[i][0][r] : acc[i][1][r];
    float* slab32 = (float*)lds_raw + (size_t)(kgrp * (NT / 64) + wave) * 32 * (32 + 4);
    store_through_slab<FM, 1, 32, EPI>(kept, slab32, m0 + wm * WM, n0 + wn * WN + 32 * kgrp, M, N,
                                       Cv, lane);
    return;
  }
  float* slab = (float*)lds_raw + (size_t)wave * 32 * (WN + 4);
  if constexpr (TAIL) {
    if (in_tail) {      // (uniform over the workgroup) the whole tile as it is, rows beyond M too
      float* part = tail_ws + ((size_t)(tile - whole) * tail_split + kpart) * BM * BN;
      store_through_slab<FM, FN, WN, EPI_STORE_F32>(acc, slab, wm * WM, wn * WN, BM, BN, part, lane);
      return;
    }
  }
  store_through_slab<FM, FN, WN, EPI>(acc, slab, m0 + wm * WM, n0 + wn * WN, M, N, Cv, lane);
#endif
}

// The partials of the tiles that gemm_bf16_tile_wdirect_kernel<.., TAIL> split along K, added
// in split order, with the product's epilogue at the tile's place.  Grid (tail tiles, BM / 8):
// a workgroup takes 8 rows of a tile, a thread 8 columns of a row (SwiGLU: 4 gate columns and
// the 4 up columns that belong to them, which lie 16 further on).
template <int BM, int BN, int EPI>
__global__ __launch_bounds__(BN) void tile_tail_reduce_kernel(
    const float* __restrict__ ws, void* __restrict__ Cv, int M, int N, int tiles_m, int tiles_n,
    int whole, int split) {
  static_assert(BN % 32 == 0 && BM % 8 == 0, "a row is BN / 8 threads");
  constexpr int TPR = BN / 8;                        // threads per row
  const int t = blockIdx.x;
  int tm, tn;
  tile_of_workgroup<(BM >= 128 ? 8 : 1024 / BM)>(whole + t, tiles_m, tiles_n, tm, tn);
  const int row = blockIdx.y * 8 + threadIdx.x / TPR, q = threadIdx.x % TPR;
  const int m = tm * BM + row;
  const int c0 = EPI == EPI_SWIGLU ? (q / 4) * 32 + (q % 4) * 4 : q * 8;
  const int c1 = EPI == EPI_SWIGLU ? c0 + 16 : c0 + 4;
  const int n = tn * BN + c0;
  if (m >= M || n >= N) return;
  const float* part = ws + ((size_t)t * split * BM + row) * BN;
  float4 x0 = float4{0.f, 0.f, 0.f, 0.f}, x1 = x0;
  for (int k = 0; k < split; ++k) {
    const float4 p0 = *(const float4*)(part + (size_t)k * BM * BN + c0);
    const float4 p1 = *(const float4*)(part + (size_t)k * BM * BN + c1);
    x0.x += p0.x; x0.y += p0.y; x0.z += p0.z; x0.w += p0.w;
    x1.x += p1.x; x1.y += p1.y; x1.z += p1.z; x1.w += p1.w;
  }
  if (EPI == EPI_SWIGLU) {
    const u32x2_t v = u32x2_t{pack_bf16x2(swiglu_f(x0.x, x1.x), swiglu_f(x0.y, x1.y)),
                              pack_bf16x2(swiglu_f(x0.z, x1.z), swiglu_f(x0.w, x1.w))};
    *(u32x2_t*)((bf16_t*)Cv + (size_t)m * (N / 2) + (n / 32) * 16 + (n % 32)) = v;
  } else if (EPI == EPI_STORE_BF16) {
    *(u32x4_t*)((bf16_t*)Cv + (size_t)m * N + n) =
        u32x4_t{pack_bf16x2(x0.x, x0.y), pack_bf16x2(x0.z, x0.w), pack_bf16x2(x1.x, x1.y),
                pack_bf16x2(x1.z, x1.w)};
  } else {
    float4* dst = (float4*)((float*)Cv + (size_t)m * N + n);
    if (EPI == EPI_ACC_F32) {
      const float4 o0 = dst[0], o1 = dst[1];
      x0 = float4{o0.x + x0.x, o0.y + x0.y, o0.z + x0.z, o0.w + x0.w};
      x1 = float4{o1.x + x1.x, o1.y + x1.y, o1.z + x1.z, o1.w + x1.w};
    }
    dst[0] = x0;
    dst[1] = x1;
  }
}

// ---------------------------------------------------------------- large M: 256-token tiles, one workgroup to a CU
// Tiles of 256 tokens x BN outputs (128, 192 or 256), one workgroup of 4 waves (2 x 2) per
// CU, each wave alone on its SIMD with a tile of 128 x BN / 2 (up to 256 accumulator
// registers).  The kernel above moves (BM + BN) / (BM * BN) bytes per flop from L2 through a
// CU's vector memory path, which at 128 x 256 tiles is as busy as the MFMAs; here it is half
// to two thirds of that, and a wave's 16 MFMAs per k-step of 16 need 8 LDS reads of 16 bytes
// a lane.  Both operands go from memory into LDS by direct-to-LDS loads, k-tiles of 32 in a
// ring of 4 stages (separate arrays, so that the compiler knows which reads wait for which
// copies): the tokens as rows of 64 bytes whose four 16-byte pieces are permuted (piece c
// of row r at place c ^ ((r >> 2) & 3): the 16 rows a quarter wave reads fall into 16
// different groups of banks), W as it lies in the pre-tiled matrix (16 outputs x 8 k are 256
// consecutive bytes).  A step's operands of the first k-step of 16 are read at the end of
// the step before; in the middle of a step the wave waits for the next tile's copies (those
// of the two tiles behind it stay in flight), meets the others (which have then read all of
// this step's tile), and the copies of the tile four ahead begin, into the stage just read.
// A wave issues one instruction at a time, so what is not an MFMA follows single MFMAs,
// evenly spread.  The sums are added in the same order as in the kernels above: the results
// are the same bits.  (Keeping W out of LDS, every wave with its own operands in four
// register sets and the waves side by side, runs at the same speed.)

// which of a k-step's cnt loads follows MFMA m of nm (-1: none)
constexpr int copy_after(int m, int nm, int cnt) {
  for (int d = 0; d < cnt; ++d)
    if (m == (d + 1) * nm / cnt - 1) return d;
  return -1;
}
// how many of the nr operand reads have been issued before MFMA m: one behind every MFMA
// without a load, and those that would be left over at the end behind the first as well
constexpr int reads_before(int m, int nm, int cnt, int nr) {
  int free_slots = 0;
  for (int k = 0; k < nm; ++k) free_slots += copy_after(k, nm, cnt) < 0;
  const int extra = nr > free_slots ? nr - free_slots : 0;
  int done = 0;
  for (int k = 0; k < m && done < nr; ++k)
    if (copy_after(k, nm, cnt) < 0) done += 1 + (k == 0 ? extra : 0);
  return done < nr ? done : nr;
}

template <int BN, int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_tile256_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ Cv, int M,
    int N, int K, int tiles_m, int tiles_n) {
  // (the host pass, which only needs the launch stub, does not know the buffer descriptor type)
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int BM = 256, NT = 256, WM = 128, WN = BN / 2, FM = WM / 32, FN = WN / 32;
  static_assert(BN == 128 || BN == 192 || BN == 256, "tile width");
  constexpr int A_PLACES = BM * 4, W_PLACES = BN * 4;    // 16-byte pieces of a k-tile of 32
  constexpr int A_CHUNKS = A_PLACES / NT, W_CHUNKS = W_PLACES / NT;     // copies per thread
  constexpr int CHUNKS = A_CHUNKS + W_CHUNKS;
  constexpr int PART1 = (CHUNKS + 1) / 2;   // a tile's copies are issued in two parts
  __shared__ u32x4_t stage0[A_PLACES + W_PLACES];
  __shared__ u32x4_t stage1[A_PLACES + W_PLACES];
  __shared__ u32x4_t stage2[A_PLACES + W_PLACES];
  __shared__ u32x4_t stage3[A_PLACES + W_PLACES];
  auto stage_of = [&](auto IDX) __attribute__((always_inline)) -> u32x4_t* {
    constexpr int I = decltype(IDX)::value;
    if constexpr (I == 0) return stage0;
    else if constexpr (I == 1) return stage1;
    else if constexpr (I == 2) return stage2;
    else return stage3;
  };

  int tm, tn;
  tile_of_workgroup<(BM >= 128 ? 8 : 1024 / BM)>(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);        // the LDS address is a scalar

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Sources, as a base all lanes share plus a 32-bit offset per lane.  Tokens: place p =
  // tid + 256 c is row p / 4 = tid / 4 + 64 c, slot p % 4, and takes piece slot ^ ((row >> 2)
  // & 3) of the row's 64 bytes (rows beyond M: the last row).  W copied into LDS: place q =
  // tid + 256 c of the stage's W part is group q / 64 = wave + 4 c of the tile's 16-row
  // groups, and inside it [8-k half h][k-step of 16][output]: lane = 32 h + 16 ks + n; in
  // the pre-tiled matrix a group's 64 k lie as [h][4 k-steps][16 outputs] pieces of 8.
  // W into registers: the operand of column block j, k-step ks: column n = n0 + wn WN + 32 j
  // + lane % 32, half lane / 32.  Groups beyond N are clamped (never stored).
  const char* a_tile = (const char*)(A + (size_t)m0 * K);
  uint32_t asrc[A_CHUNKS];
#pragma unroll
  for (int c = 0; c < A_CHUNKS; ++c) {
    const int row = tid / 4 + 64 * c, piece = (tid % 4) ^ ((tid / 16) & 3);
    asrc[c] = ((uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)K + piece * 8) * 2;
  }
  const int kt64 = K / 64;
  const int grp0 = min(n0 / 16, N / 16 - 1);
  const char* w_tile = (const char*)(W + (size_t)grp0 * kt64 * 1024);
  uint32_t wsrc[W_CHUNKS];
#pragma unroll
  for (int c = 0; c < W_CHUNKS; ++c) {
    const int grp = min(n0 / 16 + wave + 4 * c, N / 16 - 1) - grp0;
    wsrc[c] = ((uint32_t)grp * (uint32_t)kt64 * 1024 +
               ((lane / 32) * 64 + ((lane / 16) % 2) * 16 + lane % 16) * 8) * 2;
  }
  // Where k-tile t (of 32) starts in the tokens' rows and in a group's pre-tiled 64 k, as
  // offsets all lanes share; tiles behind the last one are the last one again.  (t is a
  // multiple of 4 plus a constant, so which half of the 64 k it is is known when compiling.)
  const int ktiles = K / 32, klast = ktiles - 1;
  const uint32_t last_a = (uint32_t)klast * 64, last_w = (uint32_t)(klast / 2) * 2048 + 512;
  struct TileSrc { uint32_t a; uint32_t w; };
  auto tile_src = [&](int base4, auto OFF) __attribute__((always_inline)) -> TileSrc {
    constexpr int off = decltype(OFF)::value;
    const uint32_t oa = min((uint32_t)base4 * 64 + off * 64, last_a);
    const uint32_t ow = min((uint32_t)base4 * 1024 + (off / 2) * 2048 + (off % 2) * 512, last_w);
    return TileSrc{oa, ow};
  };
  // The copies address memory through buffer descriptors (the tile's first token row, the
  // tile's first group of W; no bound that the offsets could reach): base, an offset per
  // lane and one all lanes share, so that a copy costs no address arithmetic and issues
  // faster than one with a 64-bit address per lane.
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)a_tile, 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)w_tile, 0, 0x7fffffff, 0x00020000);
  // copy number q (0 .. CHUNKS - 1) of a k-tile into stage SET
  auto copy_one = [&](TileSrc src, auto SET, auto Q) __attribute__((always_inline)) {
    constexpr int q = decltype(Q)::value;
    u32x4_t* stage = stage_of(SET);
    if constexpr (q < A_CHUNKS)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          a_rsrc, (__attribute__((address_space(3))) void*)(stage + (wave_u * 64 + q * NT)), 16,
          asrc[q], src.a, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          w_rsrc, (__attribute__((address_space(3))) void*)(stage + (A_PLACES + wave_u * 64 +
                                                                    (q - A_CHUNKS) * NT)), 16,
          wsrc[q - A_CHUNKS], src.w, 0, 0);
  };
  // MFMA operands of k-step ks (0, 1) of a stage: tokens of row block i at a_at[ks] + 128 i,
  // outputs of column block j at w_at[ks] + 128 j
  int a_at[2], w_at[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    a_at[ks] = (wm * WM + lane % 32) * 4 + ((2 * ks + lane / 32) ^ (((lane % 32) >> 2) & 3));
    w_at[ks] = A_PLACES + (wn * (WN / 16) + (lane % 32) / 16) * 64 + (lane / 32) * 32 + ks * 16 +
               lane % 16;
  }
  constexpr int NR = FM + FN;       // operand reads from LDS per k-step
  u32x4_t af[2][FM], wf[2][FN];
  // operand read number c of a k-step: the FM token blocks, then the FN output blocks
  auto read_one = [&](const u32x4_t* stage, auto KS, auto C) __attribute__((always_inline)) {
    constexpr int ks = decltype(KS)::value, c = decltype(C)::value;
    if constexpr (c < FM) af[ks][c] = stage[a_at[ks] + c * 128];
    else wf[ks][c - FM] = stage[w_at[ks] + (c - FM) * 128];
  };
  auto reads_from = [&](auto& self, const u32x4_t* stage, auto KS, auto C0, auto CNT)
                        __attribute__((always_inline)) -> void {
    constexpr int c0 = decltype(C0)::value, n = decltype(CNT)::value;
    if constexpr (n > 0) {
      read_one(stage, KS, C0);
      self(self, stage, KS, std::integral_constant<int, c0 + 1>{}, std::integral_constant<int, n - 1>{});
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // loads q0 .. q0 + n - 1 of a tile
  auto copies_from = [&](auto& self, TileSrc src, auto SET, auto Q0, auto CNT)
                         __attribute__((always_inline)) -> void {
    constexpr int q0 = decltype(Q0)::value, n = decltype(CNT)::value;
    if constexpr (n > 0) {
      copy_one(src, SET, Q0);
      self(self, src, SET, std::integral_constant<int, q0 + 1>{}, std::integral_constant<int, n - 1>{});
    }
  };
  auto copies = [&](TileSrc src, auto SET, auto Q0, auto CNT) __attribute__((always_inline)) {
    copies_from(copies_from, src, SET, Q0, CNT);
    __builtin_amdgcn_sched_barrier(0);
  };
  // the loads still in flight behind a tile's own when a step waits for it: two whole tiles
  constexpr int AHEAD = 2 * CHUNKS;
  // (and every LDS read done: the barrier frees this step's stage for the next copies, and
  // the second k-step's operands, read a few MFMAs ago, are only used behind it)
  constexpr int WAIT = 0x0070 | (AHEAD & 15) | ((AHEAD >> 4) << 14);     // vmcnt(AHEAD) lgkmcnt(0)
  // A k-step's FM * FN MFMAs on register set / stage CUR; behind them the other k-step's
  // operand reads (from read_from) and cnt loads of a later tile (from q0 on, into INTO).
  auto half_step = [&](auto KS, TileSrc src, auto INTO, auto Q0, auto CNT,
                       const u32x4_t* read_from, auto READ_KS) __attribute__((always_inline)) {
    constexpr int ks = decltype(KS)::value, q0 = decltype(Q0)::value, cnt = decltype(CNT)::value;
    constexpr int NM = FM * FN;
    auto one = [&](auto MI) __attribute__((always_inline)) {
      constexpr int m = decltype(MI)::value, i = m / FN, j = m % FN;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          *(const bf16x8_t*)&af[ks][i], *(const bf16x8_t*)&wf[ks][j], acc[i][j], 0, 0, 0);
      // Load d follows MFMA (d + 1) * NM / cnt - 1: evenly spread.  The reads follow the
      // first MFMAs that have no load (what does not fit: behind the first as well), so that
      // they have landed when the k-step ends.
      constexpr int d_here = copy_after(m, NM, cnt);
      constexpr int r0 = reads_before(m, NM, cnt, NR), r1 = reads_before(m + 1, NM, cnt, NR);
      reads_from(reads_from, read_from, READ_KS, std::integral_constant<int, r0>{},
                 std::integral_constant<int, r1 - r0>{});
      if constexpr (d_here >= 0)
        copy_one(src, INTO, std::integral_constant<int, q0 + (d_here >= 0 ? d_here : 0)>{});
      __builtin_amdgcn_sched_barrier(0);
    };
    auto run = [&](auto& self, auto MI) __attribute__((always_inline)) -> void {
      constexpr int m = decltype(MI)::value;
      if constexpr (m < NM) {
        one(MI);
        self(self, std::integral_constant<int, m + 1>{});
      }
    };
    run(run, std::integral_constant<int, 0>{});
  };
  // prologue: tiles 0, 1, 2 and the first part of tile 3; tile 0 has landed, its first operands
  copies(tile_src(0, I0{}), I0{}, I0{}, std::integral_constant<int, CHUNKS>{});
  copies(tile_src(0, I1{}), I1{}, I0{}, std::integral_constant<int, CHUNKS>{});
  copies(tile_src(0, I2{}), I2{}, I0{}, std::integral_constant<int, CHUNKS>{});
  copies(tile_src(0, I3{}), I3{}, I0{}, std::integral_constant<int, PART1>{});
  {
    constexpr int A0 = 2 * CHUNKS + PART1;
    __builtin_amdgcn_s_waitcnt(0x0f70 | (A0 & 15) | ((A0 >> 4) << 14));
  }
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  reads_from(reads_from, stage0, I0{}, I0{}, std::integral_constant<int, NR>{});
  // Step base4 + I on stage I.  First half: the first k-step's MFMAs, the second one's
  // operands read, the second part of tile + 3's loads issued (into the stage before this
  // one); then the wait for tile + 1 and the barrier; second half: the second k-step's
  // MFMAs, the next step's first operands read, the first part of tile + 4's loads issued
  // into this step's own stage, which every wave has read by now.
  auto step = [&](int base4, auto IDX) __attribute__((always_inline)) {
    constexpr int I = decltype(IDX)::value;
    using NXT = std::integral_constant<int, (I + 1) % 4>;
    using PRV = std::integral_constant<int, (I + 3) % 4>;
    half_step(I0{}, tile_src(base4, std::integral_constant<int, I + 3>{}), PRV{},
              std::integral_constant<int, PART1>{}, std::integral_constant<int, CHUNKS - PART1>{},
              stage_of(IDX), I1{});
    __builtin_amdgcn_s_waitcnt(WAIT);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    half_step(I1{}, tile_src(base4, std::integral_constant<int, I + 4>{}), IDX, I0{},
              std::integral_constant<int, PART1>{}, stage_of(NXT{}), I0{});
  };
  int kt = 0;         // (K % 128 == 0: the launch sees to it.  No test before the loop, behind
  do {                //  which loads could be moved)
    step(kt, I0{});
    step(kt, I1{});
    step(kt, I2{});
    step(kt, I3{});
    kt += 4;
  } while (kt < ktiles);
  // nothing may still be on its way into LDS when the stages become the epilogue's slabs (a
  // wave's own stage) or the workgroup ends
  __builtin_amdgcn_s_waitcnt(0x0f70);       // vmcnt(0)
  __syncthreads();
  float* slab = (float*)(wave == 0 ? stage0 : wave == 1 ? stage1 : wave == 2 ? stage2 : stage3);
  static_assert(32 * (WN + 4) * sizeof(float) <= (A_PLACES + W_PLACES) * 16 || FN == 3, "slab");
  const int mw = m0 + wm * WM, nw = n0 + wn * WN;
  if constexpr (FN == 3) {
    store_through_slab<FM, 2, 64, EPI, 0, FN>(acc, slab, mw, nw, M, N, Cv, lane);
    store_through_slab<FM, 1, 32, EPI, 2, FN>(acc, slab, mw, nw + 64, M, N, Cv, lane);
  } else {
    store_through_slab<FM, FN, WN, EPI>(acc, slab, mw, nw, M, N, Cv, lane);
  }
#endif
}

template <int BN>
static int launch_tile256(const void* A, const void* W, void* C, int M, int N, int K, int epi,
                          hipStream_t stream) {
  if (N % 16 != 0 || K % 128 != 0) return -3;
  const int tiles_m = (M + 255) / 256, tiles_n = (N + BN - 1) / BN;
  const dim3 grid(tiles_m * tiles_n), block(256);
#define ZF_T256(E)                                                                             \
  hipLaunchKernelGGL((gemm_bf16_tile256_kernel<BN, E>), grid, block, 0, stream,                \
                     (const bf16_t*)A, (const bf16_t*)W, C, M, N, K, tiles_m, tiles_n)
  if (epi == EPI_STORE_BF16) ZF_T256(EPI_STORE_BF16);
  else if (epi == EPI_STORE_F32) ZF_T256(EPI_STORE_F32);
  else if (epi == EPI_SWIGLU) ZF_T256(EPI_SWIGLU);
  else ZF_T256(EPI_ACC_F32);
#undef ZF_T256
  return (int)hipGetLastError();
}

// adds the float32 partials [ksplit, M, N] in split order and applies the epilogue (defined
// with the weight-streaming kernel below)
static int launch_reduce(const void* ws, void* C, int M, int N, int ksplit, int epi,
                         hipStream_t stream);

template <int BM, int BN, int WM, int WN, int TKM = TK, bool W2 = false, bool ADMA = false,
          int KG = 1>
static int launch_tile_wdirect(const void* A, const void* W, void* C, int M, int N, int K, int epi,
                               hipStream_t stream, void* ws = nullptr, int ksplit = 1,
                               bool reduce = true) {
  if (N % 16 != 0 || K % TKM != 0) return -3;
  // every part (and every group of waves in it) an even number of k-tiles
  if (W2 && (K / TKM) % (2 * ksplit * KG) != 0) return -3;
  if (KG > 1 && (K / TKM) % (ksplit * KG) != 0) return -3;      // the groups meet step by step
  if (ksplit > 1 && (ws == nullptr || epi == EPI_SWIGLU || ksplit > K / TKM)) return -3;
  constexpr int NT = (BM / WM) * (BN / WN) * 64 * KG;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const dim3 grid(tiles_m * tiles_n, ksplit), block(NT);
  const int final_epi = epi;
  constexpr size_t stages = (size_t)2 * BM * (TKM + 8) * sizeof(bf16_t);
  constexpr size_t slabs = (size_t)(BM / WM) * (BN / WN) * 32 * (WN + 4) * sizeof(float);
  // two groups: the column blocks handed over (half of every wave's rows, one block)
  constexpr size_t handed = (size_t)KG * (BM / WM) * (BN / WN) * (WM / 64) * 16 * 64 * sizeof(float);
  // (with the tokens copied straight into LDS the stages are arrays of the kernel's own)
  const size_t smem = KG > 1 ? handed : ADMA ? slabs : stages > slabs ? stages : slabs;
  static_assert(KG == 1 || handed >= (size_t)KG * (BM / WM) * (BN / WN) * 32 * 36 * sizeof(float),
                "the slabs of the two groups' waves fit where the blocks are handed over");
#define ZF_WD(E)                                                                              \
  do {                                                                                        \
    auto kern = gemm_bf16_tile_wdirect_kernel<BM, BN, WM, WN, E, TKM, W2, ADMA, false, KG>;   \
    if (smem > 64 * 1024 || KG > 1) {                                                         \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                                   \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                     \
    }                                                                                         \
    hipLaunchKernelGGL(kern, grid, block, smem, stream, (const bf16_t*)A, (const bf16_t*)W, C, \
                       M, N, K, tiles_m, tiles_n, 0, 1, (float*)nullptr);                     \
  } while (0)
  void* const final_c = C;
  if (ksplit > 1) {
    epi = EPI_STORE_F32;
    C = ws;
  }
  if (epi == EPI_STORE_BF16) ZF_WD(EPI_STORE_BF16);
  else if (epi == EPI_STORE_F32) ZF_WD(EPI_STORE_F32);
  else if (epi == EPI_SWIGLU) ZF_WD(EPI_SWIGLU);
  else ZF_WD(EPI_ACC_F32);
#undef ZF_WD
  if (ksplit > 1 && reduce) return launch_reduce(ws, final_c, M, N, ksplit, final_epi, stream);
  return (int)hipGetLastError();
}

// The 128 x 256 tiles with the tile order's tiles from `whole` on shared by `split` workgroups
// each along K (ws: float32 [tiles - whole][split][128][256]) and the kernel that adds their
// partials; every epilogue.
template <bool W2>
static int launch_tile_tail(const void* A, const void* W, void* C, void* ws, int M, int N, int K,
                            int epi, int whole, int split, hipStream_t stream) {
  constexpr int BM = 128, BN = 256, WM = 128, WN = 64, NT = 256;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const long long tiles = (long long)tiles_m * tiles_n;
  if (N % 16 != 0 || K % TK != 0 || ws == nullptr) return -3;
  if (split < 2 || split > K / TK || whole < 0 || whole >= tiles) return -3;
  if (W2 && (K / TK) % (2 * split) != 0) return -3;
  const long long tail = tiles - whole;
  if (whole + tail * split > 0x7fffffffLL) return -3;
  const dim3 grid((unsigned)(whole + tail * split)), block(NT);
  constexpr size_t smem = (size_t)(BM / WM) * (BN / WN) * 32 * (WN + 4) * sizeof(float);
  static_assert(smem <= 64 * 1024, "the slabs fit the default limit");
#define ZF_WT(E)                                                                              \
  do {                                                                                        \
    hipLaunchKernelGGL((gemm_bf16_tile_wdirect_kernel<BM, BN, WM, WN, E, TK, W2, true, true>), \
                       grid, block, smem, stream, (const bf16_t*)A, (const bf16_t*)W, C, M, N, \
                       K, tiles_m, tiles_n, whole, split, (float*)ws);                        \
    hipLaunchKernelGGL((tile_tail_reduce_kernel<BM, BN, E>), dim3((unsigned)tail, BM / 8),    \
                       dim3(BN), 0, stream, (const float*)ws, C, M, N, tiles_m, tiles_n,      \
                       whole, split);                                                         \
  } while (0)
  if (epi == EPI_STORE_BF16) ZF_WT(EPI_STORE_BF16);
  else if (epi == EPI_STORE_F32) ZF_WT(EPI_STORE_F32);
  else if (epi == EPI_SWIGLU) ZF_WT(EPI_SWIGLU);
  else ZF_WT(EPI_ACC_F32);
#undef ZF_WT
  return (int)hipGetLastError();
}

template <int BM, int BN, int WM, int WN, bool WT>
static int launch_tile(const void* A, const void* W, void* C, int M, int N, int K, int epi,
                       hipStream_t stream) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const int nblocks = tiles_m * tiles_n;
  const size_t smem = (size_t)2 * (BM + BN) * LDS_ROW * sizeof(bf16_t);
#define ZF_TILE_LAUNCH(E)                                                                      \
  do {                                                                                         \
    auto kern = gemm_bf16_tile_kernel<BM, BN, WM, WN, E, WT>;                                  \
    if (smem > 64 * 1024) {                                                                    \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                      \
    }                                                                                          \
    hipLaunchKernelGGL(kern, dim3(nblocks), dim3(NT), smem, stream, (const bf16_t*)A,          \
                       (const bf16_t*)W, C, M, N, K, tiles_m, tiles_n);                        \
  } while (0)
  if (epi == EPI_STORE_BF16) ZF_TILE_LAUNCH(EPI_STORE_BF16);
  else if (epi == EPI_STORE_F32) ZF_TILE_LAUNCH(EPI_STORE_F32);
  else if (epi == EPI_SWIGLU) ZF_TILE_LAUNCH(EPI_SWIGLU);
  else ZF_TILE_LAUNCH(EPI_ACC_F32);
#undef ZF_TILE_LAUNCH
  return (int)hipGetLastError();
}

// variant, plain W: 0 = 128x128 (waves 64x64), 4 = 256x256 (waves 128x64, 8 waves);
//          pre-tiled W (w_tiled; N % 16 == 0 and K % 64 == 0), taken straight from memory
//          into the MFMA operands: 6 = 128x128 (waves 64x64), 16 = 128x128 with k-tiles of 128
//          and the waves side by side (128x32: for few tiles; K % 128 == 0), 10 = 128x256
//          (waves 128x64: no two waves load the same part of W, two workgroups share a CU,
//          and W is loaded two k-tiles ahead when their number is even).  10 copies the
//          tokens straight into LDS, and so does 6 from 384 tiles on: with two workgroups to
//          most CUs that was 2 to 18 % faster (qkv at 1024 and 2048 tokens), with one 10 to
//          34 % slower (512 tokens, or 256 tiles at 1024: nothing hides the copies' longer
//          way).  7 and 11 are the tiles of 6 and 10 with the tokens through registers, for
//          comparison.  12 = the tiles of 10 with two groups of four waves in a workgroup,
//          each over half of K (K % 256 == 0): for 256 tiles or fewer, where a CU has one
//          workgroup either way.
extern "C" int zf_gemm_bf16_tile(const void* A, const void* W, void* C, int M, int N, int K,
                                 int epi, int variant, int w_tiled, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K % 8 != 0 || (epi == EPI_SWIGLU && N % 32 != 0)) return -3;
  if (w_tiled) {
    if (N % 16 != 0 || K % 64 != 0) return -3;
    if (variant == 6 && (long long)((M + 127) / 128) * ((N + 127) / 128) >= 384)
      return launch_tile_wdirect<128, 128, 64, 64, TK, false, true>(A, W, C, M, N, K, epi, stream);
    if (variant == 6 || variant == 7)
      return launch_tile_wdirect<128, 128, 64, 64>(A, W, C, M, N, K, epi, stream);
    if (variant == 16)
      return launch_tile_wdirect<128, 128, 128, 32, 128>(A, W, C, M, N, K, epi, stream);
    if (variant == 10) {
      if (K % (2 * TK) == 0)     // W two k-tiles ahead: an even number of k-tiles
        return launch_tile_wdirect<128, 256, 128, 64, TK, true, true>(A, W, C, M, N, K, epi,
                                                                      stream);
      return launch_tile_wdirect<128, 256, 128, 64, TK, false, true>(A, W, C, M, N, K, epi,
                                                                     stream);
    }
    if (variant == 20) return launch_tile256<256>(A, W, C, M, N, K, epi, stream);
    if (variant == 21) return launch_tile256<192>(A, W, C, M, N, K, epi, stream);
    if (variant == 22) return launch_tile256<128>(A, W, C, M, N, K, epi, stream);
    if (variant == 12)         // the tiles of 10 with two groups of waves, each half of K
      return launch_tile_wdirect<128, 256, 128, 64, TK, true, true, 2>(A, W, C, M, N, K, epi,
                                                                       stream);
    if (variant == 11) {       // as 10, the tokens through registers into LDS
      if (K % (2 * TK) == 0)
        return launch_tile_wdirect<128, 256, 128, 64, TK, true>(A, W, C, M, N, K, epi, stream);
      return launch_tile_wdirect<128, 256, 128, 64>(A, W, C, M, N, K, epi, stream);
    }
    return -4;
  }
  switch (variant) {
    case 0: return launch_tile<128, 128, 64, 64, false>(A, W, C, M, N, K, epi, stream);
    case 4: return launch_tile<256, 256, 128, 64, false>(A, W, C, M, N, K, epi, stream);
    default: return -4;
  }
}

// The 128 x 256 tiles of variant 10 on pre-tiled W where the tiles do not end on a whole round
// of the chip: the first `whole` tiles of the tile order run one workgroup each, the rest
// `split` workgroups each along K, so that the last round is as short as its share of the
// work (512 tokens into 34816 outputs, K = 5120: 544 tiles for 512 places, 210 -> 150 us).
// ws: float32 [tiles - whole][split][128][256].
extern "C" int zf_gemm_bf16_tile_tail(const void* A, const void* W, void* C, void* ws, int M,
                                      int N, int K, int epi, int whole, int split,
                                      hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K % 8 != 0 || (epi == EPI_SWIGLU && N % 32 != 0)) return -3;
  if (K % (2 * TK) == 0 && (K / TK) % (2 * split) == 0)
    return launch_tile_tail<true>(A, W, C, ws, M, N, K, epi, whole, split, stream);
  return launch_tile_tail<false>(A, W, C, ws, M, N, K, epi, whole, split, stream);
}

// 17 to 128 tokens on pre-tiled W.  The weight-streaming kernel below re-reads the tokens for
// every 16 * RG rows of W, which at 64 tokens is as much traffic as W itself; here a workgroup
// takes 128 rows of W, its 4 waves side by side along them, the tokens of a k-tile go through
// LDS once for all of them, and the k-tiles are 128 or 256 wide so that 32 or 64 KB of W are
// in flight per workgroup.  ksplit workgroups share a tile's K (ws: float32 [ksplit, M, N])
// when the tiles do not fill the chip.
//   M <= 32: tiles of 32 tokens, K % 256 == 0;  M <= 64: 64 tokens;  M <= 128: 128 tokens;
//   both K % 128 == 0.
// Above 128 tokens: tiles of 64 tokens again, for a few hundred tokens on a narrow output
// whose 128-token tiles would leave most CUs idle (512 tokens into 6144 outputs: 384 tiles
// of 64 x 128 against 192 of 128 x 128, 41 -> 35 us).
extern "C" int zf_gemm_bf16_mid(const void* A, const void* W, void* C, void* ws, int M, int N,
                                int K, int epi, int ksplit, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 1 || (epi == EPI_SWIGLU && N % 32 != 0)) return -3;
  if (M > 128)
    return launch_tile_wdirect<64, 128, 64, 32, 128>(A, W, C, M, N, K, epi, stream, ws, ksplit);
  if (M <= 32)
    return launch_tile_wdirect<32, 128, 32, 32, 256>(A, W, C, M, N, K, epi, stream, ws, ksplit);
  if (M <= 64)
    return launch_tile_wdirect<64, 128, 64, 32, 128>(A, W, C, M, N, K, epi, stream, ws, ksplit);
  return launch_tile_wdirect<128, 128, 128, 32, 128>(A, W, C, M, N, K, epi, stream, ws, ksplit);
}

// The same product for 17 to 128 tokens with ksplit >= 2 workgroups along K, left as float32
// partials [ksplit, M, N] in ws for a kernel of the caller's that adds them on its way.
extern "C" int zf_gemm_bf16_mid_partials(const void* A, const void* W, void* ws, int M, int N,
                                         int K, int ksplit, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 2 || ws == nullptr || M > 128) return -3;
  if (M <= 32)
    return launch_tile_wdirect<32, 128, 32, 32, 256>(A, W, ws, M, N, K, EPI_STORE_F32, stream, ws,
                                                     ksplit, false);
  if (M <= 64)
    return launch_tile_wdirect<64, 128, 64, 32, 128>(A, W, ws, M, N, K, EPI_STORE_F32, stream, ws,
                                                     ksplit, false);
  return launch_tile_wdirect<128, 128, 128, 32, 128>(A, W, ws, M, N, K, EPI_STORE_F32, stream, ws,
                                                     ksplit, false);
}

enum { NORM_NONE = 0, NORM_FOLD = 1, NORM_GIVEN = 2 };

// What the weight-streaming kernel needs to know of an RMSNorm around it.
//   before the product: NORM_FOLD   gain, eps: the rows come as the 32-bit residual stream;
//                       NORM_GIVEN  eps, sq_in [sq_groups][16]: the rows come as
//                                   bfloat16(x * gain) with the sums of x^2 per 16 columns,
//                                   as the kernel that produced x left them (EMIT);
//   after it (EMIT, with the residual epilogue): gain_out, xg_out [M, N], sq_out [N / 16][16]
//                                   for the norm that reads the sum next.
struct SkinnyNorm {
  const float* gain;
  float eps;
  const float* sq_in;
  int sq_groups;
  const float* gain_out;
  bf16_t* xg_out;
  float* sq_out;
};

// The 128 x 128 tiled product on pre-tiled W with ksplit workgroups per tile along K, for
// products whose tiles alone do not fill the chip (a few hundred tokens, a narrow output).
// ws: float32 [ksplit, M, N]; epi: store bf16, store f32 or add into f32.
extern "C" int zf_gemm_bf16_tile_splitk(const void* A, const void* W, void* C, void* ws, int M,
                                        int N, int K, int epi, int ksplit, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 2 || ksplit > 64 || epi == EPI_SWIGLU) return -3;
  if (K % 128 == 0)      // the waves side by side along the outputs: W is loaded once
    return launch_tile_wdirect<128, 128, 128, 32, 128>(A, W, C, M, N, K, epi, stream, ws, ksplit);
  return launch_tile_wdirect<128, 128, 64, 64>(A, W, C, M, N, K, epi, stream, ws, ksplit);
}

// ---------------------------------------------------------------- small M: weight streaming
// For M <= 64 the product is bound by reading W once from HBM.  A workgroup owns 16 * RG rows
// of W (output features) and all M tokens; its 8 waves (times KSPLIT workgroups along
// gridDim.y) split K between them in steps of 64: each lane loads 2 x 16 bytes of one row, 4
// lanes cover a 128-byte line.  W is the first MFMA operand, the tokens (read through L2,
// they are small, and reused for the RG row groups) the second (v_mfma_f32_16x16x32_bf16).
// The waves' partial sums are added through LDS in wave order; with KSPLIT > 1 the
// workgroups write float32 partials to a workspace [KSPLIT, M, N] that
// skinny_reduce_kernel adds in split order.  Nothing depends on timing.  No LDS staging of W:
// nothing of it is reused.
//
// NORM: the tokens come as the float32 residual stream and the RMSNorm before the product is
// folded in.  The product is linear, so  W (x * gain * inv) = inv * W (x * gain): the lanes
// feed bfloat16(x * gain) to the MFMAs, add up x^2 on the way (the workgroup sees all of K
// when there is no split over workgroups), and the epilogue scales each token's sums by
// inv = 1 / sqrt(mean(x^2) + eps), all in 32-bit  (n = x w / sqrt(mean(x^2) + eps),
// src/kernel/core/cpu.zig:38-48 of the reference).
template <int MT, int RG, int EPI, bool WT, int NORM, int NW = 8, bool EMIT = false>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_skinny_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ Cv, int M,
    int N, int K, SkinnyNorm nrm) {
  constexpr int NSS = NORM == NORM_GIVEN ? NW * 4 : NW;
  __shared__ float part[NW][RG * MT][64][4];
  __shared__ float ssum[NSS][MT][16];
  const float* __restrict__ gain = nrm.gain;
  const float eps = nrm.eps;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int n0 = blockIdx.x * (16 * RG);
  const int g = lane / 16;
  // plain layout: row pointer, k added later; pre-tiled: the lane's 16 bytes of chunk 0 of
  // the row group's first tile, tiles of 64 k are 1024 elements apart, chunk 1 is 512 on
  const bf16_t* wrow[RG];
#pragma unroll
  for (int r = 0; r < RG; ++r)
    wrow[r] = WT ? W + (size_t)(n0 / 16 + r) * (K / 64) * 1024 + lane * 8
                 : W + (size_t)min(n0 + r * 16 + lane % 16, N - 1) * K;
  const bf16_t* arow[MT];
  const float* xrow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    arow[t] = A + (size_t)min(t * 16 + lane % 16, M - 1) * K;
    xrow[t] = (const float*)A + (size_t)min(t * 16 + lane % 16, M - 1) * K;
  }
  // lanes of tokens beyond M load nothing and feed zeros
  bool tok[MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    tok[t] = t * 16 + lane % 16 < M;
    ss[t] = 0.f;
  }

  f32x4_t acc[RG][MT];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const u32x4_t zero = u32x4_t{0, 0, 0, 0};
  const int kstride = NW * 64 * gridDim.y;
  int k0 = (blockIdx.y * NW + wave) * 64;
  // What the epilogue reads from memory is asked for now, so that it has arrived when the
  // last weights have: the residual and the next norm's gains (wave 0 writes the outputs of
  // one row group and up to 16 tokens), and the producer's sums of squares.
  constexpr bool PRE_EPI = EMIT && RG * MT == 1;
  float4 pre_c = float4{0.f, 0.f, 0.f, 0.f}, pre_g = float4{0.f, 0.f, 0.f, 0.f};
  if (PRE_EPI && wave == 0 && gridDim.y == 1) {
    const int token = lane % 16, n = n0 + 4 * (lane / 16);
    if (token < M && n + 3 < N) {
      pre_c = *(const float4*)((const float*)Cv + (size_t)token * N + n);
      pre_g = *(const float4*)(nrm.gain_out + n);
    }
  }
  // the producer's sums of squares per 16 columns: thread (p, j) adds groups p, p + NSS, ...
  // of token j; the first SQ_PRE of them are asked for here, before the weights
  constexpr int SQ_PRE = NORM == NORM_GIVEN ? 16 : 1;
  float sqv[SQ_PRE];
  if (NORM == NORM_GIVEN) {
    const int j = tid % 16, p = tid / 16;
#pragma unroll
    for (int i = 0; i < SQ_PRE; ++i) {
      const int gidx = p + i * NSS;
      sqv[i] = gidx < nrm.sq_groups ? nrm.sq_in[gidx * 16 + j] : 0.f;
    }
  }
  if (WT && NORM != NORM_FOLD && (RG * MT == 1 || (RG * MT == 2 && EPI != EPI_SWIGLU))) {
    // Pre-tiled weights (no bounds checks; K % 64 == 0), up to two MFMA tiles per k-step:
    // batches of UNR k-steps in two register sets, the next batch asked for before the
    // MFMAs of the one that has arrived, so that a wave always has loads in flight.  The
    // paths below are laid out so that every wait has a known number of younger loads.
    // (Measured in a replayed graph at 1 and 8 tokens, 4096 x 4096, 4096 x 12288 and
    // 6144 x 4096: 0.1 to 1.0 us less than waiting for each batch before asking for the
    // next; the gate/up product with its three workgroups to a CU loses by it and keeps the
    // plain loop below.)
    constexpr int UNR = RG * MT == 1 ? 4 : 2;
    u32x4_t w0[2][UNR][RG], w1[2][UNR][RG], a0[2][UNR][MT], a1[2][UNR][MT];
    auto load = [&](auto BUF, int kb) {
      constexpr int B = decltype(BUF)::value;
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int kk = kb + u * kstride;
#pragma unroll
        for (int r = 0; r < RG; ++r) {
          const bf16_t* tile = wrow[r] + (size_t)(kk / 64) * 1024;
          w0[B][u][r] = __builtin_nontemporal_load((const u32x4_t*)tile);
          w1[B][u][r] = __builtin_nontemporal_load((const u32x4_t*)(tile + 512));
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          a0[B][u][t] = tok[t] ? *(const u32x4_t*)(arow[t] + kk + g * 16) : zero;
          a1[B][u][t] = tok[t] ? *(const u32x4_t*)(arow[t] + kk + g * 16 + 8) : zero;
        }
      }
    };
    auto compute = [&](auto BUF) {
      constexpr int B = decltype(BUF)::value;
#pragma unroll
      for (int u = 0; u < UNR; ++u)
#pragma unroll
        for (int r = 0; r < RG; ++r)
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *(bf16x8_t*)&w0[B][u][r], *(bf16x8_t*)&a0[B][u][t], acc[r][t], 0, 0, 0);
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                *(bf16x8_t*)&w1[B][u][r], *(bf16x8_t*)&a1[B][u][t], acc[r][t], 0, 0, 0);
          }
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    const int bstride = UNR * kstride;
    // whole batches of this wave: k0 + (nb * UNR - 1) * kstride < K
    const int nb = k0 < K ? ((K - 1 - k0) / kstride + 1) / UNR : 0;
    if (nb > 0) {
      load(B0{}, k0);
      int b = 0;
      for (; b + 2 < nb; b += 2) {
        load(B1{}, k0 + (b + 1) * bstride);
        __builtin_amdgcn_sched_barrier(0);
        compute(B0{});
        __builtin_amdgcn_sched_barrier(0);
        load(B0{}, k0 + (b + 2) * bstride);
        __builtin_amdgcn_sched_barrier(0);
        compute(B1{});
        __builtin_amdgcn_sched_barrier(0);
      }
      if (nb - b == 2) {
        load(B1{}, k0 + (b + 1) * bstride);
        __builtin_amdgcn_sched_barrier(0);
        compute(B0{});
        __builtin_amdgcn_sched_barrier(0);
        compute(B1{});
      } else {
        compute(B0{});
      }
      k0 += nb * bstride;
    }
  }
  for (; k0 < K; k0 += kstride) {
    const int k = k0 + g * 16;
    u32x4_t w0[RG], w1[RG];
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      if (WT) {       // N % 16 == 0 and K % 64 == 0: nothing to clamp, nothing to zero-fill
        const bf16_t* tile = wrow[r] + (size_t)(k0 / 64) * 1024;
        w0[r] = __builtin_nontemporal_load((const u32x4_t*)tile);
        w1[r] = __builtin_nontemporal_load((const u32x4_t*)(tile + 512));
      } else {
        w0[r] = (k < K) ? __builtin_nontemporal_load((const u32x4_t*)(wrow[r] + k)) : zero;
        w1[r] = (k + 8 < K) ? __builtin_nontemporal_load((const u32x4_t*)(wrow[r] + k + 8)) : zero;
      }
    }
    u32x4_t a0[MT], a1[MT];
    if (NORM == NORM_FOLD) {       // K % 64 == 0 here: 16 floats of x and of the gain per lane
      float4 gv[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) gv[c] = *(const float4*)(gain + k + 4 * c);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        float4 xv[4];
#pragma unroll
        for (int c = 0; c < 4; ++c)
          xv[c] = tok[t] ? *(const float4*)(xrow[t] + k + 4 * c) : float4{0.f, 0.f, 0.f, 0.f};
        uint32_t pk[8];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          ss[t] += xv[c].x * xv[c].x + xv[c].y * xv[c].y + xv[c].z * xv[c].z + xv[c].w * xv[c].w;
          pk[2 * c] = pack_bf16x2(xv[c].x * gv[c].x, xv[c].y * gv[c].y);
          pk[2 * c + 1] = pack_bf16x2(xv[c].z * gv[c].z, xv[c].w * gv[c].w);
        }
        a0[t] = u32x4_t{pk[0], pk[1], pk[2], pk[3]};
        a1[t] = u32x4_t{pk[4], pk[5], pk[6], pk[7]};
      }
    } else {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        a0[t] = (tok[t] && k < K) ? *(const u32x4_t*)(arow[t] + k) : zero;
        a1[t] = (tok[t] && k + 8 < K) ? *(const u32x4_t*)(arow[t] + k + 8) : zero;
      }
    }
#pragma unroll
    for (int r = 0; r < RG; ++r)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *(bf16x8_t*)&w0[r], *(bf16x8_t*)&a0[t], acc[r][t], 0, 0, 0);
        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *(bf16x8_t*)&w1[r], *(bf16x8_t*)&a1[t], acc[r][t], 0, 0, 0);
      }
  }
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) part[wave][r * MT + t][lane][e] = acc[r][t][e];
  if (NORM == NORM_FOLD) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float v = ss[t];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      if (lane < 16) ssum[wave][t][lane] = v;
    }
  }
  if (NORM == NORM_GIVEN) {
    // the producer of the rows left sums of squares per 16 columns: [groups][16 tokens];
    // thread (p, j) adds groups p, p + NSS, ... of token j, the rest follows in order of p
    const int j = tid % 16, p = tid / 16;
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < SQ_PRE; ++i) v += sqv[i];
    for (int gidx = p + SQ_PRE * NSS; gidx < nrm.sq_groups; gidx += NSS)
      v += nrm.sq_in[gidx * 16 + j];
    ssum[p][0][j] = v;
  }
  __syncthreads();
  // the token's 1 / sqrt(mean(x^2) + eps): the partial sums in a fixed order
  auto inv_rms = [&](int t, int j) {
    if (NORM == NORM_NONE) return 1.0f;
    float tot = 0.f;
#pragma unroll
    for (int w = 0; w < NSS; ++w) tot += ssum[w][t][j];
    return 1.0f / sqrtf(tot / (float)K + eps);
  };
  if (EPI == EPI_SWIGLU) {
    // row groups alternate gate / up: the pair (2 p, 2 p + 1) gives 16 outputs per token
    for (int item = tid; item < (RG / 2) * MT * 64; item += NW * 64) {
      const int pt = item / 64, l = item % 64;
      const int p = pt / MT, t = pt % MT;
      float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < NW; ++w)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          g[e] += part[w][(2 * p) * MT + t][l][e];
          u[e] += part[w][(2 * p + 1) * MT + t][l][e];
        }
      const int token = t * 16 + l % 16;
      if (token < M) {
        const float inv = inv_rms(t, l % 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int n = n0 / 2 + p * 16 + 4 * (l / 16) + e;      // column of the [M, N / 2] output
          if (2 * n < N)
            ((bf16_t*)Cv)[(size_t)token * (N / 2) + n] =
                float_to_bf16(swiglu_f(g[e] * inv, u[e] * inv));
        }
      }
    }
    return;
  }
  for (int item = tid; item < RG * MT * 64; item += NW * 64) {
    const int rt = item / 64, l = item % 64;
    const int r = rt / MT, t = rt % MT;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < NW; ++w)
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] += part[w][rt][l][e];
    // D[i][j]: i = 4 * (l / 16) + e is the W row (output feature), j = l % 16 the token
    const int token = t * 16 + l % 16;
    float sq = 0.f;
    if (token < M) {
      const float inv = inv_rms(t, l % 16);
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] *= inv;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = n0 + r * 16 + 4 * (l / 16) + e;
        if (n < N) {
          if (gridDim.y > 1) {
            ((float*)Cv)[((size_t)blockIdx.y * M + token) * N + n] = s[e];   // workspace
          } else {
            const size_t off = (size_t)token * N + n;
            if (EPI == EPI_STORE_BF16) {
              ((bf16_t*)Cv)[off] = float_to_bf16(s[e]);
            } else if (EPI == EPI_STORE_F32) {
              ((float*)Cv)[off] = s[e];
            } else {
              const float old = PRE_EPI ? ((const float*)&pre_c)[e] : ((float*)Cv)[off];
              const float v = old + s[e];
              ((float*)Cv)[off] = v;
              if (EMIT) {   // what the RMSNorm after this sum needs: v * gain, and v^2
                const float go = PRE_EPI ? ((const float*)&pre_g)[e] : nrm.gain_out[n];
                nrm.xg_out[off] = float_to_bf16(v * go);
                sq += v * v;
              }
            }
          }
        }
      }
    }
    if (EMIT) {
      // the 16 columns of this row group: 4 per lane, lanes l, l + 16, l + 32, l + 48 of a
      // token; every item is a whole wave here (RG * MT * 64 items, NW * 64 threads)
      sq += __shfl_xor(sq, 16, 64);
      sq += __shfl_xor(sq, 32, 64);
      if (l < 16) nrm.sq_out[(size_t)(n0 / 16 + r) * 16 + l] = sq;
    }
  }
}

// VEC: four outputs a thread with 16-byte loads (M * N a multiple of 4, so that every
// partial starts on a 16-byte boundary); else one output a thread.
template <int EPI, bool VEC>
__global__ void skinny_reduce_kernel(const float* __restrict__ ws, void* __restrict__ Cv,
                                     size_t mn, int ksplit) {
  if (VEC) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= mn) return;
    float4 s = float4{0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < ksplit; ++k) {
      const float4 p = *(const float4*)(ws + (size_t)k * mn + i);
      s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
    }
    if (EPI == EPI_STORE_BF16) {
      *(u32x2_t*)((bf16_t*)Cv + i) = u32x2_t{pack_bf16x2(s.x, s.y), pack_bf16x2(s.z, s.w)};
    } else if (EPI == EPI_STORE_F32) {
      *(float4*)((float*)Cv + i) = s;
    } else {
      float4* dst = (float4*)((float*)Cv + i);
      const float4 old = *dst;
      *dst = float4{old.x + s.x, old.y + s.y, old.z + s.z, old.w + s.w};
    }
    return;
  }
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= mn) return;
  float s = 0.f;
  for (int k = 0; k < ksplit; ++k) s += ws[(size_t)k * mn + i];
  if (EPI == EPI_STORE_BF16)
    ((bf16_t*)Cv)[i] = float_to_bf16(s);
  else if (EPI == EPI_STORE_F32)
    ((float*)Cv)[i] = s;
  else
    ((float*)Cv)[i] += s;
}

static int launch_reduce(const void* ws, void* C, int M, int N, int ksplit, int epi,
                         hipStream_t stream) {
  const size_t mn = (size_t)M * N;
  const bool vec = mn % 4 == 0;
  const unsigned blocks = (unsigned)(((vec ? mn / 4 : mn) + 255) / 256);
#define ZF_REDUCE(E)                                                                           \
  do {                                                                                         \
    if (vec)                                                                                   \
      hipLaunchKernelGGL((skinny_reduce_kernel<E, true>), dim3(blocks), dim3(256), 0, stream,  \
                         (const float*)ws, C, mn, ksplit);                                     \
    else                                                                                       \
      hipLaunchKernelGGL((skinny_reduce_kernel<E, false>), dim3(blocks), dim3(256), 0, stream, \
                         (const float*)ws, C, mn, ksplit);                                     \
  } while (0)
  if (epi == EPI_STORE_BF16) ZF_REDUCE(EPI_STORE_BF16);
  else if (epi == EPI_STORE_F32) ZF_REDUCE(EPI_STORE_F32);
  else if (epi == EPI_ACC_F32) ZF_REDUCE(EPI_ACC_F32);
  else return -3;
#undef ZF_REDUCE
  return (int)hipGetLastError();
}

// The split-K partials of a residual sum whose reader is an RMSNorm: one workgroup per token
// adds the partials in split order into the 32-bit residual row (as skinny_reduce_kernel
// does), keeps the row in registers, and writes the norm of the sum,
// n = x * gain / sqrt(mean(x^2) + eps) (src/kernel/core/cpu.zig:38-48 of the reference), as
// bfloat16: the reduce and the norm kernel in one, the row read once.  N % 4 == 0, N <= 8192
// (8 float4 per thread with 256 threads; wider rows get up to 1024 threads).
__global__ __launch_bounds__(1024) void reduce_sum_norm_kernel(
    const float* __restrict__ ws, float* __restrict__ C, const float* __restrict__ gain,
    bf16_t* __restrict__ normed, int M, int N, int ksplit, float eps) {
  __shared__ float red[16];
  const int m = blockIdx.x, n4 = N / 4, nt = blockDim.x;      // 8 * nt >= n4
  float4* row = (float4*)(C + (size_t)m * N);
  const float4* part = (const float4*)(ws + (size_t)m * N);
  const size_t kstride = (size_t)M * n4;
  float4 v[8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * nt;
    v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c < n4) {
      float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 8
      for (int k = 0; k < ksplit; ++k) {          // independent loads, added in split order
        const float4 p = part[k * kstride + c];
        s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
      }
      const float4 old = row[c];
      v[i] = make_float4(old.x + s.x, old.y + s.y, old.z + s.z, old.w + s.w);
      row[c] = v[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)N + eps);
  bf16_t* o = normed + (size_t)m * N;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * nt;
    if (c < n4) {
      const float4 g = ((const float4*)gain)[c];
      *(u32x2_t*)(o + 4 * c) = u32x2_t{pack_bf16x2(v[i].x * inv * g.x, v[i].y * inv * g.y),
                                       pack_bf16x2(v[i].z * inv * g.z, v[i].w * inv * g.w)};
    }
  }
}

// C += A W^T in 32-bit with ksplit >= 2 workgroups along K, and normed = bfloat16 RMSNorm of
// the sum's rows, from the kernel that adds the partials.  M <= 128: the kernels for 17 to 128
// tokens; above: 128 x 128 tiles.  W pre-tiled; ws: float32 [ksplit, M, N].
extern "C" int zf_gemm_bf16_splitk_sum_norm(const void* A, const void* W, void* C, void* ws,
                                            const float* gain, float eps, void* normed, int M,
                                            int N, int K, int ksplit, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 2 || ksplit > 64 || N % 16 != 0 || N > 8192 || ws == nullptr) return -3;
  int rc;
  if (M <= 32)
    rc = launch_tile_wdirect<32, 128, 32, 32, 256>(A, W, C, M, N, K, EPI_ACC_F32, stream, ws,
                                                   ksplit, false);
  else if (M <= 64)
    rc = launch_tile_wdirect<64, 128, 64, 32, 128>(A, W, C, M, N, K, EPI_ACC_F32, stream, ws,
                                                   ksplit, false);
  else if (K % 128 == 0)
    rc = launch_tile_wdirect<128, 128, 128, 32, 128>(A, W, C, M, N, K, EPI_ACC_F32, stream, ws,
                                                     ksplit, false);
  else
    rc = launch_tile_wdirect<128, 128, 64, 64>(A, W, C, M, N, K, EPI_ACC_F32, stream, ws, ksplit,
                                               false);
  if (rc != 0) return rc;
  // a thread per 4 columns up to 1024 threads: every load of a row is in flight at once
  const int threads = N / 4 >= 1024 ? 1024 : (N / 4 > 256 ? 512 : 256);
  hipLaunchKernelGGL(reduce_sum_norm_kernel, dim3(M), dim3(threads), 0, stream, (const float*)ws,
                     (float*)C, gain, (bf16_t*)normed, M, N, ksplit, eps);
  return (int)hipGetLastError();
}

// The product with 128 x 256 tiles split along K (for a long K on a narrow output at several
// hundred tokens) and the kernel that adds the partials.  (K / 64) % (2 ksplit) == 0; ws:
// float32 [ksplit, M, N]; epi: store bf16, store f32 or add into f32.
extern "C" int zf_gemm_bf16_wide_splitk(const void* A, const void* W, void* C, void* ws, int M,
                                        int N, int K, int epi, int ksplit, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 2 || ksplit > 64 || epi == EPI_SWIGLU || ws == nullptr) return -3;
  return launch_tile_wdirect<128, 256, 128, 64, TK, true, true>(A, W, C, M, N, K, epi, stream, ws,
                                                                ksplit);
}

// The same with 128 x 256 tiles (two workgroups to a CU, no two waves load the same part of
// W): for a long K on a narrow output, where few of these tiles, each split many times, run
// faster than the 128 x 128 tiles.  (K / 64) % (2 ksplit) == 0.
extern "C" int zf_gemm_bf16_wide_splitk_sum_norm(const void* A, const void* W, void* C, void* ws,
                                                 const float* gain, float eps, void* normed,
                                                 int M, int N, int K, int ksplit,
                                                 hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ksplit < 2 || ksplit > 64 || N % 16 != 0 || N > 8192 || ws == nullptr) return -3;
  const int rc = launch_tile_wdirect<128, 256, 128, 64, TK, true, true>(
      A, W, C, M, N, K, EPI_ACC_F32, stream, ws, ksplit, false);
  if (rc != 0) return rc;
  const int threads = N / 4 >= 1024 ? 1024 : (N / 4 > 256 ? 512 : 256);
  hipLaunchKernelGGL(reduce_sum_norm_kernel, dim3(M), dim3(threads), 0, stream, (const float*)ws,
                     (float*)C, gain, (bf16_t*)normed, M, N, ksplit, eps);
  return (int)hipGetLastError();
}

template <int MT, int RG, bool WT, int NORM = NORM_NONE, bool EMIT = false>
static int launch_skinny(const void* A, const void* W, void* C, void* ws, int M, int N, int K,
                         int epi, int ksplit, hipStream_t stream, SkinnyNorm nrm = SkinnyNorm{},
                         bool reduce = true) {
  constexpr int NW = 8;
  const dim3 grid((N + 16 * RG - 1) / (16 * RG), ksplit), block(NW * 64);
  void* dst = ksplit > 1 ? ws : C;
  if (NORM != NORM_NONE && (ksplit != 1 || epi == EPI_ACC_F32)) return -3;
  if (EMIT) {
    if (ksplit != 1 || epi != EPI_ACC_F32) return -3;
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, RG, EPI_ACC_F32, WT, NORM_NONE, NW, true>), grid,
                       block, 0, stream, (const bf16_t*)A, (const bf16_t*)W, dst, M, N, K, nrm);
    return (int)hipGetLastError();
  }
  if (epi == EPI_SWIGLU) {
    if (RG < 2 || ksplit != 1 || N % 32 != 0) return -3;
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, (RG < 2 ? 2 : RG), EPI_SWIGLU, WT, NORM, NW>), grid,
                       block, 0, stream, (const bf16_t*)A, (const bf16_t*)W, dst, M, N, K, nrm);
    return (int)hipGetLastError();
  }
  if (epi == EPI_STORE_BF16)
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, RG, EPI_STORE_BF16, WT, NORM, NW>), grid, block, 0,
                       stream, (const bf16_t*)A, (const bf16_t*)W, dst, M, N, K, nrm);
  else if (epi == EPI_STORE_F32)
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, RG, EPI_STORE_F32, WT, NORM, NW>), grid, block, 0,
                       stream, (const bf16_t*)A, (const bf16_t*)W, dst, M, N, K, nrm);
  else
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<MT, RG, EPI_ACC_F32, WT, NORM_NONE, NW>), grid, block, 0,
                       stream, (const bf16_t*)A, (const bf16_t*)W, dst, M, N, K, nrm);
  if (ksplit > 1 && reduce) return launch_reduce(ws, C, M, N, ksplit, epi, stream);
  return (int)hipGetLastError();
}

// C += A W^T in 32-bit by the weight-streaming kernel with ksplit >= 2 workgroups along K, and
// normed = bfloat16 RMSNorm of the sum's rows from the kernel that adds the partials: for
// narrow outputs whose row groups alone leave CUs idle (320 of them on 256 CUs).  M <= 64,
// W pre-tiled, N a multiple of 16 * rg; ws: float32 [ksplit, M, N].
extern "C" int zf_gemm_bf16_skinny_sum_norm(const void* A, const void* W, void* C, void* ws,
                                            const float* gain, float eps, void* normed, int M,
                                            int N, int K, int rg, int ksplit,
                                            hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || ksplit < 2 || ksplit > 16 || K % 64 != 0 || N % (16 * rg) != 0 || N > 8192 ||
      ws == nullptr)
    return -3;
  const int mt = (M + 15) / 16;
  int rc = -4;
#define ZF_SKS(MT, RG)                                                                         \
  rc = launch_skinny<MT, RG, true>(A, W, C, ws, M, N, K, EPI_ACC_F32, ksplit, stream,          \
                                   SkinnyNorm{}, false)
  if (rg == 1) { if (mt == 1) ZF_SKS(1, 1); else if (mt == 2) ZF_SKS(2, 1); else if (mt == 3) ZF_SKS(3, 1); else ZF_SKS(4, 1); }
  if (rg == 2) { if (mt == 1) ZF_SKS(1, 2); else if (mt == 2) ZF_SKS(2, 2); else if (mt == 3) ZF_SKS(3, 2); else ZF_SKS(4, 2); }
  if (rg == 4) { if (mt == 1) ZF_SKS(1, 4); else if (mt == 2) ZF_SKS(2, 4); else if (mt == 3) ZF_SKS(3, 4); else ZF_SKS(4, 4); }
#undef ZF_SKS
  if (rc != 0) return rc;
  const int threads = N / 4 >= 1024 ? 1024 : (N / 4 > 256 ? 512 : 256);
  hipLaunchKernelGGL(reduce_sum_norm_kernel, dim3(M), dim3(threads), 0, stream, (const float*)ws,
                     (float*)C, gain, (bf16_t*)normed, M, N, ksplit, eps);
  return (int)hipGetLastError();
}

// rg: row groups of 16 per workgroup (1, 2 or 4); ksplit: workgroups along K (1..16), which
// needs a float32 workspace of ksplit * M * N elements when > 1; w_tiled: W is pre-tiled
// (N % 16 == 0, K % 64 == 0, N a multiple of 16 * rg).
extern "C" int zf_gemm_bf16_skinny(const void* A, const void* W, void* C, void* ws, int M, int N,
                                   int K, int epi, int rg, int ksplit, int w_tiled,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K % 8 != 0 || M > 64 || ksplit < 1 || ksplit > 16 || (ksplit > 1 && ws == nullptr))
    return -3;
  const int mt = (M + 15) / 16;
  if (w_tiled && (N % (16 * rg) != 0 || K % 64 != 0)) return -3;
#define ZF_SK(MT, RG)                                                                         \
  return w_tiled ? launch_skinny<MT, RG, true>(A, W, C, ws, M, N, K, epi, ksplit, stream)     \
                 : launch_skinny<MT, RG, false>(A, W, C, ws, M, N, K, epi, ksplit, stream)
  if (rg == 1) { if (mt == 1) ZF_SK(1, 1); if (mt == 2) ZF_SK(2, 1); if (mt == 3) ZF_SK(3, 1); ZF_SK(4, 1); }
  if (rg == 2) { if (mt == 1) ZF_SK(1, 2); if (mt == 2) ZF_SK(2, 2); if (mt == 3) ZF_SK(3, 2); ZF_SK(4, 2); }
  if (rg == 4) { if (mt == 1) ZF_SK(1, 4); if (mt == 2) ZF_SK(2, 4); if (mt == 3) ZF_SK(3, 4); ZF_SK(4, 4); }
#undef ZF_SK
  return -4;
}

// The same product with the RMSNorm before it folded in: X is the float32 residual stream
// [M, K], gain float32 [K]; W must be pre-tiled, M <= 64, no split over workgroups; epi is
// store-bf16, store-f32 or SwiGLU.
extern "C" int zf_norm_gemm_bf16_skinny(const float* X, const float* gain, float eps, const void* W,
                                        void* C, int M, int N, int K, int epi, int rg,
                                        hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  const int mt = (M + 15) / 16;
  if (M > 64 || K % 64 != 0 || N % (16 * rg) != 0 || epi == EPI_ACC_F32) return -3;
  SkinnyNorm nrm{};
  nrm.gain = gain;
  nrm.eps = eps;
#define ZF_NSK(MT, RG) \
  return launch_skinny<MT, RG, true, NORM_FOLD>(X, W, C, nullptr, M, N, K, epi, 1, stream, nrm)
  if (rg == 1) { if (mt == 1) ZF_NSK(1, 1); if (mt == 2) ZF_NSK(2, 1); if (mt == 3) ZF_NSK(3, 1); ZF_NSK(4, 1); }
  if (rg == 2) { if (mt == 1) ZF_NSK(1, 2); if (mt == 2) ZF_NSK(2, 2); if (mt == 3) ZF_NSK(3, 2); ZF_NSK(4, 2); }
  if (rg == 4) { if (mt == 1) ZF_NSK(1, 4); if (mt == 2) ZF_NSK(2, 4); if (mt == 3) ZF_NSK(3, 4); ZF_NSK(4, 4); }
#undef ZF_NSK
  return -4;
}

// The same product for rows that come already multiplied by the norm's gain, as bfloat16
// XG [M <= 16, K], with the sums of squares of the un-normed rows per 16 columns,
// sq [sq_groups][16] (token j of group g at sq[g * 16 + j]), as zf_gemm_bf16_skinny_emit
// leaves them: out = (XG W^T) / sqrt(sum_g sq[g][token] / K + eps).
extern "C" int zf_gemm_bf16_skinny_given(const void* XG, const float* sq, int sq_groups, float eps,
                                         const void* W, void* C, int M, int N, int K, int epi,
                                         int rg, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K % 64 != 0 || N % (16 * rg) != 0 || epi == EPI_ACC_F32 || sq_groups < 1)
    return -3;
  SkinnyNorm nrm{};
  nrm.eps = eps;
  nrm.sq_in = sq;
  nrm.sq_groups = sq_groups;
  if (rg == 1) return launch_skinny<1, 1, true, NORM_GIVEN>(XG, W, C, nullptr, M, N, K, epi, 1, stream, nrm);
  if (rg == 2) return launch_skinny<1, 2, true, NORM_GIVEN>(XG, W, C, nullptr, M, N, K, epi, 1, stream, nrm);
  if (rg == 4) return launch_skinny<1, 4, true, NORM_GIVEN>(XG, W, C, nullptr, M, N, K, epi, 1, stream, nrm);
  return -4;
}

// C += A W^T (C the float32 residual stream [M <= 16, N], W pre-tiled) and, for the RMSNorm
// that reads C next: xg_out [M, N] = bfloat16(C * gain_out), sq_out [N / 16][16] = sums of
// C^2 over each group of 16 columns (tokens beyond M: 0).
extern "C" int zf_gemm_bf16_skinny_emit(const void* A, const void* W, float* C,
                                        const float* gain_out, void* xg_out, float* sq_out, int M,
                                        int N, int K, int rg, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K % 64 != 0 || N % (16 * rg) != 0) return -3;
  SkinnyNorm nrm{};
  nrm.gain_out = gain_out;
  nrm.xg_out = (bf16_t*)xg_out;
  nrm.sq_out = sq_out;
  if (rg == 1) return launch_skinny<1, 1, true, NORM_NONE, true>(A, W, C, nullptr, M, N, K, EPI_ACC_F32, 1, stream, nrm);
  if (rg == 2) return launch_skinny<1, 2, true, NORM_NONE, true>(A, W, C, nullptr, M, N, K, EPI_ACC_F32, 1, stream, nrm);
  return -4;
}

// ---------------------------------------------------------------- measurement: MFMAs alone
// What the matrix cores sustain on given operands with nothing else to do: every wave keeps
// four token operands (32 rows x 16 k each) and two weight operands (32 outputs x 16 k) in
// registers and runs `iters` rounds of the eight 32x32x16 products between them into eight
// accumulators, so that operands change from one instruction to the next as they do in the
// products above.  On operands that toggle the multipliers the chip's power limit, not its
// clock, sets the rate; the rate this reaches is what the tiled products are measured
// against.  src: bfloat16 [6][64][8], operand f of lane l at src[f][l] (a lane holds row or
// output l % 32, k 8 (l / 32) .. + 8); operands 0-3 tokens, 4-5 weights.  The first wave of
// the first workgroup leaves its accumulators in out [8][32][32] (accumulator n = tokens
// n % 4 against weights n / 4: iters times their product).
__global__ __launch_bounds__(256) void mfma_loop_kernel(const u32x4_t* __restrict__ src,
                                                        float* __restrict__ out, int iters) {
  const int lane = threadIdx.x % 64;
  u32x4_t a[4], b[2];
#pragma unroll
  for (int f = 0; f < 4; ++f) a[f] = src[f * 64 + lane];
#pragma unroll
  for (int f = 0; f < 2; ++f) b[f] = src[(4 + f) * 64 + lane];
  f32x16_t acc[8];
#pragma unroll
  for (int n = 0; n < 8; ++n)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[n][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < 8; ++n)
      acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&a[n % 4],
                                                       *(const bf16x8_t*)&b[n / 4], acc[n], 0, 0, 0);
  }
  if (blockIdx.x == 0 && threadIdx.x < 64) {
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        out[(n * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4) * 32 + lane % 32] = acc[n][r];
  } else {
    // (every other wave's sums must count for something, or the compiler drops its loop)
    float s = 0.f;
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[n][r];
    if (s == 1234.5678f && iters < 0) out[0] = s;
  }
}

// workgroups of four waves; 2 * 32 * 32 * 16 * 8 flops a wave and round
extern "C" int zf_mfma_loop(const void* src, float* out, int workgroups, int iters,
                            hipStream_t stream) {
  if (workgroups < 1 || workgroups > 65536 || iters < 1 || iters > (1 << 22)) return 1;
  hipLaunchKernelGGL(mfma_loop_kernel, dim3(workgroups), dim3(256), 0, stream,
                     (const u32x4_t*)src, out, iters);
  ZF_CHECK_LAUNCH();
}
