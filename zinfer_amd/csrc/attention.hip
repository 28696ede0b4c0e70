// Causal grouped-query attention over a paged cache.
//
// The key pool is laid out [page, kv head, row, hd], the value pool [page, kv head, hd, row]
// (rows of a page contiguous); token p of a sequence lies in page
// block_table[seq][p / page_size], row p % page_size.  A token at position p attends to the
// positions lo..p of its own sequence, lo = 0 or p - window + 1 (src/kernel/attention/
// basic.zig:27-76 of the reference: scores scaled after the dot product, softmax with the
// maximum subtracted, values summed in position order; query head h reads kv head h / G).
//
//  * paged_attention_wave: one wave per (token, query head), 64 keys at a time with an
//    online softmax, all in 32-bit.  Its result for a token depends only on that token's own
//    keys, never on how the batch was cut.  Any head size, any page size.
#include <type_traits>

#include "zf_common.h"

template <typename T>
__global__ __launch_bounds__(ZF_WAVE) void paged_attention_wave_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int* __restrict__ block_table, const int* __restrict__ q_start,
    const int* __restrict__ ctx_len, const int* __restrict__ seq_index, T* __restrict__ out,
    float scale, int window, int nH, int nKV, int hd, int page_size, int max_pages) {
  extern __shared__ float smem[];  // q: hd floats, p: 64 floats, acc handled in registers
  float* qs = smem;
  float* ps = smem + hd;
  int* rows = (int*)(ps + ZF_WAVE);  // (page * nKV + kvh) * page_size + row of each key
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = seq_index[t];
  const int q_len = q_start[s + 1] - q_start[s];
  const int pos = ctx_len[s] - q_len + (t - q_start[s]);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int kvh = h / (nH / nKV);
  const int* table = block_table + (size_t)s * max_pages;

  const T* qrow = q + ((size_t)t * nH + h) * hd;
  for (int i = lane; i < hd; i += ZF_WAVE) qs[i] = load_as_float<T>(qrow + i);
  __syncthreads();

  // each lane owns the output elements d = lane, lane + 64, ...  (up to 8 -> hd <= 512)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int base = lo; base <= pos; base += ZF_WAVE) {
    const int key = base + lane;
    float sc = -INFINITY;
    int row = -1;
    if (key <= pos) {
      const int page = table[key / page_size];
      row = (page * nKV + kvh) * page_size + key % page_size;
      const T* kr = k_pool + (size_t)row * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], load_as_float<T>(kr + d), dot);
      sc = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float corr = expf(m - m_new);     // exp(-inf) = 0 on the first chunk
    const float p = (key <= pos) ? expf(sc - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();
    ps[lane] = p;
    rows[lane] = row;
    __syncthreads();
    const int nk = min(ZF_WAVE, pos - base + 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= corr;
    for (int j = 0; j < nk; ++j) {
      const float pj = ps[j];
      const int rj = rows[j];
      const T* vr = v_pool + (size_t)(rj / page_size) * page_size * hd + rj % page_size;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int d = lane + i * ZF_WAVE;
        if (d < hd) acc[i] = fmaf(pj, load_as_float<T>(vr + (size_t)d * page_size), acc[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  T* orow = out + ((size_t)t * nH + h) * hd;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + i * ZF_WAVE;
    if (d < hd) store_from_float<T>(orow + d, acc[i] * inv);
  }
}

extern "C" int zf_paged_attention_wave(const void* q, const void* k_pool, const void* v_pool,
                                       int dtype, const int* block_table, const int* q_start,
                                       const int* ctx_len, const int* seq_index, void* out,
                                       float scale, int window, int T, int nH, int nKV, int hd,
                                       int page_size, int max_pages, hipStream_t stream) {
  if (T <= 0) return 0;
  if (hd > 512 || nKV <= 0 || nH % nKV != 0) return -2;
  dim3 grid(T, nH);
  const size_t smem = (size_t)(hd + 2 * ZF_WAVE) * sizeof(float);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(paged_attention_wave_kernel<float>, grid, dim3(ZF_WAVE), smem, stream,
                       (const float*)q, (const float*)k_pool, (const float*)v_pool, block_table,
                       q_start, ctx_len, seq_index, (float*)out, scale, window, nH, nKV, hd,
                       page_size, max_pages);
  else
    hipLaunchKernelGGL(paged_attention_wave_kernel<bf16_t>, grid, dim3(ZF_WAVE), smem, stream,
                       (const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool,
                       block_table, q_start, ctx_len, seq_index, (bf16_t*)out, scale, window, nH,
                       nKV, hd, page_size, max_pages);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  bfloat16 MFMA kernels.  Both compute the transposed score tile S^T = K Q^T, so that a
//  lane's score registers all belong to one query (its column): the soft-max runs in
//  registers, the probabilities are already in the operand order of the second product
//  O^T = V^T P^T, and the output accumulators of a lane belong to that same query, so the
//  running rescale is a per-lane factor.  K, V and Q go from global memory straight into MFMA
//  operands.  page_size must be a multiple of 16, hd one of 32, 64, 128, 256.  Soft-max in
//  32-bit with exp2 and the scale folded into the exponent.
//
//  Pools these kernels read are in the MFMA operand order ("tiled", written so by
//  qk_norm_rope_kv_write when it is told to): inside the block of one (page, kv head) every
//  group of 16 rows (positions) is stored as the lanes of the decode kernel consume it,
//    keys:    [hd / 32][lane = 16 * ((d % 32) / 8) + row][d % 8]        (1 KB per wave load)
//    values:  [hd / 16][lane = 16 * (row / 4) + d % 16][row % 4]        (512 B per wave load)
//  so that one wave load is consecutive memory instead of 16 pieces of 64 or 32 bytes.
// =====================================================================================
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;

// 2^x for x <= 0 as the bare v_exp_f32 (1 ulp; -inf gives 0, results below 2^-126 may come
// out as 0): exp2f() wraps the same instruction in five more that rescale such tiny results,
// which a soft-max term does not need.
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

// maximum and sum of a value over the two lanes 32 places apart, the same in both
// (v_permlane32_swap leaves the low half's values in one register and the high half's in
// the other: no trip through LDS)
__device__ __forceinline__ float max_of_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_of_halves(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return pack_bf16x2(lo, hi);
}

// keeps elements [n_lo, n_hi) of the 4 bfloat16 in v (element 0 in the low bits), zeroes the rest
__device__ __forceinline__ u32x2_t keep_range4(u32x2_t v, int n_lo, int n_hi) {
  uint64_t x = ((uint64_t)v[1] << 32) | v[0];
  n_lo = max(0, min(4, n_lo));
  n_hi = max(0, min(4, n_hi));
  uint64_t m = 0;
  if (n_hi > n_lo) {
    const uint64_t hi = n_hi == 4 ? ~0ull : ((1ull << (16 * n_hi)) - 1);
    const uint64_t lo = (1ull << (16 * n_lo)) - 1;
    m = hi & ~lo;
  }
  x &= m;
  return u32x2_t{(uint32_t)x, (uint32_t)(x >> 32)};
}

// offsets inside the block of one (page, kv head) of a tiled pool, group of 16 rows `grp`
__device__ __forceinline__ size_t tiled_k_offset(int grp, int r16, int d, int hd) {
  return (size_t)grp * 16 * hd + (d / 32) * 512 + (((d % 32) / 8) * 16 + r16) * 8 + d % 8;
}
__device__ __forceinline__ size_t tiled_v_offset(int grp, int r16, int d, int hd) {
  return (size_t)grp * 16 * hd + (d / 16) * 256 + ((r16 / 4) * 16 + d % 16) * 4 + r16 % 4;
}

// ---------------------------------------------------------------- decode: one query token
// Grid (sequence, kv head, split).  A split is the 256 keys [256 * split, 256 * split + 256)
// of the context, so which keys a split holds depends on the context length only.  Each of
// the workgroup's 4 waves takes 64 of them in one go: all key loads are issued together,
// then all value loads; the soft-max over a wave's 64 scores needs no running rescale.  The
// G query heads of the kv head are the columns of 16x16x32 MFMAs (G <= 16).  The waves'
// partials are combined through LDS in wave order; the workgroup writes one un-normalised
// partial (max, sum, O[G, hd]) that attn_decode_merge_kernel combines in split order.
// Keys and values are read once per step and come as non-temporal loads, which stream about
// a tenth faster here than loads that allocate in the caches; the grid runs kv head first,
// so that workgroups launched together read neighbouring blocks of a page.
#define DEC_SPLIT 256
#define DEC_WAVE_KEYS 64

// The scores of a wave's 64 keys against the G query columns, their soft-max terms and the
// product with the values.  kf, vf and qf are the MFMA operands as the loads leave them; m, l
// and o the wave's maximum, sum and un-normalised output.  One order of operations for every
// kernel that decodes.
//
// PATCH: key kb + pn (0 <= pn < 64; pn < 0: none) is not what kf and vf hold for it but the
// row k_new / v_new in LDS (the token's own key and value, which the cache did not hold yet
// when the loads were asked for).  Its scores come from MFMAs of their own over a tile that
// holds the row in its place, and land in the lanes and registers that hold that key's scores
// anyway: an MFMA's output element depends on its own row and column alone, so the scores, and
// with them everything after, are the bits that operands read from the cache would give.
template <int HD, bool PATCH = false>
__device__ __forceinline__ void decode_attend(const u32x4_t (&kf)[4][HD / 32],
                                              const u32x2_t (&vf)[4][HD / 16],
                                              const bf16x8_t (&qf)[HD / 32], int kb, int k_begin,
                                              int k_end, int qd, float scale_log2e, float& m,
                                              float& l, f32x4_t (&o)[HD / 16], int pn = -1,
                                              const bf16_t* k_new = nullptr,
                                              const bf16_t* v_new = nullptr) {
  f32x4_t st[4];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    st[h] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int stp = 0; stp < HD / 32; ++stp)
      st[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&kf[h][stp], qf[stp],
                                                      st[h], 0, 0, 0);
  }
  const int hn = pn / 16, jn = pn % 16, lane16 = threadIdx.x % 16;
  if constexpr (PATCH) {
    if (pn >= 0) {
      // lane (j, qd) holds of a 16-key tile the row j, elements 32 stp + 8 qd .. + 7
      f32x4_t sn = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int stp = 0; stp < HD / 32; ++stp) {
        u32x4_t kx = *(const u32x4_t*)(k_new + stp * 32 + 8 * qd);
        if (lane16 != jn) kx = u32x4_t{0, 0, 0, 0};
        sn = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8_t*)&kx, qf[stp], sn, 0, 0, 0);
      }
      // its scores: element jn % 4 of the lanes with qd = jn / 4, in group hn
#pragma unroll
      for (int h = 0; h < 4; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (h == hn && r == jn % 4 && qd == jn / 4) st[h][r] = sn[r];
    }
  }
  // st[h][r]: key kb + 16 h + 4 qd + r, query column j
  float sc[16];
#pragma unroll
  for (int h = 0; h < 4; ++h)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = kb + 16 * h + 4 * qd + r;
      const float v = (key >= k_begin && key < k_end) ? st[h][r] * scale_log2e : -INFINITY;
      sc[h * 4 + r] = v;
      m = fmaxf(m, v);
    }
  m = fmaxf(m, __shfl_xor(m, 16, 64));
  m = fmaxf(m, __shfl_xor(m, 32, 64));
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    sc[e] = exp2_raw(sc[e] - m);
    l += sc[e];
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {     // two MFMAs of 32 keys: groups 2 hh and 2 hh + 1
    u32x4_t pk = u32x4_t{pack_bf16(sc[8 * hh + 0], sc[8 * hh + 1]),
                         pack_bf16(sc[8 * hh + 2], sc[8 * hh + 3]),
                         pack_bf16(sc[8 * hh + 4], sc[8 * hh + 5]),
                         pack_bf16(sc[8 * hh + 6], sc[8 * hh + 7])};
    const bf16x8_t pf = *(bf16x8_t*)&pk;
    const int b0 = kb + 32 * hh + 4 * qd, b1 = b0 + 16;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      // stale or poisoned rows outside [k_begin, k_end) are zeroed: 0 * NaN would spoil the sum
      u32x2_t v0 = keep_range4(vf[2 * hh][dt], k_begin - b0, k_end - b0);
      u32x2_t v1 = keep_range4(vf[2 * hh + 1][dt], k_begin - b1, k_end - b1);
      if constexpr (PATCH) {
        // the lanes with qd = jn / 4 hold the values of keys 4 qd .. 4 qd + 3 at head
        // element 16 dt + j, 16 bits each
        if (pn >= 0 && hn / 2 == hh && qd == jn / 4) {
          const uint32_t vn = v_new[16 * dt + lane16];
          u32x2_t& v = hn % 2 ? v1 : v0;
          const int w = (jn % 4) / 2, sh = 16 * (jn % 2);
          v[w] = (v[w] & ~(0xffffu << sh)) | (vn << sh);
        }
      }
      u32x4_t vv = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(bf16x8_t*)&vv, pf, o[dt], 0, 0, 0);
    }
  }
}

// The four waves' partials combined through LDS in wave order; the workgroup writes one
// un-normalised partial (max, sum, O[G, hd]) per query head for its split.  With one split
// (no context beyond 256 keys) it writes the output itself, out_row[col * HD + d] =
// bfloat16(O / sum): what the merge kernel would make of a single partial, bit for bit, and
// that kernel is not launched.
template <int HD>
__device__ __forceinline__ void decode_write_partial(float (&s_o)[4][16][HD], float (&s_m)[4][16],
                                                     float (&s_l)[4][16], int wave, int j, int qd,
                                                     float m, float l,
                                                     const f32x4_t (&o)[HD / 16], int G,
                                                     size_t first_slot, int max_splits,
                                                     float* __restrict__ ws_o,
                                                     float* __restrict__ ws_ml,
                                                     bf16_t* __restrict__ out_row) {
  // this wave's partial for query column j: rows d = 16 dt + 4 qd + r
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) *(f32x4_t*)&s_o[wave][j][dt * 16 + 4 * qd] = o[dt];
  if (qd == 0) {
    s_m[wave][j] = m;
    s_l[wave][j] = l;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < G * HD; idx += 256) {
    const int col = idx / HD, d = idx % HD;
    float mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mx = fmaxf(mx, s_m[w][col]);
    float acc = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(s_m[w][col] - mx);     // a wave without keys has max -inf: weight 0
      acc += f * s_o[w][col][d];
      den += f * s_l[w][col];
    }
    if (max_splits == 1) {
      out_row[idx] = float_to_bf16(acc / den);
      continue;
    }
    const size_t slot = first_slot + (size_t)col * max_splits;   // of (sequence, head, split)
    ws_o[slot * HD + d] = acc;
    if (d == 0) {
      ws_ml[slot * 2] = mx;
      ws_ml[slot * 2 + 1] = den;
    }
  }
}

template <int HD>
__global__ __launch_bounds__(256) void attn_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, bf16_t* __restrict__ out, float scale_log2e, int window, int nH,
    int nKV, int ps, int max_pages, int max_splits) {
  __shared__ __attribute__((aligned(16))) float s_o[4][16][HD];
  __shared__ float s_m[4][16], s_l[4][16];
  const int kvh = blockIdx.x, sp = blockIdx.y, s = blockIdx.z;
  if (q_start[s + 1] - q_start[s] != 1) return;
  const int ctx = ctx_len[s], pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (max(lo, sp * DEC_SPLIT) >= min(ctx, (sp + 1) * DEC_SPLIT)) return;   // whole workgroup
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, j = lane % 16, qd = lane / 16;
  const int kb = sp * DEC_SPLIT + wave * DEC_WAVE_KEYS;
  const int k_begin = max(lo, kb), k_end = min(ctx, kb + DEC_WAVE_KEYS);
  const int G = nH / nKV;
  const int t = q_start[s];
  const int* table = block_table + (size_t)s * max_pages;
  float m = -INFINITY, l = 0.f;
  f32x4_t o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (k_begin < k_end) {
    // the four 16-key groups of this wave; a group outside [k_begin, k_end) may have no page
    // at all: it reads the group of a key that certainly exists and is masked
    const bf16_t* kg[4];
    const bf16_t* vg[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const int base = kb + 16 * h;
      const bool any = base < k_end && base + 16 > k_begin;
      const int key = any ? base : (k_begin / 16) * 16;
      const size_t blk = (((size_t)table[key / ps] * nKV + kvh) * ps + (key % ps)) * HD;
      kg[h] = k_pool + blk + lane * 8;
      vg[h] = v_pool + blk + lane * 4;
    }
    u32x4_t kf[4][HD / 32];
#pragma unroll
    for (int h = 0; h < 4; ++h)
#pragma unroll
      for (int stp = 0; stp < HD / 32; ++stp)
        kf[h][stp] = __builtin_nontemporal_load((const u32x4_t*)(kg[h] + stp * 512));
    bf16x8_t qf[HD / 32];
    {
      const bf16_t* qrow = q + ((size_t)t * nH + kvh * G + min(j, G - 1)) * HD + 8 * qd;
#pragma unroll
      for (int st = 0; st < HD / 32; ++st) {
        u32x4_t v = *(const u32x4_t*)(qrow + st * 32);
        if (j >= G) v = u32x4_t{0, 0, 0, 0};
        qf[st] = *(bf16x8_t*)&v;
      }
    }
    // values: lane (d % 16 = j, keys 4 qd .. 4 qd + 3) of head-element tile dt
    u32x2_t vf[4][HD / 16];
#pragma unroll
    for (int h = 0; h < 4; ++h)
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt)
        vf[h][dt] = __builtin_nontemporal_load((const u32x2_t*)(vg[h] + dt * 256));
    decode_attend<HD>(kf, vf, qf, kb, k_begin, k_end, qd, scale_log2e, m, l, o);
  }
  decode_write_partial<HD>(s_o, s_m, s_l, wave, j, qd, m, l, o, G,
                           ((size_t)s * nH + kvh * G) * max_splits + sp, max_splits, ws_o, ws_ml,
                           out + ((size_t)t * nH + kvh * G) * HD);
}

// What the fused decode kernel needs to do the work of the kernel before it as well (the
// per-head norm of q and k, their rotation, the new key and value into the cache).
struct DecodeFused {
  const float* q_gain;      // null: no norm
  const float* k_gain;
  float eps;
  const float* cos_t;       // [positions, hd / 2], null: no rotation
  const float* sin_t;
  const int* positions;     // [n_seqs]
  const int* slot_mapping;  // [n_seqs]: page * page_size + row of the token's own key and value
  int table_rows;           // positions the tables hold
};

// A decode step's attention from the q/k/v product's rows [n_seqs, (nH + 2 nKV) * hd], which
// it only reads: every sequence has one token, token s is sequence s's.  Grid, splits and the
// arithmetic of the attention are attn_decode_kernel's.  Before it, a workgroup norms and
// rotates its kv head's G query rows itself (into LDS, rounded to bfloat16 as the separate
// kernel leaves them in memory; every split's workgroup repeats these few hundred flops), and
// the workgroup whose split holds the token's own position does the same for the new key and
// stores it and the new value in the cache.
//
// Order.  A lane's loads return in the order it asked for them, so whatever the norm and
// rotation need from memory is asked for first and the keys right behind it: the arithmetic
// then runs while the keys' loads are in flight and waits for none of them.  At head size 128
// half of the values are asked for with the keys and half behind the arithmetic (with all 48
// loads in flight beside what the norm holds, three waves would no longer fit a SIMD's
// registers); they are needed last.  The wave that holds the token's own position cannot
// read it from the cache (the stores come later than its loads): decode_attend takes the new
// key and value from LDS instead (PATCH).
//
// The page of a 16-key group is the same for a whole wave, so the look-ups and the blocks'
// addresses are scalar and a load's address is one of them plus a lane's offset: the loads
// hold no address registers, which leaves room for what the norm holds meanwhile.
template <int HD>
__global__ __launch_bounds__(256, HD <= 128 ? 3 : 1) void attn_decode_fused_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ k_pool, bf16_t* __restrict__ v_pool,
    const int* __restrict__ block_table, const int* __restrict__ ctx_len,
    float* __restrict__ ws_o, float* __restrict__ ws_ml, bf16_t* __restrict__ out,
    float scale_log2e, int window, int nH, int nKV, int ps, int max_pages, int max_splits,
    DecodeFused fu) {
  __shared__ __attribute__((aligned(16))) float s_o[4][16][HD];
  __shared__ float s_m[4][16], s_l[4][16];
  // rows 0 .. G - 1: the query heads; row 16: the new key; row 17: the new value
  __shared__ __attribute__((aligned(16))) bf16_t s_q[18][HD + 8];
  const int kvh = blockIdx.x, sp = blockIdx.y, s = blockIdx.z;
  const int ctx = ctx_len[s], pos = ctx - 1;
  const int slot = fu.slot_mapping[s];
  // (a position beyond the tables reads their last row: wrong, but no access out of bounds)
  const int rope_pos = fu.cos_t ? min(max(fu.positions[s], 0), fu.table_rows - 1) : 0;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  if (max(lo, sp * DEC_SPLIT) >= min(ctx, (sp + 1) * DEC_SPLIT)) return;   // whole workgroup
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int lane = threadIdx.x % 64, j = lane % 16, qd = lane / 16;
  const int kb = sp * DEC_SPLIT + wave * DEC_WAVE_KEYS;
  const int k_begin = max(lo, kb), k_end = min(ctx, kb + DEC_WAVE_KEYS);
  const bool has_keys = k_begin < k_end;
  const int G = nH / nKV;
  const int* table = block_table + (size_t)s * max_pages;

  // LPH lanes to a head, 8 elements each; the workgroup takes HEADS heads at a time.  Item
  // i < G is query head kvh * G + i, item G the new key (where the split holds the token's
  // own position).
  constexpr int LPH = HD / 8, HEADS = 256 / LPH;
  constexpr int V_EARLY = HD == 128 ? 2 : 4;      // groups whose values are asked for with the keys
  const int li = threadIdx.x % LPH;
  const bool own = pos / DEC_SPLIT == sp;
  const int items = own ? G + 1 : G;
  const int row_width = (nH + 2 * nKV) * HD;
  const bf16_t* row = qkv + (size_t)s * row_width;
  struct Item {
    u32x2_t raw0, raw1;
    HeadCoef cf;
    bool active, is_q;
  };
  auto fetch = [&](int item) {
    Item it;
    it.active = item < items;
    it.is_q = item < G;
    const int head = !it.active ? 0 : it.is_q ? kvh * G + item : nH + kvh;
    it.raw0 = *(const u32x2_t*)(row + (size_t)head * HD + 4 * li);
    it.raw1 = *(const u32x2_t*)(row + (size_t)head * HD + HD / 2 + 4 * li);
    load_head_coef(it.cf, li, HD, it.is_q ? fu.q_gain : fu.k_gain, fu.cos_t, fu.sin_t, rope_pos);
    return it;
  };
  const Item first = fetch(threadIdx.x / LPH);
  u32x4_t v_new = u32x4_t{0, 0, 0, 0};
  if (own && threadIdx.x < HD / 8)      // the new value: 8 elements a lane
    v_new = *(const u32x4_t*)(row + (size_t)(nH + nKV + kvh) * HD + 8 * threadIdx.x);

  u32x4_t kf[4][HD / 32];
  u32x2_t vf[4][HD / 16];
  size_t blk[4] = {0, 0, 0, 0};
  if (has_keys) {
    // the four 16-key groups of this wave; a group outside [k_begin, k_end) may have no page
    // at all: it reads the group of a key that certainly exists and is masked
    // (the four look-ups are scalar loads: asked for together, waited for once)
    int key_of[4], page_of[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const int base = kb + 16 * h;
      const bool any = base < k_end && base + 16 > k_begin;
      key_of[h] = any ? base : (k_begin / 16) * 16;
    }
#pragma unroll
    for (int h = 0; h < 4; ++h) page_of[h] = table[key_of[h] / ps];
#pragma unroll
    for (int h = 0; h < 4; ++h)
      blk[h] = (((size_t)page_of[h] * nKV + kvh) * ps + (key_of[h] % ps)) * HD;
#pragma unroll
    for (int h = 0; h < 4; ++h)
#pragma unroll
      for (int stp = 0; stp < HD / 32; ++stp)
        kf[h][stp] = __builtin_nontemporal_load(
            (const u32x4_t*)(k_pool + blk[h] + stp * 512) + lane);
#pragma unroll
    for (int h = 0; h < V_EARLY; ++h)
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt)
        vf[h][dt] = __builtin_nontemporal_load(
            (const u32x2_t*)(v_pool + blk[h] + dt * 256) + lane);
  }
  // (nothing below may move above the loads, and none of them below it)
  __builtin_amdgcn_sched_barrier(0);

  const int page = slot / ps, r = slot % ps;
  // the block of the token's 16-row group in the pools
  const size_t grp_at = (((size_t)page * nKV + kvh) * ps + (r / 16) * 16) * HD;
  auto finish = [&](int item, const Item& it) {
    float x0[4], x1[4];
    const u32x2_t a = it.active ? it.raw0 : u32x2_t{0, 0}, b = it.active ? it.raw1 : u32x2_t{0, 0};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x0[e] = bf16_to_float((bf16_t)(a[e / 2] >> (16 * (e % 2))));
      x1[e] = bf16_to_float((bf16_t)(b[e / 2] >> (16 * (e % 2))));
    }
    head_norm_rotate<LPH>(x0, x1, HD, it.active, fu.eps, it.cf);
    if (!it.active) return;
    const u32x2_t y0 = u32x2_t{pack_bf16x2(x0[0], x0[1]), pack_bf16x2(x0[2], x0[3])};
    const u32x2_t y1 = u32x2_t{pack_bf16x2(x1[0], x1[1]), pack_bf16x2(x1[2], x1[3])};
    bf16_t* dst = s_q[it.is_q ? item : 16];
    *(u32x2_t*)(dst + 4 * li) = y0;
    *(u32x2_t*)(dst + HD / 2 + 4 * li) = y1;
    if (!it.is_q) {    // element d of row r at [d / 32][16 ((d % 32) / 8) + r % 16][d % 8]
      bf16_t* grp = k_pool + grp_at;
      const int d0 = 4 * li, d1 = HD / 2 + 4 * li;
      *(u32x2_t*)(grp + (d0 / 32) * 512 + (((d0 % 32) / 8) * 16 + r % 16) * 8 + d0 % 8) = y0;
      *(u32x2_t*)(grp + (d1 / 32) * 512 + (((d1 % 32) / 8) * 16 + r % 16) * 8 + d1 % 8) = y1;
    }
  };
  finish(threadIdx.x / LPH, first);
  // (more than HEADS items: 16 query heads to a kv head, or head size 256 with more than 7;
  // these loads queue behind the keys and values)
  for (int it0 = HEADS; it0 < items; it0 += HEADS) {
    const Item it = fetch(it0 + threadIdx.x / LPH);
    finish(it0 + threadIdx.x / LPH, it);
  }
  if (own && threadIdx.x < HD / 8) {
    *(u32x4_t*)(s_q[17] + 8 * threadIdx.x) = v_new;
    // element d of row r at [d / 16][16 (r % 16 / 4) + d % 16][r % 4]
    bf16_t* grp = v_pool + grp_at + ((r % 16) / 4) * 64 + r % 4;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = 8 * threadIdx.x + i;
      grp[(d / 16) * 256 + (d % 16) * 4] = (bf16_t)(v_new[i / 2] >> (16 * (i % 2)));
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  if (has_keys) {
#pragma unroll
    for (int h = V_EARLY; h < 4; ++h)
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt)
        vf[h][dt] = __builtin_nontemporal_load(
            (const u32x2_t*)(v_pool + blk[h] + dt * 256) + lane);
  }
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  f32x4_t o[HD / 16];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  if (has_keys) {
    bf16x8_t qf[HD / 32];
#pragma unroll
    for (int st = 0; st < HD / 32; ++st) {
      u32x4_t v = *(const u32x4_t*)(s_q[min(j, G - 1)] + st * 32 + 8 * qd);
      if (j >= G) v = u32x4_t{0, 0, 0, 0};
      qf[st] = *(bf16x8_t*)&v;
    }
    const int pn = (pos >= kb && pos < kb + DEC_WAVE_KEYS) ? pos - kb : -1;
    decode_attend<HD, true>(kf, vf, qf, kb, k_begin, k_end, qd, scale_log2e, m, l, o, pn,
                            s_q[16], s_q[17]);
  }
  decode_write_partial<HD>(s_o, s_m, s_l, wave, j, qd, m, l, o, G,
                           ((size_t)s * nH + kvh * G) * max_splits + sp, max_splits, ws_o, ws_ml,
                           out + ((size_t)s * nH + kvh * G) * HD);
}

// Combines the splits of one (sequence, head) and writes bfloat16.  One workgroup of 4 waves.
// A split's partial output is hd floats in a row: hd / 4 lanes take it as one 16-byte load
// each, so a wave load covers 256 / hd splits and the workgroup's 4 waves 1024 / hd splits
// ("slots"); slot j takes the splits first + j, first + j + slots, ... with 8 loads in
// flight: 128 splits of a 32 K context are two trips to memory (one wave of 8 loads over
// all of them took sixteen: 26 us, more than the attention kernel before it).  The first
// loads do not wait for the weights: they are asked for together with the (max, sum) pairs.
// Sums are added slot by slot and the slots in a fixed order, which the context length
// alone decides.
template <int HD>
__global__ __launch_bounds__(256) void attn_decode_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    int window, int nH, int max_splits) {
  constexpr int LPS = HD / 4;            // lanes per split
  constexpr int SLOTS = 256 / LPS;       // splits the workgroup takes at a time
  constexpr int U = 8;                   // loads in flight per lane
  __shared__ float red[4];
  __shared__ __attribute__((aligned(16))) float part[SLOTS][HD];
  __shared__ float part_den[SLOTS];
  const int s = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  if (q_start[s + 1] - q_start[s] != 1) return;
  const int ctx = ctx_len[s], pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first = lo / DEC_SPLIT, last = pos / DEC_SPLIT;
  const size_t base = ((size_t)s * nH + head) * max_splits;
  const int slot = tid / LPS, piece = tid % LPS;
  const f32x4_t* src = (const f32x4_t*)(ws_o + base * HD) + piece;     // + split * LPS
  // the first U splits of this slot, before the weights are known
  f32x4_t v[U];
  float2 ml[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int sp = min(first + slot + u * SLOTS, last);
    v[u] = src[(size_t)sp * LPS];
    ml[u] = *(const float2*)(ws_ml + (base + sp) * 2);
  }
  float mx = -INFINITY;
  for (int sp = first + tid; sp <= last; sp += 256) mx = fmaxf(mx, ws_ml[(base + sp) * 2]);
  mx = wave_max(mx);
  if (tid % 64 == 0) red[tid / 64] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float den = 0.f;
  for (int sp0 = first + slot; sp0 <= last; sp0 += U * SLOTS) {
    if (sp0 != first + slot) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int sp = min(sp0 + u * SLOTS, last);
        v[u] = src[(size_t)sp * LPS];
        ml[u] = *(const float2*)(ws_ml + (base + sp) * 2);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float w = (sp0 + u * SLOTS <= last) ? exp2f(ml[u].x - mx) : 0.f;
      den = fmaf(w, ml[u].y, den);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(w, v[u][e], acc[e]);
    }
  }
  *(f32x4_t*)&part[slot][4 * piece] = acc;
  if (piece == 0) part_den[slot] = den;
  __syncthreads();
  if (tid < HD) {
    float o = 0.f, denom = 0.f;
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) {
      o += part[j][tid];
      denom += part_den[j];
    }
    out[((size_t)q_start[s] * nH + head) * HD + tid] = float_to_bf16(o / denom);
  }
}

// ws_o: n_seqs * nH * max_splits * hd floats, ws_ml: n_seqs * nH * max_splits * 2 floats,
// max_splits >= ceil(longest context / 256); the pools are tiled.
static int launch_decode_merge(const float* ws_o, const float* ws_ml, const int* q_start,
                               const int* ctx_len, void* out, int window, int n_seqs, int nH,
                               int hd, int max_splits, hipStream_t stream) {
  if (max_splits == 1) return (int)hipGetLastError();     // the attention kernel wrote the output
#define ZF_DEC_MERGE(HD)                                                                        \
  hipLaunchKernelGGL(attn_decode_merge_kernel<HD>, dim3(n_seqs, nH), dim3(256), 0, stream, ws_o, \
                     ws_ml, q_start, ctx_len, (bf16_t*)out, window, nH, max_splits)
  if (hd == 32) ZF_DEC_MERGE(32);
  else if (hd == 64) ZF_DEC_MERGE(64);
  else if (hd == 128) ZF_DEC_MERGE(128);
  else ZF_DEC_MERGE(256);
#undef ZF_DEC_MERGE
  ZF_CHECK_LAUNCH();
}

extern "C" int zf_attn_decode_bf16(const void* q, const void* k_pool, const void* v_pool,
                                   const int* block_table, const int* q_start,
                                   const int* ctx_len, void* out, float* ws_o, float* ws_ml,
                                   float scale, int window, int n_seqs, int nH, int nKV, int hd,
                                   int page_size, int max_pages, int max_splits,
                                   hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (page_size % 16 != 0 || nKV <= 0 || nH % nKV != 0 || nH / nKV > 16) return -2;
  const float scale_log2e = scale * 1.4426950408889634f;
  dim3 grid(nKV, max_splits, n_seqs);
#define ZF_DEC(HD)                                                                              \
  hipLaunchKernelGGL(attn_decode_kernel<HD>, grid, dim3(256), 0, stream, (const bf16_t*)q,      \
                     (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_table, q_start,        \
                     ctx_len, ws_o, ws_ml, (bf16_t*)out, scale_log2e, window, nH, nKV,          \
                     page_size, max_pages, max_splits)
  if (hd == 32) ZF_DEC(32);
  else if (hd == 64) ZF_DEC(64);
  else if (hd == 128) ZF_DEC(128);
  else if (hd == 256) ZF_DEC(256);
  else return -2;
#undef ZF_DEC
  return launch_decode_merge(ws_o, ws_ml, q_start, ctx_len, out, window, n_seqs, nH, hd,
                             max_splits, stream);
}

// A decode step's attention from the q/k/v product's own rows: every sequence has one token,
// token s is sequence s's (q_start is 0, 1, ..., n_seqs).  qkv [n_seqs, (nH + 2 nKV) * hd]
// bfloat16 is read, not changed; the per-head RMSNorm of q and k (gains float32 [hd], or
// both null), their rotation (tables float32 [*, hd / 2] read at positions[s], or both null)
// and the write of the token's key and value into the tiled pools at slot_mapping[s] (the
// slot of position ctx_len[s] - 1) happen inside the attention kernel, with the arithmetic
// of zf_qk_norm_rope_kv_write.
extern "C" int zf_attn_decode_fused_bf16(const void* qkv, const float* q_gain,
                                         const float* k_gain, float eps, const float* cos_t,
                                         const float* sin_t, int table_rows,
                                         const int* positions,
                                         const int* slot_mapping, void* k_pool, void* v_pool,
                                         const int* block_table, const int* q_start,
                                         const int* ctx_len, void* out, float* ws_o,
                                         float* ws_ml, float scale, int window, int n_seqs,
                                         int nH, int nKV, int hd, int page_size, int max_pages,
                                         int max_splits, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  if (page_size % 16 != 0 || nKV <= 0 || nH % nKV != 0 || nH / nKV > 16) return -2;
  if ((q_gain == nullptr) != (k_gain == nullptr) || (cos_t == nullptr) != (sin_t == nullptr) ||
      slot_mapping == nullptr || (cos_t != nullptr && (positions == nullptr || table_rows < 1)))
    return -2;
  const DecodeFused fu{q_gain, k_gain, eps, cos_t, sin_t, positions, slot_mapping, table_rows};
  const float scale_log2e = scale * 1.4426950408889634f;
  dim3 grid(nKV, max_splits, n_seqs);
#define ZF_DEC(HD)                                                                              \
  hipLaunchKernelGGL(attn_decode_fused_kernel<HD>, grid, dim3(256), 0, stream,                  \
                     (const bf16_t*)qkv, (bf16_t*)k_pool, (bf16_t*)v_pool, block_table,         \
                     ctx_len, ws_o, ws_ml, (bf16_t*)out, scale_log2e, window, nH, nKV,          \
                     page_size, max_pages, max_splits, fu)
  if (hd == 32) ZF_DEC(32);
  else if (hd == 64) ZF_DEC(64);
  else if (hd == 128) ZF_DEC(128);
  else if (hd == 256) ZF_DEC(256);
  else return -2;
#undef ZF_DEC
  return launch_decode_merge(ws_o, ws_ml, q_start, ctx_len, out, window, n_seqs, nH, hd,
                             max_splits, stream);
}

// ---------------------------------------------------------------- prefill: portions of prompts
// One workgroup per (sequence, tile of 32 queries, kv head); wave w takes the query heads
// w, w + waves, ... of the kv head.  32x32x16 MFMAs: S^T tile of 32 keys x 32 queries,
// O^T tiles of 32 head elements x 32 queries.  A query at position p reads keys lo..p; a
// portion may start anywhere in the context (earlier pages plus its own tokens).
// Sequences with a single query token are left to the decode kernel when skip_single is set.
// POW2: the page size is 1 << ps_shift, so the page and the row of a key are a shift and a
// mask; a division by a page size known only at run time costs some 30 instructions, five
// times a tile.
template <int HD, bool POW2>
__global__ __launch_bounds__(512) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    float scale_log2e, int window, int nH, int nKV, int ps, int max_pages, int skip_single,
    int q_tiles, int nsplit, int ps_shift, float* __restrict__ ws_o, float* __restrict__ ws_ml,
    int split_keys, int max_splits, const int* __restrict__ tile_map) {
  auto page_of = [&](int key) { return POW2 ? key >> ps_shift : key / ps; };
  auto row_of = [&](int key) { return POW2 ? key & (ps - 1) : key % ps; };
  extern __shared__ float xch[];      // partials of the waves that took other key tiles
  // workgroups are handed out in the order of blockIdx.x: kv heads vary fastest and the
  // last query tiles (the longest key ranges under the causal bound) come first, so the
  // heavy tiles do not end up as the tail
  // (tile_map: the host lists the (sequence, query tile) pairs that exist, heaviest first,
  // and the grid holds no workgroup for a single token or beyond a short portion's end)
  const int kvh = blockIdx.x % nKV;
  const int qt = tile_map ? tile_map[2 * (blockIdx.x / nKV) + 1]
                          : q_tiles - 1 - (blockIdx.x / nKV) % q_tiles;
  const int s = tile_map ? tile_map[2 * (blockIdx.x / nKV)] : blockIdx.x / (nKV * q_tiles);
  const int q_len = q_start[s + 1] - q_start[s];
  if (q_len == 1 && skip_single) return;
  const int qbase = qt * 32;
  if (qbase >= q_len) return;
  const int ctx = ctx_len[s];
  const int pos0 = ctx - q_len + qbase;              // position of the tile's first query
  const int nq = min(32, q_len - qbase);
  const int p_max = pos0 + nq - 1;
  const int G = nH / nKV;
  // the wave's number as a scalar: what follows from it (its head, its key tiles, the pages
  // of the value rows) is then computed once per wave, not per lane
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), nwaves = blockDim.x / 64;
  const int lane = threadIdx.x % 64, j = lane % 32, hf = lane / 32;
  const bool q_valid = j < nq;
  const int p_j = pos0 + min(j, nq - 1);
  const int lo_j = (window > 0 && p_j - window + 1 > 0) ? p_j - window + 1 : 0;
  const int lo_min = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int lo_top = (window > 0 && p_max - window + 1 > 0) ? p_max - window + 1 : 0;
  const int* table = block_table + (size_t)s * max_pages;
  const int t_row = q_start[s] + qbase + min(j, nq - 1);
  // gridDim.y > 1: the keys are also split over workgroups, blockIdx.y taking the keys
  // [split_keys * y, split_keys * (y + 1)) (a multiple of 32, so no tile lies across an edge);
  // each writes un-normalised partials that attn_prefill_merge_kernel combines.  For portions
  // behind a long context, whose few query tiles would otherwise walk thousands of keys each.
  const int k_lo = gridDim.y > 1 ? max(lo_min, (int)blockIdx.y * split_keys) : lo_min;
  const int k_hi = gridDim.y > 1 ? min(p_max, ((int)blockIdx.y + 1) * split_keys - 1) : p_max;
  if (k_lo > k_hi) return;

  // With few query heads per kv head the waves also split the key tiles of a head between
  // them (wave `split` takes tiles split, split + nsplit, ...): under the causal bound the
  // longest chain of dependent tiles, which is what the kernel's time follows, gets nsplit
  // times shorter.  The partials are combined through LDS in split order.
  const int head_waves = nwaves / nsplit, split = wave / head_waves;
  for (int g = wave % head_waves; g < G; g += head_waves) {
    const int head = kvh * G + g;
    bf16x8_t qf[HD / 16];
    {
      const bf16_t* qrow = q + ((size_t)t_row * nH + head) * HD + 8 * hf;
#pragma unroll
      for (int st = 0; st < HD / 16; ++st) {
        u32x4_t v = *(const u32x4_t*)(qrow + st * 16);
        if (!q_valid) v = u32x4_t{0, 0, 0, 0};
        qf[st] = *(bf16x8_t*)&v;
      }
    }
    f32x16_t o[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    // The loop is software-pipelined: the key rows of the next tile and the value rows of
    // this tile are requested before this tile's scores are computed, so that two rounds of
    // memory latency overlap the MFMAs and the soft-max.
    auto load_keys = [&](int kb, u32x4_t* dst) {
      const int key = min(max(kb + j, lo_min), p_max);
      const int kpage = table[page_of(key)];
      // tiled pool: head elements 16 stp + 8 hf .. + 8 of row key % 16 of its 16-row group
      const bf16_t* kblk = k_pool + ((size_t)kpage * nKV + kvh) * ps * HD +
                           (size_t)(row_of(key) / 16) * 16 * HD + (hf * 16 + key % 16) * 8;
#pragma unroll
      for (int stp = 0; stp < HD / 16; ++stp)
        dst[stp] = *(const u32x4_t*)(kblk + (stp / 2) * 512 + (stp % 2) * 256);
    };
    const int kb0 = (k_lo / 32) * 32 + 32 * split, kstep = 32 * nsplit;
    u32x4_t kf[HD / 16];
    load_keys(kb0, kf);
    // values of a tile: keys kb + 16 u .. + 15 (one page) for u = 0, 1, into one of two
    // register sets: a tile's values are requested a whole tile before its second product
    // needs them (its keys: right after the first product of the tile before)
    u32x2_t vfs[2][2][HD / 32][2];
    bool anys[2][2];
    auto load_vals = [&](int kb, auto BUF) {
      constexpr int B = decltype(BUF)::value;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int base = kb + 16 * u;
        anys[B][u] = base <= p_max && base + 16 > lo_min;
        const int safe = anys[B][u] ? max(base, lo_min) : p_max;
        const int vpage = table[page_of(safe)];
        // tiled pool: head element 32 dt + j, rows 4 hf .. + 3 and 8 + 4 hf .. + 3 of the group
        const bf16_t* vb = v_pool + ((size_t)vpage * nKV + kvh) * ps * HD +
                           (size_t)(row_of(anys[B][u] ? base : safe) / 16) * 16 * HD +
                           (j / 16) * 256 + (hf * 16 + j % 16) * 4;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
          vfs[B][u][dt][0] = *(const u32x2_t*)(vb + dt * 512);
          vfs[B][u][dt][1] = *(const u32x2_t*)(vb + dt * 512 + 128);
        }
      }
    };
    using Buf0 = std::integral_constant<int, 0>;
    using Buf1 = std::integral_constant<int, 1>;
    auto tile = [&](int kb, auto BUF, auto OTHER) {
      constexpr int B = decltype(BUF)::value;
      load_vals(kb + kstep, OTHER);      // any kb is safe: rows are clamped into live keys
      __builtin_amdgcn_sched_barrier(0);
      // S^T: rows are the keys kb + (lane % 32), clamped into the keys that exist
      f32x16_t st;
#pragma unroll
      for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
      for (int stp = 0; stp < HD / 16; ++stp)
        st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&kf[stp], qf[stp], st, 0, 0, 0);
      load_keys(kb + kstep, kf);       // next tile's keys, in flight from here (rows clamped)
      // st[r]: key kb + 8 (r / 4) + 4 hf + r % 4, query column j
      // the scale (> 0) goes into the exponent's multiply-add: max over the raw scores
      float tmax = -INFINITY;
      if (kb + 31 <= pos0 && kb >= lo_top) {
        // every key of the tile is visible to every query of the wave: nothing to mask
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, st[r]);
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kb + 8 * (r / 4) + 4 * hf + r % 4;
          const float v = (key <= p_j && key >= lo_j) ? st[r] : -INFINITY;
          st[r] = v;
          tmax = fmaxf(tmax, v);
        }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * scale_log2e;
      const float m_new = fmaxf(m, tmax);
      // a query whose window lies wholly beyond this tile has no key here yet
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float corr = exp2_raw(m - m_use);
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        st[r] = exp2_raw(fmaf(st[r], scale_log2e, -m_use));
        psum += st[r];
      }
      psum += __shfl_xor(psum, 32, 64);
      l = l * corr + psum;
      m = m_new;
      if (__any(corr != 1.0f)) {      // after the first tiles the maxima rarely move
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[dt][r] *= corr;
      }
      const bool edge_tile = !(kb >= lo_min && kb + 16 <= p_max && kb + 32 <= ctx);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        // slots e = 0..7 <-> st[8 u + e]: keys kb + 16 u + 4 hf + e (e < 4) and
        // kb + 16 u + 8 + 4 hf + (e - 4)
        u32x4_t pk = u32x4_t{pack_bf16(st[8 * u + 0], st[8 * u + 1]),
                             pack_bf16(st[8 * u + 2], st[8 * u + 3]),
                             pack_bf16(st[8 * u + 4], st[8 * u + 5]),
                             pack_bf16(st[8 * u + 6], st[8 * u + 7])};
        const bf16x8_t pf = *(bf16x8_t*)&pk;
        // keys at or beyond ctx hold nothing of this request; keys below lo_min may lie in
        // a page that was given back: both are zeroed (0 * NaN would poison the sum)
        // (only tiles at an end of the key range have such rows: one test per wave, and the
        // masks per lane are formed behind it)
        u32x2_t keep0 = u32x2_t{~0u, ~0u}, keep1 = keep0;
        if (edge_tile) {
          const int a0 = kb + 16 * u + 4 * hf, a1 = a0 + 8;
          const int hi_lim = anys[B][u] ? ctx : 0;
          keep0 = keep_range4(keep0, lo_min - a0, hi_lim - a0);
          keep1 = keep_range4(keep1, lo_min - a1, hi_lim - a1);
        }
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
          u32x2_t v0 = vfs[B][u][dt][0], v1 = vfs[B][u][dt][1];
          if (edge_tile) {
            asm volatile("");      // a real branch: as selects this costs every tile 16 operations
            v0 = u32x2_t{v0[0] & keep0[0], v0[1] & keep0[1]};
            v1 = u32x2_t{v1[0] & keep1[0], v1[1] & keep1[1]};
          }
          u32x4_t vv = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8_t*)&vv, pf, o[dt], 0, 0, 0);
        }
      }
    };
    load_vals(kb0, Buf0{});
    for (int kb = kb0; kb <= k_hi; kb += 2 * kstep) {
      tile(kb, Buf0{}, Buf1{});
      if (kb + kstep <= k_hi) tile(kb + kstep, Buf1{}, Buf0{});
      else load_vals(kb + 2 * kstep, Buf0{});     // keeps the register sets in step (unused)
    }
    if (nsplit > 1) {     // one pass over g here: every wave comes by exactly once
      constexpr int PER_LANE = HD / 2 + 2;       // a wave's O^T values per lane, max and sum
      if (split > 0) {
        float* dst = xch + (size_t)((split - 1) * head_waves + g) * PER_LANE * 64 + lane;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[(dt * 16 + r) * 64] = o[dt][r];
        dst[(HD / 2) * 64] = m;
        dst[(HD / 2 + 1) * 64] = l;
      }
      __syncthreads();
      if (split > 0) continue;
      for (int t = 1; t < nsplit; ++t) {
        const float* src = xch + (size_t)((t - 1) * head_waves + g) * PER_LANE * 64 + lane;
        const float m_t = src[(HD / 2) * 64], l_t = src[(HD / 2 + 1) * 64];
        const float m_new = fmaxf(m, m_t);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float ca = exp2f(m - m_use), cb = exp2f(m_t - m_use);
        l = l * ca + l_t * cb;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[dt][r] = o[dt][r] * ca + src[(dt * 16 + r) * 64] * cb;
      }
    }
    if (gridDim.y > 1) {
      // this split's partial for (token, head): O^T un-normalised, running maximum and sum
      if (q_valid) {
        const size_t slot = ((size_t)t_row * nH + head) * max_splits + blockIdx.y;
        float* dst = ws_o + slot * HD;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4)
            *(f32x4_t*)(dst + dt * 32 + 8 * r4 + 4 * hf) =
                f32x4_t{o[dt][r4 * 4 + 0], o[dt][r4 * 4 + 1], o[dt][r4 * 4 + 2], o[dt][r4 * 4 + 3]};
        if (hf == 0) {
          ws_ml[slot * 2] = m;
          ws_ml[slot * 2 + 1] = l;
        }
      }
      continue;
    }
    if (q_valid) {
      const float inv = 1.0f / l;
      bf16_t* orow = out + ((size_t)t_row * nH + head) * HD;
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int d = dt * 32 + 8 * r4 + 4 * hf;
          u32x2_t w = u32x2_t{pack_bf16(o[dt][r4 * 4 + 0] * inv, o[dt][r4 * 4 + 1] * inv),
                              pack_bf16(o[dt][r4 * 4 + 2] * inv, o[dt][r4 * 4 + 3] * inv)};
          *(u32x2_t*)(orow + d) = w;
        }
    }
  }
}

// The same work with the keys and values of a tile staged once per workgroup: one workgroup
// per (sequence, tile of 32 queries, kv head, block of up to 8 of its query heads), wave w
// takes head w of the block.  Tiles of 64 keys go from the tiled pools into LDS with
// direct-to-LDS loads (no registers in between; a wave instruction copies 1 KB, 64 lanes x 16
// bytes, to one uniform LDS address + 16 bytes a lane, which is the pools' own order), two
// stages: the next tile is in flight while the waves compute this one out of LDS, each reading
// the operands at the offsets it would have read in the pool.  Against attn_prefill_kernel,
// where every wave fetches its own copy of a tile from L2 and looks up its pages lane by
// lane, the loads of a tile and their address arithmetic are shared by the heads of the group.
// The stages are two arrays, not one indexed array: the compiler then knows that reads of one
// stage do not wait for the loads into the other.
// KS = 2 (up to four heads in the block): the workgroup's waves form two groups with stages of
// their own that take the even and the odd key tiles of the same heads and combine their
// partials through LDS at the end, in a fixed order.  The kernel's time follows the longest
// chain of dependent key tiles (the last query tile under the causal bound), which gets half
// as long; used where the grid fills the chip only once or twice (short prompts).
template <int HD, bool POW2, int KS>
__global__ __launch_bounds__(512) void attn_prefill_shared_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ v_pool, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    float scale_log2e, int window, int nH, int nKV, int ps, int max_pages, int skip_single,
    int q_tiles, int head_blocks, int ps_shift, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int split_keys, int max_splits,
    const int* __restrict__ tile_map) {
  // (the host pass, which only needs the launch stub, does not know the buffer descriptor type)
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int GROUP_CHUNKS = 2 * HD;          // 16-byte pieces of 16 rows of one kv head
  constexpr int TILE_CHUNKS = 4 * GROUP_CHUNKS;  // of 64 rows: keys first, then values
  __shared__ u32x4_t stage0[2 * TILE_CHUNKS];
  __shared__ u32x4_t stage1[2 * TILE_CHUNKS];
  __shared__ u32x4_t stage2[KS == 2 ? 2 * TILE_CHUNKS : 1];      // the second group's
  __shared__ u32x4_t stage3[KS == 2 ? 2 * TILE_CHUNKS : 1];
  __shared__ float other_ml[KS == 2 ? 4 : 1][64][2];
  auto page_of = [&](int key) __attribute__((always_inline)) { return POW2 ? key >> ps_shift : key / ps; };
  auto row_of = [&](int key) __attribute__((always_inline)) { return POW2 ? key & (ps - 1) : key % ps; };
  const int kvh = blockIdx.x % nKV;
  const int hb = (blockIdx.x / nKV) % head_blocks;
  const int entry = blockIdx.x / (nKV * head_blocks);
  const int qt = tile_map ? tile_map[2 * entry + 1] : q_tiles - 1 - entry % q_tiles;
  const int s = tile_map ? tile_map[2 * entry] : entry / q_tiles;
  const int q_len = q_start[s + 1] - q_start[s];
  if (q_len == 1 && skip_single) return;
  const int qbase = qt * 32;
  if (qbase >= q_len) return;
  const int ctx = ctx_len[s];
  const int pos0 = ctx - q_len + qbase;
  const int nq = min(32, q_len - qbase);
  const int p_max = pos0 + nq - 1;
  const int G = nH / nKV;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), nwaves = blockDim.x / 64;
  const int lane = threadIdx.x % 64, j = lane % 32, hf = lane / 32;
  const bool q_valid = j < nq;
  const int p_j = pos0 + min(j, nq - 1);
  const int lo_j = (window > 0 && p_j - window + 1 > 0) ? p_j - window + 1 : 0;
  const int lo_min = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int lo_top = (window > 0 && p_max - window + 1 > 0) ? p_max - window + 1 : 0;
  const int* table = block_table + (size_t)s * max_pages;
  const int t_row = q_start[s] + qbase + min(j, nq - 1);
  const int k_lo = gridDim.y > 1 ? max(lo_min, (int)blockIdx.y * split_keys) : lo_min;
  const int k_hi = gridDim.y > 1 ? min(p_max, ((int)blockIdx.y + 1) * split_keys - 1) : p_max;
  if (k_lo > k_hi) return;      // uniform over the workgroup: before any barrier
  // waves per key group (= heads of the block), this wave's group and its place in it
  const int gw = nwaves / KS, kgrp = wave / gw, wv = wave % gw;
  const int g = hb * gw + wv;
  const bool active = g < G;
  const int head = kvh * G + min(g, G - 1);

  // groups of 16 rows that hold live keys of this request: every load is clamped into them
  const int lo_grp = (lo_min / 16) * 16, hi_grp = (p_max / 16) * 16;
  auto source_of = [&](int base) __attribute__((always_inline)) { return min(max(base, lo_grp), hi_grp); };
  // pool offsets in 16-byte pieces: a page holds nKV * ps * HD / 8 of them
  const int gpp = ps / 16;                       // groups of 16 rows in a page
  const uint32_t page_chunks = (uint32_t)nKV * ps * (HD / 8);
  const uint32_t head_chunks = (uint32_t)kvh * ps * (HD / 8);
  const u32x4_t* k_chunks = (const u32x4_t*)k_pool;
  const u32x4_t* v_chunks = (const u32x4_t*)v_pool;
  // The pages of the four groups of 16 rows of the tile at kb: lane i (mod 4) looks up group
  // i's.  A vector load, so that it is waited for with the tile's copies at the end of the
  // tile, a whole tile after it was asked for (as scalar loads the look-ups were waited for
  // at the next LDS read: some 600 cycles of every tile).
  auto pages_of = [&](int kb) __attribute__((always_inline)) {
    const int gi = source_of(kb + 16 * (lane & 3)) / 16;
    return table[POW2 ? gi >> (ps_shift - 4) : gi / gpp];
  };
  // Copies the tile at kb into `stage`; its pages were looked up a tile earlier (pg_lanes),
  // and the pages of this group's tile after it are looked up now.
  int pg_lanes = 0;
  auto issue = [&](int kb, u32x4_t* stage) __attribute__((always_inline)) {
    uint64_t at[4];
#pragma unroll
    for (int grp = 0; grp < 4; ++grp) {
      const int gi = source_of(kb + 16 * grp) / 16;
      at[grp] = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(pg_lanes, grp) * page_chunks +
                head_chunks + (uint32_t)(POW2 ? gi & (gpp - 1) : gi % gpp) * GROUP_CHUNKS;
    }
    if (kb + 64 * KS <= k_hi) pg_lanes = pages_of(kb + 64 * KS);
    for (int c0 = wv * 64; c0 < TILE_CHUNKS; c0 += 64 * gw) {
      const int grp = c0 / GROUP_CHUNKS;
      const uint64_t base = (grp == 0 ? at[0] : grp == 1 ? at[1] : grp == 2 ? at[2] : at[3]) +
                            (uint32_t)(c0 % GROUP_CHUNKS);
      // (through buffer descriptors on the 1 KB to copy: the lanes add a 32-bit offset, no
      // 64-bit address per lane; the pools may be larger than a 32-bit offset reaches)
      const __amdgpu_buffer_rsrc_t k_rsrc =
          __builtin_amdgcn_make_buffer_rsrc((void*)(k_chunks + base), 0, 1024, 0x00020000);
      const __amdgpu_buffer_rsrc_t v_rsrc =
          __builtin_amdgcn_make_buffer_rsrc((void*)(v_chunks + base), 0, 1024, 0x00020000);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          k_rsrc, (__attribute__((address_space(3))) void*)(stage + c0), 16, lane * 16, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          v_rsrc, (__attribute__((address_space(3))) void*)(stage + TILE_CHUNKS + c0), 16,
          lane * 16, 0, 0, 0);
    }
  };
  // the loads into LDS count as vector-memory operations: all of this wave's have landed,
  // then all waves meet
  auto landed = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0)
    __syncthreads();
  };

  bf16x8_t qf[HD / 16];
  {
    const bf16_t* qrow = q + ((size_t)t_row * nH + head) * HD + 8 * hf;
#pragma unroll
    for (int st = 0; st < HD / 16; ++st) {
      u32x4_t v = *(const u32x4_t*)(qrow + st * 16);
      if (!q_valid) v = u32x4_t{0, 0, 0, 0};
      qf[st] = *(bf16x8_t*)&v;
    }
  }
  f32x16_t o[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m = -INFINITY, l = 0.f;
  // the lane's places inside a stage: keys in 16-byte pieces, values in 8-byte pieces
  const int k_at = (j / 16) * GROUP_CHUNKS + hf * 16 + j % 16;
  const int v_at = (j / 16) * 64 + hf * 16 + j % 16;

  // one tile out of `stage`; the next one is requested into `next` once this tile's first
  // products are under way (every wave has left `next` behind at the barrier before)
  auto tile = [&](int kb, const u32x4_t* stage, u32x4_t* next) __attribute__((always_inline)) {
    if (kb + 64 * KS <= k_hi) issue(kb + 64 * KS, next);     // this group's next tile
    if (!active) return;
    const u32x4_t* sk = stage + k_at;
    const u32x2_t* sv = (const u32x2_t*)(stage + TILE_CHUNKS) + v_at;
    f32x16_t st[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[h][r] = 0.f;
    bool have_scores = false;
    if (__builtin_expect(kb + 63 <= pos0 && kb >= lo_top, 1)) {
      // Every key of the tile is visible to every query of the wave (so all its rows hold
      // keys of this request and were loaded from their own places): no masks.
      u32x4_t kf[2][HD / 16];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int stp = 0; stp < HD / 16; ++stp)
          kf[h][stp] = sk[2 * h * GROUP_CHUNKS + (stp / 2) * 64 + (stp % 2) * 32];
      // the two halves' products alternate: neither waits for its own last result
#pragma unroll
      for (int stp = 0; stp < HD / 16; ++stp) {
        st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&kf[0][stp], qf[stp], st[0], 0, 0, 0);
        st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&kf[1][stp], qf[stp], st[1], 0, 0, 0);
      }
      have_scores = true;
      float tmax = st[0][0];
#pragma unroll
      for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, st[0][r]);
#pragma unroll
      for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, st[1][r]);
      tmax = max_of_halves(tmax) * scale_log2e;
      // m is the exponent the running sums are held against, not always the maximum: here it
      // stays where it is unless a score exceeds it by more than 2^20 (after a query's first
      // keys that is rare; the tile then takes the path below, which moves it and rescales
      // the sums).  The terms stay far inside the range of 32-bit and bfloat16 numbers,
      // whose relative precision does not depend on their size.
      const float m_ref = (m == -INFINITY) ? tmax : m;      // nothing summed yet
      if (__builtin_expect(!__any(tmax > m_ref + 20.f), 1)) {
        m = m_ref;
        float psum = 0.f;
        auto terms = [&](int h) __attribute__((always_inline)) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            st[h][r] = exp2_raw(fmaf(st[h][r], scale_log2e, -m_ref));
            psum += st[h][r];
          }
        };
        auto values = [&](int h) __attribute__((always_inline)) {
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            u32x4_t pk = u32x4_t{pack_bf16(st[h][8 * u + 0], st[h][8 * u + 1]),
                                 pack_bf16(st[h][8 * u + 2], st[h][8 * u + 3]),
                                 pack_bf16(st[h][8 * u + 4], st[h][8 * u + 5]),
                                 pack_bf16(st[h][8 * u + 6], st[h][8 * u + 7])};
            const bf16x8_t pf = *(bf16x8_t*)&pk;
            const u32x2_t* svg = sv + (2 * h + u) * 4 * HD;
#pragma unroll
            for (int dt = 0; dt < HD / 32; ++dt) {
              const u32x2_t v0 = svg[dt * 128], v1 = svg[dt * 128 + 32];
              u32x4_t vv = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
              o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8_t*)&vv, pf, o[dt], 0, 0, 0);
            }
          }
        };
        // the second half's terms (vector ALU) are issued between the products of the first
        // half's values (matrix cores)
        terms(0);
        values(0);
        terms(1);
        l += sum_of_halves(psum);
        values(1);
        return;
      }
    }
    asm volatile("");      // a real branch: the tiles at the diagonal and at the ends
    // the second 32 keys of the tile: beyond the last key any query here reads?
    const bool two = kb + 32 <= k_hi;
    if (!have_scores) {
#pragma unroll
      for (int stp = 0; stp < HD / 16; ++stp) {
        const u32x4_t kf = sk[(stp / 2) * 64 + (stp % 2) * 32];
        st[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&kf, qf[stp], st[0], 0, 0, 0);
      }
      if (two) {
#pragma unroll
        for (int stp = 0; stp < HD / 16; ++stp) {
          const u32x4_t kf = sk[2 * GROUP_CHUNKS + (stp / 2) * 64 + (stp % 2) * 32];
          st[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)&kf, qf[stp], st[1], 0, 0, 0);
        }
      }
    }
    // st[h][r]: key kb + 32 h + 8 (r / 4) + 4 hf + r % 4, query column j
    float tmax = -INFINITY;
    if (kb + 63 <= pos0 && kb >= lo_top) {
      // every key of the tile is visible to every query of the wave: nothing to mask
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, st[h][r]);
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kb + 32 * h + 8 * (r / 4) + 4 * hf + r % 4;
          const float v = (key <= p_j && key >= lo_j && (h == 0 || two)) ? st[h][r] : -INFINITY;
          st[h][r] = v;
          tmax = fmaxf(tmax, v);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * scale_log2e;
    const float m_new = fmaxf(m, tmax);
    // a query whose window lies wholly beyond this tile has no key here yet
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = exp2_raw(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        st[h][r] = exp2_raw(fmaf(st[h][r], scale_log2e, -m_use));
        psum += st[h][r];
      }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    if (__any(corr != 1.0f)) {      // after the first tiles the maxima rarely move
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= corr;
    }
    auto packed = [&](int h, int u) __attribute__((always_inline)) {
      // slots e = 0..7 <-> st[h][8 u + e]: keys base + 4 hf + e (e < 4) and
      // base + 8 + 4 hf + (e - 4), base = kb + 32 h + 16 u
      u32x4_t pk = u32x4_t{pack_bf16(st[h][8 * u + 0], st[h][8 * u + 1]),
                           pack_bf16(st[h][8 * u + 2], st[h][8 * u + 3]),
                           pack_bf16(st[h][8 * u + 4], st[h][8 * u + 5]),
                           pack_bf16(st[h][8 * u + 6], st[h][8 * u + 7])};
      return *(bf16x8_t*)&pk;
    };
    // every group of the tile was loaded from its own place and all its rows hold keys of
    // this request: nothing to look at group by group
    if (kb >= lo_min && kb + 64 <= ctx && kb + 48 <= hi_grp) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const bf16x8_t pf = packed(h, u);
          const u32x2_t* svg = sv + (2 * h + u) * 4 * HD;
#pragma unroll
          for (int dt = 0; dt < HD / 32; ++dt) {
            const u32x2_t v0 = svg[dt * 128], v1 = svg[dt * 128 + 32];
            u32x4_t vv = u32x4_t{v0[0], v0[1], v1[0], v1[1]};
            o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8_t*)&vv, pf, o[dt], 0, 0, 0);
          }
        }
      return;
    }
    asm volatile("");      // a real branch: the tiles at the ends of the key range
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (h == 1 && !two) break;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const bf16x8_t pf = packed(h, u);
        // the rows that were loaded for this group (clamped into the live groups) and which
        // of them hold a key of this request: rows at or beyond ctx were never written, rows
        // below lo_min may be stale; both are zeroed (0 * NaN would poison the sum)
        const int src = source_of(kb + 32 * h + 16 * u);
        const int a0 = src + 4 * hf, a1 = a0 + 8;
        const u32x2_t all = u32x2_t{~0u, ~0u};
        const u32x2_t keep0 = keep_range4(all, lo_min - a0, ctx - a0);
        const u32x2_t keep1 = keep_range4(all, lo_min - a1, ctx - a1);
        const u32x2_t* svg = sv + (2 * h + u) * 4 * HD;
#pragma unroll
        for (int dt = 0; dt < HD / 32; ++dt) {
          const u32x2_t v0 = svg[dt * 128], v1 = svg[dt * 128 + 32];
          u32x4_t vv = u32x4_t{v0[0] & keep0[0], v0[1] & keep0[1], v1[0] & keep1[0],
                               v1[1] & keep1[1]};
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(bf16x8_t*)&vv, pf, o[dt], 0, 0, 0);
        }
      }
    }
  };

  // group r takes the tiles kb0 + 64 (KS i + r); every wave comes by every barrier (the
  // loop's bounds are the first group's)
  const int kb0 = (k_lo / 64) * 64;
  auto run = [&](u32x4_t* sa, u32x4_t* sb) __attribute__((always_inline)) {
    const int off = 64 * kgrp;
    if (kb0 + off <= k_hi) {
      pg_lanes = pages_of(kb0 + off);
      issue(kb0 + off, sa);
    }
    landed();
    for (int kb = kb0; kb <= k_hi; kb += 128 * KS) {
      if (kb + off <= k_hi) tile(kb + off, sa, sb);
      landed();
      if (kb + 64 * KS > k_hi) break;
      if (kb + 64 * KS + off <= k_hi) tile(kb + 64 * KS + off, sb, sa);
      landed();
    }
  };
  if (KS == 1 || kgrp == 0) run(stage0, stage1);
  else run(stage2, stage3);
  if (KS == 2) {
    // the second group's partials go through its own stages (64 floats of O^T a lane: half a
    // stage a wave) to the wave of the first group with the same head
    float* spot = (float*)((wv < 2 ? stage2 : stage3) + (wv % 2) * TILE_CHUNKS) + lane;
    if (kgrp == 1) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) spot[(dt * 16 + r) * 64] = o[dt][r];
      other_ml[wv][lane][0] = m;
      other_ml[wv][lane][1] = l;
    }
    __syncthreads();
    if (kgrp == 1) return;
    const float m_b = other_ml[wv][lane][0], l_b = other_ml[wv][lane][1];
    const float m_new = fmaxf(m, m_b);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float ca = exp2f(m - m_use), cb = exp2f(m_b - m_use);
    l = l * ca + l_b * cb;
    m = m_new;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[dt][r] = o[dt][r] * ca + spot[(dt * 16 + r) * 64] * cb;
  }
  if (!active || !q_valid) return;
  if (gridDim.y > 1) {
    // this split's partial for (token, head): O^T un-normalised, running maximum and sum
    const size_t slot = ((size_t)t_row * nH + head) * max_splits + blockIdx.y;
    float* dst = ws_o + slot * HD;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *(f32x4_t*)(dst + dt * 32 + 8 * r4 + 4 * hf) =
            f32x4_t{o[dt][r4 * 4 + 0], o[dt][r4 * 4 + 1], o[dt][r4 * 4 + 2], o[dt][r4 * 4 + 3]};
    if (hf == 0) {
      ws_ml[slot * 2] = m;
      ws_ml[slot * 2 + 1] = l;
    }
    return;
  }
  const float inv = 1.0f / l;
  bf16_t* orow = out + ((size_t)t_row * nH + head) * HD;
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const int d = dt * 32 + 8 * r4 + 4 * hf;
      u32x2_t w = u32x2_t{pack_bf16(o[dt][r4 * 4 + 0] * inv, o[dt][r4 * 4 + 1] * inv),
                          pack_bf16(o[dt][r4 * 4 + 2] * inv, o[dt][r4 * 4 + 3] * inv)};
      *(u32x2_t*)(orow + d) = w;
    }
#endif
}

// Combines the key splits of one (token, head) of a prompt portion in split order and writes
// bfloat16: token t of sequence s = seq_index[t] sits at position ctx_len[s] - q_len + (t -
// q_start[s]) and has partials from the splits that hold its keys lo .. position.
__global__ __launch_bounds__(64) void attn_prefill_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ seq_index, bf16_t* __restrict__ out, int window, int nH, int hd,
    int split_keys, int max_splits, int skip_single) {
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int s = seq_index[t];
  const int q_len = q_start[s + 1] - q_start[s];
  if (q_len == 1 && skip_single) return;
  const int pos = ctx_len[s] - q_len + (t - q_start[s]);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first = lo / split_keys, last = pos / split_keys;
  const size_t base = ((size_t)t * nH + head) * max_splits;
  float mx = -INFINITY;
  for (int sp = first; sp <= last; ++sp) mx = fmaxf(mx, ws_ml[(base + sp) * 2]);
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float denom = 0.f;
  for (int sp = first; sp <= last; ++sp) {
    const float w = exp2f(ws_ml[(base + sp) * 2] - mx);
    denom += w * ws_ml[(base + sp) * 2 + 1];
    const float* src = ws_o + (base + sp) * hd;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = lane + 64 * i;
      if (d < hd) acc[i] = fmaf(w, src[d], acc[i]);
    }
  }
  const float inv = 1.0f / denom;
  bf16_t* orow = out + ((size_t)t * nH + head) * hd;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + 64 * i;
    if (d < hd) orow[d] = float_to_bf16(acc[i] * inv);
  }
}

// tile_map (or null): int32 pairs (sequence, query tile), n_tiles of them: the workgroups that
// exist.  split_keys > 0 (a multiple of 32; ws_o: n_tokens * nH * max_splits * hd floats, ws_ml:
// n_tokens * nH * max_splits * 2, max_splits >= ceil(longest context / split_keys)): the keys
// are split over workgroups and merged by a second kernel.
// variant: 0 chooses; 1 the kernel whose waves fetch their own keys and values; 2 the kernel
// that stages them in LDS for the heads of a group (head sizes 64 and 128, splits of a
// multiple of 64 keys), -2 where it does not apply; 3 the same without the two groups of
// waves on the even and the odd key tiles.
extern "C" int zf_attn_prefill_bf16(const void* q, const void* k_pool, const void* v_pool,
                                    const int* block_table, const int* q_start,
                                    const int* ctx_len, void* out, float scale, int window,
                                    int n_seqs, int max_q_len, int nH, int nKV, int hd,
                                    int page_size, int max_pages, int skip_single,
                                    int allow_split, const int* seq_index, int n_tokens,
                                    float* ws_o, float* ws_ml, int split_keys, int max_splits,
                                    const int* tile_map, int n_tiles, int variant,
                                    hipStream_t stream) {
  if (n_seqs <= 0 || max_q_len <= 0) return 0;
  if (page_size % 16 != 0 || nKV <= 0 || nH % nKV != 0) return -2;
  if (variant < 0 || variant > 3) return -2;
  if (split_keys > 0 && (split_keys % 32 != 0 || max_splits < 1 || ws_o == nullptr ||
                         ws_ml == nullptr || seq_index == nullptr))
    return -2;
  const float scale_log2e = scale * 1.4426950408889634f;
  const int G = nH / nKV;
  const int q_tiles = (max_q_len + 31) / 32;
  if (tile_map != nullptr && n_tiles <= 0) return 0;
  int ps_shift = -1;
  for (int b = 4; b < 31; ++b)
    if (page_size == (1 << b)) ps_shift = b;
  const unsigned entries = (unsigned)(tile_map != nullptr ? n_tiles : n_seqs * q_tiles);
  // from two query heads per kv head on, the tiles staged in LDS are shared (measured: faster
  // at every length from 512 tokens to 16 K, 1.1 to 1.9 times); a lone head would be one wave
  // per workgroup and stays with the first kernel, whose waves split its key tiles
  const bool shared_ok = (hd == 64 || hd == 128) && split_keys % 64 == 0;
  if ((variant == 2 || variant == 3) && !shared_ok) return -2;
  if (variant == 2 || variant == 3 || (variant == 0 && shared_ok && G >= 2)) {
    const int heads = G < 8 ? G : 8, head_blocks = (G + heads - 1) / heads;
    dim3 sgrid(entries * head_blocks * nKV, split_keys > 0 ? max_splits : 1);
    // two groups of waves on the even and the odd key tiles where the heads leave room for
    // them and the longest chain of tiles sets the time: short contexts before the portions
    // (allow_split) and a grid that fills the chip at most twice.  (8 K keys before a
    // 2048-token portion: 14 % slower with them; a whole 2048-token prompt: 73 -> 63 us with 4
    // heads per kv head, 66 -> 45 us with 2.)
    const int ks = (variant != 3 && heads <= 4 && split_keys == 0 && allow_split && sgrid.x <= 1024) ? 2 : 1;
    const dim3 sblock(64 * heads * ks);
#define ZF_PRE_S(HD, POW2, KS)                                                                  \
  hipLaunchKernelGGL((attn_prefill_shared_kernel<HD, POW2, KS>), sgrid, sblock, 0, stream,      \
                     (const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool,            \
                     block_table, q_start, ctx_len, (bf16_t*)out, scale_log2e, window, nH, nKV, \
                     page_size, max_pages, skip_single, q_tiles, head_blocks, ps_shift, ws_o,   \
                     ws_ml, split_keys, max_splits, tile_map)
#define ZF_PRE_SK(HD, POW2)                                                                     \
  do {                                                                                          \
    if (ks == 2) ZF_PRE_S(HD, POW2, 2);                                                         \
    else ZF_PRE_S(HD, POW2, 1);                                                                 \
  } while (0)
    if (hd == 64 && ps_shift >= 0) ZF_PRE_SK(64, true);
    else if (hd == 64) ZF_PRE_SK(64, false);
    else if (ps_shift >= 0) ZF_PRE_SK(128, true);
    else ZF_PRE_SK(128, false);
#undef ZF_PRE_SK
#undef ZF_PRE_S
    if (split_keys > 0)
      hipLaunchKernelGGL(attn_prefill_merge_kernel, dim3(n_tokens, nH), dim3(64), 0, stream,
                         ws_o, ws_ml, q_start, ctx_len, seq_index, (bf16_t*)out, window, nH, hd,
                         split_keys, max_splits, skip_single);
    ZF_CHECK_LAUNCH();
  }
  dim3 grid(entries * nKV, split_keys > 0 ? max_splits : 1);
  // up to 8 waves: one per query head of the kv head, and with 4 heads or fewer several
  // waves per head that split its key tiles, as far as the partials fit into LDS
  // (allow_split: the caller expects short contexts before the portions, where the causal
  // bound leaves the tiles most unequal, and a grid that does not fill the chip many times)
  int nsplit = (allow_split && split_keys == 0 && G <= 4 && grid.x <= 1024) ? 8 / G : 1;
  const size_t per_wave = (size_t)(hd / 2 + 2) * 64 * sizeof(float);
  while (nsplit > 1 && (size_t)(nsplit - 1) * G * per_wave > 144 * 1024) --nsplit;
  const int head_waves = G < 8 ? G : 8;
  dim3 block(64 * head_waves * nsplit);
  const size_t smem = nsplit > 1 ? (size_t)(nsplit - 1) * G * per_wave : 0;
#define ZF_PRE_K(KERN)                                                                          \
  do {                                                                                          \
    if (smem > 64 * 1024) {                                                                     \
      hipError_t e = hipFuncSetAttribute((const void*)KERN,                                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
      if (e != hipSuccess) return (int)e;                                                       \
    }                                                                                           \
    hipLaunchKernelGGL(KERN, grid, block, smem, stream, (const bf16_t*)q,                       \
                       (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_table, q_start,      \
                       ctx_len, (bf16_t*)out, scale_log2e, window, nH, nKV, page_size,          \
                       max_pages, skip_single, q_tiles, nsplit, ps_shift, ws_o, ws_ml,          \
                       split_keys, max_splits, tile_map);                                       \
  } while (0)
#define ZF_PRE(HD)                                                                              \
  do {                                                                                          \
    if (ps_shift >= 0) ZF_PRE_K((attn_prefill_kernel<HD, true>));                               \
    else ZF_PRE_K((attn_prefill_kernel<HD, false>));                                            \
  } while (0)
  if (hd == 32) ZF_PRE(32);
  else if (hd == 64) ZF_PRE(64);
  else if (hd == 128) ZF_PRE(128);
  else if (hd == 256) ZF_PRE(256);
  else return -2;
#undef ZF_PRE
#undef ZF_PRE_K
  if (split_keys > 0)
    hipLaunchKernelGGL(attn_prefill_merge_kernel, dim3(n_tokens, nH), dim3(64), 0, stream, ws_o,
                       ws_ml, q_start, ctx_len, seq_index, (bf16_t*)out, window, nH, hd, split_keys,
                       max_splits, skip_single);
  ZF_CHECK_LAUNCH();
}
