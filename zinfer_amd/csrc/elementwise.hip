// Embedding gather, RMSNorm, per-head norm + rotation + cache write, SwiGLU, row gather,
// arg-max.  Formulas follow the reference's CPU kernels (src/kernel/core/cpu.zig,
// src/kernel/attention/rope.zig); all arithmetic is 32-bit, storage is float or bfloat16.
#include "zf_common.h"
#include "zf_no_alloc.h"
#include <mutex>
#include <stdio.h>

// ---------------------------------------------------------------- embedding: x[t,:] = E[id[t],:]
// times the architecture's multiplier (1 for most; the product with 1 is exact)
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int H, float scale) {
  const int t = blockIdx.x;
  const TW* row = table + (size_t)ids[t] * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = load_as_float<TW>(row + i) * scale;
}

extern "C" int zf_embed(const void* table, int table_dtype, const int* ids, float* out, int T,
                        int H, float scale, hipStream_t stream) {
  if (T <= 0) return 0;
  if (table_dtype == ZF_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(T), dim3(256), 0, stream, (const float*)table,
                       ids, out, H, scale);
  else
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(T), dim3(256), 0, stream,
                       (const bf16_t*)table, ids, out, H, scale);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- logits after the head
// x = x * scale, then, with cap > 0, x = cap * tanh(x / cap): what an architecture may ask for
// between the head's product and the sampler
__global__ void scale_cap_kernel(float* __restrict__ x, size_t n, float scale, float cap) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v = x[i] * scale;
  if (cap > 0.f) v = cap * tanhf(v / cap);
  x[i] = v;
}

extern "C" int zf_scale_cap(float* x, long long n, float scale, float cap, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(scale_cap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                     x, (size_t)n, scale, cap);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- RMSNorm over rows of width W
// n_i = x_i * w_i / sqrt(mean(x^2) + eps)      (cpu.zig:38-48,73-110)
template <typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ gain,
                               TO* __restrict__ out, int W, float eps) {
  __shared__ float red[16];
  const float* row = x + (size_t)blockIdx.x * W;
  TO* o = out + (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = row[i];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    store_from_float<TO>(o + i, row[i] * inv * gain[i]);
}

// Widths that are a multiple of 4 up to 8192: every thread keeps its part of the row in
// registers (at most 8 float4), so the row is read once and all loads are issued together.
template <typename TO>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const float* __restrict__ x,
                                                          const float* __restrict__ gain,
                                                          TO* __restrict__ out, int W, float eps) {
  __shared__ float red[16];
  const float4* row = (const float4*)(x + (size_t)blockIdx.x * W);
  const float4* g4 = (const float4*)gain;
  TO* o = out + (size_t)blockIdx.x * W;
  const int n4 = W / 4;
  float4 v[8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = c < n4 ? row[c] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      const float4 g = g4[c];
      store_from_float<TO>(o + 4 * c + 0, v[i].x * inv * g.x);
      store_from_float<TO>(o + 4 * c + 1, v[i].y * inv * g.y);
      store_from_float<TO>(o + 4 * c + 2, v[i].z * inv * g.z);
      store_from_float<TO>(o + 4 * c + 3, v[i].w * inv * g.w);
    }
  }
}

extern "C" int zf_rmsnorm(const float* x, const float* gain, void* out, int out_dtype, int T,
                          int W, float eps, hipStream_t stream) {
  if (T <= 0) return 0;
  const bool vec = (W % 4 == 0) && W <= 8192;
  if (out_dtype == ZF_F32) {
    if (vec)
      hipLaunchKernelGGL(rmsnorm_vec_kernel<float>, dim3(T), dim3(256), 0, stream, x, gain,
                         (float*)out, W, eps);
    else
      hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(T), dim3(256), 0, stream, x, gain,
                         (float*)out, W, eps);
  } else {
    if (vec)
      hipLaunchKernelGGL(rmsnorm_vec_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, x, gain,
                         (bf16_t*)out, W, eps);
    else
      hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, x, gain,
                         (bf16_t*)out, W, eps);
  }
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- per-head norm, rotation, cache write
// One wave per (token, head).  Heads 0..nH-1 are query heads, the next nKV key heads, the
// last nKV value heads, each a contiguous slice of hd elements of the token's row of `qkv`.
//   q, k: optional RMSNorm over the head (cpu.zig:50-71), optional half-split rotation
//         (x_i, x_{i+hd/2}) <- (x_i c - x_{i+hd/2} s, x_{i+hd/2} c + x_i s)   (rope.zig:92-109)
//   q -> q_out (or back in place when q_out is null)
//   k -> page `slot / page_size`, row `slot % page_size` of the key pool laid out
//        [page, kv head, row, hd]   (or back in place when slot_mapping is null)
//   v -> the value pool, laid out [page, kv head, hd, row]: the rows (positions) of a page
//        are contiguous for each element of the head, which is the operand order the
//        attention kernels' second matrix product wants
//   tiled: both pools in the MFMA attention kernels' own order inside every group of 16 rows
//        (see attention.hip); page_size % 16 == 0 and hd % 32 == 0
template <typename T>
__global__ void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
    float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping,
    T* __restrict__ k_pool, T* __restrict__ v_pool, T* __restrict__ q_out, int nH, int nKV,
    int hd, int page_size, int tiled, int table_rows) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int half = hd / 2;
  const int row_width = (nH + 2 * nKV) * hd;
  T* src = qkv + (size_t)t * row_width + (size_t)head * hd;

  if (head >= nH + nKV) {  // value head: copy into the cache
    if (slot_mapping == nullptr) return;
    const int kvh = head - nH - nKV;
    const int slot = slot_mapping[t];
    const int page = slot / page_size, r = slot % page_size;
    T* blk = v_pool + ((size_t)page * nKV + kvh) * page_size * hd;
    if (tiled) {      // the MFMA attention kernels' order inside each group of 16 rows
      T* grp = blk + (size_t)(r / 16) * 16 * hd + ((r % 16) / 4) * 64 + r % 4;
      for (int i = lane; i < hd; i += ZF_WAVE) grp[(i / 16) * 256 + (i % 16) * 4] = src[i];
    } else {
      for (int i = lane; i < hd; i += ZF_WAVE) blk[(size_t)i * page_size + r] = src[i];
    }
    return;
  }
  const bool is_q = head < nH;
  const float* gain = is_q ? q_gain : k_gain;
  T* dst;
  bool k_tiled = false;
  int r16 = 0;
  if (is_q) {
    dst = q_out ? q_out + (size_t)t * nH * hd + (size_t)head * hd : src;
  } else if (slot_mapping) {
    const int kvh = head - nH;
    const int slot = slot_mapping[t];
    const int page = slot / page_size, r = slot % page_size;
    if (tiled) {      // element d of row r goes to [d / 32][16 * ((d % 32) / 8) + r % 16][d % 8]
      k_tiled = true;
      r16 = r % 16;
      dst = k_pool + ((size_t)page * nKV + kvh) * page_size * hd + (size_t)(r / 16) * 16 * hd;
    } else {
      dst = k_pool + (((size_t)page * nKV + kvh) * page_size + r) * hd;
    }
  } else {
    dst = src;
  }
  float inv = 1.0f;
  if (gain) {
    float ss = 0.f;
    for (int i = lane; i < hd; i += ZF_WAVE) {
      const float v = load_as_float<T>(src + i);
      ss += v * v;
    }
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)hd + eps);
  }
  // (a position beyond the tables reads their last row: wrong, but no access out of bounds)
  const int pos = min(max(positions[t], 0), table_rows - 1);
  for (int i = lane; i < half; i += ZF_WAVE) {
    float x0 = load_as_float<T>(src + i);
    float x1 = load_as_float<T>(src + i + half);
    if (gain) {
      x0 = x0 * inv * gain[i];
      x1 = x1 * inv * gain[i + half];
    }
    if (cos_t) {
      const float c = cos_t[(size_t)pos * half + i], s = sin_t[(size_t)pos * half + i];
      const float r0 = x0 * c - x1 * s;
      const float r1 = x1 * c + x0 * s;
      x0 = r0;
      x1 = r1;
    }
    if (k_tiled) {
      const int d0 = i, d1 = i + half;
      store_from_float<T>(dst + (d0 / 32) * 512 + (((d0 % 32) / 8) * 16 + r16) * 8 + d0 % 8, x0);
      store_from_float<T>(dst + (d1 / 32) * 512 + (((d1 % 32) / 8) * 16 + r16) * 8 + d1 % 8, x1);
    } else {
      store_from_float<T>(dst + i, x0);
      store_from_float<T>(dst + i + half, x1);
    }
  }
}

// Four consecutive elements as one 8-byte (bfloat16) or 16-byte (float32) access; the
// address is a multiple of that size wherever the kernel below uses them (head sizes that
// are multiples of 8, rows and pools that start on 256-byte boundaries).
template <typename T> __device__ __forceinline__ void load4(const T* p, float (&x)[4]);
template <> __device__ __forceinline__ void load4<float>(const float* p, float (&x)[4]) {
  const float4 v = *(const float4*)p;
  x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
}
template <> __device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float (&x)[4]) {
  const uint2 v = *(const uint2*)p;
  x[0] = __uint_as_float(v.x << 16); x[1] = __uint_as_float(v.x & 0xffff0000u);
  x[2] = __uint_as_float(v.y << 16); x[3] = __uint_as_float(v.y & 0xffff0000u);
}
template <typename T> __device__ __forceinline__ void store4(T* p, const float (&x)[4]);
template <> __device__ __forceinline__ void store4<float>(float* p, const float (&x)[4]) {
  *(float4*)p = float4{x[0], x[1], x[2], x[3]};
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, const float (&x)[4]) {
  *(uint2*)p = uint2{pack_bf16x2(x[0], x[1]), pack_bf16x2(x[2], x[3])};
}

// The same for head sizes that are a multiple of 8 (every size in steps of 16 is): a lane
// takes 4 consecutive elements of the first half of a head and the 4 that pair with them
// under the rotation, LPH = the next power of two >= hd / 8 lanes work on a head and a wave
// takes 64 / LPH heads of one token, so that loads and stores are 8 or 16 bytes wide and
// there are far fewer waves than (token, head) pairs.
//
// PART: the rows do not come as qkv but as the float32 partials [ksplit, T, (nH + 2 nKV) * hd]
// that a product split along K left: a lane adds its elements' partials in split order and
// rounds the sum to bfloat16, as the kernel that only adds partials would have written it, and
// goes on from there (one launch less; q goes to q_out, k and v into the pools).
template <typename T, int LPH, bool PART = false, int TPB = 1>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_write_vec_kernel(
    T* __restrict__ qkv, const float* __restrict__ q_gain, const float* __restrict__ k_gain,
    float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ slot_mapping,
    T* __restrict__ k_pool, T* __restrict__ v_pool, T* __restrict__ q_out, int nH, int nKV,
    int hd, int page_size, int tiled, const float* __restrict__ partials, int ksplit,
    size_t split_stride, int Tn, int table_rows) {
  // TPB: a workgroup takes this many tokens in a row, the same lanes the same head of each:
  // what all of them need from memory is asked for before any arithmetic, and a quarter of
  // the workgroups are handed out (2048 tokens of 48 heads, one token a workgroup: 33 us for
  // 50 MB; the kernel waited for one load after the other).
  constexpr int HPW = 64 / LPH;
  const int t0 = blockIdx.x * TPB;
  const int lane = threadIdx.x % 64, li = lane % LPH;
  // four waves to a workgroup (a quarter of the workgroups to hand out: 2048 tokens of 48
  // heads took 25 us as 24576 workgroups of one wave)
  const int head = (blockIdx.y * 4 + threadIdx.x / 64) * HPW + lane / LPH;
  const int half = hd / 2;
  const int n_heads = nH + 2 * nKV;
  const bool active = head < n_heads && 4 * li < half;
  const int row_width = n_heads * hd;
  const int hh = min(head, n_heads - 1);
  const bool is_q = head < nH, is_v = head >= nH + nKV;
  float x0[TPB][4], x1[TPB][4];
  int slot[TPB], pos[TPB];
  bool live[TPB];
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) {
    const int t = min(t0 + tt, Tn - 1);
    live[tt] = active && t0 + tt < Tn;
    slot[tt] = slot_mapping ? slot_mapping[t] : 0;
    // (a position beyond the tables reads their last row: wrong, but no access out of bounds)
    pos[tt] = (cos_t && !is_v) ? min(max(positions[t], 0), table_rows - 1) : 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) x0[tt][e] = x1[tt][e] = 0.f;
    T* src = qkv + (size_t)t * row_width + (size_t)hh * hd;
    if (PART && live[tt]) {
      const float* p = partials + (size_t)t * row_width + (size_t)hh * hd + 4 * li;
      float4 s0 = float4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
      for (int k = 0; k < ksplit; ++k) {
        const float4 a = *(const float4*)(p + (size_t)k * split_stride);
        const float4 b = *(const float4*)(p + (size_t)k * split_stride + half);
        s0.x += a.x; s0.y += a.y; s0.z += a.z; s0.w += a.w;
        s1.x += b.x; s1.y += b.y; s1.z += b.z; s1.w += b.w;
      }
      x0[tt][0] = bf16_to_float(float_to_bf16(s0.x)); x0[tt][1] = bf16_to_float(float_to_bf16(s0.y));
      x0[tt][2] = bf16_to_float(float_to_bf16(s0.z)); x0[tt][3] = bf16_to_float(float_to_bf16(s0.w));
      x1[tt][0] = bf16_to_float(float_to_bf16(s1.x)); x1[tt][1] = bf16_to_float(float_to_bf16(s1.y));
      x1[tt][2] = bf16_to_float(float_to_bf16(s1.z)); x1[tt][3] = bf16_to_float(float_to_bf16(s1.w));
    } else if (live[tt]) {
      load4<T>(src + 4 * li, x0[tt]);
      load4<T>(src + half + 4 * li, x1[tt]);
    }
  }
  if (is_v) {
    if (!active || slot_mapping == nullptr) return;
    const int kvh = head - nH - nKV;
    if (TPB == 4 && tiled && sizeof(T) == 2 && live[3] && slot[0] % 4 == 0 &&
        slot[1] == slot[0] + 1 && slot[2] == slot[0] + 2 && slot[3] == slot[0] + 3) {
      // The tiled pool keeps the rows r .. r + 3 (r % 4 == 0) of a head element side by side
      // (8 bytes), and a portion's tokens lie in consecutive rows: four tokens' values of an
      // element go out as one store.  (Rows that follow one another inside a group of 4 are
      // one request's: another request's rows lie in another page.)
      const int page = slot[0] / page_size, r = slot[0] % page_size;
      uint16_t* grp = (uint16_t*)v_pool + ((size_t)page * nKV + kvh) * page_size * hd +
                      (size_t)(r / 16) * 16 * hd + ((r % 16) / 4) * 64;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int d0 = 4 * li + e, d1 = half + 4 * li + e;
        *(uint2*)(grp + (d0 / 16) * 256 + (d0 % 16) * 4) =
            uint2{pack_bf16x2(x0[0][e], x0[1][e]), pack_bf16x2(x0[2][e], x0[3][e])};
        *(uint2*)(grp + (d1 / 16) * 256 + (d1 % 16) * 4) =
            uint2{pack_bf16x2(x1[0][e], x1[1][e]), pack_bf16x2(x1[2][e], x1[3][e])};
      }
      return;
    }
#pragma unroll
    for (int tt = 0; tt < TPB; ++tt) {
      if (!live[tt]) continue;
      const int page = slot[tt] / page_size, r = slot[tt] % page_size;
      T* blk = v_pool + ((size_t)page * nKV + kvh) * page_size * hd;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int d0 = 4 * li + e, d1 = half + 4 * li + e;
        if (tiled) {
          T* grp = blk + (size_t)(r / 16) * 16 * hd + ((r % 16) / 4) * 64 + r % 4;
          store_from_float<T>(grp + (d0 / 16) * 256 + (d0 % 16) * 4, x0[tt][e]);
          store_from_float<T>(grp + (d1 / 16) * 256 + (d1 % 16) * 4, x1[tt][e]);
        } else {
          store_from_float<T>(blk + (size_t)d0 * page_size + r, x0[tt][e]);
          store_from_float<T>(blk + (size_t)d1 * page_size + r, x1[tt][e]);
        }
      }
    }
    return;
  }
  // query and key heads (lanes of value heads have left: the shuffles below stay inside
  // groups of LPH lanes, which are all of one head)
  HeadCoef cf[TPB];
  load_head_coef(cf[0], active ? li : 0, hd, is_q ? q_gain : k_gain, cos_t, sin_t, pos[0]);
#pragma unroll
  for (int tt = 1; tt < TPB; ++tt) {
    cf[tt] = cf[0];
    load_head_rotation(cf[tt], active ? li : 0, hd, cos_t, sin_t, pos[tt]);
  }
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) head_norm_rotate<LPH>(x0[tt], x1[tt], hd, live[tt], eps, cf[tt]);
#pragma unroll
  for (int tt = 0; tt < TPB; ++tt) {
    if (!live[tt]) continue;
    const int t = t0 + tt;
    T* src = qkv + (size_t)t * row_width + (size_t)hh * hd;
    T* dst0;
    T* dst1;
    if (is_q) {
      T* base = q_out ? q_out + (size_t)t * nH * hd + (size_t)head * hd : src;
      dst0 = base + 4 * li;
      dst1 = base + half + 4 * li;
    } else if (slot_mapping) {
      const int page = slot[tt] / page_size, r = slot[tt] % page_size;
      T* blk = k_pool + ((size_t)page * nKV + (head - nH)) * page_size * hd;
      if (tiled) {      // element d of row r: [d / 32][16 * ((d % 32) / 8) + r % 16][d % 8]
        T* grp = blk + (size_t)(r / 16) * 16 * hd;
        const int d0 = 4 * li, d1 = half + 4 * li;
        dst0 = grp + (d0 / 32) * 512 + (((d0 % 32) / 8) * 16 + r % 16) * 8 + d0 % 8;
        dst1 = grp + (d1 / 32) * 512 + (((d1 % 32) / 8) * 16 + r % 16) * 8 + d1 % 8;
      } else {
        dst0 = blk + (size_t)r * hd + 4 * li;
        dst1 = blk + (size_t)r * hd + half + 4 * li;
      }
    } else {
      dst0 = src + 4 * li;
      dst1 = src + half + 4 * li;
    }
    store4<T>(dst0, x0[tt]);
    store4<T>(dst1, x1[tt]);
  }
}

template <typename T, bool PART = false>
static void launch_qk_vec(T* qkv, const float* q_gain, const float* k_gain, float eps,
                          const float* cos_t, const float* sin_t, const int* positions,
                          const int* slot_mapping, T* k_pool, T* v_pool, T* q_out, int Tn, int nH,
                          int nKV, int hd, int page_size, int tiled, int table_rows,
                          hipStream_t stream, const float* partials = nullptr, int ksplit = 0) {
  const int lanes = hd / 8, heads = nH + 2 * nKV;
  const size_t split_stride = (size_t)Tn * heads * hd;
  // from a few hundred tokens on a workgroup takes four tokens in a row
  const bool rows4 = !PART && Tn >= 256;
#define ZF_QKV_T(LPH, TPB)                                                                     \
  hipLaunchKernelGGL((qk_norm_rope_kv_write_vec_kernel<T, LPH, PART, TPB>),                    \
                     dim3((Tn + TPB - 1) / TPB, (heads + 256 / LPH - 1) / (256 / LPH)),        \
                     dim3(256), 0, stream, qkv, q_gain, k_gain, eps, cos_t, sin_t, positions,  \
                     slot_mapping, k_pool, v_pool, q_out, nH, nKV, hd, page_size, tiled,       \
                     partials, ksplit, split_stride, Tn, table_rows)
#define ZF_QKV(LPH)                                                                            \
  do {                                                                                         \
    if constexpr (PART) ZF_QKV_T(LPH, 1);                                                      \
    else if (rows4) ZF_QKV_T(LPH, 4);                                                          \
    else ZF_QKV_T(LPH, 1);                                                                     \
  } while (0)
  if (lanes <= 2) ZF_QKV(2);
  else if (lanes <= 4) ZF_QKV(4);
  else if (lanes <= 8) ZF_QKV(8);
  else if (lanes <= 16) ZF_QKV(16);
  else if (lanes <= 32) ZF_QKV(32);
  else ZF_QKV(64);
#undef ZF_QKV
#undef ZF_QKV_T
}

extern "C" int zf_qk_norm_rope_kv_write(void* qkv, int dtype, const float* q_gain,
                                        const float* k_gain, float eps, const float* cos_t,
                                        const float* sin_t, const int* positions,
                                        const int* slot_mapping, void* k_pool, void* v_pool,
                                        void* q_out, int T, int nH, int nKV, int hd,
                                        int page_size, int tiled, int table_rows,
                                        const float* partials, int ksplit, hipStream_t stream) {
  if (T <= 0) return 0;
  if (tiled && (page_size % 16 != 0 || hd % 32 != 0)) return -2;
  if (cos_t != nullptr && table_rows < 1) return -2;        // table_rows: the tables' positions
  if (partials != nullptr) {
    // rows from a split product's partials: bfloat16, q to q_out, k and v into the pools
    if (dtype != ZF_BF16 || hd % 8 != 0 || hd > 512 || ksplit < 1 || q_out == nullptr ||
        slot_mapping == nullptr)
      return -2;
    launch_qk_vec<bf16_t, true>(nullptr, q_gain, k_gain, eps, cos_t, sin_t, positions,
                                slot_mapping, (bf16_t*)k_pool, (bf16_t*)v_pool, (bf16_t*)q_out,
                                T, nH, nKV, hd, page_size, tiled, table_rows, stream, partials,
                                ksplit);
    ZF_CHECK_LAUNCH();
  }
  if (hd % 8 == 0 && hd <= 512) {
    if (dtype == ZF_F32)
      launch_qk_vec<float>((float*)qkv, q_gain, k_gain, eps, cos_t, sin_t, positions, slot_mapping,
                           (float*)k_pool, (float*)v_pool, (float*)q_out, T, nH, nKV, hd,
                           page_size, tiled, table_rows, stream);
    else
      launch_qk_vec<bf16_t>((bf16_t*)qkv, q_gain, k_gain, eps, cos_t, sin_t, positions,
                            slot_mapping, (bf16_t*)k_pool, (bf16_t*)v_pool, (bf16_t*)q_out, T, nH,
                            nKV, hd, page_size, tiled, table_rows, stream);
    ZF_CHECK_LAUNCH();
  }
  dim3 grid(T, nH + 2 * nKV);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(qk_norm_rope_kv_write_kernel<float>, grid, dim3(ZF_WAVE), 0, stream,
                       (float*)qkv, q_gain, k_gain, eps, cos_t, sin_t, positions, slot_mapping,
                       (float*)k_pool, (float*)v_pool, (float*)q_out, nH, nKV, hd, page_size,
                       tiled, table_rows);
  else
    hipLaunchKernelGGL(qk_norm_rope_kv_write_kernel<bf16_t>, grid, dim3(ZF_WAVE), 0, stream,
                       (bf16_t*)qkv, q_gain, k_gain, eps, cos_t, sin_t, positions, slot_mapping,
                       (bf16_t*)k_pool, (bf16_t*)v_pool, (bf16_t*)q_out, nH, nKV, hd, page_size,
                       tiled, table_rows);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- SwiGLU on [T, 2I] -> [T, I]
// a_j = g_j / (1 + exp(-g_j)) * u_j     (cpu.zig:130-147); gate is the first I columns.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t n) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const size_t t = idx / I, j = idx % I;
  const float g = load_as_float<T>(gu + t * 2 * I + j);
  const float u = load_as_float<T>(gu + t * 2 * I + I + j);
  store_from_float<T>(out + idx, g / (1.0f + expf(-g)) * u);
}

extern "C" int zf_swiglu(const void* gu, void* out, int dtype, int T, int I,
                         hipStream_t stream) {
  const size_t n = (size_t)T * I;
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                       (const float*)gu, (float*)out, I, n);
  else
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                       (const bf16_t*)gu, (bf16_t*)out, I, n);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- cast and poison
// out[i] = in[i] in the other storage type (bfloat16 -> float32 is exact, float32 -> bfloat16
// rounds to nearest even): weights stored in one type for a build in the other are converted
// on the device after the upload.
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    store_from_float<TO>(out + i, load_as_float<TI>(in + i));
}

extern "C" int zf_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                       hipStream_t stream) {
  if (n <= 0) return 0;
  long long blocks = (n + 256 * 8 - 1) / (256 * 8);
  if (blocks > 65536) blocks = 65536;
  const dim3 grid((unsigned)blocks), block(256);
  if (in_dtype == ZF_BF16 && out_dtype == ZF_F32)
    hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)in,
                       (float*)out, (size_t)n);
  else if (in_dtype == ZF_F32 && out_dtype == ZF_BF16)
    hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)in,
                       (bf16_t*)out, (size_t)n);
  else
    return 1;
  ZF_CHECK_LAUNCH();
}

// pool[run, pages[i], :] = NaN for every run and listed page: pages that were given back hold
// nothing that may be read again, and a test that poisons them finds a kernel that does.
template <typename T>
__global__ void poison_pages_kernel(T* __restrict__ pool, const int* __restrict__ pages,
                                    size_t row, size_t pages_in_pool) {
  T* dst = pool + ((size_t)blockIdx.y * pages_in_pool + pages[blockIdx.x]) * row;
  for (size_t i = threadIdx.x; i < row; i += blockDim.x) store_from_float<T>(dst + i, NAN);
}

extern "C" int zf_poison_pages(void* pool, int dtype, const int* pages, int n_pages, int runs,
                               long long pages_in_pool, long long row, hipStream_t stream) {
  if (n_pages <= 0 || runs <= 0 || row <= 0) return 0;
  const dim3 grid(n_pages, runs), block(256);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(poison_pages_kernel<float>, grid, block, 0, stream, (float*)pool, pages,
                       (size_t)row, (size_t)pages_in_pool);
  else
    hipLaunchKernelGGL(poison_pages_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)pool, pages,
                       (size_t)row, (size_t)pages_in_pool);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- out[r,:] = x[idx[r],:]
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ idx,
                                   float* __restrict__ out, int H) {
  const float* row = x + (size_t)idx[blockIdx.x] * H;
  float* o = out + (size_t)blockIdx.x * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = row[i];
}

extern "C" int zf_gather_rows(const float* x, const int* idx, float* out, int n, int H,
                              hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n), dim3(256), 0, stream, x, idx, out, H);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- arg-max, first maximum wins
// (src/model/layers/logits.zig:47-59: strict > while walking upwards).  Two stages: every
// workgroup reduces a chunk of a row to (value, index); one workgroup per row reduces the
// chunks.  Among equal values the lower index wins at every level.
#define ARGMAX_CHUNK 4096

__device__ __forceinline__ void argmax_block_reduce(float& best, int& bi, float* sval, int* sidx) {
  sval[threadIdx.x] = best;
  sidx[threadIdx.x] = bi;
  __syncthreads();
  for (int s = blockDim.x / 2; s > 0; s >>= 1) {
    if (threadIdx.x < s) {
      const float ov = sval[threadIdx.x + s];
      const int oi = sidx[threadIdx.x + s];
      if (ov > sval[threadIdx.x] || (ov == sval[threadIdx.x] && oi < sidx[threadIdx.x])) {
        sval[threadIdx.x] = ov;
        sidx[threadIdx.x] = oi;
      }
    }
    __syncthreads();
  }
  best = sval[0];
  bi = sidx[0];
}

__global__ __launch_bounds__(256) void argmax_chunk_kernel(const float* __restrict__ logits,
                                                           float* __restrict__ pval,
                                                           int* __restrict__ pidx, int V,
                                                           int nchunks) {
  __shared__ float sval[256];
  __shared__ int sidx[256];
  const float* row = logits + (size_t)blockIdx.x * V;
  const int lo = blockIdx.y * ARGMAX_CHUNK, hi = min(V, lo + ARGMAX_CHUNK);
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    const float v = row[i];
    if (v > best) {
      best = v;
      bi = i;
    }
  }
  argmax_block_reduce(best, bi, sval, sidx);
  if (threadIdx.x == 0) {
    pval[blockIdx.x * nchunks + blockIdx.y] = best;
    pidx[blockIdx.x * nchunks + blockIdx.y] = bi;
  }
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ pval,
                                                           const int* __restrict__ pidx,
                                                           int* __restrict__ out, int nchunks) {
  __shared__ float sval[256];
  __shared__ int sidx[256];
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < nchunks; i += 256) {
    const float v = pval[blockIdx.x * nchunks + i];
    const int id = pidx[blockIdx.x * nchunks + i];
    if (v > best || (v == best && id < bi)) {
      best = v;
      bi = id;
    }
  }
  argmax_block_reduce(best, bi, sval, sidx);
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// ws: (float + int) * n * ceil(V / 4096) of scratch
extern "C" int zf_argmax(const float* logits, int* out, void* ws, int n, int V,
                         hipStream_t stream) {
  if (n <= 0) return 0;
  const int nchunks = (V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  float* pval = (float*)ws;
  int* pidx = (int*)(pval + (size_t)n * nchunks);
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(n, nchunks), dim3(256), 0, stream, logits, pval,
                     pidx, V, nchunks);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n), dim3(256), 0, stream, pval, pidx, out,
                     nchunks);
  ZF_CHECK_LAUNCH();
}

// The same arg-max with its partial results in a device array of this file instead of a buffer
// of the caller's: for callers that cannot allocate (zf_no_alloc.h).  In host code `scratch`
// is only a stand-in for the symbol, not a device address: the address of each GPU's copy is
// looked up once per device and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS * 8];

#define ZF_NO_ALLOC_MAX_DEVICES 64
static void* scratch_ptr[ZF_NO_ALLOC_MAX_DEVICES];   // per device, null until looked up
static std::mutex scratch_mutex;

static int scratch_of_current_device(void** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= ZF_NO_ALLOC_MAX_DEVICES) return 1;
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return 1;
    scratch_ptr[dev] = p;
  }
  *ptr = scratch_ptr[dev];
  return 0;
}

extern "C" int zf_argmax_no_alloc(const float* logits, int* out, int n, int V,
                                  hipStream_t stream) {
  if (logits == nullptr || out == nullptr || n < 0 || V < 1) {
    fprintf(stderr, "zf_argmax_no_alloc: bad argument (logits %p, out %p, n %d, V %d)\n",
            (const void*)logits, (void*)out, n, V);
    return ZF_NO_ALLOC_BAD_ARGUMENT;
  }
  if (n == 0) return ZF_NO_ALLOC_OK;
  const long long nchunks = ((long long)V + ARGMAX_CHUNK - 1) / ARGMAX_CHUNK;
  if ((long long)n * nchunks > ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS) {
    fprintf(stderr, "zf_argmax_no_alloc: %d rows of %d logits need %lld partial results, the "
            "fixed array holds %d\n", n, V, (long long)n * nchunks,
            ZF_ARGMAX_NO_ALLOC_MAX_PARTIALS);
    return ZF_NO_ALLOC_TOO_LARGE;
  }
  void* ws = nullptr;
  if (scratch_of_current_device(&ws) != 0) {
    fprintf(stderr, "zf_argmax_no_alloc: the address of the device array could not be had\n");
    return ZF_NO_ALLOC_NO_SCRATCH;
  }
  float* pval = (float*)ws;
  int* pidx = (int*)(pval + (size_t)n * nchunks);
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(n, (int)nchunks), dim3(256), 0, stream, logits,
                     pval, pidx, V, (int)nchunks);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n), dim3(256), 0, stream, pval, pidx, out,
                     (int)nchunks);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- decode metadata, one step on
// Between two decode steps that run without the host: every request's sampled token becomes
// its next input, its position and context length go up by one, and the slot of the new
// position is looked up in the request's block table.  One launch per cache group; only the
// launch with advance = 1 moves tokens, positions and lengths, the others (advance = 0) find
// them already moved.  The host guarantees that the tables hold a page for the new position.
__global__ void advance_decode_kernel(int* __restrict__ token_ids, int* __restrict__ positions,
                                      int* __restrict__ ctx_len, const int* __restrict__ sampled,
                                      int* __restrict__ slot_mapping,
                                      const int* __restrict__ block_table, int n, int max_pages,
                                      int page_size, int advance) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int p = positions[i];
  if (advance) {
    p += 1;
    positions[i] = p;
    ctx_len[i] += 1;
    token_ids[i] = sampled[i];
  }
  const int page = block_table[(size_t)i * max_pages + p / page_size];
  slot_mapping[i] = page * page_size + p % page_size;
}

extern "C" int zf_advance_decode(int* token_ids, int* positions, int* ctx_len, const int* sampled,
                                 int* slot_mapping, const int* block_table, int n, int max_pages,
                                 int page_size, int advance, hipStream_t stream) {
  if (n <= 0) return 0;
  if (max_pages <= 0 || page_size <= 0) return 1;
  hipLaunchKernelGGL(advance_decode_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     token_ids, positions, ctx_len, sampled, slot_mapping, block_table, n,
                     max_pages, page_size, advance);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- measurement: a read stream
// Reads `bytes` (a multiple of 16) once and does nothing else of weight: every lane takes
// 16-byte non-temporal loads, 8 in flight, a workgroup 64 KB in a row at a time, and xors
// what it read into one word per workgroup (so that no load can be dropped).  The rate
// this reaches from HBM is what the weight-streaming kernels are measured against.
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t zf_u32x4_t;
__global__ __launch_bounds__(512) void stream_read_kernel(const zf_u32x4_t* __restrict__ src,
                                                          size_t n16, uint32_t* __restrict__ sink) {
  // a workgroup takes chunks of 8 x 512 x 16 bytes = 64 KB in a row, chunk after chunk
  const size_t chunk = (size_t)8 * blockDim.x;
  uint32_t acc = 0;
  size_t c = (size_t)blockIdx.x * chunk;
  for (; c + chunk <= n16; c += (size_t)gridDim.x * chunk) {
    zf_u32x4_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = __builtin_nontemporal_load(src + c + (size_t)u * blockDim.x + threadIdx.x);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  // the last, partial chunk belongs to exactly one workgroup
  if (c < n16)
    for (size_t i = c + threadIdx.x; i < n16; i += blockDim.x) {
      const zf_u32x4_t v = __builtin_nontemporal_load(src + i);
      acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc ^= __shfl_xor(acc, o, 64);
  __shared__ uint32_t part[8];
  if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t a = 0;
    for (int w = 0; w < (int)blockDim.x / 64; ++w) a ^= part[w];
    sink[blockIdx.x] = a;
  }
}

// sink: at least `workgroups` words.  bytes % 16 == 0, 1 <= workgroups <= 65536.
extern "C" int zf_stream_read(const void* src, long long bytes, uint32_t* sink, int workgroups,
                              hipStream_t stream) {
  if (bytes <= 0) return 0;
  if (bytes % 16 != 0 || workgroups < 1 || workgroups > 65536) return 1;
  hipLaunchKernelGGL(stream_read_kernel, dim3(workgroups), dim3(512), 0, stream,
                     (const zf_u32x4_t*)src, (size_t)(bytes / 16), sink);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- debugging: a step's tables
// Every page a step's kernels will look up (the first ceil(ctx_len / page_size) entries of a
// sequence's row) must be a page of the pool, every slot a row of the pool.  Nothing traps:
// a thread that finds a bad entry writes (1 + kind, sequence or token, index, value) into
// `report` (kind 0: block table, 1: slot mapping; which of several bad entries is reported is
// left open), and the host reads it.
__global__ void check_tables_kernel(const int* __restrict__ block_table,
                                    const int* __restrict__ ctx_len,
                                    const int* __restrict__ slot_mapping, int n_seqs,
                                    int max_pages, int page_size, int num_pages, int n_tokens,
                                    int* __restrict__ report) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_seqs * max_pages) {
    const int s = i / max_pages, p = i % max_pages;
    const int ctx = ctx_len[s];
    const bool used = ctx >= 0 && p < (ctx + page_size - 1) / page_size;
    const int page = block_table[i];
    if (ctx < 0 || ctx > max_pages * page_size || (used && (page < 0 || page >= num_pages))) {
      report[1] = s;
      report[2] = p;
      report[3] = ctx < 0 || ctx > max_pages * page_size ? ctx : page;
      report[0] = 1;
    }
  }
  if (slot_mapping != nullptr && i < n_tokens) {
    const int slot = slot_mapping[i];
    if (slot < 0 || slot >= num_pages * page_size) {
      report[1] = i;
      report[2] = 0;
      report[3] = slot;
      report[0] = 2;
    }
  }
}

extern "C" int zf_check_tables(const int* block_table, const int* ctx_len,
                               const int* slot_mapping, int n_seqs, int max_pages, int page_size,
                               int num_pages, int n_tokens, int* report, hipStream_t stream) {
  if (n_seqs <= 0 || max_pages <= 0 || page_size <= 0) return 1;
  const int n = max(n_seqs * max_pages, n_tokens);
  hipLaunchKernelGGL(check_tables_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     block_table, ctx_len, slot_mapping, n_seqs, max_pages, page_size, num_pages,
                     n_tokens, report);
  ZF_CHECK_LAUNCH();
}
