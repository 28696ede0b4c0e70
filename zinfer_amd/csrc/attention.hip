// Causal grouped-query attention over a paged cache.
//
// Pools are laid out [page, kv head, row, hd]; token p of a sequence lies in page
// block_table[seq][p / page_size], row p % page_size.  A token at position p attends to the
// positions lo..p of its own sequence, lo = 0 or p - window + 1 (src/kernel/attention/
// basic.zig:27-76 of the reference: scores scaled after the dot product, softmax with the
// maximum subtracted, values summed in position order; query head h reads kv head h / G).
//
//  * paged_attention_wave: one wave per (token, query head), 64 keys at a time with an
//    online softmax, all in 32-bit.  Its result for a token depends only on that token's own
//    keys, never on how the batch was cut.  Any head size, any page size.
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
  int* rows = (int*)(ps + ZF_WAVE);  // element offset of each key's row in the pool / hd
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
      const T* vr = v_pool + (size_t)rows[j] * hd;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int d = lane + i * ZF_WAVE;
        if (d < hd) acc[i] = fmaf(pj, load_as_float<T>(vr + d), acc[i]);
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
