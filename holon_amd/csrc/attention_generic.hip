// Paged causal attention, the general kernel: any element type, any page size, any head_dim that is a multiple of 8.
// One wave per (query token, query head). Keys are visited in tiles of 64 starting at the first visible key, so the
// order of every sum depends on the token's position alone, never on how the batch was cut. Scores and softmax are
// float32. For float32 operands the two long sums (a score over head_dim, the values over the keys) are accumulated in
// float64, which this GPU does at the float32 rate: a float32 running sum over 256 products of a sharp query and key
// is off by 1e-4 of the score, and that shows in the weights of the softmax.
#include <type_traits>

#include "common.h"
#include "holon_hip.h"

#define GEN_MAX_D 512

template <typename T>
__global__ void attention_generic_kernel(const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ pages,
                                         const int32_t* __restrict__ table, int table_stride,
                                         const int32_t* __restrict__ slots, const int32_t* __restrict__ lens,
                                         const int32_t* __restrict__ query_start, int rows, int heads, int kv_heads,
                                         int head_dim, int page_size, float scale, int window) {
  __shared__ float q_s[4][GEN_MAX_D];
  __shared__ float p_s[4][WAVE];
  __shared__ int64_t v_s[4][WAVE];   // element offset of each tile key's value column
  using Acc = std::conditional_t<std::is_same<T, float>::value, double, float>;
  const int w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x;
  const bool active = blockIdx.y * 4 + w < heads;
  const int h = active ? blockIdx.y * 4 + w : 0;   // a spare wave walks head 0 and stores nothing: all reach the barriers
  // the row of token t: the last b with query_start[b] <= t
  int lo_b = 0, hi_b = rows - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) / 2;
    if (query_start[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int n = lens[b];
  const int nq = query_start[b + 1] - query_start[b];
  const int pos = n - nq + (t - query_start[b]);
  T* o = out + ((int64_t)t * heads + h) * head_dim;
  if (n <= 0 || pos < 0) {   // uniform over the block (one token per block)
    if (active) for (int d = lane; d < head_dim; d += WAVE) o[d] = Elem<T>::store(0.f);
    return;
  }
  const int hk = h / (heads / kv_heads);
  const int32_t* trow = table + (int64_t)slots[b] * table_stride;
  const int64_t plane = (int64_t)page_size * head_dim;
  const T* qp = q + ((int64_t)t * heads + h) * head_dim;
  for (int d = lane; d < head_dim; d += WAVE) q_s[w][d] = Elem<T>::load(qp[d]);
  __syncthreads();

  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  Acc acc[GEN_MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < GEN_MAX_D / WAVE; ++i) acc[i] = 0;
  constexpr int V = Elem<T>::kVec;

  for (int j0 = first; j0 <= pos; j0 += WAVE) {
    const int key = j0 + lane;
    const bool valid = key <= pos;
    float s = -INFINITY;
    int64_t voff = 0;
    if (valid) {
      const int page = trow[key / page_size];
      const int off = key - (key / page_size) * page_size;
      const T* kp = pages + (((int64_t)page * 2 + 0) * kv_heads + hk) * plane + (int64_t)off * head_dim;
      voff = (((int64_t)page * 2 + 1) * kv_heads + hk) * plane + off;
      Acc dot = 0;
      for (int d = 0; d < head_dim; d += V) {
        const uint4 raw = *reinterpret_cast<const uint4*>(kp + d);
        const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int i = 0; i < V; ++i) dot += (Acc)q_s[w][d + i] * (Acc)Elem<T>::load(e[i]);
      }
      s = (float)dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float alpha = expf(m - m_new);          // m = -inf on the first tile: alpha = 0
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[w][lane] = p;
    v_s[w][lane] = voff;
    __syncthreads();
    const int count = min(WAVE, pos - j0 + 1);
#pragma unroll
    for (int i = 0; i < GEN_MAX_D / WAVE; ++i) {
      const int d = lane + i * WAVE;
      if (d < head_dim) {
        Acc a = acc[i] * (Acc)alpha;
        for (int j = 0; j < count; ++j)
          a += (Acc)p_s[w][j] * (Acc)Elem<T>::load(pages[v_s[w][j] + (int64_t)d * page_size]);
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  if (!active) return;
#pragma unroll
  for (int i = 0; i < GEN_MAX_D / WAVE; ++i) {
    const int d = lane + i * WAVE;
    if (d < head_dim) o[d] = Elem<T>::store((float)(acc[i] / (Acc)l));
  }
}

extern "C" int holon_attention_generic(const void* q, void* out, const void* pages, const int32_t* table,
                                       int table_stride, const int32_t* slots, const int32_t* lens,
                                       const int32_t* query_start, int rows, int tokens, int heads, int kv_heads,
                                       int head_dim, int page_size, int num_pages, float scale, int window, int dtype,
                                       void* stream) {
  HOLON_CHECK(rows >= 0 && tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0,
              "attention: bad head counts %d/%d", heads, kv_heads);
  HOLON_CHECK(head_dim > 0 && head_dim % 8 == 0 && head_dim <= GEN_MAX_D,
              "attention: head_dim %d must be a multiple of 8, at most %d", head_dim, GEN_MAX_D);
  HOLON_CHECK(page_size > 0 && num_pages > 0 && window >= 0, "attention: bad page size or window");
  if (tokens == 0 || rows == 0) return 0;
  dim3 grid(tokens, (heads + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    attention_generic_kernel<float><<<grid, 4 * WAVE, 0, s>>>((const float*)q, (float*)out, (const float*)pages,
                                                              table, table_stride, slots, lens, query_start, rows,
                                                              heads, kv_heads, head_dim, page_size, scale, window);
  else
    attention_generic_kernel<bf16_t><<<grid, 4 * WAVE, 0, s>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)pages,
                                                               table, table_stride, slots, lens, query_start, rows,
                                                               heads, kv_heads, head_dim, page_size, scale, window);
  HOLON_LAUNCH_OK();
  return 0;
}
