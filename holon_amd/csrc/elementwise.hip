// Per-token operations: embedding gather, RMSNorm (plain and with the residual add), SiLU*mul, and the fused
// per-head norm + rotary embedding + cache write. Everything is computed in float32 and rounded once per result.
#include "common.h"
#include "holon_hip.h"

// ---------------------------------------------------------------------------------------------------------------
// take_slot / last_token (both or neither): token t is last_token[take_slot[t]] where take_slot[t] >= 0, a token that
// the previous step drew and that never left the device.
template <typename T>
__global__ void embedding_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ take_slot,
                                 const int32_t* __restrict__ last_token, const T* __restrict__ table,
                                 T* __restrict__ out, int hidden, int vocab, float* __restrict__ stats_out) {
  const int64_t t = blockIdx.x;
  int id = ids[t];
  if (take_slot != nullptr && take_slot[t] >= 0) id = last_token[take_slot[t]];
  id = min(max(id, 0), vocab - 1);             // (the host checks the ids it sends; a drawn token is in range)
  const T* src = table + (int64_t)id * hidden;
  T* dst = out + t * hidden;
  constexpr int V = Elem<T>::kVec;
  if (hidden % V == 0) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < hidden / V; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  }
  if (stats_out != nullptr) {     // the row's sum of squares, for a norm folded into the product that reads the row
    __shared__ float part[4];
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = Elem<T>::load(src[i]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = ss;
    __syncthreads();
    if (threadIdx.x == 0) stats_out[t] = ((part[0] + part[1]) + part[2]) + part[3];
  }
}

// stats[0][m] = sum of squares of row m (m < rows <= 16): one wave per row.
template <typename T>
__global__ void row_sumsq_kernel(const T* __restrict__ x, float* __restrict__ stats, int rows, int dim) {
  const int row = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  float ss = 0.f;
  if (row < rows)
    for (int i = lane; i < dim; i += WAVE) {
      const float v = Elem<T>::load(x[(int64_t)row * dim + i]);
      ss += v * v;
    }
  ss = wave_sum(ss);
  if (lane == 0) stats[row] = ss;
}

extern "C" int holon_row_sumsq(const void* x, float* stats, int rows, int dim, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 16 && dim > 0, "row_sumsq: %d rows of %d (at most 16 rows)", rows, dim);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32) row_sumsq_kernel<float><<<1, 16 * WAVE, 0, s>>>((const float*)x, stats, rows, dim);
  else row_sumsq_kernel<bf16_t><<<1, 16 * WAVE, 0, s>>>((const bf16_t*)x, stats, rows, dim);
  HOLON_LAUNCH_OK();
  return 0;
}

// stats_out (nullable, tokens <= 16): [16] float32, the sum of squares of every row written.
extern "C" int holon_embedding(const int32_t* ids, const int32_t* take_slot, const int32_t* last_token,
                               const void* table, void* out, int tokens, int hidden, int vocab, int dtype,
                               float* stats_out, void* stream) {
  HOLON_CHECK(tokens >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes tokens=%d hidden=%d", tokens, hidden);
  HOLON_CHECK((take_slot == nullptr) == (last_token == nullptr), "embedding: slots to take tokens from need the tokens");
  HOLON_CHECK(stats_out == nullptr || tokens <= 16, "embedding: row sums for at most 16 tokens, not %d", tokens);
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    embedding_kernel<float><<<tokens, 256, 0, s>>>(ids, take_slot, last_token, (const float*)table, (float*)out,
                                                   hidden, vocab, stats_out);
  else
    embedding_kernel<bf16_t><<<tokens, 256, 0, s>>>(ids, take_slot, last_token, (const bf16_t*)table, (bf16_t*)out,
                                                    hidden, vocab, stats_out);
  HOLON_LAUNCH_OK();
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// What is added to the residual rows when it comes as float32 sums over shares of K, parts [splits, rows, dim] (a
// product whose blocks split K): the shares added up in order, rounded to T.
template <typename T>
__device__ __forceinline__ float sum_of_parts(const float* __restrict__ parts, int splits, int64_t share, int64_t at) {
  float sum = parts[at];
  for (int s = 1; s < splits; ++s) sum += parts[s * share + at];
  return Elem<T>::round(sum);
}

// One wave per row. Pass 1: (residual += x, rounded) and the sum of squares; pass 2: scale and weight. With `parts`,
// x is the sum of the parts.
template <typename T, bool ADD>
__global__ void rmsnorm_kernel(const T* __restrict__ x, T* __restrict__ residual, const T* __restrict__ weight,
                               T* __restrict__ y, int64_t rows, int dim, float eps,
                               const float* __restrict__ parts = nullptr, int splits = 0) {
  const int lane = threadIdx.x % WAVE;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (row >= rows) return;
  const T* xr = parts ? nullptr : x + row * dim;
  T* rr = ADD ? residual + row * dim : nullptr;
  float ss = 0.f;
  for (int i = lane; i < dim; i += WAVE) {
    float v = parts ? sum_of_parts<T>(parts, splits, rows * dim, row * dim + i) : Elem<T>::load(xr[i]);
    if (ADD) {
      v = Elem<T>::round(Elem<T>::load(rr[i]) + v);
      rr[i] = Elem<T>::store(v);
    }
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  T* yr = y + row * dim;
  for (int i = lane; i < dim; i += WAVE) {
    const float v = ADD ? Elem<T>::load(rr[i]) : Elem<T>::load(xr[i]);
    yr[i] = Elem<T>::store((v * inv) * Elem<T>::load(weight[i]));
  }
}

// One block of 256 threads per row, for rows that fit the registers: 16-byte loads, the row is read once. VPT = vectors
// of 16 bytes per thread. The sum of squares is reduced inside waves, then over the four waves in wave order.
template <typename T, bool ADD, int VPT>
__global__ void __launch_bounds__(256) rmsnorm_row_kernel(const T* __restrict__ x, T* __restrict__ residual,
                                                          const T* __restrict__ weight, T* __restrict__ y, int dim,
                                                          float eps) {
  constexpr int V = Elem<T>::kVec;
  __shared__ float part[4];
  const int64_t row = blockIdx.x;
  const int nvec = dim / V;
  const uint4* xr = reinterpret_cast<const uint4*>(x + row * dim);
  uint4* rr = ADD ? reinterpret_cast<uint4*>(residual + row * dim) : nullptr;
  float vals[VPT][V];
  float ss = 0.f;
  const uint4* wr = reinterpret_cast<const uint4*>(weight);
  uint4 wraw[VPT];                              // requested now, needed after the reduction
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int v = threadIdx.x + i * 256;
    if (v < nvec) wraw[i] = wr[v];
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int v = threadIdx.x + i * 256;
    if (v < nvec) {
      uint4 raw = xr[v];
      const T* e = reinterpret_cast<const T*>(&raw);
      if (ADD) {
        uint4 rraw = rr[v];
        T* re = reinterpret_cast<T*>(&rraw);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          vals[i][j] = Elem<T>::round(Elem<T>::load(re[j]) + Elem<T>::load(e[j]));
          re[j] = Elem<T>::store(vals[i][j]);
        }
        rr[v] = rraw;
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) vals[i][j] = Elem<T>::load(e[j]);
      }
#pragma unroll
      for (int j = 0; j < V; ++j) ss += vals[i][j] * vals[i][j];
    }
  }
  ss = wave_sum(ss);
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = ss;
  __syncthreads();
  ss = ((part[0] + part[1]) + part[2]) + part[3];
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  uint4* yr = reinterpret_cast<uint4*>(y + row * dim);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int v = threadIdx.x + i * 256;
    if (v < nvec) {
      const T* we = reinterpret_cast<const T*>(&wraw[i]);
      uint4 out;
      T* oe = reinterpret_cast<T*>(&out);
#pragma unroll
      for (int j = 0; j < V; ++j) oe[j] = Elem<T>::store((vals[i][j] * inv) * Elem<T>::load(we[j]));
      yr[v] = out;
    }
  }
}

// The residual add + norm over a product that comes as float32 sums over shares of K, parts [splits, rows, dim]:
// residual += round(parts[0] + parts[1] + ...), y = rmsnorm(residual), bfloat16. One block of 1,024 threads per row,
// eight values a thread (dim <= 8,192), so that all of a thread's loads, eight shares at a time, are under way at once:
// the parts come from memory (other compute dies wrote them), and with four times the values a thread and the shares
// read one after the other the kernel took 11 us where this takes half.
__global__ void __launch_bounds__(1024) rmsnorm_parts_kernel(const float* __restrict__ parts, int splits,
                                                             bf16_t* __restrict__ residual,
                                                             const bf16_t* __restrict__ weight, bf16_t* __restrict__ y,
                                                             int dim, float eps) {
  using E = Elem<bf16_t>;
  constexpr int V = 8, AT_ONCE = 8;
  __shared__ float part[16];
  const int64_t row = blockIdx.x;
  const int v = threadIdx.x;
  const bool live = v < dim / V;
  float vals[V];
  float ss = 0.f;
  uint4 wraw;
  if (live) {
    wraw = reinterpret_cast<const uint4*>(weight)[v];
    uint4* rr = reinterpret_cast<uint4*>(residual + row * dim) + v;
    uint4 rraw = *rr;
    const float* pr = parts + (row * dim + (int64_t)v * V);
    const int64_t share = (int64_t)gridDim.x * dim;
    float sum[V];
#pragma unroll
    for (int j = 0; j < V; ++j) sum[j] = 0.f;
    for (int s0 = 0; s0 < splits; s0 += AT_ONCE) {
      float4 p[AT_ONCE][V / 4];
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u)
#pragma unroll
        for (int j = 0; j < V / 4; ++j)
          p[u][j] = s0 + u < splits ? *reinterpret_cast<const float4*>(pr + (s0 + u) * share + 4 * j)
                                    : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < AT_ONCE; ++u)
#pragma unroll
        for (int j = 0; j < V / 4; ++j) {
          sum[4 * j] += p[u][j].x;
          sum[4 * j + 1] += p[u][j].y;
          sum[4 * j + 2] += p[u][j].z;
          sum[4 * j + 3] += p[u][j].w;
        }
    }
    bf16_t* re = reinterpret_cast<bf16_t*>(&rraw);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      vals[j] = E::round(E::load(re[j]) + E::round(sum[j]));
      re[j] = E::store(vals[j]);
      ss += vals[j] * vals[j];
    }
    *rr = rraw;
  }
  ss = wave_sum(ss);
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = ss;
  __syncthreads();
  ss = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) ss += part[w];
  const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
  if (live) {
    const bf16_t* we = reinterpret_cast<const bf16_t*>(&wraw);
    uint4 out;
    bf16_t* oe = reinterpret_cast<bf16_t*>(&out);
#pragma unroll
    for (int j = 0; j < V; ++j) oe[j] = E::store((vals[j] * inv) * E::load(we[j]));
    reinterpret_cast<uint4*>(y + row * dim)[v] = out;
  }
}

template <typename T, bool ADD>
static bool launch_rmsnorm_rows(const void* x, void* residual, const void* weight, void* y, int64_t rows, int dim,
                                float eps, hipStream_t s) {
  constexpr int V = Elem<T>::kVec;
  if (dim % V != 0 || dim < 1024 || rows > 0x7fffffff) return false;
  if ((((uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)y) & 15) != 0) return false;
  const int vpt = (dim / V + 255) / 256;
#define ROWS_LAUNCH(VPT)                                                                                          \
  rmsnorm_row_kernel<T, ADD, VPT><<<(unsigned)rows, 256, 0, s>>>((const T*)x, (T*)residual, (const T*)weight, (T*)y, \
                                                                 dim, eps)
  if (vpt <= 1) ROWS_LAUNCH(1);
  else if (vpt <= 2) ROWS_LAUNCH(2);
  else if (vpt <= 4) ROWS_LAUNCH(4);
  else if (vpt <= 8) ROWS_LAUNCH(8);
  else return false;
#undef ROWS_LAUNCH
  return true;
}

extern "C" int holon_rmsnorm(const void* x, void* residual, const void* weight, void* y, int64_t rows, int dim,
                             float eps, int dtype, void* stream) {
  HOLON_CHECK(rows >= 0 && dim > 0, "rmsnorm: bad sizes rows=%lld dim=%d", (long long)rows, dim);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  bool done;
  if (dtype == HOLON_F32)
    done = residual ? launch_rmsnorm_rows<float, true>(x, residual, weight, y, rows, dim, eps, s)
                    : launch_rmsnorm_rows<float, false>(x, residual, weight, y, rows, dim, eps, s);
  else
    done = residual ? launch_rmsnorm_rows<bf16_t, true>(x, residual, weight, y, rows, dim, eps, s)
                    : launch_rmsnorm_rows<bf16_t, false>(x, residual, weight, y, rows, dim, eps, s);
  if (done) {
    HOLON_LAUNCH_OK();
    return 0;
  }
  const int waves = 4;   // narrow or odd rows: one wave per row
  const unsigned grid = (unsigned)((rows + waves - 1) / waves);
#define RMS_LAUNCH(T, ADD) \
  rmsnorm_kernel<T, ADD><<<grid, waves * WAVE, 0, s>>>((const T*)x, (T*)residual, (const T*)weight, (T*)y, rows, dim, eps)
  if (dtype == HOLON_F32) {
    if (residual) RMS_LAUNCH(float, true); else RMS_LAUNCH(float, false);
  } else {
    if (residual) RMS_LAUNCH(bf16_t, true); else RMS_LAUNCH(bf16_t, false);
  }
#undef RMS_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_rmsnorm_parts(const float* parts, int splits, void* residual, const void* weight, void* y,
                                   int64_t rows, int dim, float eps, void* stream) {
  HOLON_CHECK(rows >= 0 && rows <= 0x7fffffff && dim > 0 && splits >= 1 && parts && residual,
              "rmsnorm of parts: bad sizes rows=%lld dim=%d splits=%d", (long long)rows, dim, splits);
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = (((uintptr_t)parts | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)y) & 15) == 0;
  if (dim % 8 == 0 && dim >= 1024 && dim <= 8192 && aligned) {
    rmsnorm_parts_kernel<<<(unsigned)rows, 1024, 0, s>>>(parts, splits, (bf16_t*)residual, (const bf16_t*)weight,
                                                         (bf16_t*)y, dim, eps);
  } else {                 // narrow, odd or very wide rows: one wave per row
    const int waves = 4;
    const unsigned grid = (unsigned)((rows + waves - 1) / waves);
    rmsnorm_kernel<bf16_t, true><<<grid, waves * WAVE, 0, s>>>(nullptr, (bf16_t*)residual, (const bf16_t*)weight,
                                                               (bf16_t*)y, rows, dim, eps, parts, splits);
  }
  HOLON_LAUNCH_OK();
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t tokens, int inter) {
  const int64_t n = tokens * inter;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / inter;
    const int c = (int)(i - t * inter);
    const float g = Elem<T>::load(gu[t * 2 * inter + c]);
    const float u = Elem<T>::load(gu[t * 2 * inter + inter + c]);
    const float s = Elem<T>::round(silu<T>(g));
    out[i] = Elem<T>::store(s * u);
  }
}

// 16 bytes of gate and 16 bytes of up per thread (widths that are multiples of the vector).
template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t tokens, int inter) {
  constexpr int V = Elem<T>::kVec;
  const int per_row = inter / V;
  const int64_t n = tokens * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / per_row;
    const int c = (int)(i - t * per_row) * V;
    const uint4 graw = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + c);
    const uint4 uraw = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + inter + c);
    const T* ge = reinterpret_cast<const T*>(&graw);
    const T* ue = reinterpret_cast<const T*>(&uraw);
    uint4 oraw;
    T* oe = reinterpret_cast<T*>(&oraw);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float g = Elem<T>::load(ge[j]);
      const float sg = Elem<T>::round(silu<T>(g));
      oe[j] = Elem<T>::store(sg * Elem<T>::load(ue[j]));
    }
    *reinterpret_cast<uint4*>(out + t * inter + c) = oraw;
  }
}

extern "C" int holon_silu_mul(const void* gate_up, void* out, int64_t tokens, int inter, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && inter > 0, "silu_mul: bad sizes");
  if (tokens == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int vec = dtype == HOLON_F32 ? 4 : 8;
  if (inter % vec == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    const int64_t nv = tokens * (inter / vec);
    const unsigned vgrid = (unsigned)((nv + 255) / 256 < 16384 ? (nv + 255) / 256 : 16384);
    if (dtype == HOLON_F32)
      silu_mul_vec_kernel<float><<<vgrid, 256, 0, s>>>((const float*)gate_up, (float*)out, tokens, inter);
    else
      silu_mul_vec_kernel<bf16_t><<<vgrid, 256, 0, s>>>((const bf16_t*)gate_up, (bf16_t*)out, tokens, inter);
    HOLON_LAUNCH_OK();
    return 0;
  }
  const int64_t n = tokens * inter;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (dtype == HOLON_F32)
    silu_mul_kernel<float><<<grid, 256, 0, s>>>((const float*)gate_up, (float*)out, tokens, inter);
  else
    silu_mul_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)gate_up, (bf16_t*)out, tokens, inter);
  HOLON_LAUNCH_OK();
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// One wave per (token, head) of the merged projection. Head index h: [0, Hq) queries, [Hq, Hq+Hkv) keys, the rest
// values. The head is staged in LDS as float32 so that a lane can read its rotation partner.
#define MAX_HEAD_DIM 512
template <typename T>
__global__ void qk_norm_rope_write_kernel(const T* qkv, int64_t qkv_stride, T* q_out,
                                          int heads, int kv_heads, int head_dim, const T* __restrict__ q_weight,
                                          const T* __restrict__ k_weight, float eps, const float* __restrict__ table,
                                          int rotary_dim, const int32_t* __restrict__ positions,
                                          T* __restrict__ pages, const int32_t* __restrict__ write_page,
                                          const int32_t* __restrict__ write_off, int page_size, int total_heads) {
  __shared__ float stage[4][MAX_HEAD_DIM];
  const int w = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int t = blockIdx.x;
  const int h = blockIdx.y * 4 + w;
  const bool active = h < total_heads;   // no early return: every wave reaches the barrier below
  const T* src = qkv + (int64_t)t * qkv_stride + (int64_t)h * head_dim;
  const bool is_q = active && h < heads, is_k = active && !is_q && h < heads + kv_heads;
  float* buf = stage[w];
  if (is_q || is_k) {
    const T* weight = is_q ? q_weight : k_weight;
    float ss = 0.f;
    for (int d = lane; d < head_dim; d += WAVE) {
      const float v = Elem<T>::load(src[d]);
      buf[d] = v;
      ss += v * v;
    }
    if (weight != nullptr) {
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
      for (int d = lane; d < head_dim; d += WAVE) buf[d] = Elem<T>::round((buf[d] * inv) * Elem<T>::load(weight[d]));
    }
  }
  __syncthreads();   // rotation partners were staged by other lanes
  if (is_q || is_k) {
    T* dst;
    int64_t dstride = 1;
    if (is_q) {
      dst = q_out + ((int64_t)t * heads + h) * head_dim;
    } else {
      const int hk = h - heads;
      dst = pages + (((int64_t)write_page[t] * 2 + 0) * kv_heads + hk) * (int64_t)page_size * head_dim +
            (int64_t)write_off[t] * head_dim;
    }
    const int half = rotary_dim / 2;
    const float* cs = table != nullptr ? table + (int64_t)positions[t] * rotary_dim : nullptr;
    for (int d = lane; d < head_dim; d += WAVE) {
      float o;
      if (cs != nullptr && d < half) {
        o = buf[d] * cs[d] - buf[d + half] * cs[half + d];
      } else if (cs != nullptr && d < rotary_dim) {
        const int i = d - half;
        o = buf[d] * cs[i] + buf[i] * cs[half + i];
      } else {
        o = buf[d];
      }
      dst[d * dstride] = Elem<T>::store(o);
    }
  } else if (active) {
    const int hk = h - heads - kv_heads;
    T* dst = pages + (((int64_t)write_page[t] * 2 + 1) * kv_heads + hk) * (int64_t)page_size * head_dim +
             write_off[t];
    for (int d = lane; d < head_dim; d += WAVE) dst[(int64_t)d * page_size] = src[d];
  }
}

// Values of 16 consecutive tokens of one kv head into the cache. Inside a page values are stored transposed
// ([D, P]), so a token alone writes D scattered elements; 16 tokens that fill consecutive places of one page are
// transposed through LDS and written as 32 contiguous bytes per dim. A block of 256 threads; `tile` and `together`
// are the block's.
template <typename T, int PITCH>
__device__ __forceinline__ void v_write_group(T (*tile)[PITCH], int* together, int t0, int hk,
                                              const T* __restrict__ qkv, int64_t qkv_stride, int v_col0, int tokens,
                                              int kv_heads, int head_dim, T* __restrict__ pages,
                                              const int32_t* __restrict__ write_page,
                                              const int32_t* __restrict__ write_off, int page_size) {
  const int tid = threadIdx.x;
  const int count = min(16, tokens - t0);
  if (tid < WAVE) {                    // lane j looks at token j's place: one round of loads, not sixteen
    int pg = 0, off = 0;
    if (tid < count) { pg = write_page[t0 + tid]; off = write_off[t0 + tid]; }
    const int pg0 = __shfl(pg, 0, WAVE), off0 = __shfl(off, 0, WAVE);
    const bool ok = count == 16 && off0 % 8 == 0 && off0 + 16 <= page_size &&
                    (tid >= 16 || (pg == pg0 && off == off0 + tid));
    const bool all_ok = __all(ok);
    if (tid == 0) *together = all_ok;
  }
  const int per_row = head_dim / 8;   // head_dim % 8 == 0 (checked by the host)
  for (int q = tid; q < count * per_row; q += 256) {
    const int tk = q / per_row, c8 = (q % per_row) * 8;
    const T* src = qkv + (int64_t)(t0 + tk) * qkv_stride + v_col0 + (int64_t)hk * head_dim + c8;
    // (16-byte pieces: the caller's sizes put every piece of eight values on a 16-byte edge, here and in `tile`)
    if (sizeof(T) == 2) {
      *reinterpret_cast<uint4*>(&tile[tk][c8]) = *reinterpret_cast<const uint4*>(src);
    } else {
      *reinterpret_cast<float4*>(&tile[tk][c8]) = *reinterpret_cast<const float4*>(src);
      *reinterpret_cast<float4*>(&tile[tk][c8 + 4]) = *reinterpret_cast<const float4*>(src + 4);
    }
  }
  __syncthreads();
  const int64_t plane = (int64_t)page_size * head_dim;
  if (*together) {
    T* base = pages + (((int64_t)write_page[t0] * 2 + 1) * kv_heads + hk) * plane + write_off[t0];
    for (int r = tid; r < head_dim * 2; r += 256) {
      const int d = r / 2, half = r % 2;
      T out8[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) out8[j] = tile[half * 8 + j][d];
      T* dst = base + (int64_t)d * page_size + half * 8;
      if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(out8);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = out8[j];
      }
    }
  } else {
    for (int q = tid; q < count * head_dim; q += 256) {
      const int tk = q % count, d = q / count;
      pages[(((int64_t)write_page[t0 + tk] * 2 + 1) * kv_heads + hk) * plane + (int64_t)d * page_size +
            write_off[t0 + tk]] = tile[tk][d];
    }
  }
}

// Among the LPH lanes of a head: the sum over them, and the value LPH / 2 lanes away. With 16 lanes a head (a DPP row)
// both are register moves (rotations of the row, swaps inside a quad) that hand every lane the very values the
// shuffles by xor 8, 4, 2, 1 would: after the step by 8, lanes l and l ^ 8 hold the same, so the lane 4 before holds
// what lane l ^ 4 does. Other head sizes go through the shuffles.
template <int CTRL>
__device__ __forceinline__ float row_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
template <int LPH>
__device__ __forceinline__ float head_sum(float ss) {
  if constexpr (LPH == 16) {
    ss += row_move<0x128>(ss);     // row_ror:8
    ss += row_move<0x124>(ss);     // row_ror:4
    ss += row_move<0x4e>(ss);      // quad_perm:[2,3,0,1]
    ss += row_move<0xb1>(ss);      // quad_perm:[1,0,3,2]
  } else {
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
  }
  return ss;
}
template <int LPH>
__device__ __forceinline__ float half_away(float v) {
  if constexpr (LPH == 16) return row_move<0x128>(v);
  else return __shfl_xor(v, LPH / 2, WAVE);
}

// The same for head_dim 64, 128 or 256 with the whole head rotated (or not at all): each lane holds 8 consecutive
// values (one 16-byte load), LPH = head_dim / 8 lanes make a head, a wave holds 64 / LPH heads. The rotation partner
// of a value sits LPH / 2 lanes away; norm sums run over the LPH lanes of a head. No LDS.
template <typename T, int LPH>
__global__ void __launch_bounds__(256) qk_norm_rope_write_fast_kernel(
    const T* qkv, int64_t qkv_stride, T* q_out, int heads, int kv_heads, const T* __restrict__ q_weight,
    const T* __restrict__ k_weight, float eps, const float* __restrict__ table, const int32_t* __restrict__ positions,
    T* __restrict__ pages, const int32_t* __restrict__ write_page, const int32_t* __restrict__ write_off,
    int page_size, int total_heads, int tokens, int value_groups) {
  constexpr int D = LPH * 8;
  constexpr int HPB = 256 / LPH;                     // heads a block covers at a time
  // With many tokens the values do not go through the heads' loop (a token alone would write them an element at a
  // time): blocks behind the tokens' own take 16 tokens of one kv head each (`value_groups` groups of 16 tokens).
  __shared__ __attribute__((aligned(16))) T tile[16][D + 8];
  __shared__ int together;
  if ((int)blockIdx.x >= tokens) {
    const int v = blockIdx.x - tokens;
    v_write_group<T, D + 8>(tile, &together, (v % value_groups) * 16, v / value_groups, qkv, qkv_stride, (heads + kv_heads) * D,
                     tokens, kv_heads, D, pages, write_page, write_off, page_size);
    return;
  }
  const int t = blockIdx.x;
  const int li = threadIdx.x % LPH;                  // lane within the head
  // Everything the block reads is asked for before anything is waited for, the longest chain first: the token's
  // position (then its cosines and sines, the same for every head of the token), its place in the cache, the head's
  // values, the norm's weight. A decode step runs this kernel on rows another kernel has just written, and each
  // round trip for them costs as much as the arithmetic.
  const int pos = table != nullptr ? positions[t] : 0;
  const int wpage = pages != nullptr ? write_page[t] : 0, woff = pages != nullptr ? write_off[t] : 0;
  float co[8], si[8];
  bool have_cs = table == nullptr;
  // a block takes HPB heads, then (with fewer blocks than that along y) the next HPB, ...
  for (int h0 = blockIdx.y * HPB; h0 < total_heads; h0 += gridDim.y * HPB) {
    const int h = h0 + threadIdx.x / LPH;
    const bool active = h < total_heads;             // (shuffles below are executed by every lane)
    const int hh = active ? h : 0;
    const T* src = qkv + (int64_t)t * qkv_stride + (int64_t)hh * D + li * 8;
    const bool is_v = hh >= heads + kv_heads;
    const bool is_q = hh < heads;
    const T* weight = is_q ? q_weight : k_weight;
    float v[8];
    T w[8];
    if (sizeof(T) == 2) {
      const uint4 raw = *reinterpret_cast<const uint4*>(src);
      if (weight != nullptr) *reinterpret_cast<uint4*>(w) = *reinterpret_cast<const uint4*>(weight + li * 8);
      const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = Elem<T>::load(e[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = Elem<T>::load(src[j]);
      if (weight != nullptr) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = weight[li * 8 + j];
      }
    }
    if (!have_cs) {
      const float* cs = table + (int64_t)pos * D + (li % (LPH / 2)) * 8;   // the pair's place within the half
      const float4 c0 = *reinterpret_cast<const float4*>(cs), c1 = *reinterpret_cast<const float4*>(cs + 4);
      const float4 s0 = *reinterpret_cast<const float4*>(cs + D / 2), s1 = *reinterpret_cast<const float4*>(cs + D / 2 + 4);
      co[0] = c0.x; co[1] = c0.y; co[2] = c0.z; co[3] = c0.w; co[4] = c1.x; co[5] = c1.y; co[6] = c1.z; co[7] = c1.w;
      si[0] = s0.x; si[1] = s0.y; si[2] = s0.z; si[3] = s0.w; si[4] = s1.x; si[5] = s1.y; si[6] = s1.z; si[7] = s1.w;
      have_cs = true;
    }
    if (active && is_v) {   // a value head: transposed inside the page
      const int hk = hh - heads - kv_heads;
      T* dst = pages + (((int64_t)wpage * 2 + 1) * kv_heads + hk) * (int64_t)page_size * D + woff;
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[(int64_t)(li * 8 + j) * page_size] = Elem<T>::store(v[j]);
    }
    if (weight != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
      ss = head_sum<LPH>(ss);
      const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = Elem<T>::round((v[j] * inv) * Elem<T>::load(w[j]));
    }
    if (table != nullptr) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float other = half_away<LPH>(v[j]);
        v[j] = li < LPH / 2 ? v[j] * co[j] - other * si[j] : v[j] * co[j] + other * si[j];
      }
    }
    if (!active || is_v) continue;
    T* dst = is_q ? q_out + ((int64_t)t * heads + hh) * D + li * 8
                  : pages + (((int64_t)wpage * 2 + 0) * kv_heads + (hh - heads)) * (int64_t)page_size * D +
                        (int64_t)woff * D + li * 8;
    if (sizeof(T) == 2) {
      uint4 out;
      T* oe = reinterpret_cast<T*>(&out);
#pragma unroll
      for (int j = 0; j < 8; ++j) oe[j] = Elem<T>::store(v[j]);
      *reinterpret_cast<uint4*>(dst) = out;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[j] = Elem<T>::store(v[j]);
    }
  }
}

extern "C" int holon_qk_norm_rope_write(const void* qkv, int64_t qkv_stride, void* q_out, int tokens, int heads,
                                        int kv_heads, int head_dim, const void* q_weight, const void* k_weight,
                                        float eps, const float* table, int rotary_dim, int max_positions,
                                        const int32_t* positions, void* pages, const int32_t* write_page,
                                        const int32_t* write_off, int page_size, int num_pages, int dtype,
                                        void* stream) {
  HOLON_CHECK(tokens >= 0 && heads > 0 && kv_heads >= 0 && head_dim > 0, "qk_norm_rope_write: bad sizes");
  HOLON_CHECK(head_dim <= MAX_HEAD_DIM, "qk_norm_rope_write: head_dim %d exceeds %d", head_dim, MAX_HEAD_DIM);
  HOLON_CHECK((q_weight == nullptr) == (k_weight == nullptr) || kv_heads == 0 || pages == nullptr,
              "qk_norm_rope_write: q and k norm weights must both be given or both be absent");
  HOLON_CHECK(table == nullptr || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= head_dim && positions),
              "qk_norm_rope_write: rotary_dim %d must be even and within head_dim %d", rotary_dim, head_dim);
  HOLON_CHECK(pages == nullptr || (write_page && write_off && page_size > 0 && num_pages > 0),
              "qk_norm_rope_write: a cache needs write targets and a page size");
  if (tokens == 0) return 0;
  const int total_heads = pages != nullptr ? heads + 2 * kv_heads : heads;
  dim3 grid(tokens, (total_heads + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
  if ((head_dim == 64 || head_dim == 128 || head_dim == 256) && (table == nullptr || rotary_dim == head_dim) &&
      qkv != q_out) {
    // many tokens: the values are written 16 tokens at a time (contiguous writes) by blocks of their own behind the
    // tokens' blocks in the same launch; the heads' loop then covers queries and keys only
    const bool split_v = pages != nullptr && tokens >= 256;
    const int fast_heads = split_v ? heads + kv_heads : total_heads;
    const int lph = head_dim / 8;
    const int value_groups = split_v ? (tokens + 15) / 16 : 0;
    // many tokens: one block a token walks all its heads, with the token's cosines and sines read once
    grid = dim3(tokens + value_groups * kv_heads, tokens >= 256 ? 1 : (fast_heads + 256 / lph - 1) / (256 / lph));
#define QK_FAST(T, LPH)                                                                                            \
  qk_norm_rope_write_fast_kernel<T, LPH><<<grid, 256, 0, s>>>(                                                      \
      (const T*)qkv, qkv_stride, (T*)q_out, heads, kv_heads, (const T*)q_weight, (const T*)k_weight, eps, table,    \
      positions, (T*)pages, write_page, write_off, page_size, fast_heads, tokens, value_groups)
    if (dtype == HOLON_F32) {
      if (head_dim == 64) QK_FAST(float, 8); else if (head_dim == 128) QK_FAST(float, 16); else QK_FAST(float, 32);
    } else {
      if (head_dim == 64) QK_FAST(bf16_t, 8); else if (head_dim == 128) QK_FAST(bf16_t, 16); else QK_FAST(bf16_t, 32);
    }
#undef QK_FAST
    HOLON_LAUNCH_OK();
    return 0;
  }
#define QK_LAUNCH(T)                                                                                              \
  qk_norm_rope_write_kernel<T><<<grid, 4 * WAVE, 0, s>>>((const T*)qkv, qkv_stride, (T*)q_out, heads, kv_heads,    \
                                                        head_dim, (const T*)q_weight, (const T*)k_weight, eps,    \
                                                        table, rotary_dim, positions, (T*)pages, write_page,      \
                                                        write_off, page_size, total_heads)
  if (dtype == HOLON_F32) QK_LAUNCH(float); else QK_LAUNCH(bf16_t);
#undef QK_LAUNCH
  HOLON_LAUNCH_OK();
  return 0;
}

// ---------------------------------------------------------------------------------------------------------------
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ pages,
                                const int32_t* __restrict__ write_page, const int32_t* __restrict__ write_off,
                                int kv_heads, int head_dim, int page_size) {
  const int t = blockIdx.x, hk = blockIdx.y;
  const int64_t plane = (int64_t)page_size * head_dim;
  const T* ks = k + ((int64_t)t * kv_heads + hk) * head_dim;
  const T* vs = v + ((int64_t)t * kv_heads + hk) * head_dim;
  T* kd = pages + (((int64_t)write_page[t] * 2 + 0) * kv_heads + hk) * plane + (int64_t)write_off[t] * head_dim;
  T* vd = pages + (((int64_t)write_page[t] * 2 + 1) * kv_heads + hk) * plane + write_off[t];
  for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
    kd[d] = ks[d];
    vd[(int64_t)d * page_size] = vs[d];
  }
}

extern "C" int holon_kv_write(const void* k, const void* v, void* pages, const int32_t* write_page,
                              const int32_t* write_off, int tokens, int kv_heads, int head_dim, int page_size,
                              int num_pages, int dtype, void* stream) {
  HOLON_CHECK(tokens >= 0 && kv_heads > 0 && head_dim > 0 && page_size > 0 && num_pages > 0, "kv_write: bad sizes");
  if (tokens == 0) return 0;
  dim3 grid(tokens, kv_heads);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    kv_write_kernel<float><<<grid, WAVE, 0, s>>>((const float*)k, (const float*)v, (float*)pages, write_page,
                                                 write_off, kv_heads, head_dim, page_size);
  else
    kv_write_kernel<bf16_t><<<grid, WAVE, 0, s>>>((const bf16_t*)k, (const bf16_t*)v, (bf16_t*)pages, write_page,
                                                  write_off, kv_heads, head_dim, page_size);
  HOLON_LAUNCH_OK();
  return 0;
}
