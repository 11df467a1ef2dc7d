// Sampling on the device: argmax, and temperature / top-k / top-p / min-p sampling by inverse CDF with a counter-based
// uniform (a hash of seed and position: no generator state, so a request's draws do not depend on batching). A row
// without a filter is walked in vocabulary order; a row with one in the order its filters sort it (largest value first,
// equal values by index), which is the order the kept tokens come out of the filters in. One block per row.
#include <type_traits>

#include "common.h"
#include "holon_hip.h"

#define SAMPLE_THREADS 1024

struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {   // larger value; on ties the smaller index
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

// (nothing to choose from, a row of NaN: index 0, or 0x7fffffff with `none_is_zero` off)
__device__ ArgMax block_argmax(const float* __restrict__ row, int vocab, float temp, bool none_is_zero = true) {
  __shared__ ArgMax part[SAMPLE_THREADS / WAVE];
  __shared__ ArgMax result;
  ArgMax best{-INFINITY, 0x7fffffff};
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {   // 16-byte loads where the row allows
    const float4* row4 = reinterpret_cast<const float4*>(row);
    const int n4 = vocab / 4, step = blockDim.x;
    int i = threadIdx.x;
    for (; i + 3 * step < n4; i += 4 * step) {           // four loads under way at a time
      float4 v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = row4[i + e * step];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int at = 4 * (i + e * step);
        best = better(best, ArgMax{v[e].x / temp, at});
        best = better(best, ArgMax{v[e].y / temp, at + 1});
        best = better(best, ArgMax{v[e].z / temp, at + 2});
        best = better(best, ArgMax{v[e].w / temp, at + 3});
      }
    }
    for (; i < n4; i += step) {
      const float4 v = row4[i];
      best = better(best, ArgMax{v.x / temp, 4 * i});
      best = better(best, ArgMax{v.y / temp, 4 * i + 1});
      best = better(best, ArgMax{v.z / temp, 4 * i + 2});
      best = better(best, ArgMax{v.w / temp, 4 * i + 3});
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) best = better(best, ArgMax{row[i] / temp, i});
  }
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    ArgMax other{__shfl_xor(best.v, o, WAVE), __shfl_xor(best.i, o, WAVE)};
    best = better(best, other);
  }
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    ArgMax r = part[0];
    for (int w = 1; w < (int)blockDim.x / WAVE; ++w) r = better(r, part[w]);
    if (r.i == 0x7fffffff && none_is_zero) r.i = 0;   // a row of NaN: the first token
    result = r;
  }
  __syncthreads();
  return result;
}

__global__ void argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int vocab) {
  const ArgMax r = block_argmax(logits + (int64_t)blockIdx.x * vocab, vocab, 1.0f);
  if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

// A wide row in two kernels: block (piece, row) finds the best of its ARGMAX_PIECE values, then one wave a row the best
// of the pieces (ties go to the smaller index in both, so the answer is the one block's). One block walking 151,936
// values alone takes 17.5 us; the two kernels together 9.4.
constexpr int ARGMAX_PIECE = 4096;
constexpr int ARGMAX_MAX_PIECES = 1024;
__global__ void __launch_bounds__(SAMPLE_THREADS) argmax_pieces_kernel(const float* __restrict__ logits,
                                                                        ArgMax* __restrict__ pieces, int vocab) {
  const int lo = blockIdx.x * ARGMAX_PIECE;
  const ArgMax r = block_argmax(logits + (int64_t)blockIdx.y * vocab + lo, min(ARGMAX_PIECE, vocab - lo), 1.0f, false);
  if (threadIdx.x == 0)
    pieces[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = ArgMax{r.v, r.i == 0x7fffffff ? r.i : r.i + lo};
}
__global__ void __launch_bounds__(WAVE) argmax_of_pieces_kernel(const ArgMax* __restrict__ pieces,
                                                                int32_t* __restrict__ out, int n) {
  ArgMax best{-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < n; i += WAVE) best = better(best, pieces[(int64_t)blockIdx.x * n + i]);
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    ArgMax other{__shfl_xor(best.v, o, WAVE), __shfl_xor(best.i, o, WAVE)};
    best = better(best, other);
  }
  if (threadIdx.x == 0) out[blockIdx.x] = best.i == 0x7fffffff ? 0 : best.i;
}

// `pieces`: room for holon_argmax_pieces(vocab) pairs of (float, int32) a row, or NULL (one block a row).
extern "C" int holon_argmax_pieces(int vocab) {
  const int n = (vocab + ARGMAX_PIECE - 1) / ARGMAX_PIECE;
  return n >= 4 && n <= ARGMAX_MAX_PIECES ? n : 0;
}

extern "C" int holon_argmax(const float* logits, int32_t* out, int rows, int vocab, void* pieces, void* stream) {
  HOLON_CHECK(rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (rows == 0) return 0;
  const int n = holon_argmax_pieces(vocab);
  if (pieces != nullptr && n > 0) {
    argmax_pieces_kernel<<<dim3(n, rows), SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, (ArgMax*)pieces, vocab);
    HOLON_LAUNCH_OK();
    argmax_of_pieces_kernel<<<rows, WAVE, 0, (hipStream_t)stream>>>((const ArgMax*)pieces, out, n);
  } else {
    argmax_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, out, vocab);
  }
  HOLON_LAUNCH_OK();
  return 0;
}

// last_token[slots[r]] = tokens[r]: the drawn tokens kept on the device, by slot, for the rows of the next step that
// are scheduled before these tokens reach the host.
__global__ void store_tokens_kernel(int32_t* __restrict__ last_token, const int32_t* __restrict__ slots,
                                    const int32_t* __restrict__ tokens, int rows, int n_slots) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < rows && slots[r] >= 0 && slots[r] < n_slots) last_token[slots[r]] = tokens[r];
}

extern "C" int holon_store_tokens(int32_t* last_token, const int32_t* slots, const int32_t* tokens, int rows,
                                  int n_slots, void* stream) {
  HOLON_CHECK(rows >= 0 && n_slots > 0, "store_tokens: bad sizes");
  if (rows == 0) return 0;
  store_tokens_kernel<<<(rows + 255) / 256, 256, 0, (hipStream_t)stream>>>(last_token, slots, tokens, rows, n_slots);
  HOLON_LAUNCH_OK();
  return 0;
}

// dst[idx[r], :] = src[r, :] for rows of `width` int32 values: the block-table rows that changed since the last step,
// brought with the step's other inputs, put into the device's table.
__global__ void scatter_rows_kernel(int32_t* __restrict__ dst, const int32_t* __restrict__ idx,
                                    const int32_t* __restrict__ src, int width, int dst_rows) {
  const int r = blockIdx.x, to = idx[r];
  if (to < 0 || to >= dst_rows) return;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[(int64_t)to * width + i] = src[(int64_t)r * width + i];
}

extern "C" int holon_scatter_rows(int32_t* dst, const int32_t* idx, const int32_t* src, int rows, int width,
                                  int dst_rows, void* stream) {
  HOLON_CHECK(rows >= 0 && width > 0 && dst_rows > 0, "scatter_rows: bad sizes");
  if (rows == 0) return 0;
  scatter_rows_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(dst, idx, src, width, dst_rows);
  HOLON_LAUNCH_OK();
  return 0;
}

// lowbias32, and the uniform of (seed, position): 24 bits, in (0, 1).
__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
  return x;
}
__device__ __forceinline__ float hashed_uniform(uint64_t seed, uint64_t position) {
  uint32_t h = mix32((uint32_t)seed) ^ (uint32_t)(seed >> 32) ^ mix32((uint32_t)position);
  h = mix32(h);
  const float u = ((float)(h >> 8) + 0.5f) * 5.9604644775390625e-08f;   // 2^-24
  return fminf(u, 1.0f - 5.9604644775390625e-08f);
}

__device__ float block_sum(float v) {
  __shared__ float part[SAMPLE_THREADS / WAVE];
  __shared__ float result;
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = 0.f;
    for (int w = 0; w < (int)blockDim.x / WAVE; ++w) r += part[w];
    result = r;
  }
  __syncthreads();
  return result;
}

__device__ int block_sum_int(int v) {
  __shared__ int part[SAMPLE_THREADS / WAVE];
  __shared__ int result;
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    int r = 0;
    for (int w = 0; w < (int)blockDim.x / WAVE; ++w) r += part[w];
    result = r;
  }
  __syncthreads();
  return result;
}

// Order-preserving map of a float onto unsigned integers (larger float, larger key; equal floats, equal keys: -0 is
// made +0 first, the two being the same value with different bits).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f + 0.0f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// The law of a row: q_i = exp(x_i - max) where kept, 0 where a filter drops token i; x = logit / temperature.
// Filters in order (the reference's): top-k keeps the k largest (ties: lower index first); top-p keeps, in descending
// order, tokens whose preceding mass is <= top_p of the top-k mass (the largest always stays); min-p keeps q >= min_p
// times the largest q. A token is identified for ties by (value, index), so the kept set is exact.
// The general form: any k, any kept set, and the draw in sorted order. Bisection on the ordered keys, one pass over the
// row per step, every thread a contiguous segment of the row (so that ranks among equal values follow the index):
// exact but slow, for the rows whose kept set does not fit the fast form below.
__device__ void sample_row_general(const float* __restrict__ row, int32_t* __restrict__ out_r, int vocab, float temp,
                                   ArgMax top, int k, float p_keep, float p_min, float u) {
  const float xmax = top.v;

  // --- top-k: the k-th largest key, and how many of the tokens equal to it are kept (the first ones by index)
  uint32_t kth_key = 0;          // keep x with key > kth_key, plus the first `ties_kept` tokens with key == kth_key
  int ties_kept = 0x7fffffff;
  if (k > 0 && k < vocab) {
    uint32_t lo = 0, hi = 0xffffffffu;   // the largest key K with count(key >= K) >= k
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) / 2);
      int c = 0;
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) c += float_key(row[i] / temp) >= mid;
      if (block_sum_int(c) >= k) lo = mid; else hi = mid - 1;
    }
    kth_key = lo;
    int above = 0;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) above += float_key(row[i] / temp) > kth_key;
    ties_kept = k - block_sum_int(above);
  }
  // rank among equals needs an index-ordered count: each thread owns a contiguous segment of the row
  const int seg = (vocab + blockDim.x - 1) / blockDim.x;
  const int seg_lo = min(vocab, (int)threadIdx.x * seg), seg_hi = min(vocab, seg_lo + seg);
  __shared__ int scan_i[SAMPLE_THREADS];
  int ties_before = 0;           // tokens equal to the k-th value in earlier segments
  if (ties_kept != 0x7fffffff) {
    int mine = 0;
    for (int i = seg_lo; i < seg_hi; ++i) mine += float_key(row[i] / temp) == kth_key;
    scan_i[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
      int run = 0;
      for (int t = 0; t < (int)blockDim.x; ++t) { const int v = scan_i[t]; scan_i[t] = run; run += v; }
    }
    __syncthreads();
    ties_before = scan_i[threadIdx.x];
    __syncthreads();
  }
  auto in_top_k = [&](float x, int& tie_rank) -> bool {   // call in index order within the segment
    if (ties_kept == 0x7fffffff) return true;
    const uint32_t key = float_key(x);
    if (key > kth_key) return true;
    if (key == kth_key) return tie_rank++ < ties_kept;
    return false;
  };

  // --- mass after top-k
  float part = 0.f;
  {
    int tie_rank = ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] / temp;
      if (in_top_k(x, tie_rank)) part += expf(x - xmax);
    }
  }
  const float z_k = block_sum(part);

  // --- top-p: the smallest key K such that the mass of tokens above K (strictly) is <= top_p * z_k; tokens with
  // key >= K are kept, those equal to K as long as the mass before each stays within the bound.
  uint32_t p_key = 0;
  float p_budget = INFINITY;     // mass that may precede a token equal to p_key
  float p_each = 0.f;            // mass of one token equal to p_key
  if (p_keep < 1.0f) {
    const float bound = p_keep * z_k;
    uint32_t lo = 0, hi = float_key(xmax);   // mass_above(hi) = 0 <= bound always
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float above = 0.f;
      int tie_rank = ties_before;
      for (int i = seg_lo; i < seg_hi; ++i) {
        const float x = row[i] / temp;
        const bool kept = in_top_k(x, tie_rank);
        if (kept && float_key(x) > mid) above += expf(x - xmax);
      }
      if (block_sum(above) <= bound) hi = mid; else lo = mid + 1;
    }
    p_key = lo;
    float above = 0.f;
    int tie_rank = ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] / temp;
      const bool kept = in_top_k(x, tie_rank);
      if (kept && float_key(x) > p_key) above += expf(x - xmax);
    }
    p_budget = bound - block_sum(above);
    p_each = expf(key_float(p_key) - xmax);
  }
  // tokens equal to p_key, in index order, each preceded by (rank * p_each) more mass
  int p_ties_before = 0;
  if (p_keep < 1.0f) {
    int mine = 0, tie_rank = ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] / temp;
      const bool kept = in_top_k(x, tie_rank);
      mine += kept && float_key(x) == p_key;
    }
    scan_i[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
      int run = 0;
      for (int t = 0; t < (int)blockDim.x; ++t) { const int v = scan_i[t]; scan_i[t] = run; run += v; }
    }
    __syncthreads();
    p_ties_before = scan_i[threadIdx.x];
    __syncthreads();
  }
  const float q_floor = p_min > 0.f ? p_min : 0.f;   // min-p: q / q_max >= min_p, and q_max = exp(0) = 1

  auto law = [&](float x, int& tie_rank, int& p_rank) -> float {
    if (!in_top_k(x, tie_rank)) return 0.f;
    const float qv = expf(x - xmax);
    if (p_keep < 1.0f) {
      const uint32_t key = float_key(x);
      if (key < p_key) return 0.f;
      if (key == p_key && !((float)(p_rank++) * p_each <= p_budget)) return 0.f;
    }
    if (qv < q_floor) return 0.f;
    return qv;
  };

  // --- draw: inverse CDF in sorted order (value descending, equal values by index). The drawn token's key is the
  // smallest K with kept mass above K (strictly) <= target; among the kept tokens equal to K, the one whose rank times
  // their common mass first passes what the target leaves.
  float mine = 0.f;
  {
    int tie_rank = ties_before, p_rank = p_ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) mine += law(row[i] / temp, tie_rank, p_rank);
  }
  const float total = block_sum(mine);
  const float target = u * total;
  uint32_t d_key;
  {
    uint32_t lo = 0, hi = float_key(xmax);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float above = 0.f;
      int tie_rank = ties_before, p_rank = p_ties_before;
      for (int i = seg_lo; i < seg_hi; ++i) {
        const float x = row[i] / temp;
        const float qv = law(x, tie_rank, p_rank);
        if (float_key(x) > mid) above += qv;
      }
      if (block_sum(above) <= target) hi = mid; else lo = mid + 1;
    }
    d_key = lo;
  }
  float above = 0.f;
  int ties_mine = 0;
  {
    int tie_rank = ties_before, p_rank = p_ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] / temp;
      const float qv = law(x, tie_rank, p_rank);
      const uint32_t key = float_key(x);
      if (key > d_key) above += qv;
      ties_mine += key == d_key && qv > 0.f;
    }
  }
  above = block_sum(above);
  scan_i[threadIdx.x] = ties_mine;
  __syncthreads();
  __shared__ int n_ties_s;
  if (threadIdx.x == 0) {
    int run = 0;
    for (int t = 0; t < (int)blockDim.x; ++t) { const int v = scan_i[t]; scan_i[t] = run; run += v; }
    n_ties_s = run;
  }
  __syncthreads();
  const int d_before = scan_i[threadIdx.x], n_ties = n_ties_s;
  const float each = expf(key_float(d_key) - xmax);
  int want = each > 0.f ? (int)fminf((target - above) / each, 2147483000.f) : 0;
  want = max(0, min(want, n_ties - 1));
  __shared__ int chosen;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  if (ties_mine > 0 && d_before <= want && want < d_before + ties_mine) {   // (one thread)
    int tie_rank = ties_before, p_rank = p_ties_before, rank = d_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] / temp;
      const float qv = law(x, tie_rank, p_rank);
      if (float_key(x) == d_key && qv > 0.f && rank++ == want) { chosen = i; break; }
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) *out_r = chosen >= 0 ? chosen : top.i;
}

// ---------------------------------------------------------------------------------------------------------------
// The fast form. Masses are integers, Q = trunc(exp(x - max) * (2^32 - 256)): sums of them are exact in any order, so
// every decision below is the same whatever the threads' order, and a sum over a part of the row is exact too.
//   1. the largest value;
//   2. (top-k is set) how many tokens lie in each of 16 bands below the largest value (within 1, 2, ... 8, 12, 16,
//      ... 128); the fewest bands that are sure to hold the kept set are collected into LDS (at most SAMPLE_CANDIDATES
//      tokens) and sorted by (value descending, index ascending): the order in which top-k and top-p take tokens.
//      (top-p alone) the row's mass and token counts in 2,048 bins below the largest value say which bin holds the last
//      kept token and how many tokens precede it: a kept set that fits is collected whole and sorted, of a longer one
//      only that bin, which gives the cut. A cut that cannot be found this way is found by halving ranges, and where
//      thousands of equal values lie at the cut the row takes the general form;
//   3. top-k keeps the first k of the sorted set; top-p those whose preceding mass is <= top_p * (mass of what top-k
//      kept); both keep a prefix, so the kept set is "(value, index) at or before the last kept one": one compare;
//   4. min-p drops q < min_p (the largest q is 1): a prefix again; the draw is the inverse CDF over the integer masses
//      of the kept tokens as they lie sorted. A row without a filter is drawn in vocabulary order instead: sums of 256
//      consecutive tokens, the 256 that hold the target found among those sums, one scan of them.
#define SAMPLE_CANDIDATES 4096
#define SAMPLE_WAVES (SAMPLE_THREADS / WAVE)
#define SAMPLE_PER (SAMPLE_CANDIDATES / SAMPLE_THREADS)
#define SAMPLE_BANDS 16
#define SAMPLE_CHUNK 256
typedef unsigned long long u64;

// The band of a token d = max - x below the largest value: 0..7 for d in [0, 8) by ones, then [8, 12), [12, 16),
// [16, 24), [24, 32), [32, 48), [48, 64), [64, 96), [96, 128); SAMPLE_BANDS beyond (or for a NaN).
__device__ __forceinline__ int near_band(float d) {
  if (!(d < 128.f)) return SAMPLE_BANDS;
  const int di = (int)d;
  if (di < 8) return di;
  const int e = 31 - __clz(di);                 // 3 .. 6
  return 8 + 2 * (e - 3) + ((di >> (e - 1)) & 1);
}
__device__ __forceinline__ float band_edge(int band) {   // tokens beyond bands 0 .. band are at least this far below
  const float edges[SAMPLE_BANDS] = {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24, 32, 48, 64, 96, 128};
  return edges[band];
}

__device__ __forceinline__ uint32_t fixed_mass(float q) { return (uint32_t)(q * 4294967040.0f); }   // q in [0, 1]
__device__ __forceinline__ u64 order_key(float x, int i) {   // larger = taken earlier
  return ((u64)float_key(x) << 32) | (uint32_t)(0x7fffffff - i);
}

__device__ __forceinline__ u64 shfl_u64(u64 v, int src) {
  return ((u64)__shfl((uint32_t)(v >> 32), src, WAVE) << 32) | __shfl((uint32_t)v, src, WAVE);
}
__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, o, WAVE), hi = __shfl_xor((uint32_t)(v >> 32), o, WAVE);
    v += ((u64)hi << 32) | lo;
  }
  return v;
}
__device__ __forceinline__ u64 wave_scan_u64(u64 v, int lane) {   // inclusive, over the lanes in order
#pragma unroll
  for (int o = 1; o < WAVE; o <<= 1) {
    const uint32_t lo = __shfl_up((uint32_t)v, o, WAVE), hi = __shfl_up((uint32_t)(v >> 32), o, WAVE);
    if (lane >= o) v += ((u64)hi << 32) | lo;
  }
  return v;
}
__device__ u64 block_sum_u64(u64 v) {
  __shared__ u64 part[SAMPLE_WAVES];
  __shared__ u64 result;
  v = wave_sum_u64(v);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    u64 r = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) r += part[w];
    result = r;
  }
  __syncthreads();
  return result;
}
// The sum of `v` over the threads before this one (thread order), and the whole sum.
__device__ u64 block_scan_u64(u64 v, u64& total) {
  __shared__ u64 part[SAMPLE_WAVES];
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const u64 incl = wave_scan_u64(v, lane);
  __syncthreads();
  if (lane == WAVE - 1) part[wave] = incl;
  __syncthreads();
  u64 before = 0, all = 0;
  for (int w = 0; w < SAMPLE_WAVES; ++w) {
    if (w < wave) before += part[w];
    all += part[w];
  }
  total = all;
  return before + incl - v;
}

// f(x, i) for every token of the row, x = logit / temp, in no particular order: 16-byte loads where the row allows.
template <typename F>
__device__ __forceinline__ void for_each_token(const float* __restrict__ row, int vocab, float temp, F f) {
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    // four loads under way at a time: a block walks its row alone, and what it waits for is the loads
    const float4* row4 = reinterpret_cast<const float4*>(row);
    const int n4 = vocab / 4, step = blockDim.x;
    int i = threadIdx.x;
    for (; i + 3 * step < n4; i += 4 * step) {
      float4 v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = row4[i + e * step];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int at = 4 * (i + e * step);
        f(v[e].x / temp, at); f(v[e].y / temp, at + 1); f(v[e].z / temp, at + 2); f(v[e].w / temp, at + 3);
      }
    }
    for (; i < n4; i += step) {
      const float4 v = row4[i];
      f(v.x / temp, 4 * i); f(v.y / temp, 4 * i + 1); f(v.z / temp, 4 * i + 2); f(v.w / temp, 4 * i + 3);
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) f(row[i] / temp, i);
  }
}

// About how many tokens lie in bands 0 .. j below the largest value, for every j, into counts[] (shared): every eighth
// stretch of the row is counted (a token's place in the vocabulary says nothing about its value), a thread counting in
// 8-bit fields of two registers.
__device__ void estimate_band_counts(const float* __restrict__ row, int vocab, float temp, float xmax, int* counts,
                                     int (*band_counts)[SAMPLE_BANDS]) {
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  u64 near_lo = 0, near_hi = 0;                  // bands 0..7 and 8..15
  const int stretch = 4 * SAMPLE_THREADS;        // tokens a pass of the block covers
  for (int base = 0; base < vocab; base += 8 * stretch) {
    const int i0 = base + 4 * tid;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (i0 + e < vocab) {
        const int band = near_band(xmax - row[i0 + e] / temp);
        if (band < 8) near_lo += 1ull << (8 * band); else if (band < SAMPLE_BANDS) near_hi += 1ull << (8 * (band - 8));
      }
    }
  }
  // the fields widened to 16 bits (a wave's sum fits), added over the wave, then over the waves
  u64 wide[4];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const uint32_t four = (uint32_t)((h < 2 ? near_lo : near_hi) >> (32 * (h & 1)));
    wide[h] = wave_sum_u64((u64)(four & 0xff) | ((u64)((four >> 8) & 0xff) << 16) | ((u64)((four >> 16) & 0xff) << 32) |
                           ((u64)(four >> 24) << 48));
  }
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < SAMPLE_BANDS; ++j) band_counts[wave][j] = (int)((wide[j / 4] >> (16 * (j % 4))) & 0xffff);
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int j = 0; j < SAMPLE_BANDS; ++j) {
      for (int w = 0; w < SAMPLE_WAVES; ++w) run += band_counts[w][j];
      counts[j] = 8 * run;
    }
  }
  __syncthreads();
}

// The tokens of bands 0 .. `bands` into cand[] as order keys, in no order; returns how many there are (the same in
// every thread), of which only the first SAMPLE_CANDIDATES were stored.
__device__ int collect_bands(const float* __restrict__ row, int vocab, float temp, float xmax, int bands, u64* cand,
                             int* n_cand) {
  if (threadIdx.x == 0) *n_cand = 0;
  __syncthreads();
  const float edge = band_edge(bands);
  for_each_token(row, vocab, temp, [&](float x, int i) {
    if (xmax - x < edge) {
      const int at = atomicAdd(n_cand, 1);
      if (at < SAMPLE_CANDIDATES) cand[at] = order_key(x, i);
    }
  });
  __syncthreads();
  const int count = *n_cand;
  __syncthreads();
  return count;
}

// Bitonic sort of a[0 .. n_pad) in LDS by the whole block; n_pad is a power of two.
__device__ void bitonic_sort(u64* a, int n_pad, bool descending) {
  for (int size = 2; size <= n_pad; size <<= 1) {
    for (int stride = size / 2; stride > 0; stride >>= 1) {
      for (int i = threadIdx.x; i < n_pad; i += blockDim.x) {
        const int partner = i ^ stride;
        if (partner > i) {
          const u64 x = a[i], y = a[partner];
          const bool down = ((i & size) == 0) == descending;
          if (down ? x < y : x > y) { a[i] = y; a[partner] = x; }
        }
      }
      __syncthreads();
    }
  }
}

// Top-p alone over a kept set too large to collect. The range of values that holds the last kept token is halved
// until few enough tokens lie in it: `above` is the mass of the tokens over the range (all kept: it is within the
// bound), and more than the bound lies over the range's lower end. The tokens of the range are then collected and
// sorted, and the kept ones among them are those whose preceding mass, `above` included, is within the bound. Returns
// the order key of the last kept token, or 0 when the range cannot be narrowed (thousands of equal values).
__device__ u64 top_p_cut_wide(const float* __restrict__ row, int vocab, float temp, float xmax, u64 bound, u64* cand,
                              int* n_cand) {
  __shared__ int kept_s;
  const int tid = threadIdx.x;
  float x_hi = xmax, x_lo = xmax - 128.f;        // (what lies further below weighs nothing)
  u64 above = 0;
  for (int step = 0;; ++step) {
    const float x_mid = 0.5f * (x_lo + x_hi);
    if (step == 48 || !(x_mid > x_lo && x_mid < x_hi)) return 0;
    u64 mass = 0;
    int up = 0, down = 0;
    for_each_token(row, vocab, temp, [&](float x, int) {
      if (x > x_mid && x <= x_hi) { mass += fixed_mass(__expf(x - xmax)); ++up; }
      else if (x > x_lo && x <= x_mid) ++down;
    });
    mass = block_sum_u64(mass);
    up = block_sum_int(up);
    down = block_sum_int(down);
    int inside;
    if (above + mass <= bound) { x_hi = x_mid; above += mass; inside = down; }
    else { x_lo = x_mid; inside = up; }
    if (inside <= SAMPLE_CANDIDATES) break;
  }
  if (tid == 0) *n_cand = 0;
  __syncthreads();
  for_each_token(row, vocab, temp, [&](float x, int i) {
    if (x > x_lo && x <= x_hi) {
      const int at = atomicAdd(n_cand, 1);
      if (at < SAMPLE_CANDIDATES) cand[at] = order_key(x, i);
    }
  });
  __syncthreads();
  const int count = *n_cand;
  int n_pad = WAVE;
  while (n_pad < count) n_pad <<= 1;
  for (int i = count + tid; i < n_pad; i += blockDim.x) cand[i] = 0;
  __syncthreads();
  bitonic_sort(cand, n_pad, true);
  const int per = max(1, n_pad / SAMPLE_THREADS);
  u64 incl[SAMPLE_PER];
  u64 run = 0;
#pragma unroll
  for (int e = 0; e < SAMPLE_PER; ++e) {
    const int i = tid * per + e;
    if (e < per && i < count) run += fixed_mass(__expf(key_float((uint32_t)(cand[i] >> 32)) - xmax));
    incl[e] = run;
  }
  u64 all;
  const u64 before = above + block_scan_u64(run, all);
  int mine = 0;
#pragma unroll
  for (int e = 0; e < SAMPLE_PER; ++e) {
    const int i = tid * per + e;
    if (e < per && i < count) mine += (before + (e ? incl[e - 1] : 0)) <= bound;
  }
  const int kept = block_sum_int(mine);
  if (tid == 0) kept_s = kept;
  __syncthreads();
  // nothing of the range kept: the last kept token is the smallest over the range, i.e. any value over x_hi passes
  return kept_s > 0 ? cand[kept_s - 1] : ((u64)(float_key(x_hi) + 1u) << 32);
}

// Top-k over a kept set too large to collect (a k beyond the room, or a flat row): the same halving, by count. `above`
// tokens lie over the range and the k-th lies inside it; the range's tokens are then collected and sorted, and the
// (k - above)-th of them is the last kept one. Sets `cut` to its order key (0 when fewer than k tokens weigh anything:
// all are kept); false when the range cannot be narrowed.
__device__ bool top_k_cut_wide(const float* __restrict__ row, int vocab, float temp, float xmax, int k, u64* cand,
                               int* n_cand, u64& cut) {
  const int tid = threadIdx.x;
  float x_hi = xmax, x_lo = xmax - 128.f;        // (what lies further below weighs nothing)
  int above = 0;
  {
    int within = 0;
    for_each_token(row, vocab, temp, [&](float x, int) { within += x > x_lo; });
    if (block_sum_int(within) <= k) { cut = 0; return true; }
  }
  for (int step = 0;; ++step) {
    const float x_mid = 0.5f * (x_lo + x_hi);
    if (step == 48 || !(x_mid > x_lo && x_mid < x_hi)) return false;
    int up = 0, down = 0;
    for_each_token(row, vocab, temp, [&](float x, int) {
      if (x > x_mid && x <= x_hi) ++up;
      else if (x > x_lo && x <= x_mid) ++down;
    });
    up = block_sum_int(up);
    down = block_sum_int(down);
    int inside;
    if (above + up >= k) { x_lo = x_mid; inside = up; }
    else { above += up; x_hi = x_mid; inside = down; }
    if (inside <= SAMPLE_CANDIDATES) break;
  }
  if (tid == 0) *n_cand = 0;
  __syncthreads();
  for_each_token(row, vocab, temp, [&](float x, int i) {
    if (x > x_lo && x <= x_hi) {
      const int at = atomicAdd(n_cand, 1);
      if (at < SAMPLE_CANDIDATES) cand[at] = order_key(x, i);
    }
  });
  __syncthreads();
  const int count = *n_cand;
  int n_pad = WAVE;
  while (n_pad < count) n_pad <<= 1;
  for (int i = count + tid; i < n_pad; i += blockDim.x) cand[i] = 0;
  __syncthreads();
  bitonic_sort(cand, n_pad, true);
  cut = cand[min(count, k - above) - 1];
  __syncthreads();
  return true;
}

// ---- a row's mass by distance below its largest value -----------------------------------------------------------
// Bins of 1/64 down to 32 below the largest value (what lies further weighs nothing): the mass and the number of the
// tokens in each. With it "the last token, in sorted order, that has at most a given mass before it" (top-p's last
// kept token; the drawn token, with the target as the bound) lies in a known bin, and only that bin's tokens have to be
// collected and sorted, however many tokens precede them. The masses are integers, so the sums are exact.
#define HIST_BINS 2048
__device__ __forceinline__ int hist_bin(float d) { return d < 32.f ? (int)(d * 64.f) : HIST_BINS; }   // (a NaN: none)

// Fills the bins; returns the row's mass.
__device__ u64 mass_histogram(const float* __restrict__ row, int vocab, float temp, float xmax, u64* h_mass, int* h_cnt) {
  for (int i = threadIdx.x; i < HIST_BINS; i += blockDim.x) { h_mass[i] = 0; h_cnt[i] = 0; }
  __syncthreads();
  for_each_token(row, vocab, temp, [&](float x, int) {
    const int b = hist_bin(xmax - x);
    if (b < HIST_BINS) {
      atomicAdd(&h_mass[b], (u64)fixed_mass(__expf(x - xmax)));
      atomicAdd(&h_cnt[b], 1);
    }
  });
  __syncthreads();
  u64 mine = 0;
  for (int i = threadIdx.x; i < HIST_BINS; i += blockDim.x) mine += h_mass[i];
  return block_sum_u64(mine);
}

struct BinAt {
  int bin;        // the first bin at whose end more than the bound has gone by; HIST_BINS: the whole row is within it
  u64 before;     // the mass of the bins before it
  int n_before;   // their tokens
};
__device__ BinAt bin_past(const u64* h_mass, const int* h_cnt, u64 bound) {
  __shared__ BinAt found;
  constexpr int PER = HIST_BINS / SAMPLE_THREADS;
  const int tid = threadIdx.x;
  u64 mine = 0, n_mine = 0;
#pragma unroll
  for (int e = 0; e < PER; ++e) { mine += h_mass[tid * PER + e]; n_mine += (u64)h_cnt[tid * PER + e]; }
  u64 total, n_total;
  const u64 before = block_scan_u64(mine, total);
  const u64 n_before = block_scan_u64(n_mine, n_total);
  if (tid == 0) found = BinAt{HIST_BINS, total, (int)n_total};
  __syncthreads();
  if (before <= bound && bound < before + mine) {      // (one thread)
    u64 run = before;
    int n = (int)n_before;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const u64 m = h_mass[tid * PER + e];
      if (run + m > bound) { found = BinAt{tid * PER + e, run, n}; break; }
      run += m;
      n += h_cnt[tid * PER + e];
    }
  }
  __syncthreads();
  const BinAt at = found;
  __syncthreads();
  return at;
}

// The tokens of bins lo .. hi into cand[] as order keys, sorted (taken earlier first) and padded with zeros to a power
// of two, which `n_pad` receives; returns how many there are. The caller knows from the bins' counts that they fit.
__device__ int collect_bins_sorted(const float* __restrict__ row, int vocab, float temp, float xmax, int lo, int hi,
                                   u64* cand, int* n_cand, int& n_pad) {
  if (threadIdx.x == 0) *n_cand = 0;
  __syncthreads();
  for_each_token(row, vocab, temp, [&](float x, int i) {
    const int b = hist_bin(xmax - x);
    if (b >= lo && b <= hi) {
      const int at = atomicAdd(n_cand, 1);
      if (at < SAMPLE_CANDIDATES) cand[at] = order_key(x, i);
    }
  });
  __syncthreads();
  const int count = min(*n_cand, SAMPLE_CANDIDATES);
  n_pad = WAVE;
  while (n_pad < count) n_pad <<= 1;
  for (int i = count + threadIdx.x; i < n_pad; i += blockDim.x) cand[i] = 0;
  __syncthreads();
  bitonic_sort(cand, n_pad, true);
  return count;
}

// cand[0 .. count) sorted, `above` the mass of what precedes them all: how many of them have at most `bound` before
// them (a prefix, as the sums only grow), and in `through` the mass up to and including the last of those.
__device__ int within_bound(const u64* cand, int count, int n_pad, float xmax, u64 above, u64 bound, u64& through) {
  __shared__ u64 through_s;
  const int tid = threadIdx.x;
  const int per = max(1, n_pad / SAMPLE_THREADS);     // 1, 2 or 4
  u64 incl[SAMPLE_PER];
  u64 run = 0;
#pragma unroll
  for (int e = 0; e < SAMPLE_PER; ++e) {
    const int i = tid * per + e;
    if (e < per && i < count) run += fixed_mass(__expf(key_float((uint32_t)(cand[i] >> 32)) - xmax));
    incl[e] = run;
  }
  u64 all;
  const u64 before = above + block_scan_u64(run, all);
  int mine = 0;
#pragma unroll
  for (int e = 0; e < SAMPLE_PER; ++e) {
    const int i = tid * per + e;
    if (e < per && i < count) mine += (before + (e ? incl[e - 1] : 0)) <= bound;
  }
  const int kept = block_sum_int(mine);
  if (tid == 0) through_s = above;
  __syncthreads();
#pragma unroll
  for (int e = 0; e < SAMPLE_PER; ++e)
    if (e < per && tid * per + e == kept - 1) through_s = before + incl[e];
  __syncthreads();
  through = through_s;
  __syncthreads();
  return kept;
}

// The order key of the last token, in sorted order, with at most `bound` before it, from the bins: 0 when the bin
// that holds it has more tokens than there is room for, or when the whole row lies within the bound (the caller then
// halves ranges instead). `through`: the mass up to and including that token.
__device__ u64 last_within(const float* __restrict__ row, int vocab, float temp, float xmax, u64 bound,
                           const u64* h_mass, const int* h_cnt, u64* cand, int* n_cand, u64& through) {
  const BinAt at = bin_past(h_mass, h_cnt, bound);
  if (at.bin == HIST_BINS || h_cnt[at.bin] > SAMPLE_CANDIDATES) return 0;
  int n_pad;
  const int count = collect_bins_sorted(row, vocab, temp, xmax, at.bin, at.bin, cand, n_cand, n_pad);
  const int kept = within_bound(cand, count, n_pad, xmax, at.before, bound, through);   // >= 1: the bin's first token
  const u64 key = cand[max(kept, 1) - 1];
  __syncthreads();
  return key;
}

__global__ void __launch_bounds__(SAMPLE_THREADS) sample_kernel(
    const float* __restrict__ logits, int32_t* __restrict__ out, int vocab, const float* __restrict__ temperature,
    const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
    const int64_t* __restrict__ seeds, const void* __restrict__ positions, const int32_t* __restrict__ slots,
    int positions_i32) {
  __shared__ u64 cand[SAMPLE_CANDIDATES];      // order keys of the collected tokens, sorted; later the sums of 256 tokens
  __shared__ int counts[SAMPLE_BANDS];
  __shared__ int band_counts[SAMPLE_WAVES][SAMPLE_BANDS];
  __shared__ int n_cand, n_keep_s, pick_s;
  __shared__ u64 z_k_s;
  __shared__ u64 h_mass[HIST_BINS];
  __shared__ int h_cnt[HIST_BINS];
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const float* row = logits + (int64_t)r * vocab;
  const int pr = slots != nullptr ? slots[r] : r;     // where this row's parameters lie: by its slot, or by its place
  const float temp = temperature[pr];
  if (temp == 0.f) {
    const ArgMax a = block_argmax(row, vocab, 1.0f);
    if (tid == 0) out[r] = a.i;
    return;
  }
  const ArgMax top = block_argmax(row, vocab, temp);
  const float xmax = top.v;
  const int k = top_k[pr];
  const float p_keep = top_p[pr], p_min = min_p[pr];
  const uint64_t position = positions_i32 ? (uint64_t)((const int32_t*)positions)[r] : (uint64_t)((const int64_t*)positions)[r];
  const float u = hashed_uniform((uint64_t)seeds[pr], position);
  const bool k_on = k > 0 && k < vocab, p_on = p_keep < 1.0f;
  const int chunks = (vocab + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  const bool m_on = p_min > 0.f;
  const bool filtered = k > 0 || p_on || m_on;
  if (filtered && vocab > 255 * SAMPLE_THREADS) {      // (uniform over the block)
    sample_row_general(row, out + r, vocab, temp, top, k, p_keep, p_min, u);
    return;
  }

  // A row with a filter. Its kept set is a prefix of the sorted order; where that prefix fits the room in LDS it is
  // collected, sorted and drawn from there, else (`wide`) it is described by `cut`: tokens with order_key >= cut pass
  // top-k and top-p (0: all do), and min-p is a bound on q.
  if (filtered) {
    u64 cut = 0;
    bool wide = !(k_on || p_on || m_on);         // k >= vocab and nothing else: everything is kept, in sorted order
    bool binned = false;                         // h_mass / h_cnt hold this row
    u64 kept_mass = 0;                           // (wide, top-p alone, no min-p) the mass of the kept tokens, else 0
    if (p_on && !k_on) {
      // top-p alone: the row's mass by bins says which bin holds the last kept token and how many tokens precede it.
      // A kept set that fits the room is collected whole, sorted, and drawn from there; of a larger one only that bin.
      const u64 z_all = mass_histogram(row, vocab, temp, xmax, h_mass, h_cnt);
      binned = true;
      const u64 bound = (u64)((double)p_keep * (double)z_all);
      const BinAt at = bin_past(h_mass, h_cnt, bound);
      if (at.bin == HIST_BINS) {
        wide = true;                             // (a row whose mass rounds to the bound: everything is kept)
      } else if (at.n_before + h_cnt[at.bin] <= SAMPLE_CANDIDATES) {
        int n_pad;
        const int count = collect_bins_sorted(row, vocab, temp, xmax, 0, at.bin, cand, &n_cand, n_pad);
        u64 through;
        const int kept = within_bound(cand, count, n_pad, xmax, 0, bound, through);
        if (tid == 0) n_keep_s = kept;
        __syncthreads();
      } else {
        wide = true;
        u64 through = 0;
        cut = last_within(row, vocab, temp, xmax, bound, h_mass, h_cnt, cand, &n_cand, through);
        if (cut != 0 && !m_on) kept_mass = through;
        if (cut == 0) cut = top_p_cut_wide(row, vocab, temp, xmax, bound, cand, &n_cand);
        if (cut == 0) {                          // thousands of equal values where the cut falls
          sample_row_general(row, out + r, vocab, temp, top, k, p_keep, p_min, u);
          return;
        }
      }
    } else if (k_on || p_on) {
      u64 z_all = 0;
      if (!k_on) {                               // top-p without top-k: the mass of the whole row
        u64 mass = 0;
        for_each_token(row, vocab, temp, [&](float x, int) { mass += fixed_mass(__expf(x - xmax)); });
        z_all = block_sum_u64(mass);
      }
      wide = k_on && k > SAMPLE_CANDIDATES;      // no room for the kept set whatever the bands
      if (!wide) estimate_band_counts(row, vocab, temp, xmax, counts, band_counts);
      // Which bands to collect: the fewest that should hold twice what is needed (k tokens; 256 for top-p alone). The
      // collecting counts exactly; too many, or fewer than k, and another set of bands is tried.
      const int need = k_on ? k : 1;
      int beyond_at = -1;                        // the most bands found to hold too little of the mass
      int bands = SAMPLE_BANDS - 1;
      for (int j = SAMPLE_BANDS - 1; j >= 0; --j)
        if (counts[j] >= 2 * (k_on ? k : 256) + 64) bands = j;
      while (bands > 0 && counts[bands] > SAMPLE_CANDIDATES / 2 && counts[bands - 1] >= 2 * need) --bands;
      for (int attempt = 0; !wide; ++attempt) {
        if (attempt == 6 || bands < 0 || bands >= SAMPLE_BANDS) {
          wide = true;
          break;
        }
        const int count = collect_bands(row, vocab, temp, xmax, bands, cand, &n_cand);
        if (count > SAMPLE_CANDIDATES) {
          --bands;
          if (bands <= beyond_at) attempt = 5;    // the next fewer bands held too little: no set of bands will do
          continue;
        }
        if (count < need && count < vocab) { ++bands; continue; }
        int n_pad = WAVE;
        while (n_pad < count) n_pad <<= 1;
        for (int i = count + tid; i < n_pad; i += blockDim.x) cand[i] = 0;   // after every real key
        __syncthreads();
        bitonic_sort(cand, n_pad, true);
        // masses in sorted order: a thread holds consecutive ones and the sum of everything before them
        const int per = max(1, n_pad / SAMPLE_THREADS);     // 1, 2 or 4
        u64 incl[SAMPLE_PER];
        u64 run = 0;
#pragma unroll
        for (int e = 0; e < SAMPLE_PER; ++e) {
          const int i = tid * per + e;
          if (e < per && i < count) run += fixed_mass(__expf(key_float((uint32_t)(cand[i] >> 32)) - xmax));
          incl[e] = run;
        }
        u64 cand_mass;
        const u64 before = block_scan_u64(run, cand_mass);
        const int k_eff = k_on ? min(k, count) : count;
        if (tid == 0) n_keep_s = k_eff;
#pragma unroll
        for (int e = 0; e < SAMPLE_PER; ++e)
          if (e < per && tid * per + e == k_eff - 1) z_k_s = before + incl[e];
        __syncthreads();
        if (p_on) {
          const u64 z_k = k_on ? z_k_s : z_all;
          const u64 bound = (u64)((double)p_keep * (double)z_k);
          // the kept ones are those whose preceding mass is within the bound: a prefix, as the sums only grow
          int mine = 0;
#pragma unroll
          for (int e = 0; e < SAMPLE_PER; ++e) {
            const int i = tid * per + e;
            if (e < per && i < k_eff) mine += (before + (e ? incl[e - 1] : 0)) <= bound;
          }
          const int kept = block_sum_int(mine);
          if (tid == 0) n_keep_s = kept;
          __syncthreads();
        }
        // top-p alone, and everything collected was kept: the bound may lie past it, in bands not collected
        if (p_on && !k_on && count < vocab && n_keep_s == count) {
          __syncthreads();
          beyond_at = bands;
          ++bands;
          while (bands < SAMPLE_BANDS - 1 && counts[bands] < 4 * count) ++bands;   // a good deal more at once
          continue;
        }
        break;
      }
      if (wide) {
        // the last token top-k keeps, then the last one top-p keeps of those (what precedes a token is the same with
        // and without top-k as long as the token is within it): the kept set ends at the earlier of the two
        __syncthreads();
        bool found = true;
        u64 z_k = z_all;
        if (k_on) {
          found = top_k_cut_wide(row, vocab, temp, xmax, k, cand, &n_cand, cut);
          if (found && p_on) {
            u64 mass = 0;
            for_each_token(row, vocab, temp, [&](float x, int i) {
              if (order_key(x, i) >= cut) mass += fixed_mass(__expf(x - xmax));
            });
            z_k = block_sum_u64(mass);
          }
        }
        if (found && p_on) {
          const u64 p_cut = top_p_cut_wide(row, vocab, temp, xmax, (u64)((double)p_keep * (double)z_k), cand, &n_cand);
          found = p_cut != 0;
          cut = max(cut, p_cut);
        }
        if (!found) {                              // thousands of equal values where a cut falls
          sample_row_general(row, out + r, vocab, temp, top, k, p_keep, p_min, u);
          return;
        }
      }
    } else if (m_on) {
      // min-p alone keeps the tokens within -ln(min_p) of the largest value: the bands that reach that far
      const float reach = -__logf(p_min) + 0.01f;
      int bands = 0;
      while (bands < SAMPLE_BANDS && band_edge(bands) < reach) ++bands;
      wide = true;
      if (bands < SAMPLE_BANDS) {
        const int count = collect_bands(row, vocab, temp, xmax, bands, cand, &n_cand);
        if (count <= SAMPLE_CANDIDATES) {
          int n_pad = WAVE;
          while (n_pad < count) n_pad <<= 1;
          for (int i = count + tid; i < n_pad; i += blockDim.x) cand[i] = 0;
          __syncthreads();
          bitonic_sort(cand, n_pad, true);
          if (tid == 0) n_keep_s = count;
          __syncthreads();
          wide = false;
        }
      }
    }
    if (!wide) {
      // min-p drops q < min_p: the values only fall along the sorted order, so this keeps a prefix too
      int ok = 0;
      for (int i = tid; i < n_keep_s; i += blockDim.x) ok += __expf(key_float((uint32_t)(cand[i] >> 32)) - xmax) >= p_min;
      const int n_final = max(1, block_sum_int(ok));
      // the draw walks the kept tokens as they lie sorted: the first whose running mass exceeds the target
      int n_pad = WAVE;
      while (n_pad < n_final) n_pad <<= 1;
      const int per = max(1, n_pad / SAMPLE_THREADS);
      uint32_t m[SAMPLE_PER];
      u64 mine = 0;
#pragma unroll
      for (int e = 0; e < SAMPLE_PER; ++e) {
        const int i = tid * per + e;
        m[e] = (e < per && i < n_final) ? fixed_mass(__expf(key_float((uint32_t)(cand[i] >> 32)) - xmax)) : 0u;
        mine += m[e];
      }
      u64 total;
      const u64 before = block_scan_u64(mine, total);
      const u64 target = (u64)((double)u * (double)total);
      if (tid == 0) pick_s = -1;
      __syncthreads();
      if (mine > 0 && before <= target && target < before + mine) {   // (one thread)
        u64 run = before;
        int pick = -1;
#pragma unroll
        for (int e = 0; e < SAMPLE_PER; ++e) {
          run += m[e];
          if (pick < 0 && m[e] > 0 && run > target) pick = (int)(0x7fffffffu - (uint32_t)cand[tid * per + e]);
        }
        pick_s = pick;
      }
      __syncthreads();
      if (tid == 0) out[r] = pick_s >= 0 ? pick_s : top.i;
      return;
    }
    // The kept prefix is too long to collect. Its mass, then the token at which the sorted running mass passes the
    // target: the search for "the last token whose preceding mass is within a bound" that top-p uses, with the target as
    // the bound (what precedes a kept token is kept, so the search need not know the filters).
    __syncthreads();                            // `cand` is free from here on
    u64 total = kept_mass;
    if (total == 0) {
      u64 mass = 0;
      for_each_token(row, vocab, temp, [&](float x, int i) {
        const float q = __expf(x - xmax);
        if (order_key(x, i) >= cut && q >= p_min) mass += fixed_mass(q);
      });
      total = block_sum_u64(mass);
    }
    const u64 target = (u64)((double)u * (double)total);
    u64 hit = 0;
    if (total > 0) {
      if (!binned) mass_histogram(row, vocab, temp, xmax, h_mass, h_cnt);
      u64 through;
      hit = last_within(row, vocab, temp, xmax, target, h_mass, h_cnt, cand, &n_cand, through);
      if (hit == 0) hit = top_p_cut_wide(row, vocab, temp, xmax, target, cand, &n_cand);
    }
    if (total > 0 && hit == 0) {                 // thousands of equal values around the target
      sample_row_general(row, out + r, vocab, temp, top, k, p_keep, p_min, u);
      return;
    }
    if (tid == 0) out[r] = total > 0 ? (int)(0x7fffffffu - (uint32_t)hit) : top.i;
    return;
  }

  // no filter: the law is the mass itself, and the draw walks the vocabulary as it lies
  auto law = [&](float x, int, auto) -> uint32_t { return fixed_mass(__expf(x - xmax)); };
  u64* chunk_mass = cand;                       // [chunks]: the mass of tokens 256 c .. 256 c + 255, four to a lane
  const bool wide = (vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  auto lane_masses = [&](int c, uint32_t (&m)[4], auto all) {
    const int i0 = c * SAMPLE_CHUNK + 4 * lane;
    float x[4];
    if (wide && i0 + 3 < vocab) {
      const float4 v = *reinterpret_cast<const float4*>(row + i0);
      x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = i0 + e < vocab ? row[i0 + e] : -INFINITY;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) m[e] = i0 + e < vocab ? law(x[e] / temp, i0 + e, all) : 0u;
  };
  auto chunk_sums = [&](auto all) {
    for (int c = wave; c < chunks; c += SAMPLE_WAVES) {
      uint32_t m[4];
      lane_masses(c, m, all);
      const u64 sum = wave_sum_u64((u64)m[0] + m[1] + m[2] + m[3]);
      if (lane == 0) chunk_mass[c] = sum;
    }
  };
  chunk_sums(std::true_type{});
  if (tid == 0) pick_s = -1;
  __syncthreads();
  // a thread holds consecutive chunks; the one whose chunks hold the target names the chunk
  const int cper = (chunks + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  u64 mine = 0;
  for (int e = 0; e < cper; ++e) {
    const int c = tid * cper + e;
    if (c < chunks) mine += chunk_mass[c];
  }
  u64 total;
  const u64 before = block_scan_u64(mine, total);
  const u64 target = (u64)((double)u * (double)total);     // the first token whose running mass exceeds it
  __shared__ int chunk_s;
  __shared__ u64 chunk_before_s;
  if (mine > 0 && before <= target && target < before + mine) {   // (one thread)
    u64 run = before;
    for (int e = 0; e < cper; ++e) {
      const int c = tid * cper + e;
      const u64 m = c < chunks ? chunk_mass[c] : 0;
      if (run + m > target) { chunk_s = c; chunk_before_s = run; break; }
      run += m;
    }
  }
  __syncthreads();
  if (wave == 0) {
    uint32_t m[4];
    lane_masses(chunk_s, m, std::false_type{});
    const u64 mine4 = (u64)m[0] + m[1] + m[2] + m[3];
    u64 run = chunk_before_s + wave_scan_u64(mine4, lane) - mine4;   // the mass before this lane's four tokens
    int pick = -1;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      run += m[e];
      if (pick < 0 && run > target) pick = chunk_s * SAMPLE_CHUNK + 4 * lane + e;
    }
    const u64 hit = __ballot(pick >= 0);
    if (hit) {
      const int first = __ffsll((long long)hit) - 1;
      pick = __shfl(pick, first, WAVE);
      if (lane == 0) pick_s = pick;
    }
  }
  __syncthreads();
  if (tid == 0) out[r] = pick_s >= 0 ? pick_s : top.i;
}

extern "C" int holon_sample(const float* logits, int32_t* out, int rows, int vocab, const float* temperature,
                            const int32_t* top_k, const float* top_p, const float* min_p, const int64_t* seeds,
                            const void* positions, const int32_t* slots, int positions_i32, void* stream) {
  HOLON_CHECK(rows >= 0 && vocab > 0, "sample: bad sizes");
  HOLON_CHECK(vocab <= SAMPLE_CANDIDATES * SAMPLE_CHUNK, "sample: a vocabulary of %d tokens exceeds the %d this kernel serves",
              vocab, SAMPLE_CANDIDATES * SAMPLE_CHUNK);
  if (rows == 0) return 0;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, out, vocab, temperature, top_k, top_p,
                                                                  min_p, seeds, positions, slots, positions_i32);
  HOLON_LAUNCH_OK();
  return 0;
}

// Log-probabilities of the raw logits (before temperature): for each row the log-probability of `token[r]` and the
// `k` largest log-probabilities with their ids (ties: lower id first). One block per row: the largest value, the
// log of the sum, then the tokens nearest the largest value collected and sorted as for sampling; if no band holds
// k tokens within the room there is, k passes of argmax over the row instead.
#define LOGPROB_MAX_K 32
__global__ void __launch_bounds__(SAMPLE_THREADS) logprobs_kernel(
    const float* __restrict__ logits, const int32_t* __restrict__ tokens, int vocab, int k,
    float* __restrict__ token_lp, int32_t* __restrict__ top_ids, float* __restrict__ top_lp) {
  __shared__ u64 cand[SAMPLE_CANDIDATES];
  __shared__ int counts[SAMPLE_BANDS];
  __shared__ int band_counts[SAMPLE_WAVES][SAMPLE_BANDS];
  __shared__ int n_cand;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (int64_t)r * vocab;
  const ArgMax top = block_argmax(row, vocab, 1.0f);
  float part = 0.f;
  for_each_token(row, vocab, 1.0f, [&](float x, int) { part += expf(x - top.v); });
  const float lse = top.v + logf(block_sum(part));
  if (tid == 0) token_lp[r] = row[tokens[r]] - lse;
  if (k == 0) return;
  if (vocab <= 255 * SAMPLE_THREADS) {
    estimate_band_counts(row, vocab, 1.0f, top.v, counts, band_counts);
    int bands = SAMPLE_BANDS - 1;
    for (int j = SAMPLE_BANDS - 1; j >= 0; --j)
      if (counts[j] >= 2 * k + 64) bands = j;
    for (int attempt = 0; attempt < 6 && bands >= 0 && bands < SAMPLE_BANDS; ++attempt) {
      const int count = collect_bands(row, vocab, 1.0f, top.v, bands, cand, &n_cand);
      if (count > SAMPLE_CANDIDATES) { --bands; continue; }
      if (count < k && count < vocab) { ++bands; continue; }
      int n_pad = WAVE;
      while (n_pad < count) n_pad <<= 1;
      for (int i = count + tid; i < n_pad; i += blockDim.x) cand[i] = 0;
      __syncthreads();
      bitonic_sort(cand, n_pad, true);
      if (tid < k) {
        const u64 c = cand[tid];
        top_ids[(int64_t)r * k + tid] = (int)(0x7fffffffu - (uint32_t)c);
        top_lp[(int64_t)r * k + tid] = key_float((uint32_t)(c >> 32)) - lse;
      }
      return;
    }
  }
  // the k largest one after the other: each pass takes the first in order after the one before
  __shared__ ArgMax part_best[SAMPLE_WAVES];
  __shared__ u64 last_s;
  u64 last = ~0ull;
  for (int j = 0; j < k; ++j) {
    ArgMax best{-INFINITY, 0x7fffffff};
    for_each_token(row, vocab, 1.0f, [&](float x, int i) {
      if (order_key(x, i) < last) best = better(best, ArgMax{x, i});
    });
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
      ArgMax other{__shfl_xor(best.v, o, WAVE), __shfl_xor(best.i, o, WAVE)};
      best = better(best, other);
    }
    if (tid % WAVE == 0) part_best[tid / WAVE] = best;
    __syncthreads();
    if (tid == 0) {
      ArgMax b = part_best[0];
      for (int w = 1; w < SAMPLE_WAVES; ++w) b = better(b, part_best[w]);
      top_ids[(int64_t)r * k + j] = b.i == 0x7fffffff ? 0 : b.i;
      top_lp[(int64_t)r * k + j] = b.v - lse;
      last_s = b.i == 0x7fffffff ? 0 : order_key(b.v, b.i);
    }
    __syncthreads();
    last = last_s;
    __syncthreads();
  }
}

extern "C" int holon_logprobs(const float* logits, const int32_t* tokens, int rows, int vocab, int k, float* token_lp,
                              int32_t* top_ids, float* top_lp, void* stream) {
  HOLON_CHECK(rows >= 0 && vocab > 0 && k >= 0 && k <= LOGPROB_MAX_K && k <= vocab, "logprobs: k=%d must be at most %d",
              k, LOGPROB_MAX_K);
  if (rows == 0) return 0;
  logprobs_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, tokens, vocab, k, token_lp, top_ids, top_lp);
  HOLON_LAUNCH_OK();
  return 0;
}
