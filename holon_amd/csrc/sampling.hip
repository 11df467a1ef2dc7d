// Sampling on the device: argmax, and temperature / top-k / top-p / min-p sampling by inverse CDF in vocabulary order
// with a counter-based uniform (a hash of seed and position: no generator state, so a request's draws do not depend on
// batching). One block per row.
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

__device__ ArgMax block_argmax(const float* __restrict__ row, int vocab, float inv_temp) {
  __shared__ ArgMax part[SAMPLE_THREADS / WAVE];
  __shared__ ArgMax result;
  ArgMax best{-INFINITY, 0x7fffffff};
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {   // 16-byte loads where the row allows
    const float4* row4 = reinterpret_cast<const float4*>(row);
    for (int i = threadIdx.x; i < vocab / 4; i += blockDim.x) {
      const float4 v = row4[i];
      best = better(best, ArgMax{v.x * inv_temp, 4 * i});
      best = better(best, ArgMax{v.y * inv_temp, 4 * i + 1});
      best = better(best, ArgMax{v.z * inv_temp, 4 * i + 2});
      best = better(best, ArgMax{v.w * inv_temp, 4 * i + 3});
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) best = better(best, ArgMax{row[i] * inv_temp, i});
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
    if (r.i == 0x7fffffff) r.i = 0;   // a row of NaN or -inf: the first token
    result = r;
  }
  __syncthreads();
  return result;
}

__global__ void argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int vocab) {
  const ArgMax r = block_argmax(logits + (int64_t)blockIdx.x * vocab, vocab, 1.0f);
  if (threadIdx.x == 0) out[blockIdx.x] = r.i;
}

extern "C" int holon_argmax(const float* logits, int32_t* out, int rows, int vocab, void* stream) {
  HOLON_CHECK(rows >= 0 && vocab > 0, "argmax: bad sizes");
  if (rows == 0) return 0;
  argmax_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, out, vocab);
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

// Order-preserving map of a float onto unsigned integers (larger float, larger key).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// The law of a row: q_i = exp(x_i - max) where kept, 0 where a filter drops token i; x = logit / temperature.
// Filters in order (the reference's): top-k keeps the k largest (ties: lower index first); top-p keeps, in descending
// order, tokens whose preceding mass is <= top_p of the top-k mass (the largest always stays); min-p keeps q >= min_p
// times the largest q. A token is identified for ties by (value, index), so the kept set is exact.
__global__ void sample_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int vocab,
                              const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                              const float* __restrict__ top_p, const float* __restrict__ min_p,
                              const int64_t* __restrict__ seeds, const int64_t* __restrict__ positions) {
  const int r = blockIdx.x;
  const float* row = logits + (int64_t)r * vocab;
  const float temp = temperature[r];
  if (temp == 0.f) {
    const ArgMax a = block_argmax(row, vocab, 1.0f);
    if (threadIdx.x == 0) out[r] = a.i;
    return;
  }
  const float inv_temp = 1.0f / temp;
  const ArgMax top = block_argmax(row, vocab, inv_temp);
  const float xmax = top.v;
  const int k = top_k[r];
  const float p_keep = top_p[r], p_min = min_p[r];

  // --- top-k: the k-th largest key, and how many of the tokens equal to it are kept (the first ones by index)
  uint32_t kth_key = 0;          // keep x with key > kth_key, plus the first `ties_kept` tokens with key == kth_key
  int ties_kept = 0x7fffffff;
  if (k > 0 && k < vocab) {
    uint32_t lo = 0, hi = 0xffffffffu;   // the largest key K with count(key >= K) >= k
    while (lo < hi) {
      const uint32_t mid = lo + (uint32_t)(((uint64_t)hi - lo + 1) / 2);
      int c = 0;
      for (int i = threadIdx.x; i < vocab; i += blockDim.x) c += float_key(row[i] * inv_temp) >= mid;
      if (block_sum_int(c) >= k) lo = mid; else hi = mid - 1;
    }
    kth_key = lo;
    int above = 0;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) above += float_key(row[i] * inv_temp) > kth_key;
    ties_kept = k - block_sum_int(above);
  }
  // rank among equals needs an index-ordered count: each thread owns a contiguous segment of the row
  const int seg = (vocab + blockDim.x - 1) / blockDim.x;
  const int seg_lo = min(vocab, (int)threadIdx.x * seg), seg_hi = min(vocab, seg_lo + seg);
  __shared__ int scan_i[SAMPLE_THREADS];
  __shared__ float scan_f[SAMPLE_THREADS];
  int ties_before = 0;           // tokens equal to the k-th value in earlier segments
  if (ties_kept != 0x7fffffff) {
    int mine = 0;
    for (int i = seg_lo; i < seg_hi; ++i) mine += float_key(row[i] * inv_temp) == kth_key;
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
      const float x = row[i] * inv_temp;
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
        const float x = row[i] * inv_temp;
        const bool kept = in_top_k(x, tie_rank);
        if (kept && float_key(x) > mid) above += expf(x - xmax);
      }
      if (block_sum(above) <= bound) hi = mid; else lo = mid + 1;
    }
    p_key = lo;
    float above = 0.f;
    int tie_rank = ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float x = row[i] * inv_temp;
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
      const float x = row[i] * inv_temp;
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

  // --- draw: inverse CDF in vocabulary order over segment sums
  float mine = 0.f;
  {
    int tie_rank = ties_before, p_rank = p_ties_before;
    for (int i = seg_lo; i < seg_hi; ++i) mine += law(row[i] * inv_temp, tie_rank, p_rank);
  }
  scan_f[threadIdx.x] = mine;
  __syncthreads();
  __shared__ float total_s;
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int t = 0; t < (int)blockDim.x; ++t) { const float v = scan_f[t]; scan_f[t] = run; run += v; }
    total_s = run;
  }
  __syncthreads();
  const float before = scan_f[threadIdx.x];
  const float target = hashed_uniform((uint64_t)seeds[r], (uint64_t)positions[r]) * total_s;
  __shared__ int chosen;
  if (threadIdx.x == 0) chosen = -1;
  __syncthreads();
  // the segment whose running mass first exceeds the target; the last segment with mass takes what rounding leaves
  const float next = (threadIdx.x + 1 < blockDim.x) ? scan_f[threadIdx.x + 1] : total_s;
  const bool last_with_mass = mine > 0.f && next == total_s;
  if (mine > 0.f && ((before <= target && target < next) || (last_with_mass && target >= next))) {
    int tie_rank = ties_before, p_rank = p_ties_before, pick = -1, last = -1;
    float run = before;
    for (int i = seg_lo; i < seg_hi; ++i) {
      const float qv = law(row[i] * inv_temp, tie_rank, p_rank);
      if (qv > 0.f) {
        last = i;
        run += qv;
        if (pick < 0 && run > target) pick = i;
      }
    }
    atomicMax(&chosen, pick >= 0 ? pick : last);
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = chosen >= 0 ? chosen : top.i;
}

extern "C" int holon_sample(const float* logits, int32_t* out, int rows, int vocab, const float* temperature,
                            const int32_t* top_k, const float* top_p, const float* min_p, const int64_t* seeds,
                            const int64_t* positions, void* stream) {
  HOLON_CHECK(rows >= 0 && vocab > 0, "sample: bad sizes");
  if (rows == 0) return 0;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, out, vocab, temperature, top_k, top_p,
                                                                  min_p, seeds, positions);
  HOLON_LAUNCH_OK();
  return 0;
}

// Log-probabilities of the raw logits (before temperature): for each row the log-probability of `token[r]` and the
// `k` largest log-probabilities with their ids (ties: lower id first). One block per row; k passes of argmax over
// the row with the tokens already taken masked out.
#define LOGPROB_MAX_K 32
__global__ void logprobs_kernel(const float* __restrict__ logits, const int32_t* __restrict__ tokens, int vocab, int k,
                                float* __restrict__ token_lp, int32_t* __restrict__ top_ids,
                                float* __restrict__ top_lp) {
  const int r = blockIdx.x;
  const float* row = logits + (int64_t)r * vocab;
  const ArgMax top = block_argmax(row, vocab, 1.0f);
  float part = 0.f;
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) part += expf(row[i] - top.v);
  const float lse = top.v + logf(block_sum(part));
  if (threadIdx.x == 0) token_lp[r] = row[tokens[r]] - lse;
  __shared__ int taken[LOGPROB_MAX_K];
  __shared__ ArgMax part_best[SAMPLE_THREADS / WAVE];
  for (int j = 0; j < k; ++j) {
    ArgMax best{-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      bool skip = false;
      for (int t = 0; t < j; ++t) skip = skip || taken[t] == i;
      if (!skip) best = better(best, ArgMax{row[i], i});
    }
#pragma unroll
    for (int o = WAVE / 2; o > 0; o >>= 1) {
      ArgMax other{__shfl_xor(best.v, o, WAVE), __shfl_xor(best.i, o, WAVE)};
      best = better(best, other);
    }
    if (threadIdx.x % WAVE == 0) part_best[threadIdx.x / WAVE] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
      ArgMax b = part_best[0];
      for (int w = 1; w < (int)blockDim.x / WAVE; ++w) b = better(b, part_best[w]);
      taken[j] = b.i;
      top_ids[(int64_t)r * k + j] = b.i == 0x7fffffff ? 0 : b.i;
      top_lp[(int64_t)r * k + j] = b.v - lse;
    }
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
