// A toy kernel that a test's toy mixer brings with it: y[t] = s_t with s_t = decay * s_(t-1) + x[t] along the tokens
// of every row of a step; a row's s lives in the row's slot (float32) between steps, and a row that starts at position
// 0 starts from zero. One block per row, threads over the width. It stands for no model's kernel.
#include "common.h"

template <typename T>
__global__ void decay_scan_kernel(const T* __restrict__ x, T* __restrict__ y, float* __restrict__ state,
                                  const int32_t* __restrict__ slots, const int32_t* __restrict__ starts,
                                  const int32_t* __restrict__ query_start, int hidden, float decay) {
  const int b = blockIdx.x;
  const int64_t slot = slots[b];
  const int t0 = query_start[b], t1 = query_start[b + 1];
  const bool fresh = starts[b] == 0;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float s = fresh ? 0.f : state[slot * hidden + i];
    for (int t = t0; t < t1; ++t) {
      s = decay * s + Elem<T>::load(x[(int64_t)t * hidden + i]);
      y[(int64_t)t * hidden + i] = Elem<T>::store(s);
    }
    state[slot * hidden + i] = s;
  }
}

extern "C" int toy_decay_scan(const void* x, void* y, float* state, const int32_t* slots, const int32_t* starts,
                              const int32_t* query_start, int rows, int hidden, float decay, int dtype, void* stream) {
  if (rows < 0 || hidden <= 0 || (dtype != HOLON_F32 && dtype != HOLON_BF16)) return -1;
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HOLON_F32)
    decay_scan_kernel<float><<<rows, 256, 0, s>>>((const float*)x, (float*)y, state, slots, starts, query_start, hidden, decay);
  else
    decay_scan_kernel<bf16_t><<<rows, 256, 0, s>>>((const bf16_t*)x, (bf16_t*)y, state, slots, starts, query_start, hidden, decay);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
