// y[M, N] = x[M, K] w[N, K]^T in true float32: float32 operands on the matrix cores (v_mfma_f32_32x32x2_f32: no
// reduced-precision mode), float32 accumulation. This is the product of the 32-bit check path.
//
// Its point is a fixed order of summation. Output element (m, n) is the sum over k of x[m, k] w[n, k] taken in tiles of
// 32 k, one after the other, and inside a tile in the order the instruction adds its pairs; neither depends on M, on
// where the row lies in the batch, or on the tile of the output the element falls in (rows and columns beyond the edge
// are computed on zeros and never stored; a K that is no multiple of 32 is padded with zeros, which add nothing). So
// a token's result is bit for bit the same whether it runs alone, in a portion of a prompt or in a batch of others.
//
// A workgroup of four waves owns a 64 x 64 tile of the output, each wave a 32 x 32 quarter. Per step the workgroup
// stages 64 rows of x and 64 rows of w, 32 k wide, in LDS (rows padded to 33 floats: a wave's 32 rows then fall in 32
// different banks).
#include "common.h"
#include "holon_hip.h"

typedef float f32x16_t __attribute__((ext_vector_type(16)));

namespace {
constexpr int TM = 64, TN = 64, TK = 32, PAD = 1;

// VEC: K is a multiple of 4 and both operands are 16-byte aligned, so rows are read four floats at a time.
template <bool VEC>
__device__ __forceinline__ void stage_rows(const float* __restrict__ src, int rows, int K, int row0, int k0,
                                           float (*dst)[TK + PAD]) {
  // 64 rows x 32 floats = 512 groups of four; 256 threads take two each
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = threadIdx.x + it * 256;
    const int r = idx / (TK / 4), c = (idx % (TK / 4)) * 4;
    const int row = row0 + r, k = k0 + c;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < rows) {
      const float* p = src + (int64_t)row * K + k;
      if (VEC) {
        if (k < K) v = *reinterpret_cast<const float4*>(p);      // K % 4 == 0: a group is inside or outside whole
      } else {
        if (k + 0 < K) v.x = p[0];
        if (k + 1 < K) v.y = p[1];
        if (k + 2 < K) v.z = p[2];
        if (k + 3 < K) v.w = p[3];
      }
    }
    dst[r][c + 0] = v.x; dst[r][c + 1] = v.y; dst[r][c + 2] = v.z; dst[r][c + 3] = v.w;
  }
}

template <bool VEC>
__global__ void __launch_bounds__(256) gemm_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       float* __restrict__ y, int M, int N, int K) {
  __shared__ float xs[TM][TK + PAD];
  __shared__ float ws[TN][TK + PAD];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int r = lane % 32, half = lane / 32;
  f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (int k0 = 0; k0 < K; k0 += TK) {
    stage_rows<VEC>(x, M, K, m0, k0, xs);
    stage_rows<VEC>(w, N, K, n0, k0, ws);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; kk += 2) {
      const float a = xs[wm * 32 + r][kk + half];
      const float b = ws[wn * 32 + r][kk + half];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  // lane holds column n = r of rows 8 (i / 4) + 4 half + i % 4
  const int n = n0 + wn * 32 + r;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int m = m0 + wm * 32 + 8 * (i / 4) + 4 * half + i % 4;
    if (m < M) y[(int64_t)m * N + n] = acc[i];
  }
}
}  // namespace

extern "C" int holon_gemm_f32(const void* x, const void* w, void* y, int M, int N, int K, void* stream) {
  HOLON_CHECK(M >= 0 && N > 0 && K > 0, "gemm (float32): M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  const dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  HOLON_CHECK(grid.y <= 65535, "gemm (float32): M=%d rows exceed one launch (%d)", M, 65535 * TM);
  const bool vec = K % 4 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
  hipStream_t s = (hipStream_t)stream;
  if (vec) gemm_f32_kernel<true><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, (float*)y, M, N, K);
  else gemm_f32_kernel<false><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, (float*)y, M, N, K);
  HOLON_LAUNCH_OK();
  return 0;
}
