// y[M, N] = x[M, K] w[N, K]^T for few rows (decode steps): bfloat16 operands, float32 accumulation on the matrix
// cores, memory-bound on the weights. A workgroup owns 16 weight rows; its waves split K evenly and add their partial
// tiles through LDS in wave order, so the result does not depend on M or on anything but the shapes.
//
// v_mfma_f32_16x16x32_bf16 with the weights as A (16 rows x 32 k: lane l reads 16 contiguous bytes of row l%16) and
// the activations as B (32 k x 16 tokens: lane l reads 16 contiguous bytes of token l%16); the result tile has weight
// rows 4*(l/16)+r of token l%16 in lane l, i.e. 4 consecutive outputs of one token: one 8- or 16-byte store.
#include "common.h"
#include "holon_hip.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <int MT, int WPB, int UNROLL, typename OutT>
__global__ void __launch_bounds__(WPB * 64) gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                const bf16_t* __restrict__ w, OutT* __restrict__ y,
                                                                int M, int N, int K) {
  __shared__ f32x4_t red[WPB > 1 ? (WPB - 1) * MT * WAVE : 1];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  const int n0 = blockIdx.x * 16;
  const int kw = K / WPB;                       // this wave's slice of K (a multiple of 32)
  const bf16_t* wp = w + (int64_t)(n0 + c) * K + (int64_t)wave * kw + 8 * g;
  const bf16_t* xp = x + (int64_t)c * K + (int64_t)wave * kw + 8 * g;
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  bool have[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) have[t] = t * 16 + c < M;

  const int steps = kw / 32;
  int s = 0;
  for (; s + UNROLL <= steps; s += UNROLL) {
    bf16x8_t wf[UNROLL], xf[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) wf[u] = *reinterpret_cast<const bf16x8_t*>(wp + (s + u) * 32);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (have[t]) {
          xf[u][t] = *reinterpret_cast<const bf16x8_t*>(xp + (int64_t)t * 16 * K + (s + u) * 32);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) xf[u][t][i] = (__bf16)0.f;
        }
      }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u], xf[u][t], acc[t], 0, 0, 0);
  }
  for (; s < steps; ++s) {
    const bf16x8_t wf = *reinterpret_cast<const bf16x8_t*>(wp + s * 32);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8_t xf;
      if (have[t]) {
        xf = *reinterpret_cast<const bf16x8_t*>(xp + (int64_t)t * 16 * K + s * 32);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) xf[i] = (__bf16)0.f;
      }
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc[t], 0, 0, 0);
    }
  }
  if (WPB > 1) {
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t) red[((wave - 1) * MT + t) * WAVE + lane] = acc[t];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int ww = 1; ww < WPB; ++ww)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] += red[((ww - 1) * MT + t) * WAVE + lane];
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + c;
    if (m >= M) continue;
    OutT* yp = y + (int64_t)m * N + n0 + 4 * g;
    if constexpr (sizeof(OutT) == 4) {
      *reinterpret_cast<f32x4_t*>(yp) = acc[t];
    } else {
      ushort4 o;
      o.x = float_to_bf16(acc[t][0]); o.y = float_to_bf16(acc[t][1]);
      o.z = float_to_bf16(acc[t][2]); o.w = float_to_bf16(acc[t][3]);
      *reinterpret_cast<ushort4*>(yp) = o;
    }
  }
}

template <int MT, int WPB, typename OutT>
static void launch_skinny(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t s) {
  constexpr int UNROLL = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
  gemm_skinny_kernel<MT, WPB, UNROLL, OutT><<<N / 16, WPB * 64, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, (OutT*)y,
                                                                         M, N, K);
}

template <int MT, typename OutT>
static int pick_waves(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t s) {
  // enough waves to keep the memory system busy: aim for a few thousand, K split in multiples of 32
  const int tiles = N / 16;
  int wpb = MT >= 3 ? 8 : 16;                  // 16 waves of 3 or 4 token tiles run out of registers
  while (wpb > 1 && (K % (32 * wpb) != 0 || tiles * (wpb / 2) >= 4096)) wpb /= 2;
  switch (wpb) {
    case 16:
      if constexpr (MT < 3) launch_skinny<MT, 16, OutT>(x, w, y, M, N, K, s);
      break;
    case 8: launch_skinny<MT, 8, OutT>(x, w, y, M, N, K, s); break;
    case 4: launch_skinny<MT, 4, OutT>(x, w, y, M, N, K, s); break;
    case 2: launch_skinny<MT, 2, OutT>(x, w, y, M, N, K, s); break;
    default: launch_skinny<MT, 1, OutT>(x, w, y, M, N, K, s); break;
  }
  return 0;
}

extern "C" int holon_gemm_skinny_supported(int M, int N, int K) {
  return M >= 1 && M <= 64 && N % 16 == 0 && K % 32 == 0 && K >= 32;
}

// out_f32: 1 writes float32, 0 bfloat16.
extern "C" int holon_gemm_skinny_bf16(const void* x, const void* w, void* y, int M, int N, int K, int out_f32,
                                      void* stream) {
  HOLON_CHECK(holon_gemm_skinny_supported(M, N, K), "gemm (few rows): M=%d N=%d K=%d not served (M <= 64, N %% 16, K %% 32)",
              M, N, K);
  hipStream_t s = (hipStream_t)stream;
  const int mt = (M + 15) / 16;
#define SKINNY(MT)                                                                 \
  if (out_f32) pick_waves<MT, float>(x, w, y, M, N, K, s);                          \
  else pick_waves<MT, bf16_t>(x, w, y, M, N, K, s)
  if (mt == 1) { SKINNY(1); } else if (mt == 2) { SKINNY(2); } else if (mt == 3) { SKINNY(3); } else { SKINNY(4); }
#undef SKINNY
  HOLON_LAUNCH_OK();
  return 0;
}
