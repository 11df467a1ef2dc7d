// y[M, N] = x[M, K] w[N, K]^T for up to 16 rows (decode steps): bfloat16 operands, float32 accumulation on the matrix
// cores, memory-bound on the weights. A workgroup owns 16 weight rows; its waves split K evenly and add their partial
// tiles through LDS in wave order, so the result does not depend on M or on anything but the shapes.
//
// v_mfma_f32_16x16x32_bf16 with the weights as A (16 rows x 32 k: lane l reads 16 contiguous bytes of row l%16) and
// the activations as B (32 k x 16 tokens: lane l reads 16 contiguous bytes of token l%16); the result tile has weight
// rows 4*(l/16)+r of token l%16 in lane l, i.e. 4 consecutive outputs of one token: one 8- or 16-byte store.
//
// Two weight layouts: rows [N, K] as the checkpoint stores them, and tiles [N/16, K/32, 64 lanes, 8] in which the
// 16 bytes lane l needs for one product are at lane l's place, so that a wave's load is one contiguous kilobyte and a
// tile's whole K extent is one contiguous run (measured: 6 to 7 TB/s against 4 to 5 for the row layout).
#include "common.h"
#include "holon_hip.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// A norm folded into the product that reads it. With RMSNorm y = x * rsqrt(mean(x^2) + eps) * g in front of a product
// with W, the product of the un-normed rows with W * diag(g) (folded into the tiled copy once, after loading), scaled
// per row by rsqrt(mean(x^2) + eps) in the epilogue, is the same number with one rounding moved from the normed
// activations to the folded weights; and the norm's kernel, which moves next to nothing and costs as much as a
// quarter of a projection, is gone. The sums of squares come as partial sums `stats` [parts, 16] (float32, row m of
// the step in column m): the kernel that last wrote the rows leaves one partial per 16 columns it owned, and the
// reader adds them in a fixed order (every wave a share in ascending order, the waves in wave order, the four lane
// groups in order).
struct RowScale {
  const float* stats;   // nullptr: rows are used as they are
  int parts;
  float eps, inv_dim;
};

// The sums of squares are read 16 parts at a time: lane l of a wave takes four floats of part 16 k + l / 4, columns
// 4 (l % 4) .. + 3, so a wave's load is one contiguous kilobyte; wave w takes chunks k = w, w + WPB, ... and adds them
// in that order. The values are asked for a few at a time, at the top of each round of the weight loop, and added one
// round later: loads return in the order they were issued, so by then they have arrived behind the weights that the
// round before waited for, and the sum never makes the stream wait.
template <int WPB>
struct RowSums {
  static constexpr int Q = 4;   // loads in flight per lane
  const f32x4_t* at;            // this lane's four floats of the next chunk
  int part, parts;              // the part they belong to; how many there are
  int n;                        // loads in flight
  f32x4_t v[Q], ss;
  __device__ __forceinline__ void start(const RowScale& rs, int wave, int lane) {
    at = reinterpret_cast<const f32x4_t*>(rs.stats) + wave * 64 + lane;
    part = wave * 16 + lane / 4;
    parts = rs.stats != nullptr ? rs.parts : 0;
    n = 0;
    ss = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  __device__ __forceinline__ void turn() {   // add what the last turn asked for, ask for the next
#pragma unroll
    for (int q = 0; q < Q; ++q)
      if (q < n) ss += v[q];
    n = 0;
#pragma unroll
    for (int q = 0; q < Q; ++q)
      if (part + q * 16 * WPB < parts) {
        v[q] = at[(int64_t)q * 64 * WPB];
        n = q + 1;
      }
    at += (int64_t)n * 64 * WPB;
    part += n * 16 * WPB;
  }
  __device__ __forceinline__ f32x4_t finish() {
    do turn(); while (n > 0);
    return ss;
  }
};
// After the waves' shares have been added: the sum over the 16 lanes that hold the same four columns (lanes l, l ^ 4,
// l ^ 8, l ^ 16, l ^ 32, in that order), then column c out of lane c / 4. Every lane of column c gets the same sum.
__device__ __forceinline__ float row_sum_of_column(f32x4_t v, int c) {
#pragma unroll
  for (int o = 4; o < WAVE; o <<= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += __shfl_xor(v[i], o, WAVE);
  const float t0 = __shfl(v[0], c / 4, WAVE), t1 = __shfl(v[1], c / 4, WAVE), t2 = __shfl(v[2], c / 4, WAVE),
              t3 = __shfl(v[3], c / 4, WAVE);
  return c % 4 == 0 ? t0 : (c % 4 == 1 ? t1 : (c % 4 == 2 ? t2 : t3));
}
// The four lane groups' shares of row c, added in order; every lane of column c gets the same sum.
__device__ __forceinline__ float over_lane_groups(float v, int c) {
  const float a = __shfl(v, c, WAVE), b = __shfl(v, 16 + c, WAVE), d = __shfl(v, 32 + c, WAVE), e = __shfl(v, 48 + c, WAVE);
  return ((a + b) + d) + e;
}

// RESID: y is the residual stream, y = round(y + round(product)) in place: the add that the next norm's kernel would
// have done, with its roundings.
// NT: tiles of 16 weight rows a block owns, next to one another; its waves run them side by side over one copy of the
// activations, which halves what the activations cost where every block reads all of them. A tile's sums are the same
// whatever NT is.
template <int NT, int WPB, int UNROLL, typename OutT, bool TILED, bool RESID = false>
__global__ void __launch_bounds__(WPB * 64) gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                const bf16_t* __restrict__ w, OutT* __restrict__ y,
                                                                int M, int N, int K, int round_first, RowScale rs,
                                                                float* __restrict__ stats_out) {
  __shared__ f32x4_t red[WPB > 1 ? (WPB - 1) * NT * WAVE : 1];
  __shared__ f32x4_t red_ss[WPB > 1 ? (WPB - 1) * WAVE : 1];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  const int tile0 = blockIdx.x * NT;
  const int kw = K / WPB;                       // this wave's slice of K (a multiple of 32)
  const int steps = kw / 32;
  const bf16_t* wp[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
    wp[j] = TILED ? w + ((int64_t)(tile0 + j) * (K / 32) + (int64_t)wave * steps) * 512 + lane * 8
                  : w + (int64_t)((tile0 + j) * 16 + c) * K + (int64_t)wave * kw + 8 * g;
  constexpr int WSTEP = TILED ? 512 : 32;       // elements between one product's weights and the next
  const bf16_t* xp = x + (int64_t)c * K + (int64_t)wave * kw + 8 * g;
  const bool have = c < M;                      // token c of the step exists
  f32x4_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  RowSums<WPB> sums;
  sums.start(rs, wave, lane);
  ushort4 before[NT];                           // RESID: the residual values this lane will add to, asked for now so
  if constexpr (RESID) {                        // that they are here when the sums are
#pragma unroll
    for (int j = 0; j < NT; ++j)
      if (wave == 0 && have) before[j] = *reinterpret_cast<const ushort4*>(y + (int64_t)c * N + (tile0 + j) * 16 + 4 * g);
  }
  auto tokens = [&](int s) -> bf16x8_t {        // the activations of product s: zeros for a token that is not there
    bf16x8_t xf;
    if (have) {
      xf = *reinterpret_cast<const bf16x8_t*>(xp + s * 32);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) xf[i] = (__bf16)0.f;
    }
    return xf;
  };

  int s = 0;
  for (; s + UNROLL <= steps; s += UNROLL) {
    sums.turn();
    bf16x8_t wf[NT][UNROLL], xf[UNROLL];
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
        wf[j][u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp[j] + (int64_t)(s + u) * WSTEP));
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) xf[u] = tokens(s + u);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j][u], xf[u], acc[j], 0, 0, 0);
  }
  for (; s < steps; ++s) {
    const bf16x8_t xf = tokens(s);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const bf16x8_t wf = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp[j] + (int64_t)s * WSTEP));
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf, acc[j], 0, 0, 0);
    }
  }
  f32x4_t ss = sums.finish();
  if (WPB > 1) {
    if (wave > 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j) red[((wave - 1) * NT + j) * WAVE + lane] = acc[j];
      red_ss[(wave - 1) * WAVE + lane] = ss;
    }
    __syncthreads();
    if (wave > 0) return;
    for (int ww = 1; ww < WPB; ++ww) {
#pragma unroll
      for (int j = 0; j < NT; ++j) acc[j] += red[((ww - 1) * NT + j) * WAVE + lane];
      ss += red_ss[(ww - 1) * WAVE + lane];
    }
  }
  if (rs.stats != nullptr) {                     // the norm's scale of row c, on the float32 sums before they are rounded
    const float inv = 1.0f / sqrtf(row_sum_of_column(ss, c) * rs.inv_dim + rs.eps);
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] *= inv;
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    float mine = 0.f;                            // RESID with stats_out: the squares of the residual values written
    if (have) {
      OutT* yp = y + (int64_t)c * N + (tile0 + j) * 16 + 4 * g;
      if constexpr (sizeof(OutT) == 4) {
        f32x4_t o = acc[j];
        if (round_first) {      // the bfloat16 product, widened: what the vendor product of more rows gives, cast up
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r] = bf16_to_float(float_to_bf16(o[r]));
        }
        *reinterpret_cast<f32x4_t*>(yp) = o;
      } else {
        ushort4 o;
        o.x = float_to_bf16(acc[j][0]); o.y = float_to_bf16(acc[j][1]);
        o.z = float_to_bf16(acc[j][2]); o.w = float_to_bf16(acc[j][3]);
        if constexpr (RESID) {
          const ushort4 r = before[j];
          o.x = float_to_bf16(bf16_to_float(r.x) + bf16_to_float(o.x));
          o.y = float_to_bf16(bf16_to_float(r.y) + bf16_to_float(o.y));
          o.z = float_to_bf16(bf16_to_float(r.z) + bf16_to_float(o.z));
          o.w = float_to_bf16(bf16_to_float(r.w) + bf16_to_float(o.w));
          const float v0 = bf16_to_float(o.x), v1 = bf16_to_float(o.y), v2 = bf16_to_float(o.z), v3 = bf16_to_float(o.w);
          mine = ((v0 * v0 + v1 * v1) + v2 * v2) + v3 * v3;
        }
        *reinterpret_cast<ushort4*>(yp) = o;
      }
    }
    if constexpr (RESID) {
      if (stats_out != nullptr) {                // a tile's 16 columns of every row: one partial per row
        const float part = over_lane_groups(mine, c);
        if (g == 0) stats_out[(int64_t)(tile0 + j) * 16 + c] = part;
      }
    }
  }
}

template <int NT, int WPB, int UNROLL, typename OutT, bool RESID>
static void launch_skinny(const void* x, const void* w, void* y, int M, int N, int K, bool tiled, hipStream_t s,
                          int round_first, RowScale rs, float* stats_out) {
  const dim3 grid(N / 16 / NT), block(WPB * 64);
  if constexpr (RESID)
    gemm_skinny_kernel<NT, WPB, UNROLL, OutT, true, true><<<grid, block, 0, s>>>((const bf16_t*)x, (const bf16_t*)w,
                                                                                (OutT*)y, M, N, K, round_first, rs, stats_out);
  else if (tiled)
    gemm_skinny_kernel<NT, WPB, UNROLL, OutT, true><<<grid, block, 0, s>>>((const bf16_t*)x, (const bf16_t*)w,
                                                                          (OutT*)y, M, N, K, round_first, rs, stats_out);
  else
    gemm_skinny_kernel<NT, WPB, UNROLL, OutT, false><<<grid, block, 0, s>>>((const bf16_t*)x, (const bf16_t*)w,
                                                                           (OutT*)y, M, N, K, round_first, rs, stats_out);
}

// How many waves share a tile, from the shapes alone (a result never depends on M), and how many tiles a block owns
// (which changes no result, so it may follow M). Measured on MI355X, K 4096 to 8192, in us at 1 / 8 / 16 rows:
//   256 tiles: 16 waves, one tile (two tiles leave half the compute units without a block);
//   320 to 512 tiles: 8 waves; two tiles 9.9 / 10.7 / 12.2 (320), 11.5 / 12.3 / 13.8 (384), 14.0 / 14.6 / 15.8 (512)
//     against one 10.8 / 12.8 / 16.1, 11.9 / 14.2 / 16.8, 13.8 / 15.5 / 17.9;
//   640 tiles: 8 waves, one tile 17.2 / 20.0 / 23.1 against two 19.1 / 21.1 / 23.3;
//   9,496 tiles (float32 result): 8 waves; one tile up to 8 rows (4 rows 181 against 195, 8 rows 192 against 201), two
//     from 10 rows up (12 rows 211 against 220, 16 rows 223 against 251).
constexpr int SKINNY_WIDE_TWO_FROM = 10;   // rows from which a vocabulary's worth of tiles is walked two a block
template <typename OutT, bool RESID = false>
static int pick_waves(const void* x, const void* w, void* y, int M, int N, int K, bool tiled, hipStream_t s,
                      int round_first = 0, RowScale rs = RowScale{nullptr, 0, 0.f, 0.f}, float* stats_out = nullptr) {
  const int tiles = N / 16;
  int wpb = tiles >= 320 ? 8 : 16;
  while (wpb > 1 && K % (32 * wpb) != 0) wpb /= 2;
  const bool two = tiles % 2 == 0 && wpb <= 8 && ((tiles >= 320 && tiles <= 512) || (tiles > 4096 && M >= SKINNY_WIDE_TWO_FROM));
#define SKINNY(WPB, U)                                                                                         \
  if (two) launch_skinny<2, WPB, U, OutT, RESID>(x, w, y, M, N, K, tiled, s, round_first, rs, stats_out);     \
  else launch_skinny<1, WPB, U, OutT, RESID>(x, w, y, M, N, K, tiled, s, round_first, rs, stats_out)
  switch (wpb) {
    case 16: launch_skinny<1, 16, 8, OutT, RESID>(x, w, y, M, N, K, tiled, s, round_first, rs, stats_out); break;
    case 8: SKINNY(8, 8); break;
    case 4: if (two) { SKINNY(4, 8); } else { SKINNY(4, 16); } break;
    case 2: SKINNY(2, 8); break;
    default: SKINNY(1, 8); break;
  }
#undef SKINNY
  return 0;
}

extern "C" int holon_gemm_skinny_supported(int M, int N, int K) {
  return M >= 1 && M <= 16 && N % 16 == 0 && K % 32 == 0 && K >= 32;
}

// out_f32: 0 writes bfloat16, 1 float32 straight from the accumulators, 2 float32 values that were rounded to bfloat16
// first (the product in the operands' type, cast up). tiled: 1 when `w` is in the tile layout (see holon_tile_weight_bf16).
extern "C" int holon_gemm_skinny_bf16(const void* x, const void* w, void* y, int M, int N, int K, int out_f32,
                                      int tiled, void* stream) {
  HOLON_CHECK(holon_gemm_skinny_supported(M, N, K), "gemm (few rows): M=%d N=%d K=%d not served (M <= 16, N %% 16, K %% 32)",
              M, N, K);
  hipStream_t s = (hipStream_t)stream;
  if (out_f32) pick_waves<float>(x, w, y, M, N, K, tiled != 0, s, out_f32 == 2);
  else pick_waves<bf16_t>(x, w, y, M, N, K, tiled != 0, s);
  HOLON_LAUNCH_OK();
  return 0;
}

// The same product over rows that a folded norm has yet to scale: `w_tiled` holds W * diag(g), x the un-normed rows,
// `stats` [parts, 16] the partial sums of squares of x's rows; row m of the result is scaled by
// rsqrt(sum(stats[:, m]) / K + eps) before it is rounded.
extern "C" int holon_gemm_skinny_scaled_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K,
                                             int out_f32, const float* stats, int parts, float eps, void* stream) {
  HOLON_CHECK(holon_gemm_skinny_supported(M, N, K) && stats != nullptr && parts >= 1,
              "gemm (few rows, folded norm): M=%d N=%d K=%d parts=%d not served (M <= 16, N %% 16, K %% 32)", M, N, K, parts);
  const RowScale rs{stats, parts, eps, 1.0f / (float)K};
  hipStream_t s = (hipStream_t)stream;
  if (out_f32) pick_waves<float>(x, w_tiled, y, M, N, K, true, s, out_f32 == 2, rs);
  else pick_waves<bf16_t>(x, w_tiled, y, M, N, K, true, s, 0, rs);
  HOLON_LAUNCH_OK();
  return 0;
}

// residual[M, N] += x[M, K] w^T in place (the product rounded, then the sum rounded) over tiled weights: the output
// projection's product and the residual add that follows it, in one kernel. With `stats_out` ([N / 16, 16] float32)
// it also leaves, per block of 16 columns, the sums of squares of the residual values it wrote: what a norm over the
// new rows needs.
extern "C" int holon_gemm_skinny_add_bf16(const void* x, const void* w_tiled, void* residual, int M, int N, int K,
                                          float* stats_out, void* stream) {
  HOLON_CHECK(holon_gemm_skinny_supported(M, N, K),
              "gemm (few rows, added to the residual): M=%d N=%d K=%d not served (M <= 16, N %% 16, K %% 32)", M, N, K);
  pick_waves<bf16_t, true>(x, w_tiled, residual, M, N, K, true, (hipStream_t)stream, 0,
                           RowScale{nullptr, 0, 0.f, 0.f}, stats_out);
  HOLON_LAUNCH_OK();
  return 0;
}

// The gated form: w = [gate rows; up rows] (2I rows), y[M, I] = round(silu(round(x gate^T))) * round(x up^T), the
// roundings of the two-kernel composition. A block owns gate tile t and up tile t + I/16 and streams both.
template <int WPB, int UNROLL, bool TILED>
__global__ void __launch_bounds__(WPB * 64) gemm_skinny_glu_kernel(const bf16_t* __restrict__ x,
                                                                    const bf16_t* __restrict__ w,
                                                                    bf16_t* __restrict__ y, int M, int I, int K,
                                                                    RowScale rs) {
  __shared__ f32x4_t red[WPB > 1 ? (WPB - 1) * 2 * WAVE : 1];
  __shared__ f32x4_t red_ss[WPB > 1 ? (WPB - 1) * WAVE : 1];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  const int n0 = blockIdx.x * 16;
  const int kw = K / WPB, steps = kw / 32;
  const bf16_t* wp[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t tile = blockIdx.x + (int64_t)h * (I / 16);
    wp[h] = TILED ? w + (tile * (K / 32) + (int64_t)wave * steps) * 512 + lane * 8
                  : w + (tile * 16 + c) * K + (int64_t)wave * kw + 8 * g;
  }
  constexpr int WSTEP = TILED ? 512 : 32;
  const bf16_t* xp = x + (int64_t)c * K + (int64_t)wave * kw + 8 * g;
  const bool have = c < M;
  f32x4_t acc[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
  RowSums<WPB> sums;
  sums.start(rs, wave, lane);
  auto tokens = [&](int s) -> bf16x8_t {
    bf16x8_t xf;
    if (have) {
      xf = *reinterpret_cast<const bf16x8_t*>(xp + s * 32);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) xf[i] = (__bf16)0.f;
    }
    return xf;
  };
  int s = 0;
  for (; s + UNROLL <= steps; s += UNROLL) {
    sums.turn();
    bf16x8_t wf[2][UNROLL], xf[UNROLL];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
        wf[h][u] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp[h] + (int64_t)(s + u) * WSTEP));
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) xf[u] = tokens(s + u);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[0][u], xf[u], acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[1][u], xf[u], acc[1], 0, 0, 0);
    }
  }
  for (; s < steps; ++s) {
    const bf16x8_t w0 = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp[0] + (int64_t)s * WSTEP));
    const bf16x8_t w1 = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp[1] + (int64_t)s * WSTEP));
    const bf16x8_t xf = tokens(s);
    acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, xf, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, xf, acc[1], 0, 0, 0);
  }
  f32x4_t ss = sums.finish();
  if (WPB > 1) {
    if (wave > 0) {
#pragma unroll
      for (int h = 0; h < 2; ++h) red[((wave - 1) * 2 + h) * WAVE + lane] = acc[h];
      red_ss[(wave - 1) * WAVE + lane] = ss;
    }
    __syncthreads();
    if (wave > 0) return;
    for (int ww = 1; ww < WPB; ++ww) {
#pragma unroll
      for (int h = 0; h < 2; ++h) acc[h] += red[((ww - 1) * 2 + h) * WAVE + lane];
      ss += red_ss[(ww - 1) * WAVE + lane];
    }
  }
  if (rs.stats != nullptr) {
    const float inv = 1.0f / sqrtf(row_sum_of_column(ss, c) * rs.inv_dim + rs.eps);
    acc[0] *= inv;
    acc[1] *= inv;
  }
  if (!have) return;
  ushort4 o;
  bf16_t* oe = reinterpret_cast<bf16_t*>(&o);
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float gate = bf16_to_float(float_to_bf16(acc[0][r]));
    const float up = bf16_to_float(float_to_bf16(acc[1][r]));
    const float sg = bf16_to_float(float_to_bf16(silu<bf16_t>(gate)));
    oe[r] = float_to_bf16(sg * up);
  }
  *reinterpret_cast<ushort4*>(y + (int64_t)c * I + n0 + 4 * g) = o;
}

// `stats` (nullable, with `parts` and `eps`): x holds un-normed rows and `w` the tiled weights with the norm's weight
// folded in; rows are scaled as in holon_gemm_skinny_scaled_bf16 (tiled).
extern "C" int holon_gemm_skinny_glu_bf16(const void* x, const void* w, void* y, int M, int I, int K, int tiled,
                                          const float* stats, int parts, float eps, void* stream) {
  HOLON_CHECK(M >= 1 && M <= 16 && I % 16 == 0 && K % 128 == 0, "gated gemm (few rows): M=%d I=%d K=%d not served", M, I, K);
  HOLON_CHECK(stats == nullptr || (tiled && parts >= 1), "gated gemm (few rows, folded norm): tiled=%d parts=%d", tiled, parts);
  const RowScale rs{stats, parts, eps, 1.0f / (float)K};
  hipStream_t s = (hipStream_t)stream;
  const bool few = I / 16 < 512;   // few tile pairs: four waves share each; otherwise two (measured at 768 pairs, K 4096:
                                   // 33 us against 36 for one wave a pair at 1 and 8 rows, the same at 16)
#define GLU(WPB, U)                                                                                              \
  if (tiled) gemm_skinny_glu_kernel<WPB, U, true><<<I / 16, WPB * 64, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, \
                                                                             (bf16_t*)y, M, I, K, rs);           \
  else gemm_skinny_glu_kernel<WPB, U, false><<<I / 16, WPB * 64, 0, s>>>((const bf16_t*)x, (const bf16_t*)w,      \
                                                                        (bf16_t*)y, M, I, K, rs)
  if (few) { GLU(4, 8); } else { GLU(2, 8); }
#undef GLU
  HOLON_LAUNCH_OK();
  return 0;
}

// tiled[t][s][l][e] = w[16 t + l % 16][32 s + 8 (l / 16) + e]: the layout the few-row product streams.
// With `scale` [K]: tiled holds round(w[n][k] * scale[k]), a norm's weight folded into the columns it multiplies.
__global__ void tile_weight_kernel(const bf16_t* __restrict__ w, bf16_t* __restrict__ tiled, int N, int K,
                                   const bf16_t* __restrict__ scale) {
  const int64_t chunks = (int64_t)N * K / 8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < chunks; i += (int64_t)gridDim.x * blockDim.x) {
    const int lane = (int)(i % 64);
    const int64_t ts = i / 64;
    const int64_t step = ts % (K / 32), tile = ts / (K / 32);
    const int64_t col = step * 32 + 8 * (lane / 16);
    const int64_t src = (tile * 16 + lane % 16) * K + col;
    uint4 v = *reinterpret_cast<const uint4*>(w + src);
    if (scale != nullptr) {
      bf16_t* e = reinterpret_cast<bf16_t*>(&v);
#pragma unroll
      for (int j = 0; j < 8; ++j) e[j] = float_to_bf16(bf16_to_float(e[j]) * bf16_to_float(scale[col + j]));
    }
    *reinterpret_cast<uint4*>(tiled + i * 8) = v;
  }
}

extern "C" int holon_tile_weight_bf16(const void* w, void* tiled, int N, int K, const void* scale, void* stream) {
  HOLON_CHECK(N > 0 && K > 0 && N % 16 == 0 && K % 32 == 0, "tile_weight: N=%d K=%d must be multiples of 16 and 32", N, K);
  tile_weight_kernel<<<4096, 256, 0, (hipStream_t)stream>>>((const bf16_t*)w, (bf16_t*)tiled, N, K, (const bf16_t*)scale);
  HOLON_LAUNCH_OK();
  return 0;
}
