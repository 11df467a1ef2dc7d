// y[M, N] = x[M, K] w[N, K]^T for 17 to 64 rows (decode steps of many requests) over weights with many tiles of 16
// rows (a gated feed-forward's first product, the head): bfloat16 operands, float32 accumulation on the matrix cores.
//
// The few-row kernel streams the weights and lets every block read its rows of activations from L2; with 64 rows those
// reads cost as much as the weights. Here a block's waves walk K together and share the rows through LDS: a chunk of
// KC columns of all rows is copied in once per block by the memory pipeline itself (global_load_lds, no register and
// no LDS write instruction on the way; double buffered, the next chunk's copy under way while this one is used), each
// wave streams the weights of its own tile (from the tiled copy: a contiguous kilobyte a product) for the next chunk
// while it multiplies this one, and reads its activations as B operands from LDS. A copy's kilobyte is contiguous
// in LDS, so rows are not padded apart but swizzled: a row's 16-byte piece j sits at place j ^ (row % 16) (rows of 128
// bytes: j ^ (row / 2 % 8)), and 16 lanes that read the same piece of 16 consecutive rows touch every bank once. A
// wave sums its tile over all of K in order, so a result depends on nothing but the operands.
//
// Weights with tiles enough to fill the GPU (a gated feed-forward's first product, the head) are served whole. Narrow
// ones (a few hundred tiles: q/k/v, output and down projections) have K split over blocks as well (grid y): every
// block writes the float32 sums of its share of K, [splits, M, N], and the reader adds them up in split order (the
// residual add + norm kernel does so as it reads; `holon_sum_parts` for anyone else), so no block waits for another.
//
// v_mfma_f32_16x16x32_bf16 with the weights as A and MT tiles of 16 tokens as B, as in the few-row kernel.
#include "common.h"
#include "holon_hip.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

namespace {
// OUT: 0 bfloat16, 1 float32 of the values rounded to bfloat16 (the product in the operands' type, cast up),
//      2 the gated form, bfloat16 round(silu(round(gate))) * round(up): the first half of a block's waves own gate
//      tiles, the second half the up tiles of the same columns (I / 16 tiles further on), and the halves meet in LDS,
//      3 float32 sums over this block's share of K (block y of gridDim.y), unrounded, to y[blockIdx.y][M][N].
template <int MT, int WAVES, int KC, int OUT>
__global__ void __launch_bounds__(WAVES * 64) gemm_rows_kernel(const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w, void* __restrict__ y,
                                                               int M, int N, int K) {
  constexpr int ROWS = MT * 16, STEPS = KC / 32;
  constexpr int PPR = KC / 8;                               // 16-byte pieces a row of a chunk has
  constexpr int RPI = 64 / PPR;                             // rows one copy instruction (a kilobyte) brings
  constexpr int COPIES = ROWS / RPI;                        // instructions a chunk takes
  constexpr int XCH = (COPIES + WAVES - 1) / WAVES;         // of which a wave issues this many
  static_assert(KC == 64 || KC == 128 || KC == 256, "rows of 128, 256 or 512 bytes");
  __shared__ __attribute__((aligned(1024))) bf16_t xs[2][ROWS * KC];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  constexpr bool GATED = OUT == 2;
  constexpr int COLS = GATED ? WAVES / 2 : WAVES;            // output tiles of 16 columns a block writes
  const bool up_half = GATED && wave >= COLS;                // (gated) this wave owns an up tile
  const int col_tile = blockIdx.x * COLS + wave % COLS;      // N / 16 is a multiple of COLS
  const int tile = col_tile + (up_half ? N / 16 : 0);        // the weight's tile: up rows lie I / 16 tiles further on
  const bf16_t* wp = w + (int64_t)tile * (K / 32) * 512 + lane * 8;
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  bf16x8_t wcur[STEPS], wnext[STEPS];
  auto load_w = [&](int chunk, bf16x8_t (&to)[STEPS]) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
      to[s] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(wp + ((int64_t)chunk * STEPS + s) * 512));
  };
  // what this lane copies: of instruction j = i * WAVES + wave, row j * RPI + lane / PPR, the piece that belongs at
  // place lane % PPR (rows beyond M repeat the last row: what they give is never written)
  uint32_t x_src[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int row = (i * WAVES + wave) * RPI + lane / PPR;
    const int piece = (lane % PPR) ^ (KC == 64 ? (row / 2) % 8 : row % 16);
    x_src[i] = (uint32_t)(((int64_t)min(row, M - 1) * K + piece * 8) * 2);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&xs[0][0];
  auto copy_x = [&](int chunk, int buf) {
    const bf16_t* from = x + (int64_t)chunk * KC;
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int j = i * WAVES + wave;                       // (uniform over the wave)
      if (j < COPIES) load_to_lds16(from, x_src[i], lds0 + (uint32_t)(buf * ROWS * KC * 2 + j * 1024));
    }
  };
  // where this lane reads the B operand of product s for the tile of tokens t: row 16 t + c, piece 4 s + g
  uint32_t x_at[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) x_at[s] = (uint32_t)(c * KC + 8 * ((4 * s + g) ^ (KC == 64 ? (c / 2) % 8 : c)));
  const int chunks = K / KC / (int)gridDim.y;              // this block's share of K (all of it unless OUT == 3)
  const int first = (int)blockIdx.y * chunks;
  load_w(first, wcur);
  copy_x(first, 0);
  wait_loads_but<0>();
  __syncthreads();
  for (int ch = 0; ch < chunks; ++ch) {
    const int buf = ch & 1;
    const bool more = ch + 1 < chunks;                      // (uniform)
    if (more) {
      load_w(first + ch + 1, wnext);
      copy_x(first + ch + 1, buf ^ 1);                      // the other buffer: last read before the barrier behind us
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(&xs[buf][t * 16 * KC + x_at[s]]);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wcur[s], b, acc[t], 0, 0, 0);
      }
    if (more) {
#pragma unroll
      for (int s = 0; s < STEPS; ++s) wcur[s] = wnext[s];
    }
    wait_loads_but<0>();                                    // the next chunk's rows have landed (this wave's share)
    __syncthreads();
  }
  if constexpr (GATED) {                                     // the gate waves hand their rounded sums to the up waves
    f32x4_t* meet = reinterpret_cast<f32x4_t*>(&xs[0][0]);   // (every wave is past its last read of the rows)
    static_assert(COLS * MT * WAVE * sizeof(f32x4_t) <= sizeof(xs), "the gate tiles fit the rows' buffers");
    if (!up_half) {
#pragma unroll
      for (int t = 0; t < MT; ++t) meet[(wave * MT + t) * WAVE + lane] = acc[t];
    }
    __syncthreads();
    if (!up_half) return;
  }
  // lane holds outputs 4 g .. 4 g + 3 of the tile for token 16 t + c
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + c;
    if (m >= M) continue;
    if constexpr (OUT == 3) {
      *reinterpret_cast<f32x4_t*>((float*)y + ((int64_t)blockIdx.y * M + m) * N + col_tile * 16 + 4 * g) = acc[t];
    } else if constexpr (OUT == 1) {
      f32x4_t o;
#pragma unroll
      for (int r = 0; r < 4; ++r) o[r] = bf16_to_float(float_to_bf16(acc[t][r]));
      *reinterpret_cast<f32x4_t*>((float*)y + (int64_t)m * N + col_tile * 16 + 4 * g) = o;
    } else {
      ushort4 o;
      bf16_t* oe = reinterpret_cast<bf16_t*>(&o);
      f32x4_t gates;
      if constexpr (GATED) gates = reinterpret_cast<const f32x4_t*>(&xs[0][0])[((wave - COLS) * MT + t) * WAVE + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if constexpr (GATED) {
          const float gate = bf16_to_float(float_to_bf16(gates[r]));
          const float up = bf16_to_float(float_to_bf16(acc[t][r]));
          const float sg = bf16_to_float(float_to_bf16(silu<bf16_t>(gate)));
          oe[r] = float_to_bf16(sg * up);
        } else {
          oe[r] = float_to_bf16(acc[t][r]);
        }
      }
      *reinterpret_cast<ushort4*>((bf16_t*)y + (int64_t)m * N + col_tile * 16 + 4 * g) = o;
    }
  }
}

constexpr int ROWS_MIN_TILES = 1024;   // tiles (gated: tile pairs times two) from which the kernel fills the GPU

template <int WAVES, int KC, int OUT>
void launch_rows(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t s, int splits = 1) {
  const dim3 grid(N / 16 / (OUT == 2 ? WAVES / 2 : WAVES), splits), block(WAVES * 64);
  const int mt = (M + 15) / 16;
#define ROWS(MT) gemm_rows_kernel<MT, WAVES, KC, OUT><<<grid, block, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, y, M, N, K)
  if (mt == 2) ROWS(2); else if (mt == 3) ROWS(3); else ROWS(4);
#undef ROWS
}

// The same for 65 to 128 rows (five to eight tiles of tokens): chunks of 64 columns keep the rows' two buffers within
// the LDS a block may have without asking.
template <int WAVES, int OUT>
void launch_rows_tall(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t s, int splits) {
  const dim3 grid(N / 16 / WAVES, splits), block(WAVES * 64);
#define ROWS(MT) gemm_rows_kernel<MT, WAVES, 64, OUT><<<grid, block, 0, s>>>((const bf16_t*)x, (const bf16_t*)w, y, M, N, K)
  switch ((M + 15) / 16) {
    case 5: ROWS(5); break;
    case 6: ROWS(6); break;
    case 7: ROWS(7); break;
    default: ROWS(8); break;
  }
#undef ROWS
}
}  // namespace

// Whether holon_gemm_rows_bf16 serves this product (gated: N is the number of output columns I, the weight has 2 I rows).
extern "C" int holon_gemm_rows_supported(int M, int N, int K, int gated) {
  const int tiles = N / 16;
  return M > 16 && M <= 64 && N % 16 == 0 && K % 256 == 0 && K >= 256 && tiles % 8 == 0 &&
         tiles * (gated ? 2 : 1) >= ROWS_MIN_TILES;
}

// y[M, N] = x[M, K] w^T over tiled weights, 17 <= M <= 64; out_f32: 0 bfloat16, otherwise float32 of the values rounded
// to bfloat16. Measured on MI355X at N = 24,576, K = 4,096: 44 us at 64 rows, 39 at 32 (the vendor library 47 and 46);
// N = 151,936: 238 and 219 us (267 and 269).
extern "C" int holon_gemm_rows_bf16(const void* x, const void* w_tiled, void* y, int M, int N, int K, int out_f32,
                                    void* stream) {
  HOLON_CHECK(holon_gemm_rows_supported(M, N, K, 0), "gemm (17 to 64 rows): M=%d N=%d K=%d not served", M, N, K);
  hipStream_t s = (hipStream_t)stream;
  const bool wide = N / 16 >= 4096;          // a vocabulary's worth of tiles: longer chunks, at 64 rows eight waves
  if (out_f32) {
    if (wide && M > 48) launch_rows<8, 256, 1>(x, w_tiled, y, M, N, K, s);
    else if (wide) launch_rows<4, 256, 1>(x, w_tiled, y, M, N, K, s);
    else launch_rows<4, 128, 1>(x, w_tiled, y, M, N, K, s);
  } else {
    if (wide && M > 48) launch_rows<8, 256, 0>(x, w_tiled, y, M, N, K, s);
    else if (wide) launch_rows<4, 256, 0>(x, w_tiled, y, M, N, K, s);
    else launch_rows<4, 128, 0>(x, w_tiled, y, M, N, K, s);
  }
  HOLON_LAUNCH_OK();
  return 0;
}

// y[M, I] = round(silu(round(x gate^T))) * round(x up^T) with w = [gate; up] ([2 I, K], tiled), 17 <= M <= 64: four waves
// a block, two gate tiles and the two up tiles of the same columns; where eight waves a block (four and four, chunks of
// 256 columns: half the reads of the rows) still give a block to every compute unit, those. Measured over weights
// streamed from memory, 51200 x 5120: 94 us at 32 rows and 104 at 64 against 104 and 119 with four waves (the vendor
// library's product and SiLU-mul: 101 and 109); 24576 x 4096, where eight waves would leave 192 blocks: 39 and 46 us
// with four (the vendor library's pair: 50 and 51).
constexpr int ROWS_GLU_WIDE_BLOCKS = 256;
extern "C" int holon_gemm_rows_glu_bf16(const void* x, const void* w_tiled, void* y, int M, int I, int K, void* stream) {
  HOLON_CHECK(holon_gemm_rows_supported(M, I, K, 1), "gated gemm (17 to 64 rows): M=%d I=%d K=%d not served", M, I, K);
  if (I / 16 / 4 >= ROWS_GLU_WIDE_BLOCKS) launch_rows<8, 256, 2>(x, w_tiled, y, M, I, K, (hipStream_t)stream);
  else launch_rows<4, 128, 2>(x, w_tiled, y, M, I, K, (hipStream_t)stream);
  HOLON_LAUNCH_OK();
  return 0;
}

namespace {
constexpr int PARTS_KC = 128;          // columns of K a chunk of the split form holds
constexpr int PARTS_MAX_SPLITS = 16;
constexpr int PARTS_MAX_ROWS = 128;    // (the forms that write whole products serve up to 64)
constexpr int PARTS_WAVES = 4;         // eight were slower at every shape measured

// y[i] = round(parts[0][i] + parts[1][i] + ...) in split order, four values a thread.
__global__ void sum_parts_kernel(const float* __restrict__ parts, bf16_t* __restrict__ y, int splits, int64_t count) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= count) return;
  f32x4_t sum = *reinterpret_cast<const f32x4_t*>(parts + i);
  for (int s = 1; s < splits; ++s) sum += *reinterpret_cast<const f32x4_t*>(parts + (int64_t)s * count + i);
  ushort4 o;
  bf16_t* oe = reinterpret_cast<bf16_t*>(&o);
#pragma unroll
  for (int r = 0; r < 4; ++r) oe[r] = float_to_bf16(sum[r]);
  *reinterpret_cast<ushort4*>(y + i) = o;
}
}  // namespace

// Whether holon_gemm_rows_parts_bf16 serves this product with K cut into `splits` shares (blocks of four waves, each
// with a tile of 16 columns of its own).
extern "C" int holon_gemm_rows_parts_supported(int M, int N, int K, int splits) {
  return M > 16 && M <= PARTS_MAX_ROWS && N % 16 == 0 && (N / 16) % PARTS_WAVES == 0 && splits >= 1 &&
         splits <= PARTS_MAX_SPLITS && K > 0 && K % (PARTS_KC * splits) == 0;
}

// How many shares of K serve a narrow weight best: measured on MI355X, eight where that gives at most 1,024 blocks of
// four waves (4096 x 4096 at 64 rows: 9.4 us against the vendor library's 12.4; 4096 x 12288: 20.8 against 27.5;
// 5120 x 25600: 60 against 78), four for wider weights; 0 when the shape is not served or K has no such shares.
extern "C" int holon_gemm_rows_splits(int M, int N, int K) {
  if (N % 16 || K <= 0) return 0;
  int splits = N / 16 <= 512 ? 8 : 4;
  while (splits > 1 && K % (PARTS_KC * splits)) splits /= 2;
  return splits > 1 && holon_gemm_rows_parts_supported(M, N, K, splits) ? splits : 0;
}

// parts[s][M][N] (float32) = x[:, share s of K] w[:, share s of K]^T over tiled weights, 17 <= M <= 128: the product is
// the sum of the parts in order, which the reader takes (holon_rmsnorm_parts, holon_sum_parts).
extern "C" int holon_gemm_rows_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K,
                                          int splits, void* stream) {
  HOLON_CHECK(holon_gemm_rows_parts_supported(M, N, K, splits),
              "gemm in parts (17 to 64 rows): M=%d N=%d K=%d splits=%d not served", M, N, K, splits);
  if (M > 64) launch_rows_tall<PARTS_WAVES, 3>(x, w_tiled, parts, M, N, K, (hipStream_t)stream, splits);
  else launch_rows<PARTS_WAVES, PARTS_KC, 3>(x, w_tiled, parts, M, N, K, (hipStream_t)stream, splits);
  HOLON_LAUNCH_OK();
  return 0;
}

// y[count] (bfloat16) = the parts [splits, count] summed in order in float32, rounded once. count % 4 == 0.
extern "C" int holon_sum_parts(const void* parts, void* y, int splits, int64_t count, void* stream) {
  HOLON_CHECK(splits >= 1 && count >= 0 && count % 4 == 0, "sum of parts: splits=%d count=%lld", splits, (long long)count);
  if (count == 0) return 0;
  const int threads = 256;
  const int64_t blocks = (count / 4 + threads - 1) / threads;
  HOLON_CHECK(blocks <= 0x7fffffff, "sum of parts: %lld values are too many", (long long)count);
  sum_parts_kernel<<<(unsigned)blocks, threads, 0, (hipStream_t)stream>>>((const float*)parts, (bf16_t*)y, splits, count);
  HOLON_LAUNCH_OK();
  return 0;
}
