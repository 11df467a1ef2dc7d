// parts[s][M, N] = x[M, share s of K] w[N, share s of K]^T for 129 to 1,024 rows (prompt portions of a few hundred
// tokens) over a narrow weight with a long K (a feed-forward's second product): bfloat16 operands, float32 sums on the
// matrix cores, the shares added up by whoever reads them (the residual add + norm does so as it reads).
//
// The shape the vendor library serves worst: few tiles of output and a long K, so that its blocks walk all of K alone
// and re-read both operands from L2 (4096 x 12288 at 512 rows: 82 us, 0.63 PFLOP/s). Here K is cut into shares over
// the grid as well, and a block of four waves takes 128 rows against 4 x NT tiles of 16 columns: the rows' chunk of KC
// columns goes into LDS once a block by the memory pipeline (global_load_lds, swizzled rows, three buffers), every
// wave streams the weights of its own NT tiles from the tiled copy (a contiguous kilobyte a product) two chunks ahead
// of the one it multiplies, and each B operand read from LDS serves NT products. A tile's sums run over its share
// of K in order, so a result depends on nothing but the operands and the number of shares.
//
// Blocks are numbered so that the row blocks of one set of columns run on the same XCD (blocks go to the XCDs in
// turn), one shortly after the other: the weights they share then come out of that XCD's L2.
#include <type_traits>

#include "common.h"
#include "holon_hip.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

namespace {
constexpr int TILES_WAVES = 4;
constexpr int TILES_MT = 8;            // tiles of 16 rows a block takes: 128 rows
constexpr int TILES_KC = 64;           // columns of K a chunk holds (rows of 128 bytes in LDS)
constexpr int TILES_XCDS = 8;

template <int NT>
__global__ void __launch_bounds__(TILES_WAVES * 64, 2) gemm_tiles_kernel(const bf16_t* __restrict__ x,
                                                                          const bf16_t* __restrict__ w,
                                                                          float* __restrict__ parts, int M, int N, int K,
                                                                          int col_blocks, int row_blocks, int splits) {
  constexpr int MT = TILES_MT, WAVES = TILES_WAVES, KC = TILES_KC;
  constexpr int ROWS = MT * 16, STEPS = KC / 32;
  constexpr int PPR = KC / 8;                               // 16-byte pieces a row of a chunk has
  constexpr int RPI = 64 / PPR;                             // rows one copy instruction (a kilobyte) brings
  constexpr int COPIES = ROWS / RPI;                        // instructions a chunk takes
  constexpr int XCH = COPIES / WAVES;                       // of which a wave issues this many
  static_assert(COPIES % WAVES == 0, "every wave issues the same number of copies");
  __shared__ __attribute__((aligned(1024))) bf16_t xs[3][ROWS * KC];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  // block number -> (columns and share, row block): of TILES_XCDS * row_blocks consecutive blocks, those that are
  // TILES_XCDS apart (the same XCD) take the row blocks of one (columns, share)
  int pair, rb;
  {
    const int id = blockIdx.x, per = TILES_XCDS * row_blocks, pairs = col_blocks * splits;
    const int full = pairs / TILES_XCDS * TILES_XCDS;      // pairs that come in whole groups of TILES_XCDS
    if (id < full * row_blocks) {
      pair = id / per * TILES_XCDS + id % TILES_XCDS;
      rb = id % per / TILES_XCDS;
    } else {                                                // the rest: row blocks side by side
      const int left = id - full * row_blocks;
      pair = full + left / row_blocks;
      rb = left % row_blocks;
    }
  }
  const int cb = pair % col_blocks, split = pair / col_blocks;
  const int row0 = rb * ROWS;
  const int tile0 = (cb * WAVES + wave) * NT;
  const int64_t tile_stride = (int64_t)(K / 32) * 512;      // values of one tile of 16 columns over all of K
  const bf16_t* wp = w + (int64_t)tile0 * tile_stride;       // (the same for the wave's lanes)
  uint32_t w_at[NT];                                         // this lane's 16 bytes of tile n's kilobyte
#pragma unroll
  for (int n = 0; n < NT; ++n) w_at[n] = (uint32_t)((n * tile_stride + lane * 8) * 2);
  f32x4_t acc[MT][NT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[t][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // three sets of weight registers and three buffers of rows, in turn: chunk ch + 2 is asked for while chunk ch is
  // multiplied (one chunk is 1,024 cycles of products, and what is asked for takes longer than that to come)
  bf16x8_t wreg[3][STEPS][NT];
  // (loads the compiler does not track, like the copies of the rows: the waits are written below)
  static_assert(STEPS == 2, "a chunk's two kilobytes of a tile: offsets 0 and 1024");
  auto load_w = [&](int chunk, bf16x8_t (&to)[STEPS][NT]) {
    const bf16_t* from = wp + (int64_t)chunk * STEPS * 512;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
      load16_untracked<bf16x8_t, 0>(to[0][n], from, w_at[n]);
      load16_untracked<bf16x8_t, 1024>(to[1][n], from, w_at[n]);
    }
  };
  // what this lane copies: of instruction j = i * WAVES + wave, row j * RPI + lane / PPR, the piece that belongs at
  // place lane % PPR (rows beyond M repeat the last row: what they give is never written)
  uint32_t x_src[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int row = (i * WAVES + wave) * RPI + lane / PPR;
    const int piece = (lane % PPR) ^ ((row / 2) % 8);
    x_src[i] = (uint32_t)(((int64_t)min(row0 + row, M - 1) * K + piece * 8) * 2);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)&xs[0][0];
  auto copy_x = [&](int chunk, int buf) {
    const bf16_t* from = x + (int64_t)chunk * KC;
#pragma unroll
    for (int i = 0; i < XCH; ++i)
      load_to_lds16(from, x_src[i], lds0 + (uint32_t)(buf * ROWS * KC * 2 + (i * WAVES + wave) * 1024));
  };
  // where this lane reads the B operand of product s for the tile of rows t: row 16 t + c, piece 4 s + g
  uint32_t x_at[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) x_at[s] = (uint32_t)(c * KC + 8 * ((4 * s + g) ^ ((c / 2) % 8)));
  const int chunks = K / KC / splits;                       // this block's share of K
  const int first = split * chunks;
  constexpr int LOADS = STEPS * NT + XCH;                   // what a wave asks for per chunk
  load_w(first, wreg[0]);
  copy_x(first, 0);
  if (chunks > 1) {
    load_w(first + 1, wreg[1]);
    copy_x(first + 1, 1);
    wait_loads_but<LOADS>();
  } else {
    wait_loads_but<0>();
  }
  __syncthreads();
  auto chunk = [&](auto which, int ch) {
    constexpr int B = decltype(which)::value;               // ch % 3
    const bool ahead = ch + 2 < chunks;                     // (uniform)
    if (ahead) {
      load_w(first + ch + 2, wreg[(B + 2) % 3]);
      copy_x(first + ch + 2, (B + 2) % 3);                  // the buffer chunk ch - 1 was read from, before the barrier behind us
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8_t b = *reinterpret_cast<const bf16x8_t*>(&xs[B][t * 16 * KC + x_at[s]]);
#pragma unroll
        for (int n = 0; n < NT; ++n)
          acc[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wreg[B][s][n], b, acc[t][n], 0, 0, 0);
      }
    // chunk ch + 1 has landed (this wave's share of the rows, and its weights): all but what was just asked for
    if (ahead) wait_loads_but<LOADS>(); else wait_loads_but<0>();
    __syncthreads();
  };
  for (int ch = 0; ch < chunks; ch += 3) {
    chunk(std::integral_constant<int, 0>{}, ch);
    if (ch + 1 < chunks) chunk(std::integral_constant<int, 1>{}, ch + 1);
    if (ch + 2 < chunks) chunk(std::integral_constant<int, 2>{}, ch + 2);
  }
  // lane holds sums 4 g .. 4 g + 3 of tile n for row 16 t + c
  float* out = parts + (int64_t)split * M * N;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = row0 + t * 16 + c;
    if (m >= M) continue;
#pragma unroll
    for (int n = 0; n < NT; ++n)
      *reinterpret_cast<f32x4_t*>(out + (int64_t)m * N + (tile0 + n) * 16 + 4 * g) = acc[t][n];
  }
}

constexpr int TILES_NT = 4;
constexpr int TILES_MAX_SPLITS = 8;
}  // namespace

// Whether holon_gemm_tiles_parts_bf16 serves this product with K cut into `splits` shares.
extern "C" int holon_gemm_tiles_parts_supported(int M, int N, int K, int splits) {
  return M > 128 && M <= 1024 && N % (16 * TILES_WAVES * TILES_NT) == 0 && splits >= 1 && splits <= TILES_MAX_SPLITS &&
         K > 0 && K % (TILES_KC * splits) == 0 && K % 32 == 0 &&
         (int64_t)M * K * 2 < (int64_t)1 << 32;             // (a lane's place among the rows is a 32-bit byte offset)
}

// How many shares of K to take, 0 where the kernel does not serve the shape or is not the one to take: it is for
// weights whose K is well above their N (few output tiles, long sums), with as few shares (a power of two, at most
// eight) as give 384 blocks. Measured on MI355X with the add + norm that reads the parts, against the vendor library's
// product with its add + norm, us: 4096 x 12288 at 256 / 512 / 768 / 1,024 rows 46 / 73 / 103 / 114 against 61 / 93 /
// 111 / 135; 5120 x 25600: 120 / 171 / 210 / 291 against 268 / 278 / 303 / 362; 2560 x 9728: 37 / 57 / 63 / 87 against
// 43 / 57 / 71 / 90. With K between 1.5 and 2 times N it still wins up to 768 rows (5120 x 8192: 54 / 76 / 87 against
// 78 / 81 / 90; at 1,024 rows 119 against 111); with K = N it loses everywhere (4096 x 4096: 26 / 36 / 52 / 58 against
// 24 / 33 / 37 / 47). Blocks of eight waves (the rows read half as often) were no faster.
extern "C" int holon_gemm_tiles_splits(int M, int N, int K) {
  if (M <= 128 || M > 1024 || N <= 0 || N % (16 * TILES_WAVES * TILES_NT)) return 0;
  if (!(K >= 2 * N || (2 * (int64_t)K >= 3 * (int64_t)N && M <= 768))) return 0;
  const int blocks = N / (16 * TILES_WAVES * TILES_NT) * ((M + 127) / 128);
  int splits = 1;
  while (splits < TILES_MAX_SPLITS && blocks * splits < 384) splits *= 2;
  while (splits > 1 && K % (TILES_KC * splits)) splits /= 2;
  return holon_gemm_tiles_parts_supported(M, N, K, splits) && blocks * splits >= 128 ? splits : 0;
}

// parts[s][M][N] (float32) = x[:, share s of K] w[:, share s of K]^T over tiled weights, 129 <= M <= 1,024.
extern "C" int holon_gemm_tiles_parts_bf16(const void* x, const void* w_tiled, void* parts, int M, int N, int K,
                                           int splits, void* stream) {
  HOLON_CHECK(holon_gemm_tiles_parts_supported(M, N, K, splits),
              "gemm in parts (129 to 1,024 rows): M=%d N=%d K=%d splits=%d not served", M, N, K, splits);
  const int col_blocks = N / (16 * TILES_WAVES * TILES_NT), row_blocks = (M + 127) / 128;
  gemm_tiles_kernel<TILES_NT><<<col_blocks * row_blocks * splits, TILES_WAVES * 64, 0, (hipStream_t)stream>>>(
      (const bf16_t*)x, (const bf16_t*)w_tiled, (float*)parts, M, N, K, col_blocks, row_blocks, splits);
  HOLON_LAUNCH_OK();
  return 0;
}
