// Paged causal attention on the matrix cores, bfloat16, for head_dim in {64, 128, 256} and page sizes that are
// multiples of 16. Two kernels share one tile loop:
//   * prompt portions: one wave owns NT tiles of 16 (query, head) rows and walks the keys 0 .. its last position;
//   * decode rows: the keys of a row are split over waves, each writes an unnormalised partial (max, sum, values) and a
//     second kernel merges the partials in a fixed order.
//
// A tile's 16 rows are the G query heads of one kv head at 16/G consecutive positions (grouped-query attention: the
// heads of a group read the same keys, so each key is loaded once per group, not once per head).
//
// Operand layouts (v_mfma_f32_16x16x32_bf16: A is 16x32, B is 32x16, lane l holds 8 consecutive k of row/column l%16
// starting at 8*(l/16); the 16x16 result has rows 4*(l/16)+r, r<4, of column l%16 in lane l):
//   S^T = K Q^T: A = 16 keys x 32 dims straight from a key page (keys are rows there), B = Q^T from registers.
//     Two products cover 32 keys; their rows are permuted (row i of the first is key 8*(i/4) + i%4 of the block, of the
//     second 4 more) so that lane group g ends up with the scores of keys 8g .. 8g+7 of one query:
//     exactly the B operand of the next product, with no data movement.
//   O^T = V^T P^T: A = 16 dims x 32 keys straight from a value page (values are stored transposed inside a page, so the
//     8 keys a lane needs are one 16-byte load), B = P^T from the registers above, rounded to bfloat16.
// Softmax is online, float32, in base 2 with log2(e) folded into the scale.
#include <mutex>

#include "common.h"
#include "holon_hip.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8_t*>(p); }

// Values are fetched 32 keys at a time, so the last block of a row reaches past its last key: into slots of the page
// that an earlier request may have left anything in, or into the null page. Their probabilities are zero, but zero
// times a NaN or an infinity is a NaN in the value product: such values are replaced by zeros. `v` holds keys
// first_key .. first_key + 7.
__device__ __forceinline__ void zero_after(bf16x8_t& v, int first_key, int key_hi) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (first_key + i > key_hi) v[i] = (__bf16)0.f;
}

struct AttnArgs {
  const bf16_t* q;         // [T, Hq, D]
  bf16_t* out;             // [T, Hq, D]
  const bf16_t* pages;     // [num_pages, 2, Hkv, P*D]
  const int32_t* table;    // [slots, table_stride]
  int table_stride;
  const int32_t* slots;    // [B]
  const int32_t* lens;     // [B]
  const int32_t* qstart;   // [B+1]
  const int32_t* row_ids;  // rows this launch serves
  int heads, kv_heads, page_size;
  float scale_log2;        // scale * log2(e)
  int window;
  // decode only
  float* part_o;           // [n_rows, Hq, splits, D]
  float* part_ml;          // [n_rows, Hq, splits, 2]
  int splits, keys_per_split;
  int out_splits;          // partials a (row, head) leaves: splits / waves of a block (1: the block writes the result)
  int rows_in_order;       // every row of the step is a decode row and row_ids[i] = query_start[i] = i
  // long prompt portions only: a block runs one of its two ranges (blockIdx.z = 2 row + which), not both
  int unpaired;
};

// How the 16 rows of a tile map to (position, head) for a group of G heads.
struct TileMap {
  int rows_per_pos;   // min(G, 16)
  int pos_per_tile;   // 16 / rows_per_pos
  int head_blocks;    // ceil(G / 16)
};
__host__ __device__ inline TileMap tile_map(int group) {
  TileMap m;
  m.rows_per_pos = group < 16 ? group : 16;
  m.pos_per_tile = 16 / m.rows_per_pos;
  m.head_blocks = (group + 15) / 16;
  return m;
}

// One block of 32 keys for one tile, after the score products: mask (only where the block is not wholly visible),
// running max and sum, the probabilities as the next product's B operand, and the rescale of what was summed so far
// (only when some row's max moved: later blocks rarely move it, and the accumulators can then stay where the matrix
// cores keep them). Lane (g, c): s0[r] is key kb+8g+r against query column c, s1[r] key kb+8g+4+r.
template <int DS>
__device__ __forceinline__ bf16x8_t softmax_block(const f32x4_t& s0, const f32x4_t& s1, bool whole, int kb, int g,
                                                  int qp, int first, int key_lo, int key_hi, float scale_log2,
                                                  float& m, float& l, f32x4_t (&o)[DS]) {
  // m and the comparisons are in units of the raw scores' scale times log2(e); a score enters as one fused
  // multiply-add, exp2(s * c - m)
  float sv[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) sv[r] = r < 4 ? s0[r] : s1[r - 4];
  if (!whole) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int key = kb + 8 * g + r;
      if (!(key <= qp && key >= first && key >= key_lo && key <= key_hi)) sv[r] = -INFINITY;
    }
  }
  float mx = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
  {   // over the four lane groups: the swaps leave lane l's value beside that of lane l ^ 16, then of lane l ^ 32
    const auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    mx = fmaxf(__uint_as_float(rows[0]), __uint_as_float(rows[1]));
    const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    mx = fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
  }
  const float m_new = fmaxf(m, mx * scale_log2);          // (scale > 0: the largest raw score is the largest scaled one)
  const float m_use = m_new == -INFINITY ? 0.f : m_new;   // nothing visible yet: keep everything at zero
  bf16x8_t pb;
  float psum = 0.f;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const float p = __builtin_amdgcn_exp2f(fmaf(sv[r], scale_log2, -m_use));   // <= 0; below 2^-126 flushes to zero
    psum += p;
    pb[r] = (__bf16)p;
  }
  if (__any(m_new != m)) {
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    l *= alpha;
#pragma unroll
    for (int ds = 0; ds < DS; ++ds) o[ds] *= alpha;
    m = m_new;
  }
  l += psum;
  return pb;
}

// One wave: NT tiles against keys [key_lo, key_hi] (inclusive, as bounded per row by causality and the window).
// On return o[t][dsub] holds the unnormalised O^T, m[t] the running max (base-2 scaled), l[t] this lane's share of
// the sum (to be added over the four lane groups).
// `fresh` (nullable): the key (D values) and then the value (D values) of key number `key_hi`, in LDS, which take the
// place of what the cache holds there (a decode row's new token, whose stores to the cache may still be under way).
// `prepare()` runs once the first block's keys have been asked for and before `qf` is first read: arithmetic that
// makes the queries (a decode row's norm and rotation) then runs while those loads are under way.
struct Nothing {
  __device__ __forceinline__ void operator()() const {}
};
template <int D, int NT, typename Prepare = Nothing>
__device__ __forceinline__ void attn_tiles(const AttnArgs& a, const int32_t* __restrict__ trow, int hk,
                                           const bf16x8_t (&qf)[NT][D / 32], const int (&qpos)[NT],
                                           const int (&tile_last)[NT], const int (&tile_first)[NT], int key_lo,
                                           int key_hi,
                                           f32x4_t (&o)[NT][D / 16], float (&m)[NT], float (&l)[NT],
                                           const bf16_t* fresh = nullptr, Prepare prepare = Prepare()) {
  const int lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  const int P = a.page_size;
  const int64_t plane = (int64_t)P * D;
  const int64_t page_stride = 2 * (int64_t)a.kv_heads * plane;
  const bf16_t* kbase = a.pages + (int64_t)hk * plane;
  const bf16_t* vbase = a.pages + ((int64_t)a.kv_heads + hk) * plane;
  const int krow = 8 * (c / 4) + (c % 4);   // this lane's key (row of A) within the 32-key block, first product
  const int khalf = krow / 16, kin = krow % 16;
  const int max_page = a.table_stride - 1;

  // The block table's entries for a block of 32 keys: the page of its first 16 keys and of its last 16. They are
  // looked up two blocks ahead and kept in registers, so that no load of keys or values waits for a lookup issued
  // just before it: a wave's loads return in the order they were issued, and waiting for the newest one (a lookup)
  // would wait for every load of keys and values still under way.
  auto lookup = [&](int kb, int (&e)[2]) {
    e[0] = trow[min(kb / P, max_page)];
    e[1] = trow[min((kb + 16) / P, max_page)];
  };
  // Keys of block kb for this lane: two fragments per 32 dims (the lane's key, and the key 4 further on).
  auto load_keys = [&](int kb, const int (&e)[2], bf16x8_t (&f0)[D / 32], bf16x8_t (&f1)[D / 32]) {
    const int half_key = kb + 16 * khalf;
    const int64_t pg = (int64_t)(khalf ? e[1] : e[0]) * page_stride;
    const bf16_t* krowp = kbase + pg + (int64_t)(half_key % P + kin) * D + 8 * g;
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks) {
      f0[ks] = load8(krowp + ks * 32);
      f1[ks] = load8(krowp + 4 * D + ks * 32);
    }
  };
  const int kb_first = (key_lo / 32) * 32;
  int e_cur[2], e_next[2];
  lookup(kb_first, e_cur);
  lookup(kb_first + 32, e_next);
  bf16x8_t kf0[D / 32], kf1[D / 32];
  load_keys(kb_first, e_cur, kf0, kf1);
  prepare();
  for (int kb = kb_first; kb <= key_hi; kb += 32) {
    // values of this block (lane group g needs keys 8g .. 8g+7, for dims dsub*16 + c) and the keys of the next one
    // are requested before this block's products, so that their latency hides behind the matrix cores
    const int vkey = kb + (g >= 2 ? 16 : 0);
    const bf16_t* vrowp = vbase + (int64_t)(g >= 2 ? e_cur[1] : e_cur[0]) * page_stride + (int64_t)c * P + vkey % P +
                          8 * (g % 2);
    bf16x8_t vf[D / 16];
#pragma unroll
    for (int ds = 0; ds < D / 16; ++ds) vf[ds] = load8(vrowp + (int64_t)ds * 16 * P);
    if (kb + 31 > key_hi) {
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) zero_after(vf[ds], kb + 8 * g, key_hi);
    }
    if (fresh != nullptr && kb + 31 >= key_hi) {           // the block that holds key_hi: its key and value from LDS
      const int k0 = kb + 16 * khalf + kin;                // this lane's keys are k0 and k0 + 4
      if (k0 == key_hi || k0 + 4 == key_hi) {
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          const bf16x8_t nk = *reinterpret_cast<const bf16x8_t*>(fresh + ks * 32 + 8 * g);
          if (k0 == key_hi) kf0[ks] = nk; else kf1[ks] = nk;
        }
      }
      const int j = key_hi - (kb + 8 * g);                 // the value's place among this lane's eight keys, if any
      if (j >= 0 && j < 8) {
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) {
          const __bf16 nv = reinterpret_cast<const __bf16*>(fresh + D)[ds * 16 + c];
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (i == j) vf[ds][i] = nv;
        }
      }
    }
    bf16x8_t nf0[D / 32], nf1[D / 32];
    const bool more = kb + 32 <= key_hi;
    int e_after[2] = {0, 0};
    if (more) {
      load_keys(kb + 32, e_next, nf0, nf1);
      lookup(kb + 64, e_after);                  // (an entry past the row's keys is clamped into the table and unused)
    }
    bf16x8_t pb[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (kb > tile_last[t]) continue;   // every key of the block lies after every query of the tile
      f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf0[ks], qf[t][ks], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf1[ks], qf[t][ks], s1, 0, 0, 0);
      }
      const int qp = qpos[t];
      const int first = a.window > 0 ? qp - a.window + 1 : 0;
      const bool whole = kb + 31 <= tile_first[t] && kb >= key_lo && kb + 31 <= key_hi &&
                         (a.window <= 0 || kb >= tile_last[t] - a.window + 1);
      pb[t] = softmax_block<D / 16>(s0, s1, whole, kb, g, qp, first, key_lo, key_hi, a.scale_log2, m[t], l[t], o[t]);
    }
#pragma unroll
    for (int ds = 0; ds < D / 16; ++ds) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        if (kb > tile_last[t]) continue;
        o[t][ds] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[ds], pb[t], o[t][ds], 0, 0, 0);
      }
    }
    if (more) {
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks) {
        kf0[ks] = nf0[ks];
        kf1[ks] = nf1[ks];
      }
      e_cur[0] = e_next[0]; e_cur[1] = e_next[1];
      e_next[0] = e_after[0]; e_next[1] = e_after[1];
    }
  }
}

// Column c of tile (first position index `p0`): which query token, head and position it is, or invalid.
struct RowRef {
  bool valid;
  int token, head, qpos;
};
__device__ __forceinline__ RowRef row_ref(const TileMap& tm, int c, int p0, int hb, int hk, int group, int qs, int nq,
                                          int n) {
  RowRef r;
  const int pi = c / tm.rows_per_pos, hi = hb * 16 + c % tm.rows_per_pos;
  const int qi = p0 + pi;
  r.valid = pi < tm.pos_per_tile && qi < nq && hi < group;
  r.token = qs + qi;
  r.head = hk * group + hi;
  r.qpos = n - nq + qi;
  return r;
}

template <int D, int NT>
__global__ void __launch_bounds__(256) attn_prefill_kernel(AttnArgs a) {
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int g = lane / 16, c = lane % 16;
  const int b = a.row_ids[blockIdx.z];
  const int group = a.heads / a.kv_heads;
  const TileMap tm = tile_map(group);
  const int hk = blockIdx.y / tm.head_blocks, hb = blockIdx.y % tm.head_blocks;
  const int qs = a.qstart[b], nq = a.qstart[b + 1] - qs, n = a.lens[b];
  // Tiles of 16 rows along the row's positions. A wave takes NT of them: with NT = 2 the w-th from the start and the
  // w-th from the end, so that every wave walks about the same number of keys under the causal mask.
  const int n_tiles = (nq + tm.pos_per_tile - 1) / tm.pos_per_tile;
  const int wi = blockIdx.x * 4 + wave;
  if (n <= 0 || wi >= (n_tiles + NT - 1) / NT) return;
  const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;

  bf16x8_t qf[NT][D / 32];
  int qpos[NT], tile_last[NT], tile_first[NT];   // a tile's rows sit at positions tile_first .. tile_last
  RowRef rr[NT];
  int key_hi = 0, key_lo = 0x7fffffff;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int tile = NT == 1 ? n_tiles - 1 - wi : (t == 0 ? wi : n_tiles - 1 - wi);
    if (t == 1 && tile <= wi) tile = n_tiles;          // an odd count: the middle tile is the first one's alone
    const int p0 = tile * tm.pos_per_tile;
    rr[t] = row_ref(tm, c, p0, hb, hk, group, qs, nq, n);
    qpos[t] = rr[t].valid ? rr[t].qpos : -1;   // an unused row sees no key
    const int last_qi = min(nq, p0 + tm.pos_per_tile) - 1;
    tile_last[t] = p0 < nq ? n - nq + last_qi : -1;
    tile_first[t] = n - nq + p0;
    key_hi = max(key_hi, tile_last[t]);
    if (p0 < nq) key_lo = min(key_lo, a.window > 0 ? max(0, n - nq + p0 - a.window + 1) : 0);
    const bf16_t* qp = a.q + ((int64_t)rr[t].token * a.heads + rr[t].head) * D + 8 * g;
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks) {
      if (rr[t].valid) {
        qf[t][ks] = load8(qp + ks * 32);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) qf[t][ks][i] = (__bf16)0.f;
      }
    }
  }
  f32x4_t o[NT][D / 16];
  float m[NT], l[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    m[t] = -INFINITY;
    l[t] = 0.f;
#pragma unroll
    for (int ds = 0; ds < D / 16; ++ds) o[t][ds] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  attn_tiles<D, NT>(a, trow, hk, qf, qpos, tile_last, tile_first, key_lo, key_hi, o, m, l);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    float lt = l[t];
    lt += __shfl_xor(lt, 16, WAVE);
    lt += __shfl_xor(lt, 32, WAVE);
    if (!rr[t].valid) continue;
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    bf16_t* op = a.out + ((int64_t)rr[t].token * a.heads + rr[t].head) * D + 4 * g;
#pragma unroll
    for (int ds = 0; ds < D / 16; ++ds) {
      ushort4 w;
      w.x = float_to_bf16(o[t][ds][0] * inv);
      w.y = float_to_bf16(o[t][ds][1] * inv);
      w.z = float_to_bf16(o[t][ds][2] * inv);
      w.w = float_to_bf16(o[t][ds][3] * inv);
      *reinterpret_cast<ushort4*>(op + ds * 16) = w;
    }
  }
}

// A barrier that waits for this wave's LDS traffic only. __syncthreads() also waits for every global load in flight
// (vmcnt(0)), which would make each stage wait for the loads it has just requested for a later stage.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Prompt portions, staged through LDS: a block of four waves owns 4*NT consecutive tiles (for four heads a group: 32
// positions with NT = 2) and walks the keys in stages of 32; each stage's keys and transposed values are copied from
// the pages into LDS once per block (double buffered: the next stage's loads are in flight while this one is
// multiplied) and every wave takes its matrix-core operands from there, so a key is read from the cache once per
// block, not once per wave. Keys are stored in LDS in the order the two score products want their rows (lane c reads
// row c, then row 16 + c), which with a row pitch of D + 8 makes the 16-byte reads conflict-free; value rows have a
// pitch of 40. To even out the causal mask, a block does two position ranges: the b-th from the start and the b-th
// from the end.
template <int D, int NT>
__global__ void __launch_bounds__(256) attn_prefill_lds_kernel(AttnArgs a) {
  constexpr int KP = D + 8;    // pitch of a key row in LDS (elements)
  constexpr int VP = 40;       // pitch of a value row: 32 keys + 8
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][32 * KP];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][D * VP];
  constexpr int PG = 4096;     // the row's first block-table entries, kept in LDS: page lookups then do not queue
  __shared__ int32_t pg_lds[PG];   // behind the vector loads in flight
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, tid = threadIdx.x;
  const int g = lane / 16, c = lane % 16;
  const int b = a.row_ids[blockIdx.z];
  const int group = a.heads / a.kv_heads;
  const TileMap tm = tile_map(group);
  const int hk = blockIdx.y / tm.head_blocks, hb = blockIdx.y % tm.head_blocks;
  const int qs = a.qstart[b], nq = a.qstart[b + 1] - qs, n = a.lens[b];
  const int n_tiles = (nq + tm.pos_per_tile - 1) / tm.pos_per_tile;
  constexpr int TPB = 4 * NT;                                  // tiles a block owns per range
  const int n_ranges = (n_tiles + TPB - 1) / TPB;
  if (n <= 0 || (int)blockIdx.x >= (n_ranges + 1) / 2) return;   // uniform over the block
  const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;
  const int P = a.page_size;
  const int64_t plane = (int64_t)P * D;
  const int64_t page_stride = 2 * (int64_t)a.kv_heads * plane;
  const bf16_t* kbase = a.pages + (int64_t)hk * plane;
  const bf16_t* vbase = a.pages + ((int64_t)a.kv_heads + hk) * plane;
  const int max_page = min(a.table_stride, PG) - 1;

  // every entry a stage can ask for: the last stage's second half may lie one page past the row's tokens (the table
  // holds a valid page id there, the null page or any other: the keys are masked), so the whole row is copied
  for (int i = tid; i < min(PG, a.table_stride); i += 256) pg_lds[i] = trow[i];
  // this thread's share of a stage's copy: D/64 chunks of keys and as many of values, 16 bytes each
  constexpr int KCH = D / 8;                                   // chunks per key row
  constexpr int ROUNDS = D / 64;                               // 32 keys x D and D x 32 values: 4 D chunks each, 256 threads
  static_assert(D == 64 || D == 128, "the LDS kernel copies one or two chunks of each kind per thread");
  int k_key[ROUNDS], k_col[ROUNDS], k_dst[ROUNDS], v_d[ROUNDS], v_kc[ROUNDS], v_dst[ROUNDS];
#pragma unroll
  for (int i = 0; i < ROUNDS; ++i) {
    const int q = tid + 256 * i;
    k_key[i] = q / KCH;
    k_col[i] = (q % KCH) * 8;
    const int j = k_key[i];
    const int row = (j % 8 < 4) ? 4 * (j / 8) + j % 8 : 16 + 4 * (j / 8) + (j % 8 - 4);
    k_dst[i] = row * KP + k_col[i];
    v_d[i] = q / 4;                                            // 4 chunks of 8 keys per value row
    v_kc[i] = q % 4;
    v_dst[i] = v_d[i] * VP + v_kc[i] * 8;
  }

  for (int pass = 0; pass < 2; ++pass) {
    const int range = pass == 0 ? (int)blockIdx.x : n_ranges - 1 - (int)blockIdx.x;
    if (pass == 1 && range <= (int)blockIdx.x) break;          // an odd count: the middle range was done in pass 0
    bf16x8_t qf[NT][D / 32];
    int qpos[NT], tile_last[NT], tile_first[NT];
    RowRef rr[NT];
    int key_hi = -1, key_lo = 0x7fffffff;                      // over the whole block (all waves walk the same stages)
    {
      const int p_lo = range * TPB * tm.pos_per_tile;
      const int p_hi = min(nq, p_lo + TPB * tm.pos_per_tile) - 1;
      key_hi = n - nq + p_hi;
      key_lo = a.window > 0 ? max(0, n - nq + p_lo - a.window + 1) : 0;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int tile = range * TPB + wave * NT + t;
      const int p0 = tile * tm.pos_per_tile;
      rr[t] = row_ref(tm, c, p0, hb, hk, group, qs, nq, n);
      qpos[t] = rr[t].valid ? rr[t].qpos : -1;
      tile_last[t] = p0 < nq ? n - nq + min(nq, p0 + tm.pos_per_tile) - 1 : -1;
      tile_first[t] = n - nq + p0;
      const bf16_t* qp = a.q + ((int64_t)rr[t].token * a.heads + rr[t].head) * D + 8 * g;
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks) {
        if (rr[t].valid) {
          qf[t][ks] = load8(qp + ks * 32);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) qf[t][ks][i] = (__bf16)0.f;
        }
      }
    }
    f32x4_t o[NT][D / 16];
    float m[NT], l[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      m[t] = -INFINITY;
      l[t] = 0.f;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) o[t][ds] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    // Two register sets keep the loads of the next two stages in flight (a load from the cache takes longer than a
    // stage's products; with one block per compute unit nothing else hides it). No branches around the loads: a
    // stage past the end re-reads the last one.
    struct Regs { bf16x8_t k[ROUNDS], v[ROUNDS]; };
    Regs r0, r1;
    const int kb_last = (key_hi / 32) * 32;
    auto fetch = [&](int kb_want, Regs& r) {   // this thread's chunks of a stage, into registers
      const int kb = min(kb_want, kb_last);
      // a stage is two groups of 16 keys, each inside one page: two table entries, the same for every thread (scalar
      // loads, which do not queue behind the vector loads in flight)
      const int i0 = min(kb / P, max_page), i1 = min((kb + 16) / P, max_page);   // (kb <= key_hi < n: inside the row)
      // (uniform over the block: kept in scalar registers, so the 64-bit page offsets are scalar arithmetic)
      const int64_t pg0 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i0]) * page_stride;
      const int64_t pg1 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i1]) * page_stride;
      const int off0 = kb % P, off1 = (kb + 16) % P;
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        const bool hi = k_key[i] >= 16;
        r.k[i] = load8(kbase + (hi ? pg1 : pg0) + (int64_t)((hi ? off1 - 16 : off0) + k_key[i]) * D + k_col[i]);
        const bool vhi = v_kc[i] >= 2;
        r.v[i] = load8(vbase + (vhi ? pg1 : pg0) + (int64_t)v_d[i] * P + (vhi ? off1 : off0) + 8 * (v_kc[i] % 2));
      }
    };
    auto stash = [&](int buf, const Regs& r) {
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        *reinterpret_cast<bf16x8_t*>(&k_lds[buf][k_dst[i]]) = r.k[i];
        *reinterpret_cast<bf16x8_t*>(&v_lds[buf][v_dst[i]]) = r.v[i];
      }
    };
    // One stage: LDS buffer `buf` holds the keys kb .. kb+31. `next` holds stage kb+32, which goes to the other
    // buffer after the products and is then refilled with stage kb+96 (`other` holds kb+64 meanwhile).
    auto stage = [&](int kb, int buf, Regs& next) {
      bool any = false;
#pragma unroll
      for (int t = 0; t < NT; ++t) any = any || kb <= tile_last[t];
      if (any) {
        bf16x8_t kf0[D / 32], kf1[D / 32];
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          kf0[ks] = *reinterpret_cast<const bf16x8_t*>(&k_lds[buf][c * KP + ks * 32 + 8 * g]);
          kf1[ks] = *reinterpret_cast<const bf16x8_t*>(&k_lds[buf][(16 + c) * KP + ks * 32 + 8 * g]);
        }
        bf16x8_t pb[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          if (kb > tile_last[t]) continue;
          f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < D / 32; ++ks) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf0[ks], qf[t][ks], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf1[ks], qf[t][ks], s1, 0, 0, 0);
          }
          const int qp = qpos[t];
          const int first = a.window > 0 ? qp - a.window + 1 : 0;
          const bool whole = kb + 31 <= tile_first[t] && (a.window <= 0 || kb >= tile_last[t] - a.window + 1);
          pb[t] = softmax_block<D / 16>(s0, s1, whole, kb, g, qp, first, 0, 0x7fffffff, a.scale_log2, m[t], l[t], o[t]);
        }
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) {
          bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(&v_lds[buf][(ds * 16 + c) * VP + 8 * g]);
          if (kb + 31 > key_hi) zero_after(vf, kb + 8 * g, key_hi);
#pragma unroll
          for (int t = 0; t < NT; ++t) {
            if (kb > tile_last[t]) continue;
            o[t][ds] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[t], o[t][ds], 0, 0, 0);
          }
        }
      }
      stash(buf ^ 1, next);
      fetch(kb + 96, next);
      lds_barrier();
    };
    const int kb_first = (key_lo / 32) * 32;
    lds_barrier();               // the previous pass has finished reading both buffers
    fetch(kb_first, r0);
    fetch(kb_first + 32, r1);
    stash(0, r0);
    fetch(kb_first + 64, r0);
    lds_barrier();
    for (int kb = kb_first; kb <= key_hi; kb += 64) {   // even stages: buffer 0, next in r1; odd stages: buffer 1, r0
      stage(kb, 0, r1);
      if (kb + 32 <= key_hi) stage(kb + 32, 1, r0);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      float lt = l[t];
      lt += __shfl_xor(lt, 16, WAVE);
      lt += __shfl_xor(lt, 32, WAVE);
      if (!rr[t].valid) continue;
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      bf16_t* op = a.out + ((int64_t)rr[t].token * a.heads + rr[t].head) * D + 4 * g;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) {
        ushort4 w;
        w.x = float_to_bf16(o[t][ds][0] * inv);
        w.y = float_to_bf16(o[t][ds][1] * inv);
        w.z = float_to_bf16(o[t][ds][2] * inv);
        w.w = float_to_bf16(o[t][ds][3] * inv);
        *reinterpret_cast<ushort4*>(op + ds * 16) = w;
      }
    }
  }
}

// The same with tiles of 32 rows and the 32x32x16 products: a stage's keys and values, read from LDS once by a wave,
// serve twice the rows, and a wave's share of the step's barriers and page lookups halves. For long prompts.
//   S^T (32 keys x 32 queries) = K Q^T: A = 32 keys x 16 dims from LDS, B = Q^T from registers (lane l: query l%32,
//     dims 8*(l/32) .. +7 of the 16); the result has, in lane l, query l%32 and rows 8i + 4*(l/32) + r (i, r < 4).
//     Keys sit in LDS so that row 8i + 4h + r is key 16*(i/2) + 8h + 4*(i%2) + r of the stage: the scores a lane then
//     holds for i < 2 are those of keys 8h .. 8h+7 of the stage's first 16 keys, for i >= 2 of its last 16: the B
//     operands of the two value products, with no data movement.
//   O^T (32 dims x 32 queries) += V^T P^T: A = 32 dims x 16 keys from LDS (values are transposed there as in the
//     pages), B = P^T from the registers above.
typedef float f32x16_t __attribute__((ext_vector_type(16)));
#ifndef UNPAIR_BELOW
#define UNPAIR_BELOW 512
#endif

struct TileMap32 {
  int rows_per_pos;   // min(G, 32)
  int pos_per_tile;   // 32 / rows_per_pos
};
__host__ __device__ inline TileMap32 tile_map32(int group) {
  TileMap32 m;
  m.rows_per_pos = group < 32 ? group : 32;
  m.pos_per_tile = 32 / m.rows_per_pos;
  return m;
}

template <int D>
__global__ void __launch_bounds__(256, D == 128 ? 2 : 3) attn_prefill_wide_kernel(AttnArgs a) {
  constexpr int KP = D + 8;    // pitch of a key row in LDS (elements)
  constexpr int VP = 40;       // pitch of a value row: 32 keys + 8
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][32 * KP];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][D * VP];
  constexpr int PG = 4096;
  __shared__ int32_t pg_lds[PG];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, tid = threadIdx.x;
  const int h = lane / 32, c = lane % 32;
  const int b = a.row_ids[a.unpaired ? blockIdx.z / 2 : blockIdx.z];
  const int group = a.heads / a.kv_heads;      // <= 32 (the host checks)
  const TileMap32 tm = tile_map32(group);
  const int hk = blockIdx.x;          // (blocks are dealt to the XCDs in turn: a kv head's blocks share an L2)
  const int qs = a.qstart[b], nq = a.qstart[b + 1] - qs, n = a.lens[b];
  const int n_tiles = (nq + tm.pos_per_tile - 1) / tm.pos_per_tile;
  const int n_ranges = (n_tiles + 3) / 4;      // a block owns four tiles per range, one a wave
  if (n <= 0 || (int)blockIdx.y >= (n_ranges + 1) / 2) return;   // uniform over the block
  const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;
  const int P = a.page_size;
  const int64_t plane = (int64_t)P * D;
  const int64_t page_stride = 2 * (int64_t)a.kv_heads * plane;
  const bf16_t* kbase = a.pages + (int64_t)hk * plane;
  const bf16_t* vbase = a.pages + ((int64_t)a.kv_heads + hk) * plane;
  const int max_page = min(a.table_stride, PG) - 1;
  for (int i = tid; i < min(PG, a.table_stride); i += 256) pg_lds[i] = trow[i];
  constexpr int KCH = D / 8;
  constexpr int ROUNDS = D / 64;
  static_assert(D == 64 || D == 128, "the LDS kernels copy one or two chunks of each kind per thread");
  // What a thread copies per stage: ROUNDS 16-byte pieces of keys and of values. With D = 128 a round is one half
  // of the stage (keys 0-15, then 16-31), so that every lane of a round reads the same page and an address is a
  // scalar base plus a lane offset that never changes; with D = 64 the one round covers both halves.
  constexpr bool HALVES = ROUNDS == 2;
  int k_half[ROUNDS], k_off[ROUNDS], k_dst[ROUNDS], v_half[ROUNDS], v_off[ROUNDS], v_dst[ROUNDS];
#pragma unroll
  for (int i = 0; i < ROUNDS; ++i) {
    const int q = tid + 256 * i;
    const int j = q / KCH, col = (q % KCH) * 8;                // key j of the stage goes to row 8i' + 4h' + r
    const int row = 8 * (2 * (j / 16) + (j % 8) / 4) + 4 * ((j % 16) / 8) + j % 4;
    k_half[i] = j / 16;
    k_off[i] = (j % 16) * D + col;
    k_dst[i] = row * KP + col;
    const int vd = HALVES ? tid / 2 : tid / 4, vkc = HALVES ? 2 * i + tid % 2 : tid % 4;   // dim, chunk of 8 keys
    v_half[i] = vkc / 2;
    v_off[i] = vd * P + 8 * (vkc % 2);
    v_dst[i] = vd * VP + vkc * 8;
  }
  // the row of this lane's column: position c / rows_per_pos of the tile, head c % rows_per_pos of the group
  const int pi = c / tm.rows_per_pos, hi = c % tm.rows_per_pos;

  // Paired, a block runs range x and then its mirror image, which together see the same number of keys in every block.
  // Unpaired, the two are blocks of their own, the long one first in launch order: twice the blocks for short prompts.
  const int pass_lo = a.unpaired ? 1 - (int)(blockIdx.z % 2) : 0, pass_hi = a.unpaired ? pass_lo + 1 : 2;
  for (int pass = pass_lo; pass < pass_hi; ++pass) {
    const int range = pass == 0 ? (int)blockIdx.y : n_ranges - 1 - (int)blockIdx.y;
    if (pass == 1 && range <= (int)blockIdx.y) break;
    const int p_lo = range * 4 * tm.pos_per_tile;
    const int p_hi = min(nq, p_lo + 4 * tm.pos_per_tile) - 1;
    const int key_hi = n - nq + p_hi;                          // over the whole block (all waves walk the same stages)
    const int key_lo = a.window > 0 ? max(0, n - nq + p_lo - a.window + 1) : 0;
    const int p0 = (range * 4 + wave) * tm.pos_per_tile;       // this wave's tile
    const int qi = p0 + pi;
    const bool valid = pi < tm.pos_per_tile && qi < nq && hi < group;
    const int token = qs + qi, head = hk * group + hi;
    const int qpos = valid ? n - nq + qi : -1;
    const int tile_last = p0 < nq ? n - nq + min(nq, p0 + tm.pos_per_tile) - 1 : -1;
    const int tile_first = n - nq + p0;
    bf16x8_t qf[D / 16];
    {
      const bf16_t* qp = a.q + ((int64_t)token * a.heads + head) * D + 8 * h;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) {
        if (valid) {
          qf[ds] = load8(qp + ds * 16);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) qf[ds][i] = (__bf16)0.f;
        }
      }
    }
    f32x16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    struct Regs { bf16x8_t k[ROUNDS], v[ROUNDS]; };
    Regs r0, r1;
    const int kb_last = (key_hi / 32) * 32;
    auto fetch = [&](int kb_want, Regs& r) {
      const int kb = min(kb_want, kb_last);
      const int i0 = min(kb / P, max_page), i1 = min((kb + 16) / P, max_page);
      const int64_t pg0 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i0]) * page_stride;
      const int64_t pg1 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i1]) * page_stride;
      const int off0 = kb % P, off1 = (kb + 16) % P;
      const bf16_t* kh[2] = {kbase + pg0 + (int64_t)off0 * D, kbase + pg1 + (int64_t)off1 * D};   // the halves' first keys
      const bf16_t* vh[2] = {vbase + pg0 + off0, vbase + pg1 + off1};
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        if constexpr (HALVES) {
          r.k[i] = load8(kh[i] + (uint32_t)k_off[i]);
          r.v[i] = load8(vh[i] + (uint32_t)v_off[i]);
        } else {
          r.k[i] = load8((k_half[i] ? kh[1] : kh[0]) + (uint32_t)k_off[i]);
          r.v[i] = load8((v_half[i] ? vh[1] : vh[0]) + (uint32_t)v_off[i]);
        }
      }
    };
    auto stash = [&](int buf, const Regs& r) {
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        *reinterpret_cast<bf16x8_t*>(&k_lds[buf][k_dst[i]]) = r.k[i];
        *reinterpret_cast<bf16x8_t*>(&v_lds[buf][v_dst[i]]) = r.v[i];
      }
    };
    // `last`: the stage holds the row's last key (std::true_type) and may reach past it; nothing is staged behind it.
    auto stage = [&](auto last, int kb, int buf, Regs& next) {
      if (kb <= tile_last) {
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
        bf16x8_t kf[D / 16];                       // all of a stage's key fragments are asked for at once
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds)
          kf[ds] = *reinterpret_cast<const bf16x8_t*>(&k_lds[buf][c * KP + ds * 16 + 8 * h]);
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds], qf[ds], sc, 0, 0, 0);
        bf16x8_t vf[D / 32][2];                    // and its value fragments before the softmax that they wait for
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          vf[db][0] = *reinterpret_cast<const bf16x8_t*>(&v_lds[buf][(db * 32 + c) * VP + 8 * h]);
          vf[db][1] = *reinterpret_cast<const bf16x8_t*>(&v_lds[buf][(db * 32 + c) * VP + 16 + 8 * h]);
          if constexpr (decltype(last)::value) {
            zero_after(vf[db][0], kb + 8 * h, key_hi);
            zero_after(vf[db][1], kb + 16 + 8 * h, key_hi);
          }
        }
        // value idx = 4i + r of this lane is key kb + 16*(i/2) + 8h + 4*(i%2) + r against query column c
        const int first = a.window > 0 ? qpos - a.window + 1 : 0;
        const bool whole = kb + 31 <= tile_first && (a.window <= 0 || kb >= tile_last - a.window + 1);
        float sv[16];
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) sv[idx] = sc[idx];
        if (!whole) {
#pragma unroll
          for (int idx = 0; idx < 16; ++idx) {
            const int i = idx / 4, r = idx % 4;
            const int key = kb + 16 * (i / 2) + 8 * h + 4 * (i % 2) + r;
            if (!(key <= qpos && key >= first)) sv[idx] = -INFINITY;
          }
        }
        float mx = sv[0];
#pragma unroll
        for (int idx = 1; idx < 16; ++idx) mx = fmaxf(mx, sv[idx]);
        {                                          // the other half of the keys is in lane l ^ 32
          const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
          mx = fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
        }
        const float m_new = fmaxf(m, mx * a.scale_log2);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        bf16x8_t pb0, pb1;
        float psum = 0.f;
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) {
          const float p = __builtin_amdgcn_exp2f(fmaf(sv[idx], a.scale_log2, -m_use));
          psum += p;
          if (idx < 8) pb0[idx] = (__bf16)p; else pb1[idx - 8] = (__bf16)p;
        }
        if (__any(m_new != m)) {
          const float alpha = __builtin_amdgcn_exp2f(m - m_use);
          l *= alpha;
#pragma unroll
          for (int db = 0; db < D / 32; ++db) o[db] *= alpha;
          m = m_new;
        }
        l += psum;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][0], pb0, o[db], 0, 0, 0);
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][1], pb1, o[db], 0, 0, 0);
        }
      }
      if constexpr (!decltype(last)::value) {
        stash(buf ^ 1, next);
        fetch(kb + 96, next);
        lds_barrier();
      }
    };
    const int kb_first = (key_lo / 32) * 32;
    lds_barrier();               // the previous pass has finished reading both buffers
    fetch(kb_first, r0);
    fetch(kb_first + 32, r1);
    stash(0, r0);
    fetch(kb_first + 64, r0);
    lds_barrier();
    int kb = kb_first;
    for (; kb + 32 < kb_last; kb += 64) {        // pairs of stages that both lie before the last one
      stage(std::false_type{}, kb, 0, r1);
      stage(std::false_type{}, kb + 32, 1, r0);
    }
    if (kb < kb_last) {
      stage(std::false_type{}, kb, 0, r1);
      stage(std::true_type{}, kb + 32, 1, r0);
    } else {
      stage(std::true_type{}, kb, 0, r1);
    }
    float lt = l + __shfl_xor(l, 32, WAVE);
    if (valid) {
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      bf16_t* op = a.out + ((int64_t)token * a.heads + head) * D + 4 * h;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ushort4 w;
          w.x = float_to_bf16(o[db][4 * i + 0] * inv);
          w.y = float_to_bf16(o[db][4 * i + 1] * inv);
          w.z = float_to_bf16(o[db][4 * i + 2] * inv);
          w.w = float_to_bf16(o[db][4 * i + 3] * inv);
          *reinterpret_cast<ushort4*>(op + db * 32 + 8 * i) = w;
        }
    }
  }
}

#ifndef PAIR_VALU_PER_MFMA
#define PAIR_VALU_PER_MFMA 16   // vector instructions the scheduler is asked to put between two matrix products
#endif
// The same with two tiles of 32 rows a wave (a block: 256 rows, 64 positions of a group of four heads). A stage's
// keys and values are read from the cache into LDS once for twice the rows (the staged kernels are bound by what the
// blocks of a launch read through L2: every block reads every key before its rows), a wave reads them from LDS once
// for both tiles, and the two tiles are independent work in one instruction stream: one tile's exponentials are issued
// between the other tile's matrix products. Stages that both tiles see whole run without masks (`MASK` false); the
// stages at the diagonal, with a window, and the last one run the masked form.
template <bool MASK>
__device__ __forceinline__ void scores_to_probs(const f32x16_t& sc, int kb, int h, int qpos, int first,
                                                float scale_log2, float m, float& m_new, float& psum, bf16x8_t& pb0,
                                                bf16x8_t& pb1) {
  float sv[16];
#pragma unroll
  for (int idx = 0; idx < 16; ++idx) sv[idx] = sc[idx];
  if constexpr (MASK) {
#pragma unroll
    for (int idx = 0; idx < 16; ++idx) {
      const int i = idx / 4, r = idx % 4;
      const int key = kb + 16 * (i / 2) + 8 * h + 4 * (i % 2) + r;
      if (!(key <= qpos && key >= first)) sv[idx] = -INFINITY;
    }
  }
  float mx = fmaxf(fmaxf(sv[0], sv[1]), sv[2]);
#pragma unroll
  for (int idx = 3; idx + 1 < 16; idx += 2) mx = fmaxf(fmaxf(mx, sv[idx]), sv[idx + 1]);
  mx = fmaxf(mx, sv[15]);
  {                                          // the other half of the keys is in lane l ^ 32
    const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
    mx = fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
  }
  m_new = fmaxf(m, mx * scale_log2);
  const float m_use = m_new == -INFINITY ? 0.f : m_new;
  psum = 0.f;
#pragma unroll
  for (int idx = 0; idx < 16; ++idx) {
    const float p = __builtin_amdgcn_exp2f(fmaf(sv[idx], scale_log2, -m_use));
    psum += p;
    if (idx < 8) pb0[idx] = (__bf16)p; else pb1[idx - 8] = (__bf16)p;
  }
}

// The same for head_dim 128 with a stage's keys and values copied from the cache into LDS by the memory pipeline
// itself (global_load_lds: 16 bytes a lane, a wave's 64 lanes into one contiguous kilobyte of LDS), two stages ahead
// of the one being multiplied, into three buffers in turn: no registers hold a stage on its way, and no instruction
// writes LDS. A wave's kilobyte has to be contiguous, so rows cannot be padded apart; instead each 16-byte piece
// sits at place `piece ^ (row % 16)` of its key's 256-byte row (values: each half of the stage's keys apart, a dim's 16
// keys a row of 32 bytes, place `piece ^ (row / 8 % 2)`), which a lane's source address arranges and a lane's read
// undoes: 16 lanes that read the same piece of 16 consecutive rows then touch every bank once, as with padded rows.
// Every copy instruction reads one page, so its lanes share a scalar base and their own offsets never change.
// The compiler does not know these loads (it would wait for all of them before every read of LDS): they are issued
// from inline assembly, and the one wait per stage that they need (all but the newest stage's four loads a lane) is
// written by hand in front of the stage's barrier. Nothing else loads from memory inside the loop.
// A block's staging of 32-key stages at head_dim 128 through three LDS buffers: what each lane copies, where it reads.
struct StagedCopies {
  static constexpr int D = 128;
  static constexpr int K_BYTES = 32 * D * 2, V_BYTES = D * 32 * 2, STAGE_BYTES = K_BYTES + V_BYTES;   // 8 KB + 8 KB
  static constexpr int BUFFERS = 3, PG = 4096;
  const unsigned char* lds;      // BUFFERS * STAGE_BYTES, aligned to 1,024
  const int32_t* pg;             // the row's block table, in LDS
  const bf16_t* kbase;
  const bf16_t* vbase;
  int64_t page_stride;
  int P, max_page, second, wave;
  uint32_t lds0, k_src[2], v_src[2], k_at[D / 16], v_at[2];

  // What this lane copies per stage: two pieces of keys and two of values (instruction q = 2 * wave + i of eight;
  // waves 0 and 1 copy the stage's first 16 keys, which lie in one page, waves 2 and 3 its last 16).
  // Keys: kilobyte q holds rows 4 q .. 4 q + 3; row 8 i' + 4 h' + r holds key 16 (i' / 2) + 8 h' + 4 (i' % 2) + r of
  // the stage (the order the score product's result wants), so rows 0-15 are the first half. Values: kilobyte q holds
  // dims 32 (q % 4) .. + 31 of half q / 4, two pieces a dim: keys 0-7 and 8-15 of the half.
  // Where it reads: keys, row c, piece 2 ds + h; values, half t, row 32 db + c, piece h (lane = 32 h + c).
  __device__ __forceinline__ void init(const unsigned char* stage_lds, const int32_t* pg_lds, const AttnArgs& a, int hk) {
    lds = stage_lds;
    pg = pg_lds;
    P = a.page_size;
    const int64_t plane = (int64_t)P * D;
    page_stride = 2 * (int64_t)a.kv_heads * plane;
    kbase = a.pages + (int64_t)hk * plane;
    vbase = a.pages + ((int64_t)a.kv_heads + hk) * plane;
    max_page = min(a.table_stride, PG) - 1;
    const int lane = threadIdx.x % WAVE, h = lane / 32, c = lane % 32;
    wave = threadIdx.x / WAVE;
    second = __builtin_amdgcn_readfirstlane(wave / 2);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = 2 * wave + i;
      const int row = 4 * q + lane / 16, piece = (lane % 16) ^ (row % 16);
      const int key = 16 * ((row / 8) / 2) + 8 * ((row % 8) / 4) + 4 * ((row / 8) % 2) + row % 4;
      k_src[i] = (uint32_t)(((key % 16) * D + piece * 8) * 2);
      const int dim = 32 * (q % 4) + lane / 2, vpiece = (lane % 2) ^ ((dim / 8) % 2);
      v_src[i] = (uint32_t)((dim * P + 8 * vpiece) * 2);
    }
    lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)stage_lds;
#pragma unroll
    for (int ds = 0; ds < D / 16; ++ds) k_at[ds] = (uint32_t)(c * (D * 2) + 16 * ((2 * ds + h) ^ (c % 16)));
#pragma unroll
    for (int t = 0; t < 2; ++t) v_at[t] = (uint32_t)(K_BYTES + t * (V_BYTES / 2) + c * 32 + 16 * (h ^ ((c / 8) % 2)));
  }
  // four loads a lane: the stage at kb (a stage past kb_last copies the last one again) into buffer `buf`
  __device__ __forceinline__ void copy(int kb_want, int kb_last, int buf) const {
    const int kb = min(kb_want, kb_last) + 16 * second;         // this wave's half of the stage: 16 keys of one page
    const int64_t at = (int64_t)__builtin_amdgcn_readfirstlane(pg[min(kb / P, max_page)]) * page_stride;
    const int off = kb % P;
    const bf16_t* kh = kbase + at + (int64_t)off * D;
    const bf16_t* vh = vbase + at + off;
    const uint32_t to = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)buf * STAGE_BYTES + (uint32_t)wave * 2048);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      load_to_lds16(kh, k_src[i], to + 1024 * i);
      load_to_lds16(vh, v_src[i], to + K_BYTES + 1024 * i);
    }
  }
  static constexpr int LOADS = 4;                               // of a lane, per stage
  __device__ __forceinline__ bf16x8_t key(int buf, int ds) const {
    return *reinterpret_cast<const bf16x8_t*>(lds + buf * STAGE_BYTES + k_at[ds]);
  }
  __device__ __forceinline__ bf16x8_t value(int buf, int db, int t) const {
    return *reinterpret_cast<const bf16x8_t*>(lds + buf * STAGE_BYTES + v_at[t] + db * 1024);
  }
  static __device__ __forceinline__ int after(int buf) { return buf == BUFFERS - 1 ? 0 : buf + 1; }
  static __device__ __forceinline__ int before(int buf) { return buf == 0 ? BUFFERS - 1 : buf - 1; }
};

__global__ void __launch_bounds__(256, 2) attn_prefill_dma_kernel(AttnArgs a) {
  using SC = StagedCopies;
  constexpr int D = SC::D;
  __shared__ __attribute__((aligned(1024))) unsigned char stage_lds[SC::BUFFERS * SC::STAGE_BYTES];
  __shared__ int32_t pg_lds[SC::PG];
  static_assert(sizeof(stage_lds) + sizeof(pg_lds) <= 64 * 1024, "a block's static LDS; two blocks share a compute unit");
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, tid = threadIdx.x;
  const int h = lane / 32, c = lane % 32;
  const int b = a.row_ids[a.unpaired ? blockIdx.z / 2 : blockIdx.z];
  const int group = a.heads / a.kv_heads;      // <= 32 (the host checks)
  const TileMap32 tm = tile_map32(group);
  const int hk = blockIdx.x;          // (blocks are dealt to the XCDs in turn: a kv head's blocks share an L2)
  const int qs = a.qstart[b], nq = a.qstart[b + 1] - qs, n = a.lens[b];
  const int n_tiles = (nq + tm.pos_per_tile - 1) / tm.pos_per_tile;
  const int n_ranges = (n_tiles + 3) / 4;      // a block owns four tiles per range, one a wave
  if (n <= 0 || (int)blockIdx.y >= (n_ranges + 1) / 2) return;   // uniform over the block
  const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;
  for (int i = tid; i < min(SC::PG, a.table_stride); i += 256) pg_lds[i] = trow[i];
  SC sc_;
  sc_.init(stage_lds, pg_lds, a, hk);
  const int pi = c / tm.rows_per_pos, hi = c % tm.rows_per_pos;

  const int pass_lo = a.unpaired ? 1 - (int)(blockIdx.z % 2) : 0, pass_hi = a.unpaired ? pass_lo + 1 : 2;
  for (int pass = pass_lo; pass < pass_hi; ++pass) {
    const int range = pass == 0 ? (int)blockIdx.y : n_ranges - 1 - (int)blockIdx.y;
    if (pass == 1 && range <= (int)blockIdx.y) break;
    const int p_lo = range * 4 * tm.pos_per_tile;
    const int p_hi = min(nq, p_lo + 4 * tm.pos_per_tile) - 1;
    const int key_hi = n - nq + p_hi;                          // over the whole block (all waves walk the same stages)
    const int key_lo = a.window > 0 ? max(0, n - nq + p_lo - a.window + 1) : 0;
    const int p0 = (range * 4 + wave) * tm.pos_per_tile;       // this wave's tile
    const int qi = p0 + pi;
    const bool valid = pi < tm.pos_per_tile && qi < nq && hi < group;
    const int token = qs + qi, head = hk * group + hi;
    const int qpos = valid ? n - nq + qi : -1;
    const int tile_last = p0 < nq ? n - nq + min(nq, p0 + tm.pos_per_tile) - 1 : -1;
    const int tile_first = n - nq + p0;
    bf16x8_t qf[D / 16];
    {
      const bf16_t* qp = a.q + ((int64_t)token * a.heads + head) * D + 8 * h;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) {
        if (valid) {
          qf[ds] = load8(qp + ds * 16);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) qf[ds][i] = (__bf16)0.f;
        }
      }
    }
    f32x16_t o[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int kb_last = (key_hi / 32) * 32;
    // `last`: the stage holds the row's last key (std::true_type) and may reach past it
    auto stage = [&](auto last, int kb, int buf) {
      if (kb <= tile_last) {
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
        bf16x8_t kf[D / 16];                       // all of a stage's key fragments are asked for at once
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) kf[ds] = sc_.key(buf, ds);
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds], qf[ds], sc, 0, 0, 0);
        bf16x8_t vf[D / 32][2];                    // and its value fragments before the softmax that they wait for
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          vf[db][0] = sc_.value(buf, db, 0);
          vf[db][1] = sc_.value(buf, db, 1);
          if constexpr (decltype(last)::value) {
            zero_after(vf[db][0], kb + 8 * h, key_hi);
            zero_after(vf[db][1], kb + 16 + 8 * h, key_hi);
          }
        }
        // value idx = 4i + r of this lane is key kb + 16*(i/2) + 8h + 4*(i%2) + r against query column c
        const int first = a.window > 0 ? qpos - a.window + 1 : 0;
        const bool whole = kb + 31 <= tile_first && (a.window <= 0 || kb >= tile_last - a.window + 1);
        float sv[16];
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) sv[idx] = sc[idx];
        if (!whole) {
#pragma unroll
          for (int idx = 0; idx < 16; ++idx) {
            const int i = idx / 4, r = idx % 4;
            const int key = kb + 16 * (i / 2) + 8 * h + 4 * (i % 2) + r;
            if (!(key <= qpos && key >= first)) sv[idx] = -INFINITY;
          }
        }
        float mx = sv[0];
#pragma unroll
        for (int idx = 1; idx < 16; ++idx) mx = fmaxf(mx, sv[idx]);
        {                                          // the other half of the keys is in lane l ^ 32
          const auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
          mx = fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
        }
        const float m_new = fmaxf(m, mx * a.scale_log2);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        bf16x8_t pb0, pb1;
        float psum = 0.f;
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) {
          const float p = __builtin_amdgcn_exp2f(fmaf(sv[idx], a.scale_log2, -m_use));
          psum += p;
          if (idx < 8) pb0[idx] = (__bf16)p; else pb1[idx - 8] = (__bf16)p;
        }
        if (__any(m_new != m)) {
          const float alpha = __builtin_amdgcn_exp2f(m - m_use);
          l *= alpha;
#pragma unroll
          for (int db = 0; db < D / 32; ++db) o[db] *= alpha;
          m = m_new;
        }
        l += psum;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][0], pb0, o[db], 0, 0, 0);
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][1], pb1, o[db], 0, 0, 0);
        }
      }
    };
    const int kb_first = (key_lo / 32) * 32;
    wait_loads_but<0>();         // (a stage past the end of the pass before may still be on its way into a buffer)
    lds_barrier();               // the previous pass has finished reading the buffers; the table is in LDS
    sc_.copy(kb_first, kb_last, 0);
    sc_.copy(kb_first + 32, kb_last, 1);
    wait_loads_but<SC::LOADS>();
    lds_barrier();
    int buf = 0;
    for (int kb = kb_first; kb < kb_last; kb += 32) {          // every stage before the last one
      sc_.copy(kb + 64, kb_last, SC::before(buf));             // two stages on, into the buffer read a stage ago
      stage(std::false_type{}, kb, buf);
      wait_loads_but<SC::LOADS>();                             // the next stage has landed (this wave's share of it)
      lds_barrier();
      buf = SC::after(buf);
    }
    stage(std::true_type{}, kb_last, buf);
    float lt = l + __shfl_xor(l, 32, WAVE);
    if (valid) {
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      bf16_t* op = a.out + ((int64_t)token * a.heads + head) * D + 4 * h;
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          ushort4 w;
          w.x = float_to_bf16(o[db][4 * i + 0] * inv);
          w.y = float_to_bf16(o[db][4 * i + 1] * inv);
          w.z = float_to_bf16(o[db][4 * i + 2] * inv);
          w.w = float_to_bf16(o[db][4 * i + 3] * inv);
          *reinterpret_cast<ushort4*>(op + db * 32 + 8 * i) = w;
        }
    }
  }
  wait_loads_but<0>();           // nothing of this wave is on its way into LDS when the block ends
}

template <int D>
__global__ void __launch_bounds__(256, 1) attn_prefill_pair_kernel(AttnArgs a) {
  constexpr int KP = D + 8;    // pitch of a key row in LDS (elements)
  constexpr int VP = 40;       // pitch of a value row: 32 keys + 8
  __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][32 * KP];
  __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][D * VP];
  constexpr int PG = 4096;
  __shared__ int32_t pg_lds[PG];
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, tid = threadIdx.x;
  const int h = lane / 32, c = lane % 32;
  const int b = a.row_ids[a.unpaired ? blockIdx.z / 2 : blockIdx.z];
  const int group = a.heads / a.kv_heads;      // <= 32 (the host checks)
  const TileMap32 tm = tile_map32(group);
  const int hk = blockIdx.x;          // (blocks are dealt to the XCDs in turn: a kv head's blocks share an L2)
  const int qs = a.qstart[b], nq = a.qstart[b + 1] - qs, n = a.lens[b];
  const int n_tiles = (nq + tm.pos_per_tile - 1) / tm.pos_per_tile;
  constexpr int TPB = 8;                       // tiles a block owns per range: two a wave, side by side
  const int n_ranges = (n_tiles + TPB - 1) / TPB;
  if (n <= 0 || (int)blockIdx.y >= (n_ranges + 1) / 2) return;   // uniform over the block
  const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;
  const int P = a.page_size;
  const int64_t plane = (int64_t)P * D;
  const int64_t page_stride = 2 * (int64_t)a.kv_heads * plane;
  const bf16_t* kbase = a.pages + (int64_t)hk * plane;
  const bf16_t* vbase = a.pages + ((int64_t)a.kv_heads + hk) * plane;
  const int max_page = min(a.table_stride, PG) - 1;
  for (int i = tid; i < min(PG, a.table_stride); i += 256) pg_lds[i] = trow[i];
  constexpr int KCH = D / 8;
  constexpr int ROUNDS = D / 64;
  static_assert(D == 64 || D == 128, "the LDS kernels copy one or two chunks of each kind per thread");
  constexpr bool HALVES = ROUNDS == 2;         // (what a thread copies per stage: as in attn_prefill_wide_kernel)
  int k_half[ROUNDS], k_off[ROUNDS], k_dst[ROUNDS], v_half[ROUNDS], v_off[ROUNDS], v_dst[ROUNDS];
#pragma unroll
  for (int i = 0; i < ROUNDS; ++i) {
    const int q = tid + 256 * i;
    const int j = q / KCH, col = (q % KCH) * 8;
    const int row = 8 * (2 * (j / 16) + (j % 8) / 4) + 4 * ((j % 16) / 8) + j % 4;
    k_half[i] = j / 16;
    k_off[i] = (j % 16) * D + col;
    k_dst[i] = row * KP + col;
    const int vd = HALVES ? tid / 2 : tid / 4, vkc = HALVES ? 2 * i + tid % 2 : tid % 4;
    v_half[i] = vkc / 2;
    v_off[i] = vd * P + 8 * (vkc % 2);
    v_dst[i] = vd * VP + vkc * 8;
  }
  const int pi = c / tm.rows_per_pos, hi = c % tm.rows_per_pos;

  const int pass_lo = a.unpaired ? 1 - (int)(blockIdx.z % 2) : 0, pass_hi = a.unpaired ? pass_lo + 1 : 2;
  for (int pass = pass_lo; pass < pass_hi; ++pass) {
    const int range = pass == 0 ? (int)blockIdx.y : n_ranges - 1 - (int)blockIdx.y;
    if (pass == 1 && range <= (int)blockIdx.y) break;
    const int p_lo = range * TPB * tm.pos_per_tile;
    const int p_hi = min(nq, p_lo + TPB * tm.pos_per_tile) - 1;
    const int key_hi = n - nq + p_hi;                          // over the whole block (all waves walk the same stages)
    const int key_lo = a.window > 0 ? max(0, n - nq + p_lo - a.window + 1) : 0;
    bool valid[2];
    int token[2], qpos[2], tile_last[2], tile_first[2];
    const int head = hk * group + hi;
    bf16x8_t qf[2][D / 16];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int p0 = (range * TPB + wave * 2 + t) * tm.pos_per_tile;
      const int qi = p0 + pi;
      valid[t] = pi < tm.pos_per_tile && qi < nq && hi < group;
      token[t] = qs + qi;
      qpos[t] = valid[t] ? n - nq + qi : -1;
      tile_last[t] = p0 < nq ? n - nq + min(nq, p0 + tm.pos_per_tile) - 1 : -1;
      tile_first[t] = n - nq + p0;
      const bf16_t* qp = a.q + ((int64_t)token[t] * a.heads + head) * D + 8 * h;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) {
        if (valid[t]) {
          qf[t][ds] = load8(qp + ds * 16);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) qf[t][ds][i] = (__bf16)0.f;
        }
      }
    }
    f32x16_t o[2][D / 32];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[t][db][i] = 0.f;
    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};

    struct Regs { bf16x8_t k[ROUNDS], v[ROUNDS]; };
    Regs r0, r1;
    const int kb_last = (key_hi / 32) * 32;
    auto fetch = [&](int kb_want, Regs& r) {
      const int kb = min(kb_want, kb_last);
      const int i0 = min(kb / P, max_page), i1 = min((kb + 16) / P, max_page);
      const int64_t pg0 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i0]) * page_stride;
      const int64_t pg1 = (int64_t)__builtin_amdgcn_readfirstlane(pg_lds[i1]) * page_stride;
      const int off0 = kb % P, off1 = (kb + 16) % P;
      const bf16_t* kh[2] = {kbase + pg0 + (int64_t)off0 * D, kbase + pg1 + (int64_t)off1 * D};
      const bf16_t* vh[2] = {vbase + pg0 + off0, vbase + pg1 + off1};
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        if constexpr (HALVES) {
          r.k[i] = load8(kh[i] + (uint32_t)k_off[i]);
          r.v[i] = load8(vh[i] + (uint32_t)v_off[i]);
        } else {
          r.k[i] = load8((k_half[i] ? kh[1] : kh[0]) + (uint32_t)k_off[i]);
          r.v[i] = load8((v_half[i] ? vh[1] : vh[0]) + (uint32_t)v_off[i]);
        }
      }
    };
    auto stash = [&](int buf, const Regs& r) {
#pragma unroll
      for (int i = 0; i < ROUNDS; ++i) {
        *reinterpret_cast<bf16x8_t*>(&k_lds[buf][k_dst[i]]) = r.k[i];
        *reinterpret_cast<bf16x8_t*>(&v_lds[buf][v_dst[i]]) = r.v[i];
      }
    };
    // what follows a tile's probabilities: the rescale of its sums when some row's max moved, then its sum
    auto settle = [&](int t, float m_new, float psum) {
      if (__any(m_new != m[t])) {
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m[t] - m_use);
        l[t] *= alpha;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) o[t][db] *= alpha;
        m[t] = m_new;
      }
      l[t] += psum;
    };
    // One stage. `masked`: some row of the wave's tiles does not see the whole stage (the diagonal, a window);
    // `last`: the stage holds the row's last key and may reach past it; nothing is staged behind it.
    auto stage = [&](auto masked, auto last, int kb, int buf, Regs& next) {
      constexpr bool MASK = decltype(masked)::value, LAST = decltype(last)::value;
      const bool on0 = !MASK || kb <= tile_last[0], on1 = !MASK || kb <= tile_last[1];   // (uniform over the wave)
      if (on0 || on1) {
        bf16x8_t kf[D / 16];
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds)
          kf[ds] = *reinterpret_cast<const bf16x8_t*>(&k_lds[buf][c * KP + ds * 16 + 8 * h]);
        f32x16_t sc0, sc1;
#pragma unroll
        for (int i = 0; i < 16; ++i) { sc0[i] = 0.f; sc1[i] = 0.f; }
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) sc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds], qf[0][ds], sc0, 0, 0, 0);
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds) sc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds], qf[1][ds], sc1, 0, 0, 0);
        bf16x8_t vf[D / 32][2];
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          vf[db][0] = *reinterpret_cast<const bf16x8_t*>(&v_lds[buf][(db * 32 + c) * VP + 8 * h]);
          vf[db][1] = *reinterpret_cast<const bf16x8_t*>(&v_lds[buf][(db * 32 + c) * VP + 16 + 8 * h]);
          if constexpr (LAST) {
            zero_after(vf[db][0], kb + 8 * h, key_hi);
            zero_after(vf[db][1], kb + 16 + 8 * h, key_hi);
          }
        }
        float m_new, psum;
        bf16x8_t pb0, pb1;
        if (on0) {
          scores_to_probs<MASK>(sc0, kb, h, qpos[0], a.window > 0 ? qpos[0] - a.window + 1 : 0, a.scale_log2, m[0],
                                m_new, psum, pb0, pb1);
          if constexpr (!MASK) {     // the second tile's score products, one at a time between the first tile's exponentials
            __builtin_amdgcn_sched_group_barrier(0x008, D / 16, 0);
#pragma unroll
            for (int i = 0; i < D / 16; ++i) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
              __builtin_amdgcn_sched_group_barrier(0x002, PAIR_VALU_PER_MFMA, 0);
            }
          }
          settle(0, m_new, psum);
#pragma unroll
          for (int db = 0; db < D / 32; ++db) {
            o[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][0], pb0, o[0][db], 0, 0, 0);
            o[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][1], pb1, o[0][db], 0, 0, 0);
          }
        }
        if (on1) {
          scores_to_probs<MASK>(sc1, kb, h, qpos[1], a.window > 0 ? qpos[1] - a.window + 1 : 0, a.scale_log2, m[1],
                                m_new, psum, pb0, pb1);
          if constexpr (!MASK) {     // the first tile's value products between the second tile's exponentials
#pragma unroll
            for (int i = 0; i < D / 16; ++i) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
              __builtin_amdgcn_sched_group_barrier(0x002, PAIR_VALU_PER_MFMA, 0);
            }
          }
          settle(1, m_new, psum);
#pragma unroll
          for (int db = 0; db < D / 32; ++db) {
            o[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][0], pb0, o[1][db], 0, 0, 0);
            o[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][1], pb1, o[1][db], 0, 0, 0);
          }
        }
      }
      if constexpr (!LAST) {
        stash(buf ^ 1, next);
        fetch(kb + 96, next);
        lds_barrier();
      }
    };
    // a stage is unmasked when every row of both tiles sees all of it: it ends at or before the first tile's first
    // position, and there is no window
    auto step = [&](auto last, int kb, int buf, Regs& next) {
      if (a.window <= 0 && kb + 31 <= tile_first[0]) stage(std::false_type{}, last, kb, buf, next);
      else stage(std::true_type{}, last, kb, buf, next);
    };
    const int kb_first = (key_lo / 32) * 32;
    lds_barrier();               // the previous pass has finished reading both buffers
    fetch(kb_first, r0);
    fetch(kb_first + 32, r1);
    stash(0, r0);
    fetch(kb_first + 64, r0);
    lds_barrier();
    int kb = kb_first;
    for (; kb + 32 < kb_last; kb += 64) {        // pairs of stages that both lie before the last one
      step(std::false_type{}, kb, 0, r1);
      step(std::false_type{}, kb + 32, 1, r0);
    }
    if (kb < kb_last) {
      step(std::false_type{}, kb, 0, r1);
      stage(std::true_type{}, std::true_type{}, kb + 32, 1, r0);
    } else {
      stage(std::true_type{}, std::true_type{}, kb, 0, r1);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const float lt = l[t] + __shfl_xor(l[t], 32, WAVE);
      if (valid[t]) {
        const float inv = lt > 0.f ? 1.0f / lt : 0.f;
        bf16_t* op = a.out + ((int64_t)token[t] * a.heads + head) * D + 4 * h;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            ushort4 w;
            w.x = float_to_bf16(o[t][db][4 * i + 0] * inv);
            w.y = float_to_bf16(o[t][db][4 * i + 1] * inv);
            w.z = float_to_bf16(o[t][db][4 * i + 2] * inv);
            w.w = float_to_bf16(o[t][db][4 * i + 3] * inv);
            *reinterpret_cast<ushort4*>(op + db * 32 + 8 * i) = w;
          }
      }
    }
  }
}

// What the decode kernel needs to take the step's raw q/k/v projection itself (`qkv` [T, (Hq + 2 Hkv) D]) instead of
// queries that another kernel has normed and rotated and keys that it has stored: per-head RMSNorm weights (both or
// neither), the rotation table (cos | sin of every position, over the whole head, or none), where each token's key
// and value go in the cache.
struct FusedArgs {
  const bf16_t* qkv;
  int64_t qkv_stride;
  const bf16_t* q_weight;
  const bf16_t* k_weight;
  float eps;
  const float* table;          // [max_positions, D]; a decode row's token sits at position len - 1
  int max_positions;           // (a longer row, which the engine never makes, would read the table's last row)
  bf16_t* pages;               // the cache, written for the row's new token
  const int32_t* write_page;   // [T]
  const int32_t* write_off;    // [T]
};

// The row's new key and value from the raw projection: RMSNorm over the head and rotation for the key, the value as
// it is. One wave: lanes 0 .. D/8 - 1 hold eight dims each of the key, the next D/8 lanes of the value. `make` leaves
// both in LDS (`fresh`: the key's D values, then the value's) and in the lanes' registers; `store` sends them to the
// cache (the value transposed inside its page). The roundings are those of the norm + rotation + write kernel
// (elementwise.hip).
template <int D>
struct NewKeyValue {
  static constexpr int LPH = D / 8;
  uint4 mine;       // role 0: the key's eight values as stored; role 1: the value's
  int li, role;

  __device__ __forceinline__ void make(const AttnArgs& a, const FusedArgs& f, int token, int pos, int hk, bf16_t* fresh) {
    const int lane = threadIdx.x % WAVE;
    li = lane % LPH;
    role = lane / LPH;                                   // 0: the key, 1: the value, beyond: nothing to store
    const int head = a.heads + (role == 1 ? a.kv_heads : 0) + hk;
    const bf16_t* src = f.qkv + (int64_t)token * f.qkv_stride + (int64_t)head * D + li * 8;
    const uint4 raw = *reinterpret_cast<const uint4*>(src);
    const bf16_t* e = reinterpret_cast<const bf16_t*>(&raw);
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = bf16_to_float(e[j]);
    if (f.k_weight != nullptr) {
      const uint4 wraw = *reinterpret_cast<const uint4*>(f.k_weight + li * 8);
      const bf16_t* w = reinterpret_cast<const bf16_t*>(&wraw);
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[j] * v[j];
#pragma unroll
      for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, WAVE);
      const float inv = 1.0f / sqrtf(ss / (float)D + f.eps);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (float)(__bf16)((v[j] * inv) * bf16_to_float(w[j]));
    }
    if (f.table != nullptr) {
      const float* cs = f.table + (int64_t)pos * D + (li % (LPH / 2)) * 8;
      float co[8], si[8];
      *reinterpret_cast<float4*>(co) = *reinterpret_cast<const float4*>(cs);
      *reinterpret_cast<float4*>(co + 4) = *reinterpret_cast<const float4*>(cs + 4);
      *reinterpret_cast<float4*>(si) = *reinterpret_cast<const float4*>(cs + D / 2);
      *reinterpret_cast<float4*>(si + 4) = *reinterpret_cast<const float4*>(cs + D / 2 + 4);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float other = __shfl_xor(v[j], LPH / 2, WAVE);
        v[j] = li < LPH / 2 ? v[j] * co[j] - other * si[j] : v[j] * co[j] + other * si[j];
      }
    }
    mine = raw;
    if (role == 0) {
      __bf16* oe = reinterpret_cast<__bf16*>(&mine);
#pragma unroll
      for (int j = 0; j < 8; ++j) oe[j] = (__bf16)v[j];
    }
    if (role < 2) *reinterpret_cast<uint4*>(fresh + role * D + li * 8) = mine;
  }

  __device__ __forceinline__ void store(const AttnArgs& a, const FusedArgs& f, int token, int hk) const {
    const int P = a.page_size;
    const int64_t plane = (int64_t)P * D;
    const int wpage = f.write_page[token], woff = f.write_off[token];
    if (role == 0) {
      *reinterpret_cast<uint4*>(f.pages + (((int64_t)wpage * 2) * a.kv_heads + hk) * plane + (int64_t)woff * D + li * 8) = mine;
    } else if (role == 1) {
      const bf16_t* e = reinterpret_cast<const bf16_t*>(&mine);
      bf16_t* dst = f.pages + (((int64_t)wpage * 2 + 1) * a.kv_heads + hk) * plane + woff;
#pragma unroll
      for (int j = 0; j < 8; ++j) dst[(int64_t)(li * 8 + j) * P] = e[j];
    }
  }
};

// Decode rows: block (split, kv head x head block, row), one wave. Partials go to part_o / part_ml.
// FUSED: the queries come raw from the step's q/k/v projection and are normed and rotated here (each wave its own
// copy: a few hundred values), and the wave whose keys end with the row's new token norms and rotates that token's key
// and keeps it and the value in LDS, from where they take their place among the wave's operands; it stores them into
// the cache as the last thing it does (a store before the loads would make every later load wait for it), and no
// other wave reads that place. A decode row's token sits at position len - 1. The kernel that did all this for decode
// steps is gone.
// A block's waves take consecutive shares of the row's keys and their partials are combined through LDS in wave order
// (waves 1.. leave theirs there, wave 0 adds them up); with one block a (row, kv head) the block writes the result
// itself and no merge kernel follows.
template <int D, bool FUSED>
__global__ void __launch_bounds__(512) attn_decode_kernel(AttnArgs a, FusedArgs f) {
  extern __shared__ __attribute__((aligned(16))) float red[];   // [waves - 1][16 D values, 16 maxima, 16 sums]
  __shared__ __attribute__((aligned(16))) bf16_t fresh_lds[FUSED ? 2 * D : 8];
  constexpr int PART = 16 * D + 32;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE, waves = blockDim.x / WAVE;
  const int g = lane / 16, c = lane % 16;
  const int ri = blockIdx.z;
  const int b = a.rows_in_order ? ri : a.row_ids[ri];
  const int group = a.heads / a.kv_heads;
  const TileMap tm = tile_map(group);
  const int hk = blockIdx.y / tm.head_blocks, hb = blockIdx.y % tm.head_blocks;
  const int split = blockIdx.x * waves + wave;
  const int qs = a.rows_in_order ? b : a.qstart[b], n = a.lens[b];
  const RowRef rr = row_ref(tm, c, 0, hb, hk, group, qs, 1, n);
  // the keys this row can see, cut into `splits` ranges of keys_per_split
  const int qp_row = n - 1;
  const int first = a.window > 0 ? max(0, qp_row - a.window + 1) : 0;
  // every split gets an equal share of this row's own keys (a multiple of 32), whatever length the launch was
  // shaped for: a row shorter than the longest one still keeps all its waves busy
  const int base = (first / 32) * 32;
  const int share = max(32, ((qp_row - base + a.splits) / a.splits + 31) / 32 * 32);
  const int key_lo = base + split * share;
  const int key_hi = min(qp_row, key_lo + share - 1);
  const bool empty = n <= 0 || key_lo > key_hi;           // (uniform over the wave) a partial that weighs nothing
  const bool writer = FUSED && !empty && key_hi == qp_row;   // its keys end with the row's new token
  f32x4_t o[1][D / 16];
  float m[1] = {-INFINITY}, l[1] = {0.f};
#pragma unroll
  for (int ds = 0; ds < D / 16; ++ds) o[0][ds] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  NewKeyValue<D> fresh;
  if (!empty) {
    const int32_t* trow = a.table + (int64_t)a.slots[b] * a.table_stride;
    bf16x8_t qf[1][D / 32];
    // FUSED: what makes the queries is asked for now (lane (g, c) holds dims 32 ks + 8 g .. + 7 of head c: the raw
    // values, the norm's weights, the cosines and sines of the row's position) and turned into `qf` inside attn_tiles,
    // while the first keys are on their way
    uint4 qraw[D / 32], wraw[D / 32];
    float4 cs[D / 64][4];
    if constexpr (FUSED) {
      const bf16_t* qptr = f.qkv + (int64_t)rr.token * f.qkv_stride + (int64_t)rr.head * D + 8 * g;
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks) {
        qraw[ks] = uint4{0u, 0u, 0u, 0u};
        if (rr.valid) qraw[ks] = *reinterpret_cast<const uint4*>(qptr + ks * 32);
        if (f.q_weight != nullptr) wraw[ks] = *reinterpret_cast<const uint4*>(f.q_weight + ks * 32 + 8 * g);
      }
      if (f.table != nullptr) {
        const float* t0 = f.table + (int64_t)min(qp_row, f.max_positions - 1) * D + 8 * g;
#pragma unroll
        for (int ks = 0; ks < D / 64; ++ks) {
          cs[ks][0] = *reinterpret_cast<const float4*>(t0 + ks * 32);
          cs[ks][1] = *reinterpret_cast<const float4*>(t0 + ks * 32 + 4);
          cs[ks][2] = *reinterpret_cast<const float4*>(t0 + D / 2 + ks * 32);
          cs[ks][3] = *reinterpret_cast<const float4*>(t0 + D / 2 + ks * 32 + 4);
        }
      }
      if (writer) {                      // one wave of the block at most; what it leaves in LDS only it reads
        fresh.make(a, f, qs, min(qp_row, f.max_positions - 1), hk, fresh_lds);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
    } else {
      const bf16_t* qptr = a.q + ((int64_t)rr.token * a.heads + rr.head) * D + 8 * g;
#pragma unroll
      for (int ks = 0; ks < D / 32; ++ks) {
        if (rr.valid) {
          qf[0][ks] = load8(qptr + ks * 32);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) qf[0][ks][i] = (__bf16)0.f;
        }
      }
    }
    auto make_queries = [&]() {
      if constexpr (FUSED) {
        float qv[D / 32][8];
        float ss = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          const bf16_t* e = reinterpret_cast<const bf16_t*>(&qraw[ks]);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            qv[ks][j] = bf16_to_float(e[j]);
            ss += qv[ks][j] * qv[ks][j];
          }
        }
        if (f.q_weight != nullptr) {     // the sum of squares over the four lane groups, then round((x inv) w)
          ss += __shfl_xor(ss, 16, WAVE);
          ss += __shfl_xor(ss, 32, WAVE);
          const float inv = 1.0f / sqrtf(ss / (float)D + f.eps);
#pragma unroll
          for (int ks = 0; ks < D / 32; ++ks) {
            const bf16_t* w = reinterpret_cast<const bf16_t*>(&wraw[ks]);
#pragma unroll
            for (int j = 0; j < 8; ++j) qv[ks][j] = (float)(__bf16)((qv[ks][j] * inv) * bf16_to_float(w[j]));
          }
        }
        if (f.table != nullptr) {        // dim i turns with dim i + D/2: fragment ks + D/64 of the same lane
#pragma unroll
          for (int ks = 0; ks < D / 64; ++ks) {
            const float* co = reinterpret_cast<const float*>(&cs[ks][0]);
            const float* si = reinterpret_cast<const float*>(&cs[ks][2]);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float lo = qv[ks][j], hi = qv[ks + D / 64][j];
              qv[ks][j] = lo * co[j] - hi * si[j];
              qv[ks + D / 64][j] = hi * co[j] + lo * si[j];
            }
          }
        }
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks)
#pragma unroll
          for (int j = 0; j < 8; ++j) qf[0][ks][j] = (__bf16)qv[ks][j];
      }
    };
    int qpos[1] = {rr.valid ? qp_row : -1}, tile_last[1] = {qp_row}, tile_first[1] = {qp_row};
    attn_tiles<D, 1>(a, trow, hk, qf, qpos, tile_last, tile_first, max(key_lo, first), key_hi, o, m, l,
                     writer ? fresh_lds : nullptr, make_queries);
  }
  float lt = l[0];
  lt += __shfl_xor(lt, 16, WAVE);
  lt += __shfl_xor(lt, 32, WAVE);
  float mt = m[0];
  if (waves > 1) {                       // the block's partials, added up in wave order by wave 0
    if (wave > 0) {
      float* mine = red + (int64_t)(wave - 1) * PART;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) *reinterpret_cast<f32x4_t*>(mine + (ds * WAVE + lane) * 4) = o[0][ds];
      if (g == 0) { mine[16 * D + c] = mt; mine[16 * D + 16 + c] = lt; }
    }
    __syncthreads();
    if (wave == 0) {
      for (int w = 1; w < waves; ++w) {
        const float* theirs = red + (int64_t)(w - 1) * PART;
        const float mw = theirs[16 * D + c], lw = theirs[16 * D + 16 + c];
        const float m_new = fmaxf(mt, mw);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(mt - m_use), beta = __builtin_amdgcn_exp2f(mw - m_use);
        lt = lt * alpha + lw * beta;
#pragma unroll
        for (int ds = 0; ds < D / 16; ++ds)
          o[0][ds] = o[0][ds] * alpha + *reinterpret_cast<const f32x4_t*>(theirs + (ds * WAVE + lane) * 4) * beta;
        mt = m_new;
      }
    }
  }
  if (wave == 0 && rr.valid) {
    if (a.out_splits == 1) {             // the row's whole result: normalised and rounded here
      const float inv = lt > 0.f ? 1.0f / lt : 0.f;
      bf16_t* op = a.out + ((int64_t)rr.token * a.heads + rr.head) * D + 4 * g;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) {
        ushort4 w;
        w.x = float_to_bf16(o[0][ds][0] * inv);
        w.y = float_to_bf16(o[0][ds][1] * inv);
        w.z = float_to_bf16(o[0][ds][2] * inv);
        w.w = float_to_bf16(o[0][ds][3] * inv);
        *reinterpret_cast<ushort4*>(op + ds * 16) = w;
      }
    } else {
      const int64_t cell = ((int64_t)ri * a.heads + rr.head) * a.out_splits + blockIdx.x;
      float* po = a.part_o + cell * D + 4 * g;
#pragma unroll
      for (int ds = 0; ds < D / 16; ++ds) *reinterpret_cast<f32x4_t*>(po + ds * 16) = o[0][ds];
      if (g == 0) { a.part_ml[cell * 2] = mt; a.part_ml[cell * 2 + 1] = lt; }
    }
  }
  if constexpr (FUSED) {
    if (writer) fresh.store(a, f, qs, hk);
  }
}

// out[row, head, :] = sum_i 2^(m_i - M) o_i / sum_i 2^(m_i - M) l_i over the splits (at most 64). One block of four
// waves per (row, head): thread (group, d4) adds the partials of splits group, group + NG, ... for four dims, all of
// its loads under way at once; the groups' sums are then added in group order. The order of every sum depends on
// the number of splits and the head size alone.
template <int D>
__global__ void __launch_bounds__(256) attn_merge_kernel(const float* __restrict__ part_o,
                                                         const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                                                         const int32_t* __restrict__ row_ids,
                                                         const int32_t* __restrict__ qstart, int heads, int splits) {
  constexpr int LANES = D / 4;            // threads across one partial
  constexpr int NG = 256 / LANES;         // groups of splits
  constexpr int PER = (64 + NG - 1) / NG; // splits a thread may own
  __shared__ float weight[64];
  __shared__ float inv_denom;
  __shared__ f32x4_t sums[NG][LANES];
  const int ri = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int token = qstart[row_ids[ri]];
  const float* ml = part_ml + ((int64_t)ri * heads + h) * splits * 2;
  const float* po = part_o + ((int64_t)ri * heads + h) * splits * D;
  const int group = tid / LANES, d0 = 4 * (tid % LANES);
  f32x4_t v[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i)            // asked for before the weights are known: an empty split's values are dropped
    v[i] = *reinterpret_cast<const f32x4_t*>(po + (int64_t)min(group + i * NG, splits - 1) * D + d0);
  if (tid < WAVE) {
    float m_s = -INFINITY, l_s = 0.f;
    if (tid < splits) {
      const float2 x = *reinterpret_cast<const float2*>(ml + 2 * tid);
      m_s = x.x;
      l_s = x.y;
    }
    if (!(l_s > 0.f)) m_s = -INFINITY;
    const float big = wave_max(m_s);
    const float w_s = l_s > 0.f ? exp2f(m_s - big) : 0.f;
    float denom = 0.f;                     // in split order
    for (int s = 0; s < splits; ++s) denom += __shfl(w_s * l_s, s, WAVE);
    weight[tid] = w_s;
    if (tid == 0) inv_denom = denom > 0.f ? 1.0f / denom : 0.f;
  }
  __syncthreads();
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int sp = group + i * NG;
    const float w = sp < splits ? weight[sp] : 0.f;
    if (w > 0.f) acc += w * v[i];
  }
  sums[group][tid % LANES] = acc;
  __syncthreads();
  if (group == 0) {
#pragma unroll
    for (int gq = 1; gq < NG; ++gq) acc += sums[gq][tid];
    const float inv = inv_denom;
    ushort4 o;
    o.x = float_to_bf16(acc[0] * inv); o.y = float_to_bf16(acc[1] * inv);
    o.z = float_to_bf16(acc[2] * inv); o.w = float_to_bf16(acc[3] * inv);
    *reinterpret_cast<ushort4*>(out + ((int64_t)token * heads + h) * D + d0) = o;
  }
}

#ifndef PAIR_VALU_PER_MFMA
#define PAIR_VALU_PER_MFMA 16
#endif
#ifndef PAIR_UNPAIR_BELOW
#define PAIR_UNPAIR_BELOW 512
#endif
// Long prompt portions of groups of up to 32 heads whose stages pass registers on their way into LDS (head_dim 64; 128
// when the direct copies are switched off): two tiles of 32 rows a wave from PAIR_FROM_KEYS keys on (measured, 32 heads
// over 8 kv heads of 128, portions of 4,096 tokens, us a layer, one tile against two: behind 4,096 tokens 616 and 636,
// behind 12,288 tokens 1,366 and 1,279, behind 28,672 tokens 2,625 and 2,441; whole prompts of 2,048 and 4,096 tokens
// 78 and 101, 208 and 298: short rows have too few blocks of 256 rows to fill the GPU).
// holon_attention_prefill_form: 0 never, 1 by that rule, 2 always (tests run both forms at the same sizes); returns
// what was set before; a negative argument only asks.
constexpr int PAIR_FROM_KEYS = 12288;
static int g_prefill_pair = 1;
extern "C" int holon_attention_prefill_form(int form) {
  const int was = g_prefill_pair;
  if (form >= 0 && form <= 2) g_prefill_pair = form;
  return was;
}

// Whether long portions at head_dim 128 (groups of up to 32 heads) have their stages copied into LDS by the memory
// pipeline, one tile of 32 rows a wave (1, the default), or through registers, one or two tiles a wave (0; tests run
// both); returns what was set before; a negative argument only asks. Measured, 32 heads over 8 kv heads, portions of
// 4,096 tokens, us a layer, direct against the better of the register forms: a whole prompt of 2,048 tokens 65 and 76,
// of 4,096 tokens 204 and 204; behind 4,096 tokens 552 and 603, behind 12,288 tokens 1,108 and 1,221, behind 28,672
// tokens 2,206 and 2,246 (0.93 PFLOP/s), behind 61,440 tokens 4,624 and 4,430; 64 heads over 8: 0.97 PFLOP/s behind 28,672.
static int g_prefill_dma = 1;
extern "C" int holon_attention_prefill_copies(int direct) {
  const int was = g_prefill_dma;
  if (direct == 0 || direct == 1) g_prefill_dma = direct;
  return was;
}

static bool mfma_serves(int head_dim, int page_size) {
  return (head_dim == 64 || head_dim == 128 || head_dim == 256) && page_size % 16 == 0;
}

extern "C" int holon_attention_mfma_supported(int head_dim, int page_size, int dtype) {
  return dtype == HOLON_BF16 && mfma_serves(head_dim, page_size);
}

extern "C" int holon_attention_prefill_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                            int table_stride, const int32_t* slots, const int32_t* lens,
                                            const int32_t* query_start, const int32_t* row_ids, int n_rows,
                                            int max_query, int max_len, int heads, int kv_heads, int head_dim,
                                            int page_size, float scale, int window, void* stream) {
  HOLON_CHECK(mfma_serves(head_dim, page_size), "attention (matrix cores): head_dim %d / page %d not served", head_dim,
              page_size);
  HOLON_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && window >= 0 && table_stride > 0,
              "attention: bad sizes");
  if (n_rows <= 0 || max_query <= 0) return 0;
  AttnArgs a{};
  a.q = (const bf16_t*)q; a.out = (bf16_t*)out; a.pages = (const bf16_t*)pages; a.table = table;
  a.table_stride = table_stride; a.slots = slots; a.lens = lens; a.qstart = query_start; a.row_ids = row_ids;
  a.heads = heads; a.kv_heads = kv_heads; a.page_size = page_size;
  a.scale_log2 = scale * 1.4426950408889634f; a.window = window;
  const TileMap tm = tile_map(heads / kv_heads);
  const int nt = head_dim == 256 ? 1 : 2;
  const int tiles = (max_query + tm.pos_per_tile - 1) / tm.pos_per_tile;
  if (head_dim != 256 && tiles >= 16 && max_len <= 4096 * page_size) {
    // long portions: keys and values staged through LDS, shared by four waves (rows of up to 4096 pages). Two tiles a
    // wave share each stage among twice the rows (measured: 4,096 tokens 340 -> 287 us, 32,768 tokens 17.0 -> 13.3 ms)
    // but halve the blocks: below two blocks a compute unit one tile a wave is faster (2,048 tokens: 95 against 113 us).
    const int ranges2 = (tiles + 7) / 8;
    const int64_t blocks2 = (int64_t)((ranges2 + 1) / 2) * kv_heads * tm.head_blocks * n_rows;
    hipStream_t ls = (hipStream_t)stream;
    const TileMap32 tm32 = tile_map32(heads / kv_heads);
    const int ranges32 = ((max_query + tm32.pos_per_tile - 1) / tm32.pos_per_tile + 3) / 4;
    const int ranges_pair = ((max_query + tm32.pos_per_tile - 1) / tm32.pos_per_tile + 7) / 8;
    const bool direct = g_prefill_dma && head_dim == 128 && heads / kv_heads <= 32;   // (then one tile a wave is the faster)
    if (!direct && heads / kv_heads <= 32 &&
        (g_prefill_pair == 2 || (g_prefill_pair == 1 && max_len >= PAIR_FROM_KEYS))) {
      // two tiles of 32 rows a wave
      a.unpaired = (int64_t)((ranges_pair + 1) / 2) * kv_heads * n_rows < PAIR_UNPAIR_BELOW ? 1 : 0;
      dim3 lgrid(kv_heads, (ranges_pair + 1) / 2, a.unpaired ? 2 * n_rows : n_rows);   // (x: the kv head, see below)
      if (head_dim == 64) attn_prefill_pair_kernel<64><<<lgrid, 256, 0, ls>>>(a);
      else attn_prefill_pair_kernel<128><<<lgrid, 256, 0, ls>>>(a);
    } else if (heads / kv_heads <= 32) {   // tiles of 32 rows (measured faster at every length: 2,048 tokens 89 against 95 us,
                                    // 32,768 tokens 11.1 against 13.3 ms); larger groups keep tiles of 16
      // fewer than two paired blocks a compute unit: the ranges of a pair as blocks of their own, so that a second
      // wave on every SIMD hides the first one's waits
      a.unpaired = (int64_t)((ranges32 + 1) / 2) * kv_heads * n_rows < UNPAIR_BELOW ? 1 : 0;
      // x: the kv head. Blocks are dealt to the XCDs in turn, so with 8 kv heads every block of a head runs on the
      // same XCD and finds the keys its neighbours have just read in that XCD's L2 (behind 28,672 tokens 2,246 -> 2,119 us)
      dim3 lgrid(kv_heads, (ranges32 + 1) / 2, a.unpaired ? 2 * n_rows : n_rows);
      if (head_dim == 64) attn_prefill_wide_kernel<64><<<lgrid, 256, 0, ls>>>(a);
      else if (direct) attn_prefill_dma_kernel<<<lgrid, 256, 0, ls>>>(a);
      else attn_prefill_wide_kernel<128><<<lgrid, 256, 0, ls>>>(a);
    } else if (blocks2 >= 512) {
      dim3 lgrid((ranges2 + 1) / 2, kv_heads * tm.head_blocks, n_rows);
      if (head_dim == 64) attn_prefill_lds_kernel<64, 2><<<lgrid, 256, 0, ls>>>(a);
      else attn_prefill_lds_kernel<128, 2><<<lgrid, 256, 0, ls>>>(a);
    } else {
      const int ranges = (tiles + 3) / 4;
      dim3 lgrid((ranges + 1) / 2, kv_heads * tm.head_blocks, n_rows);
      if (head_dim == 64) attn_prefill_lds_kernel<64, 1><<<lgrid, 256, 0, ls>>>(a);
      else attn_prefill_lds_kernel<128, 1><<<lgrid, 256, 0, ls>>>(a);
    }
    HOLON_LAUNCH_OK();
    return 0;
  }
  dim3 grid(((tiles + nt - 1) / nt + 3) / 4, kv_heads * tm.head_blocks, n_rows);
  hipStream_t s = (hipStream_t)stream;
  if (head_dim == 64) attn_prefill_kernel<64, 2><<<grid, 256, 0, s>>>(a);
  else if (head_dim == 128) attn_prefill_kernel<128, 2><<<grid, 256, 0, s>>>(a);
  else attn_prefill_kernel<256, 1><<<grid, 256, 0, s>>>(a);
  HOLON_LAUNCH_OK();
  return 0;
}

// The decode launch both entry points share: the split kernel, then the ordered merge.
static int decode_launch(const void* q, void* out, const void* pages, const int32_t* table, int table_stride,
                         const int32_t* slots, const int32_t* lens, const int32_t* query_start, const int32_t* row_ids,
                         int n_rows, int max_len, int heads, int kv_heads, int head_dim, int page_size, float scale,
                         int window, float* part_o, float* part_ml, int splits, int keys_per_split, void* stream,
                         const FusedArgs* fused = nullptr, int waves = 1, int rows_in_order = 0) {
  HOLON_CHECK(mfma_serves(head_dim, page_size), "attention (matrix cores): head_dim %d / page %d not served", head_dim,
              page_size);
  HOLON_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && window >= 0 && table_stride > 0,
              "attention: bad sizes");
  HOLON_CHECK(splits > 0 && splits <= 64 && keys_per_split > 0 && keys_per_split % 32 == 0,
              "attention decode: %d splits of %d keys (1 to 64 splits of a multiple of 32 keys)", splits, keys_per_split);
  HOLON_CHECK(waves >= 1 && waves <= 8 && splits % waves == 0 && (waves - 1) * (16 * head_dim + 32) * 4 <= 64 * 1024,
              "attention decode: %d waves a block for %d splits of head_dim %d (1 to 8, a divisor of the splits, "
              "partials within 64 KB of LDS)", waves, splits, head_dim);
  HOLON_CHECK(splits == waves || (part_o && part_ml), "attention decode: %d splits over blocks need a workspace",
              splits / waves);
  const int span = window > 0 ? (window < max_len ? window + 31 : max_len) : max_len;
  HOLON_CHECK((int64_t)splits * keys_per_split >= span, "attention decode: %d splits of %d keys do not cover %d keys",
              splits, keys_per_split, span);
  if (n_rows <= 0) return 0;
  AttnArgs a{};
  a.q = (const bf16_t*)q; a.out = (bf16_t*)out; a.pages = (const bf16_t*)pages; a.table = table;
  a.table_stride = table_stride; a.slots = slots; a.lens = lens; a.qstart = query_start; a.row_ids = row_ids;
  a.heads = heads; a.kv_heads = kv_heads; a.page_size = page_size;
  a.scale_log2 = scale * 1.4426950408889634f; a.window = window;
  a.part_o = part_o; a.part_ml = part_ml; a.splits = splits; a.keys_per_split = keys_per_split;
  a.out_splits = splits / waves; a.rows_in_order = rows_in_order;
  const TileMap tm = tile_map(heads / kv_heads);
  dim3 grid(a.out_splits, kv_heads * tm.head_blocks, n_rows);
  hipStream_t s = (hipStream_t)stream;
  const int threads = waves * WAVE;
  const size_t lds = (size_t)(waves - 1) * (16 * head_dim + 32) * sizeof(float);
  if (fused != nullptr) {
    if (head_dim == 64) attn_decode_kernel<64, true><<<grid, threads, lds, s>>>(a, *fused);
    else if (head_dim == 128) attn_decode_kernel<128, true><<<grid, threads, lds, s>>>(a, *fused);
    else attn_decode_kernel<256, true><<<grid, threads, lds, s>>>(a, *fused);
  } else {
    const FusedArgs none{};
    if (head_dim == 64) attn_decode_kernel<64, false><<<grid, threads, lds, s>>>(a, none);
    else if (head_dim == 128) attn_decode_kernel<128, false><<<grid, threads, lds, s>>>(a, none);
    else attn_decode_kernel<256, false><<<grid, threads, lds, s>>>(a, none);
  }
  HOLON_LAUNCH_OK();
  if (a.out_splits == 1) return 0;       // every block has written its row's result
  splits = a.out_splits;
  dim3 mgrid(n_rows, heads);
  if (head_dim == 64)
    attn_merge_kernel<64><<<mgrid, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, row_ids, query_start, heads, splits);
  else if (head_dim == 128)
    attn_merge_kernel<128><<<mgrid, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, row_ids, query_start, heads, splits);
  else
    attn_merge_kernel<256><<<mgrid, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, row_ids, query_start, heads, splits);
  HOLON_LAUNCH_OK();
  return 0;
}

extern "C" int holon_attention_decode_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                           int table_stride, const int32_t* slots, const int32_t* lens,
                                           const int32_t* query_start, const int32_t* row_ids, int n_rows, int max_len,
                                           int heads, int kv_heads, int head_dim, int page_size, float scale,
                                           int window, float* part_o, float* part_ml, int splits, int keys_per_split,
                                           void* stream) {
  return decode_launch(q, out, pages, table, table_stride, slots, lens, query_start, row_ids, n_rows, max_len, heads,
                       kv_heads, head_dim, page_size, scale, window, part_o, part_ml, splits, keys_per_split, stream);
}

// The same with `waves` waves a block (1 to 8, a divisor of `splits`): a block's waves combine their partials through
// LDS, so a (row, head) leaves splits / waves partials (part_o [n_rows, heads, splits / waves, head_dim], part_ml
// likewise) and, when that is one, none at all: the block writes the result and the workspace may be NULL.
// rows_in_order: every row of the step is a decode row, row_ids[i] = i and query_start[i] = i (neither is then read).
extern "C" int holon_attention_decode_waves_bf16(const void* q, void* out, const void* pages, const int32_t* table,
                                                 int table_stride, const int32_t* slots, const int32_t* lens,
                                                 const int32_t* query_start, const int32_t* row_ids, int n_rows,
                                                 int max_len, int heads, int kv_heads, int head_dim, int page_size,
                                                 float scale, int window, float* part_o, float* part_ml, int splits,
                                                 int keys_per_split, int waves, int rows_in_order, void* stream) {
  return decode_launch(q, out, pages, table, table_stride, slots, lens, query_start, row_ids, n_rows, max_len, heads,
                       kv_heads, head_dim, page_size, scale, window, part_o, part_ml, splits, keys_per_split, stream,
                       nullptr, waves, rows_in_order);
}

// Decode rows straight from the step's raw q/k/v projection: per-head norm, rotation and the cache write of each
// row's new token happen inside the attention kernel. `qkv` [T, (heads + 2 kv_heads) head_dim]; q_weight / k_weight
// (both or neither) the per-head RMSNorm weights; rope_table [max_positions, head_dim] (cos | sin) or NULL. A row's
// token is taken to sit at position len - 1 (what a decode row is).
extern "C" int holon_attention_decode_fused_bf16(const void* qkv, void* out, void* pages, const int32_t* table,
                                                 int table_stride, const int32_t* slots, const int32_t* lens,
                                                 const int32_t* query_start, const int32_t* row_ids, int n_rows,
                                                 int max_len, int heads, int kv_heads, int head_dim, int page_size,
                                                 float scale, int window, const void* q_weight, const void* k_weight,
                                                 float eps, const float* rope_table, int max_positions,
                                                 const int32_t* write_page, const int32_t* write_off, float* part_o,
                                                 float* part_ml, int splits, int keys_per_split, int waves,
                                                 int rows_in_order, void* stream) {
  HOLON_CHECK((q_weight == nullptr) == (k_weight == nullptr), "attention decode (fused): q and k norm weights come together");
  HOLON_CHECK(qkv && pages && write_page && write_off, "attention decode (fused): the projection, the cache and write "
              "targets are needed");
  HOLON_CHECK(rope_table == nullptr || max_positions >= 1, "attention decode (fused): a rotation table of %d positions",
              max_positions);
  FusedArgs f{};
  f.qkv = (const bf16_t*)qkv; f.qkv_stride = (int64_t)(heads + 2 * kv_heads) * head_dim;
  f.q_weight = (const bf16_t*)q_weight; f.k_weight = (const bf16_t*)k_weight; f.eps = eps;
  f.table = rope_table; f.max_positions = max_positions; f.pages = (bf16_t*)pages;
  f.write_page = write_page; f.write_off = write_off;
  return decode_launch(nullptr, out, pages, table, table_stride, slots, lens, query_start, row_ids, n_rows, max_len,
                       heads, kv_heads, head_dim, page_size, scale, window, part_o, part_ml, splits, keys_per_split,
                       stream, &f, waves, rows_in_order);
}

// ---- decode attention for callers that cannot allocate ------------------------------------------------------------
// The split partials live in a file-scope device array instead of a workspace the caller brings. Each GPU holds its own
// copy of the array at its own address, which is looked up once per device; host code uses that address and never the
// array's name. Nothing in it has to start at zero: the merge reads only partials that the split kernel of the same
// call wrote (an empty split writes a weight of zero, and its values are then dropped unread). Every call on a GPU
// shares that GPU's array, so two calls that overlap on one GPU (two streams, two threads) race on it.
static __device__ __align__(256) float scratch[HOLON_DECODE_SCRATCH_BYTES / sizeof(float)];

static constexpr int kMaxDevices = 64;
static float* g_scratch[kMaxDevices];          // per device: where that device's copy of `scratch` lies
static std::mutex g_scratch_lock;

// The current device's copy of the array, looked up at the first call on that device.
static int decode_scratch(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  HOLON_CHECK(e == hipSuccess, "attention decode (static): hipGetDevice: %s", hipGetErrorString(e));
  HOLON_CHECK(dev >= 0 && dev < kMaxDevices, "attention decode (static): device %d beyond the %d this library tracks",
              dev, kMaxDevices);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (g_scratch[dev] == nullptr) {
    void* found = nullptr;
    e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    HOLON_CHECK(e == hipSuccess && found != nullptr, "attention decode (static): hipGetSymbolAddress: %s",
                hipGetErrorString(e));
    g_scratch[dev] = (float*)found;
  }
  *ptr = g_scratch[dev];
  return 0;
}

extern "C" int holon_decode_scratch_init(void) {
  float* ptr = nullptr;
  return decode_scratch(&ptr);
}

extern "C" int64_t holon_decode_scratch_bytes(void) { return HOLON_DECODE_SCRATCH_BYTES; }

extern "C" int holon_attention_decode_bf16_static(const void* q, void* out, const void* pages, const int32_t* table,
                                                  int table_stride, const int32_t* slots, const int32_t* lens,
                                                  const int32_t* query_start, const int32_t* row_ids, int n_rows,
                                                  int max_len, int heads, int kv_heads, int head_dim, int page_size,
                                                  float scale, int window, int splits, int keys_per_split,
                                                  void* stream) {
  HOLON_CHECK(n_rows >= 0 && heads > 0 && splits > 0 && head_dim > 0, "attention decode (static): bad sizes");
  // part_o [n_rows, heads, splits, head_dim] then part_ml [n_rows, heads, splits, 2], the second on a 256-byte edge
  const int64_t cells = (int64_t)n_rows * heads * splits;
  const int64_t o_floats = (cells * head_dim + 63) / 64 * 64;
  const int64_t need = (o_floats + cells * 2) * (int64_t)sizeof(float);
  HOLON_CHECK(need <= HOLON_DECODE_SCRATCH_BYTES,
              "attention decode (static): %d rows x %d heads x %d splits of head_dim %d need %lld bytes of partials; the "
              "built-in buffer holds %lld (use holon_attention_decode_bf16 with a workspace of your own)",
              n_rows, heads, splits, head_dim, (long long)need, (long long)HOLON_DECODE_SCRATCH_BYTES);
  float* base = nullptr;
  if (decode_scratch(&base) != 0) return -1;
  return decode_launch(q, out, pages, table, table_stride, slots, lens, query_start, row_ids, n_rows, max_len, heads,
                       kv_heads, head_dim, page_size, scale, window, base, base + o_floats, splits, keys_per_split,
                       stream);
}
