// Shared device helpers for the gfx950 kernels: element types, rounding, wave and block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef uint16_t bf16_t;   // bfloat16 kept as its bit pattern; all arithmetic is float32

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round to nearest, ties to even (what torch's .bfloat16() does); NaN stays NaN. The hardware's conversion
// (v_cvt_pk_bf16_f32): one instruction where the same in integer arithmetic takes seven.
__device__ __forceinline__ bf16_t float_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int kVec = 4;   // elements in 16 bytes
  static __device__ __forceinline__ float load(float v) { return v; }
  static __device__ __forceinline__ float store(float v) { return v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Elem<bf16_t> {
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float load(bf16_t v) { return bf16_to_float(v); }
  static __device__ __forceinline__ bf16_t store(float v) { return float_to_bf16(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_to_float(float_to_bf16(v)); }
};

// silu(g) = g / (1 + exp(-g)). For float32 results the library's exp and a true division; for bfloat16 results (8 bits
// are kept) the hardware's exp2 and reciprocal, whose error of about 2^-22 vanishes in the rounding.
template <typename T> __device__ __forceinline__ float silu(float g);
template <> __device__ __forceinline__ float silu<float>(float g) { return g / (1.0f + expf(-g)); }
template <> __device__ __forceinline__ float silu<bf16_t>(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// A copy from memory straight into LDS (global_load_lds_dwordx4): 16 bytes a lane, the wave's 64 lanes into one
// contiguous kilobyte of LDS at `lds_wave_base` (the same for every lane); the source is a base every lane shares, in
// scalar registers, plus a byte offset of the lane's own. The compiler does not know these loads (known ones make it
// wait for all of them before every read of LDS): a kernel that issues them writes its own waits (`wait_loads_but`)
// in front of the barrier that publishes what they brought. They count among the wave's loads like any other, in
// the order of issue.
// M0 holds the wave's place in LDS for the instruction behind it; nothing the compiler writes in these kernels uses M0.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t lane_bytes, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(lane_bytes), "s"(base), "s"(lds_wave_base) : "memory", "m0");
}
// A 16-byte load into registers that the compiler does not track either, for kernels whose other loads are the copies
// above: the compiler counts only the loads it knows, so where both kinds are under way the waits it inserts before a
// known load's first use come out wrong for the mix (far too early a wait, measured). The caller waits
// (`wait_loads_but`) before the first use, and keeps the result where it is until then (no copy of it may be made
// before the wait: the register still holds what it held before). OFFSET: a constant added to the address, 0 to 4095.
template <typename V, int OFFSET>
__device__ __forceinline__ void load16_untracked(V& to, const void* base, uint32_t lane_bytes) {
  static_assert(sizeof(V) == 16 && OFFSET >= 0 && OFFSET < 4096, "one 16-byte vector, an offset the instruction holds");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(to) : "v"(lane_bytes), "s"(base), "n"(OFFSET) : "memory");
}
#pragma clang diagnostic pop
template <int N>
__device__ __forceinline__ void wait_loads_but() {          // until at most N of this wave's loads are under way
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}


// Host side: every entry point returns 0 or a negative code and leaves a message for holon_last_error().
void holon_set_error(const char* fmt, ...);
#define HOLON_CHECK(cond, ...)        \
  do {                                \
    if (!(cond)) {                    \
      holon_set_error(__VA_ARGS__);   \
      return -1;                      \
    }                                 \
  } while (0)
#define HOLON_LAUNCH_OK()                                                        \
  do {                                                                           \
    hipError_t e_ = hipGetLastError();                                           \
    if (e_ != hipSuccess) {                                                      \
      holon_set_error("%s: launch failed: %s", __func__, hipGetErrorString(e_)); \
      return -2;                                                                 \
    }                                                                            \
  } while (0)

enum { HOLON_F32 = 0, HOLON_BF16 = 1 };
