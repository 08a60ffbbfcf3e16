// Shared device helpers and host-side error plumbing for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // raw bfloat16 bit pattern

typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define EXO_WAVE 64

__device__ __forceinline__ float bf2f(bf16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t f2bf(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(bf16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf2(float lo, float hi) {
  bf16x2_t r;
  r[0] = (__bf16)lo;
  r[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ float bf_lo(uint32_t v) {
  return __builtin_bit_cast(float, v << 16);
}
__device__ __forceinline__ float bf_hi(uint32_t v) {
  return __builtin_bit_cast(float, v & 0xffff0000u);
}
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                         __builtin_bit_cast(bf16x2_t, b), acc, false);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
// sum over aligned sub-groups of `width` lanes (power of two <= 64)
__device__ __forceinline__ float group_sum(float v, int width) {
  for (int o = width >> 1; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- cross-lane sums on the DPP path (no LDS traffic) ----
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_get(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
// sum over the wave; the total lands in lane 63
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
  v += dpp_get<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
  v += dpp_get<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
  v += dpp_get<0x141, 0xf>(v);  // row_half_mirror
  v += dpp_get<0x140, 0xf>(v);  // row_mirror: every lane holds its row-of-16 total
  v += dpp_get<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_get<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// sum over aligned runs of W (8 or 16) lanes, in every lane of the run
template <int W>
__device__ __forceinline__ float run_sum(float v) {
  v += dpp_get<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
  v += dpp_get<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
  v += dpp_get<0x141, 0xf>(v);  // row_half_mirror
  if (W == 16) v += dpp_get<0x140, 0xf>(v);  // row_mirror
  return v;
}

// Hand-over of results to another workgroup without a device-wide fence: the producer
// writes its values with device-scope stores, then every storing wave waits here until all
// of its outstanding vector-memory operations have completed (on gfx9 stores count in
// vmcnt and are acknowledged once they are visible at the scope they were issued with),
// then the workgroup barrier, then ONE thread bumps the arrival counter with a
// device-scope read-modify-write.  A consumer that saw the counter value loads the values
// at device scope.  The chain  store(sc1) -> vmcnt(0) -> s_barrier -> RMW(agent) ->
// load(sc1)  orders the values before the counter without writing the L2 back.
__device__ __forceinline__ void wait_own_stores_done() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- host side -------------------------------------------------------------
#define EXO_OK 0
#define EXO_ERR_ARG (-1)
#define EXO_ERR_HIP (-2)

void exo_set_error(const char* fmt, ...);
// records the kernel instance a launcher chose (read back with exo_last_variant())
void exo_note_variant(const char* fmt, ...);

#define EXO_REQUIRE(cond, ...)      \
  do {                              \
    if (!(cond)) {                  \
      exo_set_error(__VA_ARGS__);   \
      return EXO_ERR_ARG;           \
    }                               \
  } while (0)

#define EXO_CHECK_LAUNCH(name)                                               \
  do {                                                                       \
    hipError_t e__ = hipGetLastError();                                      \
    if (e__ != hipSuccess) {                                                 \
      exo_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));  \
      return EXO_ERR_HIP;                                                    \
    }                                                                        \
  } while (0)

static inline int exo_ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
