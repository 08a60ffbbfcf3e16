// Packing-format kernels: unpack codes, dequantize, embedding gather-dequant.
// Also owns the library's error string.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/exo_mi355x.h"
#include "common.h"

// Dequantised bf16 weights are formed the way bf16 arithmetic forms them, one
// rounding per operation: bf16(bf16(s*q) + b).  Set to 0 for a single rounding of
// the float32 fma.  One setting is compiled in; there is no runtime switch.
#ifndef EXO_DEQUANT_TWO_ROUNDINGS
#define EXO_DEQUANT_TWO_ROUNDINGS 1
#endif

static thread_local char g_err[512] = "";

void exo_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* exo_last_error(void) { return g_err; }

// Which kernel instance and launch shape the calling thread's latest matmul / attention
// entry point chose (diagnostic: lets a test assert that a shape reached the instance it
// was written for).
static thread_local char g_variant[256] = "";

void exo_note_variant(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_variant, sizeof(g_variant), fmt, ap);
  va_end(ap);
}

extern "C" const char* exo_last_variant(void) { return g_variant; }
extern "C" int exo_abi_version(void) { return 1; }
extern "C" int exo_dequant_two_roundings(void) { return EXO_DEQUANT_TWO_ROUNDINGS; }

__device__ __forceinline__ bf16_t dq_one(float s, float b, uint32_t q) {
#if EXO_DEQUANT_TWO_ROUNDINGS
  return f2bf(bf2f(f2bf(s * (float)q)) + b);
#else
  return f2bf(fmaf(s, (float)q, b));
#endif
}

// ------------------------------------------------------------------ unpack codes
template <int BITS>
__global__ __launch_bounds__(256) void unpack_kernel(const uint32_t* __restrict__ w,
                                                     uint8_t* __restrict__ out,
                                                     int64_t n_words) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_words) return;
  uint32_t v = w[i];
  if (BITS == 4) {
    uint32_t lo = v & 0x0f0f0f0fu, hi = (v >> 4) & 0x0f0f0f0fu;
    // bytes of lo = codes 0,2,4,6; bytes of hi = codes 1,3,5,7
    uint2 o;
    o.x = __builtin_amdgcn_perm(hi, lo, 0x05010400u);  // c0,c1,c2,c3
    o.y = __builtin_amdgcn_perm(hi, lo, 0x07030602u);  // c4,c5,c6,c7
    reinterpret_cast<uint2*>(out)[i] = o;
  } else {
    reinterpret_cast<uint32_t*>(out)[i] = v;  // 4 codes, already byte ordered
  }
}

extern "C" int exo_unpack_codes(const uint32_t* w, uint8_t* out, int64_t n_words, int bits,
                                exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_unpack_codes: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(n_words >= 0 && w && out, "exo_unpack_codes: null pointer or negative size");
  if (n_words == 0) return EXO_OK;
  dim3 grid(exo_ceil_div(n_words, 256));
  if (bits == 4)
    unpack_kernel<4><<<grid, 256, 0, (hipStream_t)stream>>>(w, out, n_words);
  else
    unpack_kernel<8><<<grid, 256, 0, (hipStream_t)stream>>>(w, out, n_words);
  EXO_CHECK_LAUNCH("exo_unpack_codes");
  return EXO_OK;
}

// ------------------------------------------------------------------ dequantize
// One thread per packed word: 8 (4-bit) or 4 (8-bit) outputs.  `row_map` (may be
// null) maps output row -> source row for the embedding gather.
template <int BITS>
__global__ __launch_bounds__(256) void dequant_kernel(
    const uint32_t* __restrict__ w, const bf16_t* __restrict__ scales,
    const bf16_t* __restrict__ biases, bf16_t* __restrict__ out,
    const int32_t* __restrict__ row_map, int64_t rows, int K, int vocab) {
  constexpr int PER = 32 / BITS;
  const int wpr = K / PER;  // words per row
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * wpr) return;
  int64_t r = i / wpr;
  int c = (int)(i - r * wpr);
  int64_t src = r;
  if (row_map) {
    int id = row_map[r];
    src = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  }
  uint32_t v = w[src * wpr + c];
  int g = (c * PER) >> 6;
  float s = bf2f(scales[src * (K >> 6) + g]);
  float b = bf2f(biases[src * (K >> 6) + g]);
  bf16_t o[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) o[j] = dq_one(s, b, (v >> (BITS * j)) & ((1u << BITS) - 1));
  bf16_t* dst = out + r * (int64_t)K + (int64_t)c * PER;
  if (BITS == 4) {
    uint4 p;
    p.x = o[0] | ((uint32_t)o[1] << 16);
    p.y = o[2] | ((uint32_t)o[3] << 16);
    p.z = o[4] | ((uint32_t)o[5] << 16);
    p.w = o[6] | ((uint32_t)o[7] << 16);
    *reinterpret_cast<uint4*>(dst) = p;
  } else {
    uint2 p;
    p.x = o[0] | ((uint32_t)o[1] << 16);
    p.y = o[2] | ((uint32_t)o[3] << 16);
    *reinterpret_cast<uint2*>(dst) = p;
  }
}

static int launch_dequant(const uint32_t* w, const bf16_t* s, const bf16_t* b, bf16_t* out,
                          const int32_t* row_map, int64_t rows, int K, int vocab, int bits,
                          hipStream_t st) {
  int64_t n = rows * (K / (32 / bits));
  if (n == 0) return EXO_OK;
  dim3 grid(exo_ceil_div(n, 256));
  if (bits == 4)
    dequant_kernel<4><<<grid, 256, 0, st>>>(w, s, b, out, row_map, rows, K, vocab);
  else
    dequant_kernel<8><<<grid, 256, 0, st>>>(w, s, b, out, row_map, rows, K, vocab);
  return EXO_OK;
}

extern "C" int exo_dequantize(const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, uint16_t* out, int64_t rows, int K,
                              int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_dequantize: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_dequantize: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(K > 0 && K % 64 == 0, "exo_dequantize: K=%d must be a positive multiple of 64", K);
  EXO_REQUIRE(rows >= 0 && w && scales && biases && out, "exo_dequantize: null pointer");
  launch_dequant(w, scales, biases, out, nullptr, rows, K, 0, bits, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_dequantize");
  return EXO_OK;
}

extern "C" int exo_embed_dequant(const int32_t* ids, const uint32_t* w, const uint16_t* scales,
                                 const uint16_t* biases, uint16_t* out, int n_ids, int vocab,
                                 int K, int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_embed_dequant: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_embed_dequant: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(K > 0 && K % 64 == 0, "exo_embed_dequant: K=%d must be a positive multiple of 64", K);
  EXO_REQUIRE(n_ids >= 0 && vocab > 0 && ids && w && scales && biases && out,
              "exo_embed_dequant: null pointer or bad size");
  launch_dequant(w, scales, biases, out, ids, n_ids, K, vocab, bits, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_embed_dequant");
  return EXO_OK;
}
