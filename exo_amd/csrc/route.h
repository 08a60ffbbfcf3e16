// MoE routing of one token by one wave: softmax over E <= 256 router logits, the k largest
// probabilities.  Shared by the stand-alone top-k launch and by the expert GEMV that does
// its own routing, so both select the same experts with the same bits.
#pragma once
#include "common.h"

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_max_u32(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false);
  return o > v ? o : v;
}
// maximum over the wave, as a wave-uniform value (a six-step DPP reduction into lane 63)
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = dpp_max_u32<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
  v = dpp_max_u32<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
  v = dpp_max_u32<0x141, 0xf>(v);  // row_half_mirror
  v = dpp_max_u32<0x140, 0xf>(v);  // row_mirror: every lane holds its row-of-16 maximum
  v = dpp_max_u32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_max_u32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_max_f32(float v) {
  const int o = __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), CTRL,
                                            ROW_MASK, 0xf, false);
  return fmaxf(__builtin_bit_cast(float, o), v);
}
__device__ __forceinline__ float wave_max_f32_uniform(float v) {
  v = dpp_max_f32<0xB1, 0xf>(v);
  v = dpp_max_f32<0x4E, 0xf>(v);
  v = dpp_max_f32<0x141, 0xf>(v);
  v = dpp_max_f32<0x140, 0xf>(v);
  v = dpp_max_f32<0x142, 0xa>(v);
  v = dpp_max_f32<0x143, 0xc>(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum_uniform(float v) {
  v = wave_sum_to_lane63(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// The probabilities are float32 softmax values rounded to bf16.  The k selections run on
// packed keys (bf16 probability bits << 16 | 0xFFFF - expert): one unsigned maximum per
// selection finds the largest probability and, among equals, the lowest expert id; a
// taken key becomes 0.  On return lane j < k holds the expert id and the probability of
// the j-th selection (descending), `tot` the sum of the k probabilities in every lane.
// The logits of one token as raw 16-bit patterns, lane l holding experts l, l + 64, l + 128 and
// l + 192.  Unconditional loads (indices past E re-read the last logit, dropped afterwards) into
// 32-bit registers: the four requests go out back to back and one wait covers them.
__device__ __forceinline__ void route_load(const bf16_t* __restrict__ logits, int E, int lane,
                                           uint32_t (&raw)[4]) {
  const uint16_t* l16 = reinterpret_cast<const uint16_t*>(logits);
#pragma unroll
  for (int i = 0; i < 4; ++i) raw[i] = l16[min(lane + 64 * i, E - 1)];
}

__device__ __forceinline__ void route_topk_regs(const uint32_t (&raw)[4], int E, int k, int lane,
                                                int& my_id, float& my_p, float& tot) {
  float v[4];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = lane + 64 * i;
    v[i] = (e < E) ? __builtin_bit_cast(float, raw[i] << 16) : -INFINITY;
    mx = fmaxf(mx, v[i]);
  }
  mx = wave_max_f32_uniform(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] = (lane + 64 * i < E) ? expf(v[i] - mx) : 0.f;
    sum += v[i];
  }
  sum = wave_sum_uniform(sum);
  uint32_t key[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = lane + 64 * i;
    key[i] = (e < E) ? (((uint32_t)f2bf(v[i] / sum) << 16) | (uint32_t)(0xFFFF - e)) : 0u;
  }
  my_id = 0;
  my_p = 0.f;
  tot = 0.f;
  for (int j = 0; j < k; ++j) {
    uint32_t best = key[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) best = key[i] > best ? key[i] : best;
    best = wave_max_u32(best);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (key[i] == best) key[i] = 0u;
    const float bv = bf2f((bf16_t)(best >> 16));
    tot += bv;
    if (lane == j) {
      my_id = 0xFFFF - (int)(best & 0xFFFFu);
      my_p = bv;
    }
  }
}

__device__ __forceinline__ void route_topk_wave(const bf16_t* __restrict__ logits, int E, int k,
                                                int lane, int& my_id, float& my_p, float& tot) {
  uint32_t raw[4];
  route_load(logits, E, lane, raw);
  route_topk_regs(raw, E, k, lane, my_id, my_p, tot);
}

// score of a selection as the block uses it: the probability, or (renorm) the probability
// over the bf16-rounded sum of the k selected ones
__device__ __forceinline__ bf16_t route_score(float p, float tot, int renorm) {
  return renorm ? f2bf(p / bf2f(f2bf(tot))) : f2bf(p);
}
