// Bandwidth-bound small ops: residual+RMSNorm, RoPE + KV append (+ per-head norm),
// SwiGLU, MoE routing/combination, greedy sampling reductions.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "route.h"

namespace {

// ---------------------------------------------------------------- add + RMSNorm
// One workgroup per row; each thread keeps up to 4 x 8 elements in registers.
constexpr int kNormThreads = 256;
constexpr int kNormMaxChunks = 4;  // H <= 256*8*4 = 8192

__device__ __forceinline__ float block_sum_256(float v, float* sh) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) sh[wave] = v;
  __syncthreads();
  float r = sh[0] + sh[1] + sh[2] + sh[3];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ res,
    const bf16_t* __restrict__ w, bf16_t* __restrict__ h_out, bf16_t* __restrict__ n_out,
    int H, float eps) {
  __shared__ float sh[4];
  const size_t row = (size_t)blockIdx.x * H;
  float v[kNormMaxChunks][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kNormMaxChunks; ++i) {
    const int e0 = (threadIdx.x + i * kNormThreads) * 8;
    if (e0 < H) {
      uint4 a = *reinterpret_cast<const uint4*>(x + row + e0);
      const uint32_t* a4 = reinterpret_cast<const uint32_t*>(&a);
      if (res) {
        uint4 r = *reinterpret_cast<const uint4*>(res + row + e0);
        const uint32_t* r4 = reinterpret_cast<const uint32_t*>(&r);
        uint4 o;
        uint32_t* o4 = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o4[e] = pack_bf2(bf_lo(a4[e]) + bf_lo(r4[e]), bf_hi(a4[e]) + bf_hi(r4[e]));
          v[i][2 * e] = bf_lo(o4[e]);
          v[i][2 * e + 1] = bf_hi(o4[e]);
        }
        if (h_out) *reinterpret_cast<uint4*>(h_out + row + e0) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[i][2 * e] = bf_lo(a4[e]);
          v[i][2 * e + 1] = bf_hi(a4[e]);
        }
        if (h_out) *reinterpret_cast<uint4*>(h_out + row + e0) = a;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(v[i][e], v[i][e], ss);
    }
  }
  ss = block_sum_256(ss, sh);
  const float inv = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int i = 0; i < kNormMaxChunks; ++i) {
    const int e0 = (threadIdx.x + i * kNormThreads) * 8;
    if (e0 < H) {
      uint4 wv = *reinterpret_cast<const uint4*>(w + e0);
      const uint32_t* w4 = reinterpret_cast<const uint32_t*>(&wv);
      uint4 o;
      uint32_t* o4 = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o4[e] = pack_bf2(v[i][2 * e] * inv * bf_lo(w4[e]), v[i][2 * e + 1] * inv * bf_hi(w4[e]));
      *reinterpret_cast<uint4*>(n_out + row + e0) = o;
    }
  }
}

// ------------------------------------------------------ RoPE + KV append (+ head norm)
// blockIdx.x = token, blockIdx.y = a run of 4 * kRopeHeadsPerWave heads; each wave takes
// kRopeHeadsPerWave heads and requests all of them before it works on the first (a short
// prompt is one latency chain per wave: 12 heads in turn took 7.9 us at 126 tokens).  Lane
// i < D/2 owns the pair (i, i + D/2) of every head.  The angle's cosine and sine come from
// the table ((cos, sin) per position and pair, as the decode step uses) when the position is
// inside it, else from a precise sincosf (the angle reaches thousands of radians) of the
// same product - the table holds exactly those values.
constexpr int kRopeHeadsPerWave = 3;
__global__ __launch_bounds__(256) void rope_kv_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ q_out, bf16_t* __restrict__ kc,
    bf16_t* __restrict__ vc, const int32_t* __restrict__ pos, const float* __restrict__ inv_freq,
    const float2* __restrict__ tab, int tab_rows, const bf16_t* __restrict__ qn,
    const bf16_t* __restrict__ kn, float eps, int T, int Hq, int Hkv, int D, int S_max) {
  const int tok = blockIdx.x;  // b*T + t
  const int b = tok / T, t = tok - b * T;
  const int i = threadIdx.x & 63, wave = threadIdx.x >> 6, half = D >> 1;
  const bool active = i < half;
  const int p = pos[b] + t;
  const int nh = Hq + 2 * Hkv;  // heads [0,Hq) are q, [Hq,Hq+Hkv) k, then v
  const int h0 = ((int)blockIdx.y * 4 + wave) * kRopeHeadsPerWave;
  bf16_t lo[kRopeHeadsPerWave], hi[kRopeHeadsPerWave];
#pragma unroll
  for (int u = 0; u < kRopeHeadsPerWave; ++u) {
    lo[u] = 0;
    hi[u] = 0;
    if (active && h0 + u < nh) {
      const bf16_t* src = qkv + (size_t)tok * nh * D + (size_t)(h0 + u) * D;
      lo[u] = src[i];
      hi[u] = src[i + half];
    }
  }
  float sn = 0.f, cs = 1.f;
  if (active) {
    if (tab && p < tab_rows) {
      const float2 v = tab[(size_t)p * half + i];
      cs = v.x;
      sn = v.y;
    } else {
      sincosf((float)p * inv_freq[i], &sn, &cs);
    }
  }
#pragma unroll
  for (int u = 0; u < kRopeHeadsPerWave; ++u) {
    const int head = h0 + u;
    if (head >= nh) break;
    if (head >= Hq + Hkv) {  // v: copy into the cache
      if (active && p < S_max) {
        bf16_t* dst = vc + (((size_t)b * Hkv + (head - Hq - Hkv)) * S_max + p) * D;
        dst[i] = lo[u];
        dst[i + half] = hi[u];
      }
      continue;
    }
    float x1 = bf2f(lo[u]), x2 = bf2f(hi[u]);
    const bool is_q = head < Hq;
    const bf16_t* nw = is_q ? qn : kn;
    if (nw) {  // per-head RMSNorm, rounded to bf16 like a separate rms_norm call
      const float ss = wave_sum(x1 * x1 + x2 * x2);
      const float inv = rsqrtf(ss / (float)D + eps);
      if (active) {
        x1 = bf2f(f2bf(x1 * inv * bf2f(nw[i])));
        x2 = bf2f(f2bf(x2 * inv * bf2f(nw[i + half])));
      }
    }
    if (!active) continue;
    const bf16_t o1 = f2bf(x1 * cs - x2 * sn);
    const bf16_t o2 = f2bf(x2 * cs + x1 * sn);
    if (is_q) {
      bf16_t* dst = q_out + (size_t)tok * Hq * D + (size_t)head * D;
      dst[i] = o1;
      dst[i + half] = o2;
    } else if (p < S_max) {
      bf16_t* dst = kc + (((size_t)b * Hkv + (head - Hq)) * S_max + p) * D;
      dst[i] = o1;
      dst[i + half] = o2;
    }
  }
}

// ------------------------------------------------------------------------ SwiGLU
__global__ __launch_bounds__(256) void swiglu_kernel(const bf16_t* __restrict__ g,
                                                     const bf16_t* __restrict__ u,
                                                     bf16_t* __restrict__ out, int64_t n) {
  int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (i + 1 < n) {
    const uint32_t gv = *reinterpret_cast<const uint32_t*>(g + i);
    const uint32_t uv = *reinterpret_cast<const uint32_t*>(u + i);
    const float g0 = bf_lo(gv), g1 = bf_hi(gv);
    *reinterpret_cast<uint32_t*>(out + i) = pack_bf2(
        g0 / (1.f + __expf(-g0)) * bf_lo(uv), g1 / (1.f + __expf(-g1)) * bf_hi(uv));
  } else if (i < n) {
    const float g0 = bf2f(g[i]);
    out[i] = f2bf(g0 / (1.f + __expf(-g0)) * bf2f(u[i]));
  }
}

// ------------------------------------------------------------------- MoE routing
// One wave per row (route.h).
__global__ __launch_bounds__(64) void router_topk_kernel(const bf16_t* __restrict__ logits,
                                                         int32_t* __restrict__ idx,
                                                         bf16_t* __restrict__ scores, int E,
                                                         int k, int renorm) {
  const int row = blockIdx.x, lane = threadIdx.x;
  int my_id;
  float my_p, tot;
  route_topk_wave(logits + (size_t)row * E, E, k, lane, my_id, my_p, tot);
  if (lane < k) {
    idx[(size_t)row * k + lane] = my_id;
    scores[(size_t)row * k + lane] = route_score(my_p, tot, renorm);
  }
}

// ------------------------------------------------------------------ MoE combine
__global__ __launch_bounds__(256) void moe_combine_kernel(const bf16_t* __restrict__ y,
                                                          const bf16_t* __restrict__ scores,
                                                          const bf16_t* __restrict__ res,
                                                          bf16_t* __restrict__ out, int topk,
                                                          int H) {
  const int t = blockIdx.y;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= H) return;
  float acc = 0.f;
  for (int j = 0; j < topk; ++j) {
    const float s = bf2f(scores[(size_t)t * topk + j]);
    acc += bf2f(f2bf(bf2f(y[((size_t)t * topk + j) * H + e]) * s));
  }
  float o = bf2f(f2bf(acc));
  if (res) o += bf2f(res[(size_t)t * H + e]);
  out[(size_t)t * H + e] = f2bf(o);
}

// The same sums for H a multiple of 8 (16-byte aligned rows): 8 elements per thread, the
// expert rows of four slots requested together.  Slot order and rounding points as above.
__global__ __launch_bounds__(256) void moe_combine_vec_kernel(const bf16_t* __restrict__ y,
                                                              const bf16_t* __restrict__ scores,
                                                              const bf16_t* __restrict__ res,
                                                              bf16_t* __restrict__ out, int topk,
                                                              int H) {
  const int t = blockIdx.y;
  const int e = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (e >= H) return;
  float acc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[k] = 0.f;
  const bf16_t* yt = y + (size_t)t * topk * H + e;
  for (int j0 = 0; j0 < topk; j0 += 4) {
    uint4 v[4];
    float sc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = min(j0 + u, topk - 1);
      v[u] = *reinterpret_cast<const uint4*>(yt + (size_t)j * H);
      sc[u] = bf2f(scores[(size_t)t * topk + j]);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (j0 + u < topk) {
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          acc[2 * k] += bf2f(f2bf(bf_lo(w[k]) * sc[u]));
          acc[2 * k + 1] += bf2f(f2bf(bf_hi(w[k]) * sc[u]));
        }
      }
    }
  }
  float o[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = bf2f(f2bf(acc[k]));
  if (res) {
    const uint4 rv = *reinterpret_cast<const uint4*>(res + (size_t)t * H + e);
    const uint32_t w[4] = {rv.x, rv.y, rv.z, rv.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      o[2 * k] += bf_lo(w[k]);
      o[2 * k + 1] += bf_hi(w[k]);
    }
  }
  uint4 ov;
  ov.x = pack_bf2(o[0], o[1]);
  ov.y = pack_bf2(o[2], o[3]);
  ov.z = pack_bf2(o[4], o[5]);
  ov.w = pack_bf2(o[6], o[7]);
  *reinterpret_cast<uint4*>(out + (size_t)t * H + e) = ov;
}

// -------------------------------------------------- argmax + logsumexp over logits
// Stage 1: grid (kArgBlocks, rows): per block (max, argmax, sum exp(x - max)).
// Stage 2: one wave per row merges the blocks.
constexpr int kArgBlocks = 64;

__global__ __launch_bounds__(256) void argmax_stage1(const bf16_t* __restrict__ logits,
                                                     float* __restrict__ ws, int V) {
  __shared__ float smax[4], ssum[4];
  __shared__ int sidx[4];
  const int row = blockIdx.y;
  const bf16_t* src = logits + (size_t)row * V;
  // rows of 16-byte multiples (every vocabulary here): the block's share is whole 8-element
  // chunks, up to two per thread, which stay in registers for the second pass
  const bool vec = (V & 7) == 0 && (V >> 3) <= kArgBlocks * 512 && ((uintptr_t)logits & 15) == 0;
  const int per = vec ? (((V >> 3) + kArgBlocks - 1) / kArgBlocks) << 3 : (V + kArgBlocks - 1) / kArgBlocks;
  const int lo = min((int)blockIdx.x * per, V), hi = min(lo + per, V);
  float mx = -INFINITY;
  int mi = 0x7fffffff;
  float xv[16];
  if (vec) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int i0 = lo + (threadIdx.x + 256 * u) * 8;
      uint4 v = make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);  // -inf
      if (i0 < hi) v = *reinterpret_cast<const uint4*>(src + i0);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        xv[8 * u + 2 * k] = bf_lo(w[k]);
        xv[8 * u + 2 * k + 1] = bf_hi(w[k]);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (xv[8 * u + k] > mx) {
          mx = xv[8 * u + k];
          mi = i0 + k;
        }
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
      const float x = bf2f(src[i]);
      if (x > mx) {
        mx = x;
        mi = i;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(mx, o, 64);
    const int oi = __shfl_xor(mi, o, 64);
    if (ov > mx || (ov == mx && oi < mi)) {
      mx = ov;
      mi = oi;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    smax[wave] = mx;
    sidx[wave] = mi;
  }
  __syncthreads();
  float bm = smax[0];
  int bi = sidx[0];
#pragma unroll
  for (int w = 1; w < 4; ++w)
    if (smax[w] > bm || (smax[w] == bm && sidx[w] < bi)) {
      bm = smax[w];
      bi = sidx[w];
    }
  float se = 0.f;
  if (bm > -INFINITY) {
    if (vec) {
#pragma unroll
      for (int k = 0; k < 16; ++k) se += expf(xv[k] - bm);  // padding is -inf: exp = 0
    } else {
      for (int i = lo + threadIdx.x; i < hi; i += 256) se += expf(bf2f(src[i]) - bm);
    }
  }
  se = wave_sum(se);
  if (lane == 0) ssum[wave] = se;
  __syncthreads();
  if (threadIdx.x == 0) {
    float* d = ws + ((size_t)row * kArgBlocks + blockIdx.x) * 4;
    d[0] = bm;
    d[1] = __int_as_float(bi);
    d[2] = ssum[0] + ssum[1] + ssum[2] + ssum[3];
  }
}

__global__ __launch_bounds__(64) void argmax_stage2(const float* __restrict__ ws,
                                                    int32_t* __restrict__ token,
                                                    float* __restrict__ lse,
                                                    float* __restrict__ logprob,
                                                    int32_t* __restrict__ pos_inc) {
  const int row = blockIdx.x, lane = threadIdx.x;
  const float* s = ws + ((size_t)row * kArgBlocks + lane) * 4;
  float mx = s[0];
  int mi = __float_as_int(s[1]);
  const float bm = mx, bs = s[2];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(mx, o, 64);
    const int oi = __shfl_xor(mi, o, 64);
    if (ov > mx || (ov == mx && oi < mi)) {
      mx = ov;
      mi = oi;
    }
  }
  float se = (bm > -INFINITY) ? bs * expf(bm - mx) : 0.f;
  se = wave_sum(se);
  if (lane == 0) {
    const float l = mx + logf(se);
    token[row] = mi;
    if (lse) lse[row] = l;
    if (logprob) logprob[row] = mx - l;
    if (pos_inc) pos_inc[row] += 1;
  }
}

}  // namespace

extern "C" int exo_add_rmsnorm(const uint16_t* x, const uint16_t* residual,
                               const uint16_t* weight, uint16_t* h_out, uint16_t* n_out,
                               int rows, int H, float eps, exo_stream_t stream) {
  EXO_REQUIRE(x && weight && n_out, "exo_add_rmsnorm: null pointer");
  EXO_REQUIRE(rows >= 0 && H > 0 && H % 8 == 0 && H <= kNormThreads * 8 * kNormMaxChunks,
              "exo_add_rmsnorm: H=%d must be a multiple of 8 and <= %d", H,
              kNormThreads * 8 * kNormMaxChunks);
  if (rows == 0) return EXO_OK;
  add_rmsnorm_kernel<<<dim3(rows), kNormThreads, 0, (hipStream_t)stream>>>(
      x, residual, weight, h_out, n_out, H, eps);
  EXO_CHECK_LAUNCH("exo_add_rmsnorm");
  return EXO_OK;
}

extern "C" int exo_rope_kv_append_tab(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_cache,
                                      uint16_t* v_cache, const int32_t* pos,
                                      const float* inv_freq, const float* rope_table,
                                      int table_rows, const uint16_t* q_norm_w,
                                      const uint16_t* k_norm_w, float eps, int B, int T, int Hq,
                                      int Hkv, int D, int S_max, exo_stream_t stream) {
  EXO_REQUIRE(qkv && q_out && k_cache && v_cache && pos && inv_freq,
              "exo_rope_kv_append: null pointer");
  EXO_REQUIRE(B > 0 && T > 0 && Hq > 0 && Hkv > 0 && S_max > 0,
              "exo_rope_kv_append: non-positive size");
  EXO_REQUIRE(D == 64 || D == 128, "exo_rope_kv_append: head_dim %d not supported (64, 128)", D);
  EXO_REQUIRE(!rope_table || table_rows > 0, "exo_rope_kv_append: table without rows");
  EXO_REQUIRE((int64_t)B * T <= 0x7fffffff / 2, "exo_rope_kv_append: too many tokens");
  const int runs = exo_ceil_div(Hq + 2 * Hkv, 4 * kRopeHeadsPerWave);
  rope_kv_kernel<<<dim3(B * T, runs), 256, 0, (hipStream_t)stream>>>(
      qkv, q_out, k_cache, v_cache, pos, inv_freq, reinterpret_cast<const float2*>(rope_table),
      table_rows, q_norm_w, k_norm_w, eps, T, Hq, Hkv, D, S_max);
  EXO_CHECK_LAUNCH("exo_rope_kv_append");
  return EXO_OK;
}

extern "C" int exo_rope_kv_append(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_cache,
                                  uint16_t* v_cache, const int32_t* pos, const float* inv_freq,
                                  const uint16_t* q_norm_w, const uint16_t* k_norm_w, float eps,
                                  int B, int T, int Hq, int Hkv, int D, int S_max,
                                  exo_stream_t stream) {
  return exo_rope_kv_append_tab(qkv, q_out, k_cache, v_cache, pos, inv_freq, nullptr, 0, q_norm_w,
                                k_norm_w, eps, B, T, Hq, Hkv, D, S_max, stream);
}

extern "C" int exo_swiglu(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n,
                          exo_stream_t stream) {
  EXO_REQUIRE(gate && up && out && n >= 0, "exo_swiglu: null pointer or negative size");
  if (n == 0) return EXO_OK;
  swiglu_kernel<<<dim3(exo_ceil_div((n + 1) / 2, 256)), 256, 0, (hipStream_t)stream>>>(
      gate, up, out, n);
  EXO_CHECK_LAUNCH("exo_swiglu");
  return EXO_OK;
}

extern "C" int exo_router_topk(const uint16_t* logits, int32_t* idx, uint16_t* scores, int rows,
                               int E, int k, int renorm, exo_stream_t stream) {
  EXO_REQUIRE(logits && idx && scores, "exo_router_topk: null pointer");
  EXO_REQUIRE(E > 0 && E <= 256 && k > 0 && k <= 16 && k <= E && rows >= 0,
              "exo_router_topk: need 0<E<=256, 0<k<=min(16,E); got E=%d k=%d", E, k);
  if (rows == 0) return EXO_OK;
  router_topk_kernel<<<dim3(rows), 64, 0, (hipStream_t)stream>>>(logits, idx, scores, E, k,
                                                                  renorm);
  EXO_CHECK_LAUNCH("exo_router_topk");
  return EXO_OK;
}

extern "C" int exo_moe_combine(const uint16_t* y, const uint16_t* scores,
                               const uint16_t* residual, uint16_t* out, int T, int topk, int H,
                               exo_stream_t stream) {
  EXO_REQUIRE(y && scores && out, "exo_moe_combine: null pointer");
  EXO_REQUIRE(T >= 0 && topk > 0 && H > 0 && T <= 65535, "exo_moe_combine: bad size");
  if (T == 0) return EXO_OK;
  const bool vec = H % 8 == 0 &&
                   (((uintptr_t)y | (uintptr_t)residual | (uintptr_t)out) & 15) == 0;
  if (vec)
    moe_combine_vec_kernel<<<dim3(exo_ceil_div(H / 8, 256), T), 256, 0, (hipStream_t)stream>>>(
        y, scores, residual, out, topk, H);
  else
    moe_combine_kernel<<<dim3(exo_ceil_div(H, 256), T), 256, 0, (hipStream_t)stream>>>(
        y, scores, residual, out, topk, H);
  EXO_CHECK_LAUNCH("exo_moe_combine");
  return EXO_OK;
}

extern "C" int64_t exo_argmax_workspace(int rows) {
  return (int64_t)rows * kArgBlocks * 4 * (int64_t)sizeof(float);
}

extern "C" int exo_argmax_logsumexp(const uint16_t* logits, int32_t* token, float* lse,
                                    float* logprob, float* workspace, int32_t* pos_inc,
                                    int rows, int V, exo_stream_t stream) {
  EXO_REQUIRE(logits && token && workspace, "exo_argmax_logsumexp: null pointer");
  EXO_REQUIRE(rows >= 0 && rows <= 65535 && V > 0, "exo_argmax_logsumexp: bad size");
  if (rows == 0) return EXO_OK;
  argmax_stage1<<<dim3(kArgBlocks, rows), 256, 0, (hipStream_t)stream>>>(logits, workspace, V);
  argmax_stage2<<<dim3(rows), 64, 0, (hipStream_t)stream>>>(workspace, token, lse, logprob,
                                                           pos_inc);
  EXO_CHECK_LAUNCH("exo_argmax_logsumexp");
  return EXO_OK;
}
