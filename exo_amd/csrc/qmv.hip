// Fused dequant-GEMV for decode (M <= 16): y = x @ dq(W)^T on MLX affine-packed W.
//
// HBM-bound design for gfx950:
//  * every lane streams 16-byte pieces ("chunks") of a packed row with
//    global_load_dwordx4; a row is covered by LPR lanes (power of two, 64 when the
//    row is long enough) so that each load instruction of a wave reads 1 KiB that is
//    contiguous per row; 8 such loads are in flight per lane before any is consumed.
//  * codes are never converted one by one: a 4-bit word w gives four bf16x2 registers
//    (w >> 4t) & 0x000F000F | 0x43004300 = (128+q_t, 128+q_{t+4}); v_dot2_f32_bf16
//    multiplies them with the matching activation pair in float32.  The +128 is
//    removed with the per-chunk activation sum: sum x*q = D - 128*sum(x).
//    8-bit codes are treated as two nibbles against (x, 16x).
//  * per chunk (half / quarter of a 64-group):  acc += s*(D - 128*Sx) + b*Sx.
//  * activations sit in LDS, pre-permuted to the register order above and laid out
//    so a wave's ds_read_b128 is conflict-free; per-chunk sums are precomputed once
//    per workgroup.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "qmv_internal.h"
#include "route.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kUnits = 8;  // 16-byte loads in flight per lane

struct QmvParams {
  const bf16_t* x;         // [M,K]
  const uint32_t* w[2];    // packed [N, WPR]   ([1] only for the swiglu pair)
  const bf16_t* s[2];      // [N, K/64]
  const bf16_t* b[2];
  const bf16_t* residual;  // [M,N] or null
  bf16_t* y;               // [M,N]
  int M, N, K;
  int wpr;       // words per row
  int lpr_log2;  // lanes per row
  int iters;     // chunks per lane per row
  int slots;     // ceil(N / (64/LPR)): wave-wide row sets
  int spw;       // slots per wave
  int ragged;    // N is not a multiple of 64/LPR: the last slot has rows >= N
  // gather (MoE) mode: blockIdx.y = (token, slot) pair; expert = idx[pair]
  const int32_t* idx;  // [T*topk] or null
  int E, topk, x_rows;
  // the same with ONE matrix: blockIdx.y = row of x and of y (topk = x_rows = 1, idx null)
  int each_row;
  // gather mode that routes by itself: every wave repeats the softmax + top-k of its token
  // over route[token, :E] (idx null) and takes the expert of its slot; the first workgroup
  // of a token's first slot also writes the token's indices and scores out
  const bf16_t* route;   // [T, E] router logits or null
  int32_t* route_idx;    // [T*topk]
  bf16_t* route_scores;  // [T*topk]
  int route_renorm;
  // fused RMSNorm of the input rows: x <- bf16(x * rsqrt(mean(x^2) + eps) * norm_w)
  const bf16_t* norm_w;  // [K] or null
  float eps;
};

// sum over the 256 threads of the workgroup, for MT values at once
template <int MT>
__device__ __forceinline__ void block_sum(float (&v)[MT], float* red /* [4*MT] */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const float t = wave_sum(v[m]);
    if (lane == 0) red[wave * MT + m] = t;
  }
  __syncthreads();
#pragma unroll
  for (int m = 0; m < MT; ++m)
    v[m] = red[m] + red[MT + m] + red[2 * MT + m] + red[3 * MT + m];
  __syncthreads();
}

// 8 (4-bit layout) or 4 (8-bit layout) bf16 values of one word: v <- bf16(v * inv * w)
template <int BITS>
__device__ __forceinline__ void norm_word(uint4& xv, const uint4& wv, float inv) {
  xv.x = pack_bf2(bf_lo(xv.x) * inv * bf_lo(wv.x), bf_hi(xv.x) * inv * bf_hi(wv.x));
  xv.y = pack_bf2(bf_lo(xv.y) * inv * bf_lo(wv.y), bf_hi(xv.y) * inv * bf_hi(wv.y));
  if (BITS == 4) {
    xv.z = pack_bf2(bf_lo(xv.z) * inv * bf_lo(wv.z), bf_hi(xv.z) * inv * bf_hi(wv.z));
    xv.w = pack_bf2(bf_lo(xv.w) * inv * bf_lo(wv.w), bf_hi(xv.w) * inv * bf_hi(wv.w));
  }
}
template <int BITS>
__device__ __forceinline__ float sumsq_word(const uint4& xv) {
  float s = bf_lo(xv.x) * bf_lo(xv.x) + bf_hi(xv.x) * bf_hi(xv.x) +
            bf_lo(xv.y) * bf_lo(xv.y) + bf_hi(xv.y) * bf_hi(xv.y);
  if (BITS == 4)
    s += bf_lo(xv.z) * bf_lo(xv.z) + bf_hi(xv.z) * bf_hi(xv.z) +
         bf_lo(xv.w) * bf_lo(xv.w) + bf_hi(xv.w) * bf_hi(xv.w);
  return s;
}
// dot2 register order of one word's activations, with the sum of the stored values
// (8-bit stores x and 16x) and of the plain values
template <int BITS>
__device__ __forceinline__ uint4 permute_word(const uint4& xv, float& stored, float& truesum) {
  uint4 o;
  if (BITS == 4) {
    o.x = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);  // (x0,x4)
    o.y = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);  // (x1,x5)
    o.z = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);  // (x2,x6)
    o.w = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);  // (x3,x7)
    truesum = (bf_lo(o.x) + bf_hi(o.x)) + (bf_lo(o.y) + bf_hi(o.y)) +
              (bf_lo(o.z) + bf_hi(o.z)) + (bf_lo(o.w) + bf_hi(o.w));
    stored = truesum;
  } else {
    const uint32_t a = __builtin_amdgcn_perm(xv.y, xv.x, 0x05040100u);   // (x0,x2)
    const uint32_t c2 = __builtin_amdgcn_perm(xv.y, xv.x, 0x07060302u);  // (x1,x3)
    o.x = a;
    o.y = pack_bf2(bf_lo(a) * 16.f, bf_hi(a) * 16.f);
    o.z = c2;
    o.w = pack_bf2(bf_lo(c2) * 16.f, bf_hi(c2) * 16.f);
    truesum = (bf_lo(a) + bf_hi(a)) + (bf_lo(c2) + bf_hi(c2));
    stored = truesum + ((bf_lo(o.y) + bf_hi(o.y)) + (bf_lo(o.w) + bf_hi(o.w)));
  }
  return o;
}

// (ROUTE: the (gate, up) pair of a routed expert - two rows per wave or so, where a
// workgroup-wide staging with its barriers costs more than four waves normalising alike)
template <int MT, int ITERS, int NMAT, bool ROUTE = false>
constexpr bool kRowsXR = (MT == 1 && ITERS <= 2 && (NMAT == 1 || ROUTE));

template <int BITS>
__device__ __forceinline__ uint4 load_word_x(const bf16_t* base, int wi) {
  if (BITS == 4) return *reinterpret_cast<const uint4*>(base + (size_t)wi * 8);
  const uint2 v = *reinterpret_cast<const uint2*>(base + (size_t)wi * 4);
  return make_uint4(v.x, v.y, 0, 0);
}

// Stage x (rows m0..m0+MT) into LDS in dot2 register order; compute chunk sums.
// xs layout per m: uint4[(j*4 + t) * LPR + sl]  for chunk c = sl + j*LPR, word t.
// sx layout per m: float2[c] = (128 * sum(stored), sum(x)).
template <int BITS, int MT>
__device__ __forceinline__ void stage_x(const QmvParams& p, const bf16_t* x, uint4* xs,
                                        float2* sx, float* red) {
  const int cpr = p.wpr >> 2;
  const int lpr_mask = (1 << p.lpr_log2) - 1;
  float inv[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) inv[m] = 1.f;
  if (p.norm_w) {
    float ss[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) ss[m] = 0.f;
    for (int wi = threadIdx.x; wi < p.wpr; wi += kThreads)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        if (m < p.M) ss[m] += sumsq_word<BITS>(load_word_x<BITS>(x + (size_t)m * p.K, wi));
    block_sum<MT>(ss, red);
#pragma unroll
    for (int m = 0; m < MT; ++m) inv[m] = rsqrtf(ss[m] / (float)p.K + p.eps);
  }
  for (int wi = threadIdx.x; wi < p.wpr; wi += kThreads) {
    const int c = wi >> 2, t = wi & 3;
    const int j = c >> p.lpr_log2, sl = c & lpr_mask;
    const int dst = (((j << 2) + t) << p.lpr_log2) + sl;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      uint4 o = make_uint4(0, 0, 0, 0);
      float stored = 0.f, truesum = 0.f;
      if (m < p.M) {
        uint4 xv = load_word_x<BITS>(x + (size_t)m * p.K, wi);
        if (p.norm_w) norm_word<BITS>(xv, load_word_x<BITS>(p.norm_w, wi), inv[m]);
        o = permute_word<BITS>(xv, stored, truesum);
      }
      xs[(size_t)m * p.wpr + dst] = o;
      stored += __shfl_xor(stored, 1, 64);
      truesum += __shfl_xor(truesum, 1, 64);
      stored += __shfl_xor(stored, 2, 64);
      truesum += __shfl_xor(truesum, 2, 64);
      if (t == 0) sx[(size_t)m * cpr + c] = make_float2(128.f * stored, truesum);
    }
  }
}

// Which 16-byte chunk of a row a lane takes in unit j of the row-streaming kernel.  Units
// come in pairs (2d, 2d+1) that interleave their quantisation groups: the lanes of a
// group own the groups 2g and 2g+1 of the pair, one in each unit, so the (scale, bias) of
// both units sit next to each other and come in ONE 32-bit load instead of two 16-bit
// ones.  A wave instruction of a pair still covers whole 64-byte pieces of every 128-byte
// line of the 2 KiB span.  An odd last unit keeps the linear order.
template <int BITS, int ITERS>
__device__ __forceinline__ int chunk_of(int j, int lane) {
  constexpr int LG = BITS == 4 ? 2 : 4;  // lanes (chunks) per group
  if ((ITERS & 1) && j == ITERS - 1) return 64 * j + lane;
  return 128 * (j >> 1) + 2 * LG * (lane / LG) + LG * (j & 1) + (lane % LG);
}
template <int BITS, int ITERS>
__device__ __forceinline__ void unit_lane_of(int c, int& j, int& lane) {
  constexpr int LG = BITS == 4 ? 2 : 4;
  if ((ITERS & 1) && c >= 64 * (ITERS - 1)) {
    j = ITERS - 1;
    lane = c - 64 * (ITERS - 1);
    return;
  }
  const int r = c & 127;
  j = 2 * (c >> 7) + ((r / LG) & 1);
  lane = (r / (2 * LG)) * LG + (r % LG);
}

// Two-phase staging for the row-streaming kernel (wpr == 256*ITERS, so every thread
// owns exactly ITERS words per activation row): the global loads are issued first and
// consumed after the first weight batches are in flight.
template <int BITS, int MT, int ITERS>
struct XStage {
  uint4 r[MT][ITERS];  // 8-bit uses .x/.y only
  uint4 nw[ITERS];     // norm weights of the same words (when fused)
};

template <int BITS, int MT, int ITERS>
__device__ __forceinline__ void stage_x_load(const QmvParams& p, const bf16_t* x,
                                             XStage<BITS, MT, ITERS>& st) {
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int wi = threadIdx.x + it * kThreads;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      st.r[m][it] = make_uint4(0, 0, 0, 0);
      if (m < p.M) st.r[m][it] = load_word_x<BITS>(x + (size_t)m * p.K, wi);
    }
    if (p.norm_w) st.nw[it] = load_word_x<BITS>(p.norm_w, wi);
  }
}

template <int BITS, int MT, int ITERS>
__device__ __forceinline__ void stage_x_store(const QmvParams& p, XStage<BITS, MT, ITERS>& st,
                                              uint4* xs, float2* sx, float* red) {
  constexpr int WPR = 256 * ITERS, CPR = 64 * ITERS;
  if (p.norm_w) {
    float ss[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      ss[m] = 0.f;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) ss[m] += sumsq_word<BITS>(st.r[m][it]);
    }
    block_sum<MT>(ss, red);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float inv = rsqrtf(ss[m] / (float)p.K + p.eps);
#pragma unroll
      for (int it = 0; it < ITERS; ++it) norm_word<BITS>(st.r[m][it], st.nw[it], inv);
    }
  }
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int wi = threadIdx.x + it * kThreads;
    const int c = wi >> 2, t = wi & 3;
    int j, sl;
    unit_lane_of<BITS, ITERS>(c, j, sl);
    const int dst = (((j << 2) + t) << 6) + sl;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      float stored, truesum;
      const uint4 o = permute_word<BITS>(st.r[m][it], stored, truesum);
      xs[m * WPR + dst] = o;
      stored += __shfl_xor(stored, 1, 64);
      truesum += __shfl_xor(truesum, 1, 64);
      stored += __shfl_xor(stored, 2, 64);
      truesum += __shfl_xor(truesum, 2, 64);
      if (t == 0) sx[m * CPR + j * 64 + sl] = make_float2(128.f * stored, truesum);
    }
  }
}

template <int BITS>
__device__ __forceinline__ void unpack_word(uint32_t w, uint32_t (&pr)[4]) {
  // nibble t and nibble t+4 of the word as (128+n_t, 128+n_{t+4}) in bf16
  pr[0] = (w & 0x000F000Fu) | 0x43004300u;
  pr[1] = ((w >> 4) & 0x000F000Fu) | 0x43004300u;
  pr[2] = ((w >> 8) & 0x000F000Fu) | 0x43004300u;
  pr[3] = ((w >> 12) & 0x000F000Fu) | 0x43004300u;
}
// Same, with the mask and the exponent pattern held in registers (gfx9 VOP3 takes no
// literals), so each pair is one v_and_or_b32.
__device__ __forceinline__ void unpack_word_r(uint32_t w, uint32_t mask, uint32_t magic,
                                              uint32_t (&pr)[4]) {
  pr[0] = (w & mask) | magic;
  pr[1] = ((w >> 4) & mask) | magic;
  pr[2] = ((w >> 8) & mask) | magic;
  pr[3] = ((w >> 12) & mask) | magic;
}

// NMAT == 2: the pair (gate, up) with the SwiGLU epilogue.
// ROUTE: the instantiation that can do the routing itself (p.route; MT == 1, the pair only)
template <int BITS, int MT, int NMAT, bool ROUTE = false>
__global__ __launch_bounds__(kThreads) void qmv_kernel(const QmvParams p) {
  extern __shared__ uint4 smem[];
  uint4* xs = smem;
  float2* sx = reinterpret_cast<float2*>(smem + (size_t)MT * p.wpr);
  constexpr int U = kUnits / NMAT;
  constexpr int GSHIFT = (BITS == 4) ? 1 : 2;  // chunks per group, log2

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int lpr = 1 << p.lpr_log2;
  const int rpwi = 64 >> p.lpr_log2;  // rows per wave instruction
  const int sl = lane & (lpr - 1);
  const int sub = lane >> p.lpr_log2;
  const int G = p.K >> 6;
  const int cpr = p.wpr >> 2;

  const int gw = blockIdx.x * kWaves + wave;
  const int s_begin = min(gw * p.spw, p.slots);
  const int s_end = min(s_begin + p.spw, p.slots);
  const int total = (s_end - s_begin) * p.iters;

  // gather mode: this workgroup's (token, slot) pair selects expert, x row and y row
  const bf16_t* xin = p.x;
  bf16_t* yout = p.y;
  size_t ew = 0, eg = 0;
  if (p.idx || p.each_row || (ROUTE && p.route)) {
    const int pair = blockIdx.y;
    if (ROUTE && p.route) {  // wave 0 repeats the routing of the token, the others wait
      __shared__ int s_expert;
      const int t = pair / p.topk, slot = pair - t * p.topk;
      if (wave == 0) {
        int my_id;
        float my_p, tot;
        route_topk_wave(p.route + (size_t)t * p.E, p.E, p.topk, lane, my_id, my_p, tot);
        if (blockIdx.x == 0 && slot == 0 && lane < p.topk) {
          p.route_idx[(size_t)t * p.topk + lane] = my_id;
          p.route_scores[(size_t)t * p.topk + lane] = route_score(my_p, tot, p.route_renorm);
        }
        if (lane == slot) s_expert = my_id;
      }
      __syncthreads();
      const int e = __builtin_amdgcn_readfirstlane(s_expert);
      ew = (size_t)e * p.N * p.wpr;
      eg = (size_t)e * p.N * G;
    } else if (p.idx) {
      int e = p.idx[pair];
      e = e < 0 ? 0 : (e >= p.E ? p.E - 1 : e);  // memory safety only: the host rejects such ids
      ew = (size_t)e * p.N * p.wpr;
      eg = (size_t)e * p.N * G;
    }
    xin += (size_t)(p.x_rows == 1 ? pair / p.topk : pair) * p.K;
    yout += (size_t)pair * p.N;
  }

  const int row0 = s_begin * rpwi + sub;
  const size_t slot_words = (size_t)rpwi * p.wpr;  // words between slots
  const int j_words = lpr * 4;
  const uint32_t* wl[NMAT];
  const bf16_t* sl_s[NMAT];
  const bf16_t* sl_b[NMAT];
#pragma unroll
  for (int a = 0; a < NMAT; ++a) {
    wl[a] = p.w[a] + ew + (size_t)row0 * p.wpr + sl * 4;
    sl_s[a] = p.s[a] + eg + (size_t)row0 * G + (sl >> GSHIFT);
    sl_b[a] = p.b[a] + eg + (size_t)row0 * G + (sl >> GSHIFT);
  }
  const int slot_groups = rpwi * G;
  const int j_groups = lpr >> GSHIFT;

  uint4 wv[NMAT][U];
  bf16_t sc[NMAT][U], bi[NMAT][U];

  // unit u -> (slot, j); issue the first batch of weight loads before staging x so
  // the HBM latency overlaps the prologue.
  auto issue = [&](int u0) {
    int slot = u0 / p.iters;  // once per batch
    int j = u0 - slot * p.iters;
#pragma unroll
    for (int i = 0; i < U; ++i) {
      const int last = (u0 + i >= total);  // clamp: re-read the final unit
      size_t wo = (size_t)slot * slot_words + (size_t)j * j_words;
      size_t so = (size_t)slot * slot_groups + (size_t)j * j_groups;
      if (p.ragged) {  // rows past N re-read row N-1 (their results are not stored)
        const int over = (s_begin + slot) * rpwi + sub - (p.N - 1);
        if (over > 0) {
          wo -= (size_t)over * p.wpr;
          so -= (size_t)over * G;
        }
      }
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        wv[a][i] = *reinterpret_cast<const uint4*>(wl[a] + wo);
        sc[a][i] = sl_s[a][so];
        bi[a][i] = sl_b[a][so];
      }
      if (!last && u0 + i + 1 < total) {
        if (++j == p.iters) {
          j = 0;
          ++slot;
        }
      }
    }
  };

  if (total > 0) issue(0);
  __shared__ float s_red[4 * MT];
  stage_x<BITS, MT>(p, xin, xs, sx, s_red);
  __syncthreads();
  if (total <= 0) return;

  float acc[NMAT][MT];
#pragma unroll
  for (int a = 0; a < NMAT; ++a)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[a][m] = 0.f;

  int slot = 0, j = 0;  // of the unit being consumed
  for (int u0 = 0; u0 < total; u0 += U) {
    // registers of this batch -> locals, then prefetch the next batch
    uint4 cw[NMAT][U];
    float cs[NMAT][U], cb[NMAT][U];
#pragma unroll
    for (int a = 0; a < NMAT; ++a)
#pragma unroll
      for (int i = 0; i < U; ++i) {
        cw[a][i] = wv[a][i];
        cs[a][i] = bf2f(sc[a][i]);
        cb[a][i] = bf2f(bi[a][i]);
      }
    if (u0 + U < total) issue(u0 + U);

#pragma unroll
    for (int i = 0; i < U; ++i) {
      if (u0 + i < total) {
        const int c = sl + (j << p.lpr_log2);
        float d[NMAT][MT];
#pragma unroll
        for (int a = 0; a < NMAT; ++a)
#pragma unroll
          for (int m = 0; m < MT; ++m) d[a][m] = 0.f;
        const uint32_t* cwi[NMAT];
#pragma unroll
        for (int a = 0; a < NMAT; ++a) cwi[a] = reinterpret_cast<const uint32_t*>(&cw[a][i]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          uint32_t pr[NMAT][4];
#pragma unroll
          for (int a = 0; a < NMAT; ++a) unpack_word<BITS>(cwi[a][t], pr[a]);
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const uint4 xv = xs[(size_t)m * p.wpr + ((((j << 2) + t) << p.lpr_log2) + sl)];
#pragma unroll
            for (int a = 0; a < NMAT; ++a) {
              d[a][m] = dot2_bf16(pr[a][0], xv.x, d[a][m]);
              d[a][m] = dot2_bf16(pr[a][1], xv.y, d[a][m]);
              d[a][m] = dot2_bf16(pr[a][2], xv.z, d[a][m]);
              d[a][m] = dot2_bf16(pr[a][3], xv.w, d[a][m]);
            }
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float2 sm = sx[(size_t)m * cpr + c];
#pragma unroll
          for (int a = 0; a < NMAT; ++a) {
            acc[a][m] = fmaf(cs[a][i], d[a][m] - sm.x, acc[a][m]);
            acc[a][m] = fmaf(cb[a][i], sm.y, acc[a][m]);
          }
        }
        if (++j == p.iters) {  // row finished: reduce over its lanes and store
          const int row = (s_begin + slot) * rpwi + sub;
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float r[NMAT];
#pragma unroll
            for (int a = 0; a < NMAT; ++a) {
              float v = acc[a][m];
              v += __shfl_xor(v, 1, 64);
              if (p.lpr_log2 > 1) v += __shfl_xor(v, 2, 64);
              if (p.lpr_log2 > 2) v += __shfl_xor(v, 4, 64);
              if (p.lpr_log2 > 3) v += __shfl_xor(v, 8, 64);
              if (p.lpr_log2 > 4) v += __shfl_xor(v, 16, 64);
              if (p.lpr_log2 > 5) v += __shfl_xor(v, 32, 64);
              r[a] = v;
              acc[a][m] = 0.f;
            }
            if (sl == 0 && m < p.M && row < p.N) {
              const size_t o = (size_t)m * p.N + row;
              float out;
              if (NMAT == 2) {
                const float g = bf2f(f2bf(r[0])), up = bf2f(f2bf(r[NMAT - 1]));
                out = g / (1.f + __expf(-g)) * up;
              } else {
                out = r[0];
                if (p.residual) out = bf2f(f2bf(out)) + bf2f(p.residual[o]);
              }
              yout[o] = f2bf(out);
            }
          }
          j = 0;
          ++slot;
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------
// Fast path: rows long enough that 64 lanes x 16 B tile them exactly
// (K*bits/128 = 64*ITERS chunks).  One row per wave instruction, so the flat unit
// index u = row*ITERS + j addresses weights (u * 1 KiB), scales and biases
// (u * 64>>GSHIFT elements) linearly: no per-unit address arithmetic beyond a scalar
// add.  ITERS is a template parameter: the per-row loop, the LDS offsets of x and the
// point where a row ends are all static.
template <int BITS, int MT, int NMAT, int ITERS, bool ROUTE = false>
__global__ __launch_bounds__(kThreads) void qmv_rows_kernel(const QmvParams p) {
  extern __shared__ uint4 smem[];
  uint4* xs = smem;
  float2* sx = reinterpret_cast<float2*>(smem + (size_t)MT * p.wpr);
  constexpr int GSHIFT = (BITS == 4) ? 1 : 2;
  constexpr int UG = 64 >> GSHIFT;  // scale elements per unit
  // NBUF register buffers of one batch each.  The (gate, up) pair on short rows takes four
  // batches of one row instead of two of two: the arithmetic on a batch then starts when a
  // quarter of the wave's loads has landed (measured: 1.5 us off the 14336x4096 pair; for a
  // single matrix the extra live registers cost more than the finer batches gain)
  constexpr int NBUF = (NMAT == 2 && ITERS <= 2) ? 4 : 2;
  constexpr int R0 = (16 / NBUF) / (ITERS * NMAT);
  constexpr int R = R0 < 1 ? 1 : R0;  // rows per batch
  constexpr int UB = R * ITERS;       // units per batch and matrix
  constexpr int CPR = 64 * ITERS;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = p.K >> 6;

  // balanced contiguous row range of this wave
  const int nwaves = gridDim.x * kWaves;
  const int gw = blockIdx.x * kWaves + wave;
  const int base = p.N / nwaves, rem = p.N - base * nwaves;
  const int r0 = gw * base + min(gw, rem);
  const int r1 = r0 + base + (gw < rem ? 1 : 0);
  const int nrows = r1 - r0;

  const bf16_t* xin = p.x;
  bf16_t* yout = p.y;
  const int pair = blockIdx.y;  // gather modes: (token, slot) of this workgroup
  if (p.idx || p.each_row || (ROUTE && p.route)) {
    xin += (size_t)(p.x_rows == 1 ? pair / p.topk : pair) * p.K;
    yout += (size_t)pair * p.N;
  }
  const char* wb[NMAT];
  const char* sb[NMAT];
  const char* bb[NMAT];
  // Base pointers of this workgroup's matrices.  Gather modes: the expert of its pair.
  // Routing mode: wave 0 repeats the routing of the token, the others wait at one barrier;
  // called once the activation loads are on their way, so that their latency covers it.
  // In the register-resident layout every wave repeats it from logits it requested first
  // (route_raw): no barrier at all.
  constexpr bool XR = kRowsXR<MT, ITERS, NMAT, ROUTE>;
  __shared__ int s_expert;
  uint32_t route_raw[4] = {0, 0, 0, 0};
  auto select_matrices = [&]() {
    size_t ew = 0, eg = 0;
    if (ROUTE && XR && p.route) {
      const int t = pair / p.topk, slot = pair - t * p.topk;
      int my_id;
      float my_p, tot;
      route_topk_regs(route_raw, p.E, p.topk, lane, my_id, my_p, tot);
      if (blockIdx.x == 0 && slot == 0 && wave == 0 && lane < p.topk) {
        p.route_idx[(size_t)t * p.topk + lane] = my_id;
        p.route_scores[(size_t)t * p.topk + lane] = route_score(my_p, tot, p.route_renorm);
      }
      const int e = __builtin_amdgcn_readlane(my_id, slot);
      ew = (size_t)e * p.N * p.wpr;
      eg = (size_t)e * p.N * G;
    } else if (ROUTE && p.route) {
      const int t = pair / p.topk, slot = pair - t * p.topk;
      if (wave == 0) {
        int my_id;
        float my_p, tot;
        route_topk_wave(p.route + (size_t)t * p.E, p.E, p.topk, lane, my_id, my_p, tot);
        if (blockIdx.x == 0 && slot == 0 && lane < p.topk) {
          p.route_idx[(size_t)t * p.topk + lane] = my_id;
          p.route_scores[(size_t)t * p.topk + lane] = route_score(my_p, tot, p.route_renorm);
        }
        if (lane == slot) s_expert = my_id;
      }
      __syncthreads();
      const int e = __builtin_amdgcn_readfirstlane(s_expert);
      ew = (size_t)e * p.N * p.wpr;
      eg = (size_t)e * p.N * G;
    } else if (p.idx) {
      int e = p.idx[pair];
      e = e < 0 ? 0 : (e >= p.E ? p.E - 1 : e);  // memory safety only: the host rejects such ids
      ew = (size_t)e * p.N * p.wpr;
      eg = (size_t)e * p.N * G;
    }
#pragma unroll
    for (int a = 0; a < NMAT; ++a) {
      wb[a] = reinterpret_cast<const char*>(p.w[a] + ew);
      sb[a] = reinterpret_cast<const char*>(p.s[a] + eg);
      bb[a] = reinterpret_cast<const char*>(p.b[a] + eg);
    }
  };
  struct Batch {
    uint4 w[NMAT][UB];
    // (scale, bias) words: a unit pair shares the word of its even unit (low half: even
    // unit, high half: odd unit); an unpaired last unit holds its value in the low half
    uint32_t s[NMAT][UB], b[NMAT][UB];
    // residual of row i of the batch in lane i (single activation row only): requested
    // with the weights, so that the epilogue of a row does not wait for it
    bf16_t res;
  };

  auto issue = [&](Batch& bt, int row_first) {
    if (MT == 1 && NMAT == 1) {
      bt.res = 0;
      if (p.residual && lane < R) bt.res = p.residual[min(row_first + lane, r1 - 1)];
    }
#pragma unroll
    for (int i = 0; i < UB; ++i) {
      // rows past the end of the range re-read its last row (results are dropped)
      const int row = min(row_first + i / ITERS, r1 - 1);
      const int j = i % ITERS;
      const bool paired = !((ITERS & 1) && j == ITERS - 1);
      const size_t wofs = (size_t)row * (ITERS * 1024) + chunk_of<BITS, ITERS>(j, lane) * 16;
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        bt.w[a][i] = *reinterpret_cast<const uint4*>(wb[a] + wofs);
        if (paired) {
          if ((j & 1) == 0) {
            const size_t sofs = ((size_t)row * G + UG * j) * 2 + (lane >> GSHIFT) * 4;
            bt.s[a][i] = *reinterpret_cast<const uint32_t*>(sb[a] + sofs);
            bt.b[a][i] = *reinterpret_cast<const uint32_t*>(bb[a] + sofs);
          }
        } else {
          const size_t sofs = ((size_t)row * G + UG * j + (lane >> GSHIFT)) * 2;
          bt.s[a][i] = *reinterpret_cast<const bf16_t*>(sb[a] + sofs);
          bt.b[a][i] = *reinterpret_cast<const bf16_t*>(bb[a] + sofs);
        }
      }
    }
  };

  // Short rows: the compiler keeps the (loop-invariant) activations in registers.
  // Long rows: that would cost hundreds of VGPRs and the occupancy that hides HBM
  // latency, so the LDS offset is made opaque per batch and x is re-read from LDS.
  constexpr bool X_IN_REGS = ITERS * MT <= 2;
  // XR: a single activation row whose share per lane (ITERS * 64 bytes) fits in
  // registers.  Every wave then holds the whole row across its lanes: no LDS, no
  // barrier, and the fused RMSNorm needs only a wave reduction.
  uint4 xr[XR ? ITERS : 1][4];
  float2 sxr[XR ? ITERS : 1];
  int xlane = lane;
  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));

  auto compute = [&](const Batch& bt, int rb) {
    if (!X_IN_REGS) asm volatile("" : "+v"(xlane));
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = rb + r;
      if (row < r1) {
        float acc[NMAT][MT];
#pragma unroll
        for (int a = 0; a < NMAT; ++a)
#pragma unroll
          for (int m = 0; m < MT; ++m) acc[a][m] = 0.f;
#pragma unroll
        for (int j = 0; j < ITERS; ++j) {
          const int i = r * ITERS + j;
          // d starts at -128*Sx so the offset of the (128+q) trick needs no extra op
          float2 sm[MT];
          float d[NMAT][MT];
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            sm[m] = XR ? sxr[XR ? j : 0] : sx[m * CPR + j * 64 + xlane];
#pragma unroll
            for (int a = 0; a < NMAT; ++a) d[a][m] = -sm[m].x;
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            uint32_t pr[NMAT][4];
#pragma unroll
            for (int a = 0; a < NMAT; ++a)
              unpack_word_r(reinterpret_cast<const uint32_t*>(&bt.w[a][i])[t], kmask, kmagic, pr[a]);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              const uint4 xv = XR ? xr[XR ? j : 0][t] : xs[m * (4 * CPR) + (j * 4 + t) * 64 + xlane];
#pragma unroll
              for (int a = 0; a < NMAT; ++a) {
                d[a][m] = dot2_bf16(pr[a][0], xv.x, d[a][m]);
                d[a][m] = dot2_bf16(pr[a][1], xv.y, d[a][m]);
                d[a][m] = dot2_bf16(pr[a][2], xv.z, d[a][m]);
                d[a][m] = dot2_bf16(pr[a][3], xv.w, d[a][m]);
              }
            }
          }
#pragma unroll
          for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int a = 0; a < NMAT; ++a) {
              // odd unit of a pair: high half of the even unit's word
              const bool hi = (j & 1) && !((ITERS & 1) && j == ITERS - 1);
              const int is = hi ? i - 1 : i;
              const float sc = hi ? bf_hi(bt.s[a][is]) : bf_lo(bt.s[a][is]);
              const float bi = hi ? bf_hi(bt.b[a][is]) : bf_lo(bt.b[a][is]);
              acc[a][m] = fmaf(sc, d[a][m], acc[a][m]);
              acc[a][m] = fmaf(bi, sm[m].y, acc[a][m]);
            }
          }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          float rsum[NMAT];
#pragma unroll
          for (int a = 0; a < NMAT; ++a) rsum[a] = wave_sum_to_lane63(acc[a][m]);
          float resv = 0.f;
          if (MT == 1 && NMAT == 1)
            resv = bf2f((bf16_t)__builtin_amdgcn_readlane((int)bt.res, r));
          if (lane == 63 && m < p.M) {
            const size_t o = (size_t)m * p.N + row;
            float out;
            if (NMAT == 2) {
              const float g = bf2f(f2bf(rsum[0])), up = bf2f(f2bf(rsum[NMAT - 1]));
              out = g / (1.f + __expf(-g)) * up;
            } else {
              out = rsum[0];
              if (p.residual)
                out = bf2f(f2bf(out)) + ((MT == 1 && NMAT == 1) ? resv : bf2f(p.residual[o]));
            }
            yout[o] = f2bf(out);
          }
        }
      }
    }
  };

  // Order of the prologue: activations first (they sit in L2 and are waited for with
  // the weight loads still outstanding), then two weight batches, then the LDS staging.
  Batch buf[NBUF];
  if (XR) {
    if (nrows <= 0) return;  // (wave 0 of a workgroup, which records the routing, always has rows)
    // (no branch, so that the order of the requests below is the order written: launched
    // with expert ids instead of logits, the instance loads one activation in their place)
    if (ROUTE) {
      route_load(p.route ? p.route + (size_t)(pair / p.topk) * p.E : xin, p.route ? p.E : 1, lane, route_raw);
      __builtin_amdgcn_sched_barrier(0);
    }
    uint4 raw[ITERS][4], nwv[ITERS][4];
    // routing instance: without a norm the weight words are loaded from the activations and
    // not used - a branch per load would split the requests over basic blocks, and the wait
    // for the logits must not cover them.  (The plain instance keeps the branch: the extra
    // loads cost the o projection, which has no norm, 0.26 of its 4.65 us.)
    const bf16_t* nw_src = p.norm_w ? p.norm_w : xin;
#pragma unroll
    for (int j = 0; j < ITERS; ++j)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int wi = 4 * chunk_of<BITS, ITERS>(j, lane) + t;
        raw[j][t] = load_word_x<BITS>(xin, wi);
        if (ROUTE || p.norm_w) nwv[j][t] = load_word_x<BITS>(nw_src, wi);
      }
    // (the routing waits for its logits only: the activation loads above go out before that wait)
    if (ROUTE) __builtin_amdgcn_sched_barrier(0);
    select_matrices();
    issue(buf[0], r0);
    if (p.norm_w) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < ITERS; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) ss += sumsq_word<BITS>(raw[j][t]);
      ss = wave_sum_to_lane63(ss);
      ss = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ss), 63));
      const float inv = rsqrtf(ss / (float)p.K + p.eps);
#pragma unroll
      for (int j = 0; j < ITERS; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) norm_word<BITS>(raw[j][t], nwv[j][t], inv);
    }
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      float stored = 0.f, truesum = 0.f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float st_, ts_;
        xr[XR ? j : 0][t] = permute_word<BITS>(raw[j][t], st_, ts_);
        stored += st_;
        truesum += ts_;
      }
      sxr[XR ? j : 0] = make_float2(128.f * stored, truesum);
    }
    // the second batch only now: the raw activations and norm weights are dead, so
    // the register peak stays at what the main loop needs
    asm volatile("" ::: "memory");
#pragma unroll
    for (int b = 1; b < NBUF; ++b)
      if (nrows > b * R) issue(buf[b], r0 + b * R);
  } else {
    XStage<BITS, MT, ITERS> xst;
    stage_x_load<BITS, MT, ITERS>(p, xin, xst);
    select_matrices();
    if (nrows > 0) issue(buf[0], r0);
    __shared__ float s_red[4 * MT];
    stage_x_store<BITS, MT, ITERS>(p, xst, xs, sx, s_red);
    __syncthreads();
    if (nrows <= 0) return;
#pragma unroll
    for (int b = 1; b < NBUF; ++b)
      if (nrows > b * R) issue(buf[b], r0 + b * R);
  }

  // the register buffers in rotation: NBUF - 1 batches are in flight while one is
  // consumed, without copying registers
  int rb = r0;
  if (NBUF == 2) {
    for (;;) {
      compute(buf[0], rb);
      rb += R;
      if (rb >= r1) break;
      if (rb + R < r1) issue(buf[0], rb + R);
      compute(buf[1], rb);
      rb += R;
      if (rb >= r1) break;
      if (rb + R < r1) issue(buf[1], rb + R);
    }
  } else {
    for (;;) {
#pragma unroll
      for (int b = 0; b < NBUF; ++b) {
        compute(buf[b], rb);
        rb += R;
        if (rb >= r1) return;
        if (rb + (NBUF - 1) * R < r1) issue(buf[b], rb + (NBUF - 1) * R);
      }
    }
  }
}


// ---------------------------------------------------------------------------
// Long rows (4 or more KiB-units per row, one activation row, no fused norm): the NW
// waves of a workgroup split K.  Wave w owns unit w of every row of the workgroup's row
// range, so its share of x (16 registers) never leaves the wave: no LDS staging of the
// activations and no barrier before the first product.  The partial sums of a batch of
// rows meet in LDS (one barrier per batch, two partial-sum buffers in alternation) and
// are added in wave order, so the result does not depend on timing.
template <int BITS, int NW>
__global__ __launch_bounds__(64 * NW) void qmv_ksplit_kernel(const QmvParams p) {
  constexpr int GSHIFT = (BITS == 4) ? 1 : 2;
  constexpr int UG = 64 >> GSHIFT;  // scale elements per unit
  constexpr int R = 4;              // rows per batch
  __shared__ float red[2][R][NW];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = p.K >> 6;

  // balanced contiguous row range of this workgroup
  const int base = p.N / (int)gridDim.x, rem = p.N - base * (int)gridDim.x;
  const int r0 = (int)blockIdx.x * base + min((int)blockIdx.x, rem);
  const int r1 = r0 + base + ((int)blockIdx.x < rem ? 1 : 0);
  if (r0 >= r1) return;

  const char* wb = reinterpret_cast<const char*>(p.w[0]) + (size_t)wave * 1024 + lane * 16;
  const char* sb = reinterpret_cast<const char*>(p.s[0]) + ((size_t)wave * UG + (lane >> GSHIFT)) * 2;
  const char* bb = reinterpret_cast<const char*>(p.b[0]) + ((size_t)wave * UG + (lane >> GSHIFT)) * 2;

  struct Batch {
    uint4 w[R];
    bf16_t s[R], b[R];
  };
  auto issue = [&](Batch& bt, int row_first) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int row = min(row_first + i, r1 - 1);  // rows past the end: dropped later
      bt.w[i] = *reinterpret_cast<const uint4*>(wb + (size_t)row * (NW * 1024));
      bt.s[i] = *reinterpret_cast<const bf16_t*>(sb + (size_t)row * G * 2);
      bt.b[i] = *reinterpret_cast<const bf16_t*>(bb + (size_t)row * G * 2);
    }
  };

  // this lane's 16-byte chunk of x (unit `wave`, chunk `lane`), in dot2 register order
  uint4 xr[4];
  float2 sxr;
  {
    uint4 raw[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) raw[t] = load_word_x<BITS>(p.x, 4 * (64 * wave + lane) + t);
    float stored = 0.f, truesum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float st_, ts_;
      xr[t] = permute_word<BITS>(raw[t], st_, ts_);
      stored += st_;
      truesum += ts_;
    }
    sxr = make_float2(128.f * stored, truesum);
  }
  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));

  auto compute = [&](const Batch& bt, int rb, int parity) {
    float acc[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      float d = -sxr.x;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        uint32_t pr[4];
        unpack_word_r(reinterpret_cast<const uint32_t*>(&bt.w[i])[t], kmask, kmagic, pr);
        d = dot2_bf16(pr[0], xr[t].x, d);
        d = dot2_bf16(pr[1], xr[t].y, d);
        d = dot2_bf16(pr[2], xr[t].z, d);
        d = dot2_bf16(pr[3], xr[t].w, d);
      }
      acc[i] = fmaf(bf2f(bt.s[i]), d, bf2f(bt.b[i]) * sxr.y);
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const float t = wave_sum_to_lane63(acc[i]);
      if (lane == 63) red[parity][i][wave] = t;
    }
    __syncthreads();
    if (threadIdx.x < R) {
      const int row = rb + (int)threadIdx.x;
      if (row < r1) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) t += red[parity][threadIdx.x][w];
        if (p.residual) t = bf2f(f2bf(t)) + bf2f(p.residual[row]);
        p.y[row] = f2bf(t);
      }
    }
  };

  Batch ba, bb2;
  issue(ba, r0);
  if (r0 + R < r1) issue(bb2, r0 + R);
  int rb = r0, parity = 0;
  for (;;) {
    compute(ba, rb, parity);
    rb += R;
    parity ^= 1;
    if (rb >= r1) break;
    if (rb + R < r1) issue(ba, rb + R);
    compute(bb2, rb, parity);
    rb += R;
    parity ^= 1;
    if (rb >= r1) break;
    if (rb + R < r1) issue(bb2, rb + R);
  }
}

template <int BITS, int NW>
int launch_ksplit(const QmvParams& p, hipStream_t st) {
  // 16 waves per CU; at least one batch of four rows per workgroup
  const int per_cu = 16 / NW < 1 ? 1 : 16 / NW;
  int grid = 256 * per_cu;
  const int max_grid = (p.N + 3) / 4;
  if (grid > max_grid) grid = max_grid;
  exo_note_variant("qmv_ksplit<%d,%d> grid=%d", BITS, NW, grid);
  qmv_ksplit_kernel<BITS, NW><<<dim3(grid), dim3(64 * NW), 0, st>>>(p);
  return EXO_OK;
}


// ---------------------------------------------------------------------------
// Decode-side SwitchGLU down projection fused with the weighted sum over the token's
// top-k experts and the residual (mx.gather_qmm + the `(y * scores[..., None]).sum(-2)`
// of the MoE block + `h + r`):
//   out[t,n] = bf16( bf16( sum_j bf16( bf16(W[e_j][n,:] . x[t,j,:]) * score[t,j] ) ) + res[t,n] )
// - the same rounding points as exo_gather_qmv followed by exo_moe_combine.
// blockIdx.y = token; a workgroup has one wave per expert slot.  Wave j stages ITS
// activation row x[t,j,:], multiplies kDownRW (1, 2 or 4) sets of 64/LPR rows of expert e_j (all its
// loads in flight from the start) and leaves bf16(bf16(dot) * score_j) in LDS; the first
// wave adds the k contributions in slot order.  The launch is latency-bound, hence the
// many short waves.
struct DownCombineParams {
  const bf16_t* x;       // [T, topk, K]
  const uint32_t* w;     // [E, N, wpr]
  const bf16_t* s;       // [E, N, K/64]
  const bf16_t* b;
  const int32_t* idx;    // [T, topk]
  const bf16_t* scores;  // [T, topk]
  const bf16_t* residual;  // [T, N] or null
  bf16_t* out;           // [T, N]
  int topk, E, N, K, wpr, lpr_log2, iters;
};

constexpr int kDownMaxIters = 4;  // 16-byte chunks per lane and expert row
constexpr int kDownMaxTopk = 8;

// ITERS: 16-byte chunks per lane and row, a template parameter so that no weight load sits
// behind a branch (a value loaded behind one is waited for where the branches join, in front
// of the loads of the following rows)
template <int BITS, int kDownRW, int ITERS>
__global__ __launch_bounds__(64 * kDownMaxTopk) void moe_down_combine_kernel(
    const DownCombineParams p) {
  extern __shared__ uint4 smem[];
  constexpr int GSHIFT = (BITS == 4) ? 1 : 2;
  const int cpr = p.wpr >> 2;
  const int lane = threadIdx.x & 63;
  const int slot = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // one wave per slot
  uint4* xs = smem + (size_t)slot * p.wpr;                                                // [wpr]
  float2* sx = reinterpret_cast<float2*>(smem + (size_t)p.topk * p.wpr) + (size_t)slot * cpr;  // [cpr]
  __shared__ float contrib[kDownMaxTopk][kDownRW * 64];

  const int lpr = 1 << p.lpr_log2;
  const int rpwi = 64 >> p.lpr_log2;
  const int sl = lane & (lpr - 1), sub = lane >> p.lpr_log2;
  const int G = p.K >> 6;
  const int t = blockIdx.y;
  const int row0 = (int)blockIdx.x * (kDownRW * rpwi);

  int e = p.idx[(size_t)t * p.topk + slot];
  e = e < 0 ? 0 : (e >= p.E ? p.E - 1 : e);  // memory safety only: the host rejects such ids
  const float score = bf2f(p.scores[(size_t)t * p.topk + slot]);

  // The first 256 words of this slot's activation row are requested first (they sit in L2 and
  // are waited for with the weight loads still in flight - loads return in order), then every
  // weight load of the wave, then the row is staged: word wi -> xs[(j*4 + w4) * LPR + sl] in
  // dot2 order, per-chunk sums to sx[chunk]; four consecutive lanes hold one chunk
  const bf16_t* xt = p.x + ((size_t)t * p.topk + slot) * p.K;
  uint4 raw0[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) raw0[u] = load_word_x<BITS>(xt, min(u * 64 + lane, p.wpr - 1));
  __builtin_amdgcn_sched_barrier(0);  // (left alone, the compiler moves these behind the weight loads)
  uint4 wv[kDownRW][ITERS];
  // (scale, bias): one 32-bit register each - held as 16-bit values the compiler packs two of
  // them into a register and waits for each pair right behind its loads, so that a row's loads
  // went out only once the previous row's scales had arrived
  uint32_t sv[kDownRW][ITERS], bv[kDownRW][ITERS];
#pragma unroll
  for (int i = 0; i < kDownRW; ++i) {
    const int row = min(row0 + i * rpwi + sub, p.N - 1);  // rows past N: not stored
    const size_t r = (size_t)e * p.N + row;
    const uint32_t* wp = p.w + r * p.wpr + sl * 4;
    const bf16_t* sp = p.s + r * G + (sl >> GSHIFT);
    const bf16_t* bp = p.b + r * G + (sl >> GSHIFT);
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
      wv[i][j] = *reinterpret_cast<const uint4*>(wp + (size_t)j * lpr * 4);
      sv[i][j] = sp[j * (lpr >> GSHIFT)];
      bv[i][j] = bp[j * (lpr >> GSHIFT)];
    }
  }

  {
    for (int base = 0; base < p.wpr; base += 64 * 4) {
      uint4 raw[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        raw[u] = base == 0 ? raw0[u] : load_word_x<BITS>(xt, min(base + u * 64 + lane, p.wpr - 1));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int wi = base + u * 64 + lane;
        const int c = wi >> 2, w4 = wi & 3;
        const int j = c >> p.lpr_log2, csl = c & (lpr - 1);
        float stored, truesum;
        const uint4 o = permute_word<BITS>(raw[u], stored, truesum);
        stored += __shfl_xor(stored, 1, 64);
        truesum += __shfl_xor(truesum, 1, 64);
        stored += __shfl_xor(stored, 2, 64);
        truesum += __shfl_xor(truesum, 2, 64);
        if (wi < p.wpr) {
          xs[(((j << 2) + w4) << p.lpr_log2) + csl] = o;
          if (w4 == 0) sx[c] = make_float2(128.f * stored, truesum);
        }
      }
    }
  }
  // xs and sx of a slot belong to its wave alone: its own LDS writes are complete before its
  // reads, no workgroup barrier
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();

  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));
#pragma unroll
  for (int i = 0; i < kDownRW; ++i) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < ITERS; ++j) {
        const float2 sm = sx[(j << p.lpr_log2) + sl];
        float d = -sm.x;
#pragma unroll
        for (int w4 = 0; w4 < 4; ++w4) {
          uint32_t pr[4];
          unpack_word_r(reinterpret_cast<const uint32_t*>(&wv[i][j])[w4], kmask, kmagic, pr);
          const uint4 xv = xs[(((j << 2) + w4) << p.lpr_log2) + sl];
          d = dot2_bf16(pr[0], xv.x, d);
          d = dot2_bf16(pr[1], xv.y, d);
          d = dot2_bf16(pr[2], xv.z, d);
          d = dot2_bf16(pr[3], xv.w, d);
        }
        acc = fmaf(bf_lo(sv[i][j]), d, acc);
        acc = fmaf(bf_lo(bv[i][j]), sm.y, acc);
      }
    acc = group_sum(acc, lpr);
    if (sl == 0) contrib[slot][i * rpwi + sub] = bf2f(f2bf(bf2f(f2bf(acc)) * score));
  }
  __syncthreads();

  if (slot == 0) {
    for (int r = lane; r < kDownRW * rpwi; r += 64) {  // r = i * rpwi + sub
      const int row = row0 + r;
      if (row < p.N) {
        float total = 0.f;
        for (int j = 0; j < p.topk; ++j) total += contrib[j][r];
        float o = bf2f(f2bf(total));
        if (p.residual) o += bf2f(p.residual[(size_t)t * p.N + row]);
        p.out[(size_t)t * p.N + row] = f2bf(o);
      }
    }
  }
}

struct Plan {
  int lpr_log2, iters, slots, spw, grid, ragged;
  size_t lds;
};

bool make_plan(int N, int K, int bits, int mt, Plan* pl) {
  const int wpr = K * bits / 32;
  const int cpr = wpr / 4;  // 16-byte chunks per row
  if (cpr * 4 != wpr || cpr == 0) return false;
  const int lmin = bits == 4 ? 1 : 2;  // a lane group must span whole 64-groups
  int l = 6;
  while (l > lmin && (cpr % (1 << l)) != 0) --l;
  if ((cpr % (1 << l)) != 0) return false;
  const int rpwi = 64 >> l;
  if ((int64_t)N * wpr >= (int64_t)1 << 31) return false;
  pl->lpr_log2 = l;
  pl->iters = cpr >> l;
  pl->slots = (N + rpwi - 1) / rpwi;
  pl->ragged = (N % rpwi) != 0;
  pl->lds = (size_t)mt * ((size_t)wpr * 16 + (size_t)cpr * 8);
  const int wg_per_cu = pl->lds <= 40 * 1024 ? 2 : 1;
  int max_waves = 256 * wg_per_cu * kWaves;
  // at least ~4 units of work per wave so the x staging is amortised
  int min_spw = (4 + pl->iters - 1) / pl->iters;
  int spw = (pl->slots + max_waves - 1) / max_waves;
  if (spw < min_spw) spw = min_spw;
  pl->spw = spw;
  pl->grid = (pl->slots + spw * kWaves - 1) / (spw * kWaves);
  return true;
}

#ifndef EXO_QMV_GATHER_WGS  // tuning builds: workgroups of a gather launch in all
#define EXO_QMV_GATHER_WGS 0
#endif
template <int BITS, int MT, int NMAT, int ITERS>
int launch_rows(const QmvParams& p, const Plan& pl, int pairs, hipStream_t st) {
  constexpr bool CAN_ROUTE = MT == 1 && NMAT == 2;
  // (the routing instance also takes the launches with given expert ids: one arithmetic for
  // both, so routing inside the launch changes no bit of the result)
  const bool route = CAN_ROUTE && (p.route || p.idx);
  auto kern = route ? qmv_rows_kernel<BITS, MT, NMAT, ITERS, CAN_ROUTE>
                    : qmv_rows_kernel<BITS, MT, NMAT, ITERS, false>;
  static bool attr_set[2] = {false, false};
  bool& attr_done = attr_set[route ? 1 : 0];
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  // waves get contiguous, balanced row ranges; 4 workgroups per CU (LDS permitting) and
  // at least one full batch of rows per wave
  int per_cu = pl.lds <= 36 * 1024 ? 4 : (pl.lds <= 72 * 1024 ? 2 : 1);
  // up to 8 per CU for the (gate, up) pair, so that a 14336-row pair runs as 1792
  // workgroups of exactly two rows per wave (15.8 -> 15.1 us), and for one-unit rows
  // (128256x2048: 35.4 -> 33.4 us)
  // (the rules marked 'single' were measured with one activation row and one launch per
  // matrix; the two-row tile was slower with them)
  const bool single = MT == 1 && pairs == 1;
  if (single && per_cu == 4 && (NMAT == 2 || ITERS == 1)) per_cu = 8;
  int grid = 256 * per_cu;
  // (gather mode, several (token, slot) pairs: half of that - the launch is latency-bound
  // and twice as many workgroups finish sooner; a quarter was slower again)
  int min_rows = (8 + ITERS * NMAT - 1) / (ITERS * NMAT);
  // (8 units per row: two rows per wave, 4096x8192 8-bit 11.9 -> 10.8 us)
  if (single && ITERS * NMAT == 8) min_rows = 2;
  if (pairs > 1 && min_rows > 1) min_rows /= 2;
  // short matrices: fewer rows per wave while that grid would stay under 160 workgroups
  // (2048x2048: 64 -> 256 workgroups, 4.0 -> 2.9 us; 2048x4096: 3.5 -> 3.2 us)
  while (min_rows > 1 && p.N / (min_rows * kWaves) < 160) min_rows /= 2;
  int max_grid = (p.N + min_rows * kWaves - 1) / (min_rows * kWaves);
  if (grid > max_grid) grid = max_grid;
  if (pairs > 1 && !p.each_row) {  // (rows of one small matrix keep the single-row grid)
    // gather mode (one launch covers `pairs` (token, slot) products, blockIdx.y each): every
    // wave normalises its token's activations first, so two rows per wave at least, and a
    // grid that is resident at once (three workgroups per CU at this kernel's registers).
    // Measured in the whole decode step, workgroups in all -> tokens/s: 768x2048 4-bit
    // (gate, up), 8 pairs: 256 624, 384 628, 512 643, 768 627, 1536 (one row per wave) 551;
    // 16 pairs: 512 966, 768 973, 1024 944, 1536 957; 32 pairs: 256 1289, 512 1385, 768 1384,
    // 1536 1400; 64 pairs: 512 2050, 768 2074, 1536 2064; 128 pairs: 512 2814, 768 2956,
    // 1536 2891; 1536x4096, 8 pairs: 512 480, 768 482, 1024 480, 1536 471.
    const int wgs = EXO_QMV_GATHER_WGS > 0 ? EXO_QMV_GATHER_WGS : ((pairs <= 8 && ITERS == 1) ? 512 : 768);
    const int share = wgs / pairs < 1 ? 1 : wgs / pairs;
    const int two_rows = (p.N + 2 * kWaves - 1) / (2 * kWaves);
    grid = two_rows < share ? two_rows : share;
  }
  if (single) {
    // The same number of workgroups on each of the 256 CUs: a grid between two multiples
    // of 256 leaves some CUs with one workgroup more than the others for the whole launch
    // (6144x4096 with fused norm: 384 workgroups 7.5 us, 320: 8.2, 512: 6.9, 256: 6.2;
    // 5120x2048: 160 workgroups 4.4 us, 256: 3.8).
    if (grid >= 160 && grid < 256 && p.N >= 256 * kWaves) grid = 256;
    if (grid > 256) {
      grid -= grid % 256;
      // ... and, where one exists in the upper half, a multiple that gives every wave the
      // same number of rows (9216x4096 8-bit: 1024 workgroups 12.4 us, 768: 11.7)
      for (int g = grid; g >= 256 && 2 * g > grid; g -= 256)
        if (p.N % (g * kWaves) == 0) {
          grid = g;
          break;
        }
    }
  }
#ifdef EXO_QMV_GRID_OVERRIDE  // tuning builds: {N, grid} pairs for launches of one activation row
  if (single) {
    static const int ov[][2] = {EXO_QMV_GRID_OVERRIDE};
    for (auto& o : ov)
      if (o[0] == p.N * (NMAT == 2 ? -1 : 1) && o[1] > 0) grid = o[1];
  }
#endif
  if (grid < 1) grid = 1;
  exo_note_variant("qmv_rows<%d,%d,%d,%d,%s> grid=%dx%d", BITS, MT, NMAT, ITERS, route ? "true" : "false",
                   grid, pairs);
  const bool in_regs = route ? kRowsXR<MT, ITERS, NMAT, CAN_ROUTE> : kRowsXR<MT, ITERS, NMAT>;
  kern<<<dim3(grid, pairs), dim3(kThreads), in_regs ? 0 : pl.lds, st>>>(p);
  return EXO_OK;
}

template <int BITS, int MT, int NMAT>
int launch_one(const QmvParams& p, const Plan& pl, int pairs, hipStream_t st) {
  if (MT == 1 && NMAT == 1 && pl.lpr_log2 == 6 && !pl.ragged && !p.norm_w && !p.idx && !p.each_row &&
      !p.route && p.M == 1) {
    // measured against the row kernel: ahead at 14 units per row (8-bit, K = 14336: 17.0
    // vs 18.3 us for 4096 rows), level at 7 and 8, behind at 4
    if (pl.iters == 14) return launch_ksplit<BITS, 14>(p, st);
  }
  if (MT <= 2 && pl.lpr_log2 == 6 && !pl.ragged) {
    constexpr int MTR = MT <= 2 ? MT : 1;  // (no instantiation for larger tiles)
    switch (pl.iters) {
      case 1: return launch_rows<BITS, MTR, NMAT, 1>(p, pl, pairs, st);
      case 2: return launch_rows<BITS, MTR, NMAT, 2>(p, pl, pairs, st);
      case 4: return launch_rows<BITS, MTR, NMAT, 4>(p, pl, pairs, st);
      case 7: return launch_rows<BITS, MTR, NMAT, 7>(p, pl, pairs, st);
      case 8: return launch_rows<BITS, MTR, NMAT, 8>(p, pl, pairs, st);
      case 14: return launch_rows<BITS, MTR, NMAT, 14>(p, pl, pairs, st);
      default: break;
    }
  }
  constexpr bool CAN_ROUTE = MT == 1 && NMAT == 2;
  const bool route = CAN_ROUTE && p.route;
  auto kern = route ? qmv_kernel<BITS, MT, NMAT, CAN_ROUTE> : qmv_kernel<BITS, MT, NMAT, false>;
  static bool attr_set[2] = {false, false};
  bool& attr_done = attr_set[route ? 1 : 0];
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  exo_note_variant("qmv_generic<%d,%d,%d,%s> grid=%dx%d", BITS, MT, NMAT, route ? "true" : "false",
                   pl.grid, pairs);
  kern<<<dim3(pl.grid, pairs), dim3(kThreads), pl.lds, st>>>(p);
  return EXO_OK;
}

struct Gather {
  const int32_t* idx = nullptr;
  int pairs = 1, E = 0, topk = 1, x_rows = 1;
  bool each_row = false;  // no indices: `pairs` rows of x against the one matrix
  // no indices either: the kernel routes from these logits and writes indices and scores
  const bf16_t* route = nullptr;
  int32_t* route_idx = nullptr;
  bf16_t* route_scores = nullptr;
  int route_renorm = 0;
};

template <int NMAT>
int qmv_dispatch(const bf16_t* x, const uint32_t* const* w, const bf16_t* const* s,
                 const bf16_t* const* b, const bf16_t* residual, bf16_t* y, int M, int N,
                 int K, int bits, hipStream_t st, const char* name,
                 const Gather& ga = Gather(), const bf16_t* norm_w = nullptr, float eps = 0.f) {
  // M is processed in tiles of at most 4 rows (bounded by LDS: the whole K of every
  // row of the tile is resident); each tile re-streams W.
  int m0 = 0;
  while (m0 < M) {
    int mt = (M - m0 >= 4) ? 4 : ((M - m0 >= 2) ? 2 : 1);
    if (ga.idx || ga.each_row || ga.route) mt = 1;
    Plan pl;
    for (;;) {
      if (!make_plan(N, K, bits, mt, &pl)) {
        exo_set_error("%s: unsupported shape N=%d K=%d bits=%d", name, N, K, bits);
        return EXO_ERR_ARG;
      }
      if (pl.lds <= 150 * 1024 || mt == 1) break;
      mt >>= 1;
    }
    if (pl.lds > 150 * 1024) {
      exo_set_error("%s: K=%d too large for the LDS-resident activation tile", name, K);
      return EXO_ERR_ARG;
    }
    QmvParams p;
    p.x = x + (size_t)m0 * K;
    for (int a = 0; a < 2; ++a) {
      p.w[a] = w[a < NMAT ? a : 0];
      p.s[a] = s[a < NMAT ? a : 0];
      p.b[a] = b[a < NMAT ? a : 0];
    }
    p.residual = residual ? residual + (size_t)m0 * N : nullptr;
    p.y = y + (size_t)m0 * N;
    p.M = (M - m0 < mt) ? (M - m0) : mt;
    p.N = N;
    p.K = K;
    p.wpr = K * bits / 32;
    p.lpr_log2 = pl.lpr_log2;
    p.iters = pl.iters;
    p.slots = pl.slots;
    p.spw = pl.spw;
    p.ragged = pl.ragged;
    p.idx = ga.idx;
    p.E = ga.E;
    p.topk = ga.topk;
    p.x_rows = ga.x_rows;
    p.each_row = ga.each_row ? 1 : 0;
    p.route = ga.route;
    p.route_idx = ga.route_idx;
    p.route_scores = ga.route_scores;
    p.route_renorm = ga.route_renorm;
    p.norm_w = norm_w;
    p.eps = eps;
    const int pairs = (ga.idx || ga.each_row || ga.route) ? ga.pairs : 1;
    int rc;
    if (bits == 4) {
      rc = mt == 4   ? launch_one<4, 4, NMAT>(p, pl, pairs, st)
           : mt == 2 ? launch_one<4, 2, NMAT>(p, pl, pairs, st)
                     : launch_one<4, 1, NMAT>(p, pl, pairs, st);
    } else {
      rc = mt == 4   ? launch_one<8, 4, NMAT>(p, pl, pairs, st)
           : mt == 2 ? launch_one<8, 2, NMAT>(p, pl, pairs, st)
                     : launch_one<8, 1, NMAT>(p, pl, pairs, st);
    }
    if (rc != EXO_OK) return rc;
    m0 += mt;
  }
  return EXO_OK;
}

int check_gather(const char* name, int T, int topk, int x_rows, int E) {
  EXO_REQUIRE(T >= 0 && topk > 0 && E > 0, "%s: bad T=%d topk=%d E=%d", name, T, topk, E);
  EXO_REQUIRE(x_rows == 1 || x_rows == topk, "%s: x_rows=%d must be 1 or topk=%d", name, x_rows,
              topk);
  EXO_REQUIRE((int64_t)T * topk <= 65535, "%s: T*topk=%lld exceeds the decode-sized limit 65535",
              name, (long long)T * topk);
  return EXO_OK;
}

int check_common(const char* name, int M, int N, int K, int bits, int group_size) {
  EXO_REQUIRE(bits == 4 || bits == 8, "%s: bits must be 4 or 8, got %d", name, bits);
  EXO_REQUIRE(group_size == 64, "%s: group_size must be 64, got %d", name, group_size);
  EXO_REQUIRE(M >= 0 && M <= 16, "%s: M=%d outside [0,16]; use exo_qmm", name, M);
  EXO_REQUIRE(N > 0 && K > 0 && K % 64 == 0, "%s: bad shape N=%d K=%d (K %% 64 != 0?)", name,
              N, K);
  return EXO_OK;
}

// Exactly two rows over a short reduction run faster on the dot2 kernel with a two-row
// activation tile (1.3-1.4 x the one-row time) than on the matrix-core GEMV (about 2 x);
// from three rows on, and for long rows whose activations no longer stay in registers,
// the matrix cores win.  (Rows of more than 4 KiB of codes - 8-bit beyond K = 4096 - would take
// the two-row tile's instances that spill registers.)
inline bool two_rows_on_dot2(int M, int K, int bits) { return M == 2 && (int64_t)K * bits <= 8192 * 4; }

// A matrix this small (a MoE router: 128 x 2048 4-bit = 128 KiB) under 2...16 rows is a
// latency-bound launch: one set of single-row workgroups per row (blockIdx.y), each reading
// the matrix from L2, finishes in the time of the one-row launch (3.5 us), where the
// matrix-core tile with its staging of all rows and its K merge takes 6.8 us at four rows.
#ifndef EXO_EACH_ROW_MAX_BYTES
#define EXO_EACH_ROW_MAX_BYTES (1 << 20)
#endif
constexpr int64_t kEachRowMaxBytes = EXO_EACH_ROW_MAX_BYTES;

}  // namespace

extern "C" int exo_qmv(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M,
                       int N, int K, int bits, int group_size, exo_stream_t stream) {
  return exo_norm_qmv(x, nullptr, 0.f, w, scales, biases, residual, y, M, N, K, bits, group_size,
                      stream);
}

// Activation rows that take the 4x4x4 matrix-core kernel (qmv_quad.hip) where its shape
// rules admit the matrix.  Measured on the Llama-3.1-8B layer matrices (4-bit), us per launch,
// this kernel | the kernels below: two rows 19.7 | 21.8 (gate/up pair), 11.5 | 16.0 (down),
// 8.2 | 9.4 (qkv), 5.4 | 7.3 (o); four rows 21.7 | 22.6, 14.4 | 16.3, 9.9 | 10.9, 6.6 | 8.5;
// one row 19.1 | 17.1, 11.1 | 10.0 and from five rows on (two operand sets) it is behind too.
#ifndef EXO_QMV_QUAD_MIN_M
#define EXO_QMV_QUAD_MIN_M 2
#endif
#ifndef EXO_QMV_QUAD_MAX_M
#define EXO_QMV_QUAD_MAX_M 4
#endif
// From this many activation rows the 16x16x32 matrix-core kernel (qmv_w16.hip) takes the
// matrices its shape rules admit, in tiles of 16 rows.
#ifndef EXO_QMV_W16_MIN_M
#define EXO_QMV_W16_MIN_M 5
#endif

static int norm_qmv_impl(const uint16_t* x, const uint16_t* norm_weight, float eps,
                         const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                         const uint16_t* residual, uint16_t* y, void* workspace, int M, int N,
                         int K, int bits, int group_size, exo_stream_t stream) {
  int rc = check_common("exo_qmv", M, N, K, bits, group_size);
  if (rc) return rc;
  EXO_REQUIRE(x && w && scales && biases && y, "exo_qmv: null pointer");
  if (M == 0) return EXO_OK;
  if (M >= 2 && !residual && (int64_t)N * K * bits / 8 <= kEachRowMaxBytes) {
    const uint32_t* ws[1] = {w};
    const bf16_t* ss[1] = {scales};
    const bf16_t* bs[1] = {biases};
    Gather ga;
    ga.each_row = true;
    ga.pairs = M;
    rc = qmv_dispatch<1>(x, ws, ss, bs, nullptr, y, 1, N, K, bits, (hipStream_t)stream, "exo_qmv",
                         ga, norm_weight, eps);
    if (rc) return rc;
    EXO_CHECK_LAUNCH("exo_qmv");
    return EXO_OK;
  }
  if (M >= EXO_QMV_QUAD_MIN_M && M <= EXO_QMV_QUAD_MAX_M &&
      exo_qmv_quad_ok(M, N, K, bits, norm_weight != nullptr)) {
    rc = exo_qmv_quad_launch(x, norm_weight, eps, w, scales, biases, nullptr, nullptr, nullptr,
                             residual, y, M, N, K, bits, (hipStream_t)stream);
    if (rc) return rc;
    EXO_CHECK_LAUNCH("exo_qmv");
    return EXO_OK;
  }
  if (M >= EXO_QMV_W16_MIN_M &&
      exo_qmv_w16_ok(M < 16 ? M : 16, N, K, bits, norm_weight != nullptr, false, workspace != nullptr)) {
    for (int m0 = 0; m0 < M; m0 += 16) {
      const int mt = (M - m0 < 16) ? (M - m0) : 16;
      rc = exo_qmv_w16_launch(x + (size_t)m0 * K, norm_weight, eps, w, scales, biases, nullptr,
                              nullptr, nullptr, residual ? residual + (size_t)m0 * N : nullptr,
                              y + (size_t)m0 * N, mt, N, K, workspace, (hipStream_t)stream);
      if (rc) return rc;
    }
    EXO_CHECK_LAUNCH("exo_qmv");
    return EXO_OK;
  }
  // two or more rows: the matrix-core GEMV streams W once per tile of up to 16 rows
  // (with a workspace; without one a tile is as many rows as the LDS holds whole)
  int cap = (M >= 2 && !two_rows_on_dot2(M, K, bits)) ? exo_qmv_mfma_max_rows(K, bits) : 0;
  if (cap > 0 && workspace) cap = 16;
  if (cap >= 2) {
    int m0 = 0;
    while (M - m0 >= 2) {
      const int mt = (M - m0 < cap) ? (M - m0) : cap;
      rc = exo_qmv_mfma_launch(x + (size_t)m0 * K, norm_weight, eps, w, scales, biases, nullptr,
                               nullptr, nullptr,
                               residual ? residual + (size_t)m0 * N : nullptr, y + (size_t)m0 * N,
                               mt, N, K, bits, workspace, (hipStream_t)stream);
      if (rc) return rc;
      m0 += mt;
    }
    EXO_CHECK_LAUNCH("exo_qmv");
    if (m0 == M) return EXO_OK;
    x += (size_t)m0 * K;  // a single left-over row takes the dot2 kernel below
    y += (size_t)m0 * N;
    if (residual) residual += (size_t)m0 * N;
    M -= m0;
  }
  const uint32_t* ws[1] = {w};
  const bf16_t* ss[1] = {scales};
  const bf16_t* bs[1] = {biases};
  rc = qmv_dispatch<1>(x, ws, ss, bs, residual, y, M, N, K, bits, (hipStream_t)stream,
                       "exo_qmv", Gather(), norm_weight, eps);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_qmv");
  return EXO_OK;
}

extern "C" int exo_norm_qmv(const uint16_t* x, const uint16_t* norm_weight, float eps,
                            const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* residual, uint16_t* y, int M, int N, int K,
                            int bits, int group_size, exo_stream_t stream) {
  return norm_qmv_impl(x, norm_weight, eps, w, scales, biases, residual, y, nullptr, M, N, K,
                       bits, group_size, stream);
}

extern "C" int64_t exo_qmv_workspace(int N) {
  return N > 0 ? (int64_t)exo_qmv_mfma_workspace(N) : 0;
}

extern "C" int exo_norm_qmv_ws(const uint16_t* x, const uint16_t* norm_weight, float eps,
                               const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, const uint16_t* residual, uint16_t* y,
                               void* workspace, int64_t workspace_bytes, int M, int N, int K,
                               int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(!workspace || (workspace_bytes >= exo_qmv_workspace(N) &&
                             ((uintptr_t)workspace & 255) == 0),
              "exo_norm_qmv_ws: workspace of %lld bytes, need %lld (256-byte aligned)",
              (long long)workspace_bytes, (long long)exo_qmv_workspace(N));
  return norm_qmv_impl(x, norm_weight, eps, w, scales, biases, residual, y, workspace, M, N, K,
                       bits, group_size, stream);
}

extern "C" int exo_qmv_swiglu(const uint16_t* x, const uint32_t* wg, const uint16_t* sg,
                              const uint16_t* bg, const uint32_t* wu, const uint16_t* su,
                              const uint16_t* bu, uint16_t* y, int M, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
  return exo_norm_qmv_swiglu(x, nullptr, 0.f, wg, sg, bg, wu, su, bu, y, M, N, K, bits,
                             group_size, stream);
}

extern "C" int exo_norm_qmv_swiglu(const uint16_t* x, const uint16_t* norm_weight, float eps,
                                   const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                                   const uint32_t* wu, const uint16_t* su, const uint16_t* bu,
                                   uint16_t* y, int M, int N, int K, int bits, int group_size,
                                   exo_stream_t stream) {
  return exo_norm_qmv_swiglu_ws(x, norm_weight, eps, wg, sg, bg, wu, su, bu, y, nullptr, 0, M, N,
                                K, bits, group_size, stream);
}

extern "C" int exo_norm_qmv_swiglu_ws(const uint16_t* x, const uint16_t* norm_weight, float eps,
                                      const uint32_t* wg, const uint16_t* sg,
                                      const uint16_t* bg, const uint32_t* wu,
                                      const uint16_t* su, const uint16_t* bu, uint16_t* y,
                                      void* workspace, int64_t workspace_bytes, int M, int N,
                                      int K, int bits, int group_size, exo_stream_t stream) {
  int rc = check_common("exo_qmv_swiglu", M, N, K, bits, group_size);
  if (rc) return rc;
  EXO_REQUIRE(x && wg && sg && bg && wu && su && bu && y, "exo_qmv_swiglu: null pointer");
  EXO_REQUIRE(!workspace || (workspace_bytes >= exo_qmv_workspace(2 * N) &&
                             ((uintptr_t)workspace & 255) == 0),
              "exo_norm_qmv_swiglu_ws: workspace of %lld bytes, need %lld (256-byte aligned)",
              (long long)workspace_bytes, (long long)exo_qmv_workspace(2 * N));
  if (M == 0) return EXO_OK;
  if (M >= EXO_QMV_QUAD_MIN_M && M <= EXO_QMV_QUAD_MAX_M &&
      exo_qmv_quad_ok(M, N, K, bits, norm_weight != nullptr)) {
    rc = exo_qmv_quad_launch(x, norm_weight, eps, wg, sg, bg, wu, su, bu, nullptr, y, M, N, K, bits,
                             (hipStream_t)stream);
    if (rc) return rc;
    EXO_CHECK_LAUNCH("exo_qmv_swiglu");
    return EXO_OK;
  }
  if (M >= EXO_QMV_W16_MIN_M && exo_qmv_w16_ok(M < 16 ? M : 16, N, K, bits, norm_weight != nullptr, true, false)) {
    for (int m0 = 0; m0 < M; m0 += 16) {
      const int mt = (M - m0 < 16) ? (M - m0) : 16;
      rc = exo_qmv_w16_launch(x + (size_t)m0 * K, norm_weight, eps, wg, sg, bg, wu, su, bu, nullptr,
                              y + (size_t)m0 * N, mt, N, K, nullptr, (hipStream_t)stream);
      if (rc) return rc;
    }
    EXO_CHECK_LAUNCH("exo_qmv_swiglu");
    return EXO_OK;
  }
  // two or more rows: both projections in one matrix-core launch per tile of up to 16 rows
  if (workspace && M >= 2 && !two_rows_on_dot2(M, K, bits) && exo_qmv_mfma_max_rows(K, bits) > 0) {
    int m0 = 0;
    while (M - m0 >= 2) {
      const int mt = (M - m0 < 16) ? (M - m0) : 16;
      rc = exo_qmv_mfma_launch(x + (size_t)m0 * K, norm_weight, eps, wg, sg, bg, wu, su, bu,
                               nullptr, y + (size_t)m0 * N, mt, N, K, bits, workspace,
                               (hipStream_t)stream);
      if (rc) return rc;
      m0 += mt;
    }
    EXO_CHECK_LAUNCH("exo_qmv_swiglu");
    if (m0 == M) return EXO_OK;
    x += (size_t)m0 * K;  // a single left-over row takes the dot2 kernel below
    y += (size_t)m0 * N;
    M -= m0;
  }
  const uint32_t* ws[2] = {wg, wu};
  const bf16_t* ss[2] = {sg, su};
  const bf16_t* bs[2] = {bg, bu};
  rc = qmv_dispatch<2>(x, ws, ss, bs, nullptr, y, M, N, K, bits, (hipStream_t)stream,
                       "exo_qmv_swiglu", Gather(), norm_weight, eps);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_qmv_swiglu");
  return EXO_OK;
}

extern "C" int exo_gather_qmv(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const int32_t* idx, uint16_t* y, int T,
                              int topk, int x_rows, int E, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
  int rc = check_common("exo_gather_qmv", 1, N, K, bits, group_size);
  if (rc) return rc;
  rc = check_gather("exo_gather_qmv", T, topk, x_rows, E);
  if (rc) return rc;
  EXO_REQUIRE(x && w && scales && biases && idx && y, "exo_gather_qmv: null pointer");
  if (T == 0) return EXO_OK;
  const uint32_t* ws[1] = {w};
  const bf16_t* ss[1] = {scales};
  const bf16_t* bs[1] = {biases};
  Gather ga;
  ga.idx = idx;
  ga.pairs = T * topk;
  ga.E = E;
  ga.topk = topk;
  ga.x_rows = x_rows;
  rc = qmv_dispatch<1>(x, ws, ss, bs, nullptr, y, 1, N, K, bits, (hipStream_t)stream,
                       "exo_gather_qmv", ga);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_gather_qmv");
  return EXO_OK;
}

extern "C" int exo_norm_gather_qmv_swiglu(const uint16_t* x, const uint16_t* norm_weight,
                                          float eps, const uint32_t* wg, const uint16_t* sg,
                                          const uint16_t* bg, const uint32_t* wu,
                                          const uint16_t* su, const uint16_t* bu,
                                          const int32_t* idx, uint16_t* y, int T, int topk, int E,
                                          int N, int K, int bits, int group_size,
                                          exo_stream_t stream) {
  int rc = check_common("exo_gather_qmv_swiglu", 1, N, K, bits, group_size);
  if (rc) return rc;
  rc = check_gather("exo_gather_qmv_swiglu", T, topk, 1, E);
  if (rc) return rc;
  EXO_REQUIRE(x && wg && sg && bg && wu && su && bu && idx && y,
              "exo_gather_qmv_swiglu: null pointer");
  if (T == 0) return EXO_OK;
  const uint32_t* ws[2] = {wg, wu};
  const bf16_t* ss[2] = {sg, su};
  const bf16_t* bs[2] = {bg, bu};
  Gather ga;
  ga.idx = idx;
  ga.pairs = T * topk;
  ga.E = E;
  ga.topk = topk;
  ga.x_rows = 1;
  rc = qmv_dispatch<2>(x, ws, ss, bs, nullptr, y, 1, N, K, bits, (hipStream_t)stream,
                       "exo_gather_qmv_swiglu", ga, norm_weight, eps);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_gather_qmv_swiglu");
  return EXO_OK;
}

extern "C" int exo_gather_qmv_swiglu(const uint16_t* x, const uint32_t* wg, const uint16_t* sg,
                                     const uint16_t* bg, const uint32_t* wu, const uint16_t* su,
                                     const uint16_t* bu, const int32_t* idx, uint16_t* y, int T,
                                     int topk, int E, int N, int K, int bits, int group_size,
                                     exo_stream_t stream) {
  return exo_norm_gather_qmv_swiglu(x, nullptr, 0.f, wg, sg, bg, wu, su, bu, idx, y, T, topk, E,
                                    N, K, bits, group_size, stream);
}

extern "C" int exo_norm_route_gather_qmv_swiglu(
    const uint16_t* x, const uint16_t* norm_weight, float eps, const uint16_t* router_logits,
    int renorm, int32_t* idx_out, uint16_t* scores_out, const uint32_t* wg, const uint16_t* sg,
    const uint16_t* bg, const uint32_t* wu, const uint16_t* su, const uint16_t* bu, uint16_t* y,
    int T, int topk, int E, int N, int K, int bits, int group_size, exo_stream_t stream) {
  int rc = check_common("exo_norm_route_gather_qmv_swiglu", 1, N, K, bits, group_size);
  if (rc) return rc;
  rc = check_gather("exo_norm_route_gather_qmv_swiglu", T, topk, 1, E);
  if (rc) return rc;
  EXO_REQUIRE(x && router_logits && idx_out && scores_out && wg && sg && bg && wu && su && bu && y,
              "exo_norm_route_gather_qmv_swiglu: null pointer");
  EXO_REQUIRE(E <= 256 && topk <= 16 && topk <= E,
              "exo_norm_route_gather_qmv_swiglu: need E<=256, topk<=min(16,E); got E=%d topk=%d", E,
              topk);
  if (T == 0) return EXO_OK;
  const uint32_t* ws[2] = {wg, wu};
  const bf16_t* ss[2] = {sg, su};
  const bf16_t* bs[2] = {bg, bu};
  Gather ga;
  ga.pairs = T * topk;
  ga.E = E;
  ga.topk = topk;
  ga.x_rows = 1;
  ga.route = router_logits;
  ga.route_idx = idx_out;
  ga.route_scores = scores_out;
  ga.route_renorm = renorm;
  rc = qmv_dispatch<2>(x, ws, ss, bs, nullptr, y, 1, N, K, bits, (hipStream_t)stream,
                       "exo_norm_route_gather_qmv_swiglu", ga, norm_weight, eps);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_norm_route_gather_qmv_swiglu");
  return EXO_OK;
}

extern "C" int exo_gather_qmv_combine(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                                      const uint16_t* biases, const int32_t* idx,
                                      const uint16_t* scores, const uint16_t* residual,
                                      uint16_t* out, uint16_t* scratch, int T, int topk, int E,
                                      int N, int K, int bits, int group_size,
                                      exo_stream_t stream) {
  int rc = check_common("exo_gather_qmv_combine", 1, N, K, bits, group_size);
  if (rc) return rc;
  rc = check_gather("exo_gather_qmv_combine", T, topk, topk, E);
  if (rc) return rc;
  EXO_REQUIRE(x && w && scales && biases && idx && scores && out,
              "exo_gather_qmv_combine: null pointer");
  Plan pl;
  const bool fused = make_plan(N, K, bits, 1, &pl) && pl.iters <= kDownMaxIters &&
                     topk <= kDownMaxTopk && T <= 65535;
  if (!fused) {
    EXO_REQUIRE(scratch, "exo_gather_qmv_combine: topk=%d K=%d needs the scratch buffer", topk, K);
    rc = exo_gather_qmv(x, w, scales, biases, idx, scratch, T, topk, topk, E, N, K, bits,
                        group_size, stream);
    if (rc) return rc;
    return exo_moe_combine(scratch, scores, residual, out, T, topk, N, stream);
  }
  DownCombineParams p;
  p.x = x;
  p.w = w;
  p.s = scales;
  p.b = biases;
  p.idx = idx;
  p.scores = scores;
  p.residual = residual;
  p.out = out;
  p.topk = topk;
  p.E = E;
  p.N = N;
  p.K = K;
  p.wpr = K * bits / 32;
  p.lpr_log2 = pl.lpr_log2;
  p.iters = pl.iters;
  const int rpwi = 64 >> pl.lpr_log2;
  // as many row sets per wave (4, 2 or 1) as leave 512 workgroups per token: every wave stages
  // its slot's activation row, which more rows amortise, but the launch is latency-bound and
  // wants a wide grid (Qwen3-30B, 2048 outputs in sets of 8: one set, 256 workgroups, 482 ->
  // 509 tok/s over two; Qwen3-235B, 4096 outputs in sets of 2, whole step: one set 457 tok/s,
  // two 478, four - 512 workgroups - 490, eight 481)
#ifdef EXO_DOWN_RW
  const int rw = EXO_DOWN_RW;
#else
  const int rw = exo_ceil_div(N, 4 * rpwi) >= 512 ? 4 : (exo_ceil_div(N, 2 * rpwi) >= 512 ? 2 : 1);
#endif
  const dim3 grid(exo_ceil_div(N, rw * rpwi), T);
  const size_t lds = (size_t)topk * ((size_t)p.wpr * 16 + (size_t)(p.wpr / 4) * 8);
  exo_note_variant("moe_down_combine<%d,%d,%d> grid=%dx%d", bits, rw, pl.iters, (int)grid.x, (int)grid.y);
#define EXO_DOWN_CASE(B_, RW_, IT_)                                                       \
  if (bits == B_ && rw == RW_ && pl.iters == IT_)                                          \
    moe_down_combine_kernel<B_, RW_, IT_><<<grid, 64 * topk, lds, (hipStream_t)stream>>>(p);
#define EXO_DOWN_ITERS(B_, RW_) \
  EXO_DOWN_CASE(B_, RW_, 1) EXO_DOWN_CASE(B_, RW_, 2) EXO_DOWN_CASE(B_, RW_, 3) EXO_DOWN_CASE(B_, RW_, 4)
  EXO_DOWN_ITERS(4, 1)
  EXO_DOWN_ITERS(4, 2)
  EXO_DOWN_ITERS(8, 1)
  EXO_DOWN_ITERS(8, 2)
  EXO_DOWN_ITERS(4, 4)
  EXO_DOWN_ITERS(8, 4)
#undef EXO_DOWN_ITERS
#undef EXO_DOWN_CASE
  EXO_CHECK_LAUNCH("exo_gather_qmv_combine");
  return EXO_OK;
}
