// Fused dequant-GEMV for 2..16 activation rows (batched decode) on the matrix cores.
//
// y[M,N] = x[M,K] @ dq(W)[N,K]^T with M <= 16.  Still HBM-bound (W is streamed once),
// but the multiply-accumulate moves from the VALU to v_mfma_f32_32x32x16_bf16, so the
// cost per streamed KiB does not grow with M:
//  * a wave owns 32 weight rows; lane (r = lane%32, kq = lane/32) loads 16 B = 4 packed
//    words of row r, the lane pair covering 8 consecutive words (one 4-bit group, half
//    an 8-bit group) per load instruction;
//  * word t of every lane is unpacked to (128+nibble) bf16 pairs (v_and_or_b32, exact)
//    and is the B operand of MFMA step t; the A operand is the matching slice of the
//    activation rows, pre-permuted in LDS (rows >= M are don't-care lanes);
//  * D[m][r] of a whole group is scaled on the way out:
//      acc += s[r,g] * (D - 128*Sx[m,g]) + b[r,g] * Sx[m,g]
//    with the group sums Sx of the activations precomputed in LDS;
//  * the four waves of a workgroup split K, so that 32 rows already occupy a whole CU;
//    partial sums meet in LDS once per 32-row block.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "qmv_internal.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kStepsPerSuper = 8;  // 16-byte loads in flight per lane and buffer

struct MfmaParams {
  const bf16_t* x;         // [M,K]
  const uint32_t* w;       // [N, wpr]
  const bf16_t* s;         // [N, K/64]
  const bf16_t* b;
  const bf16_t* residual;  // [M,N] or null
  bf16_t* y;               // [M,N]
  const bf16_t* norm_w;    // [K] or null (fused RMSNorm of x)
  float eps;
  int M, N, K, wpr, G;
  int gw;  // groups per wave (multiple of the groups per super-step)
};

template <int BITS>
__device__ __forceinline__ uint4 load_word_x(const bf16_t* base, int wi) {
  if (BITS == 4) return *reinterpret_cast<const uint4*>(base + (size_t)wi * 8);
  const uint2 v = *reinterpret_cast<const uint2*>(base + (size_t)wi * 4);
  return make_uint4(v.x, v.y, 0, 0);
}
template <int BITS>
__device__ __forceinline__ float sumsq_word(const uint4& v) {
  float s = bf_lo(v.x) * bf_lo(v.x) + bf_hi(v.x) * bf_hi(v.x) + bf_lo(v.y) * bf_lo(v.y) +
            bf_hi(v.y) * bf_hi(v.y);
  if (BITS == 4)
    s += bf_lo(v.z) * bf_lo(v.z) + bf_hi(v.z) * bf_hi(v.z) + bf_lo(v.w) * bf_lo(v.w) +
         bf_hi(v.w) * bf_hi(v.w);
  return s;
}
template <int BITS>
__device__ __forceinline__ void norm_word(uint4& xv, const uint4& wv, float inv) {
  xv.x = pack_bf2(bf_lo(xv.x) * inv * bf_lo(wv.x), bf_hi(xv.x) * inv * bf_hi(wv.x));
  xv.y = pack_bf2(bf_lo(xv.y) * inv * bf_lo(wv.y), bf_hi(xv.y) * inv * bf_hi(wv.y));
  if (BITS == 4) {
    xv.z = pack_bf2(bf_lo(xv.z) * inv * bf_lo(wv.z), bf_hi(xv.z) * inv * bf_hi(wv.z));
    xv.w = pack_bf2(bf_lo(xv.w) * inv * bf_lo(wv.w), bf_hi(xv.w) * inv * bf_hi(wv.w));
  }
}
// activations of one packed word in the register order of the unpacked nibble pairs
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
  } else {  // byte codes as two nibbles against (x, 16x)
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

// MR = D registers in use: 4 covers M <= 8, 8 covers M <= 16.
template <int BITS, int MR>
__global__ __launch_bounds__(kThreads) void qmv_mfma_kernel(const MfmaParams p) {
  constexpr int WPG = 64 * BITS / 32;          // words per group: 8 / 16
  constexpr int SPG = WPG / 8;                  // load steps per group: 1 / 2
  constexpr int SSG = kStepsPerSuper / SPG;     // groups per super-step: 8 / 4
  extern __shared__ uint4 smem[];
  const int MT = p.M;
  uint4* xs = smem;                                            // [wpr/8][4][2][MT]
  float2* sxs = reinterpret_cast<float2*>(smem + (size_t)p.wpr * MT);  // [G][MT]
  float* red = reinterpret_cast<float*>(sxs + (size_t)p.G * MT);        // [4][MR][64]
  __shared__ float s_red[kWaves * 16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, kq = lane >> 5;

  // ---- stage the activations: optional RMSNorm, permute, group sums
  {
    float inv[16];
#pragma unroll
    for (int m = 0; m < 16; ++m) inv[m] = 1.f;
    if (p.norm_w) {
      float ss[16];
#pragma unroll
      for (int m = 0; m < 16; ++m) ss[m] = 0.f;
      for (int wi = tid; wi < p.wpr; wi += kThreads)
#pragma unroll
        for (int m = 0; m < 16; ++m)
          if (m < MT) ss[m] += sumsq_word<BITS>(load_word_x<BITS>(p.x + (size_t)m * p.K, wi));
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        if (m < MT) {
          const float t = wave_sum(ss[m]);
          if (lane == 0) s_red[wave * 16 + m] = t;
        }
      }
      __syncthreads();
#pragma unroll
      for (int m = 0; m < 16; ++m)
        if (m < MT)
          inv[m] = rsqrtf((s_red[m] + s_red[16 + m] + s_red[32 + m] + s_red[48 + m]) / (float)p.K +
                          p.eps);
    }
    for (int wi = tid; wi < p.wpr; wi += kThreads) {
      const int step = wi >> 3, q2 = (wi >> 2) & 1, t = wi & 3;
      const int dst = ((step * 4 + t) * 2 + q2) * MT;
      uint4 nw = make_uint4(0, 0, 0, 0);
      if (p.norm_w) nw = load_word_x<BITS>(p.norm_w, wi);
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        if (m < MT) {
          uint4 xv = load_word_x<BITS>(p.x + (size_t)m * p.K, wi);
          if (p.norm_w) norm_word<BITS>(xv, nw, inv[m]);
          float stored, truesum;
          xs[dst + m] = permute_word<BITS>(xv, stored, truesum);
          // sum over the WPG consecutive words (threads) of the group
#pragma unroll
          for (int o = 1; o < WPG; o <<= 1) {
            stored += __shfl_xor(stored, o, 64);
            truesum += __shfl_xor(truesum, o, 64);
          }
          if ((wi & (WPG - 1)) == 0) sxs[(wi / WPG) * MT + m] = make_float2(128.f * stored, truesum);
        }
      }
    }
  }
  __syncthreads();

  // D register q of this lane is activation row a(q); rows >= M are don't-care
  const int Rg = kq;
  int a_of[MR];
#pragma unroll
  for (int q = 0; q < MR; ++q) a_of[q] = min(8 * (q >> 2) + 4 * Rg + (q & 3), MT - 1);
  const int a_lane = min(r, MT - 1);  // A-operand row of this lane

  const int NB = (p.N + 31) >> 5;
  const int g_begin = wave * p.gw;                 // this wave's share of K
  const int g_end = min(p.G, g_begin + p.gw);
  const int n_super = p.gw / SSG;                  // same for every wave of the block

  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));

  struct Buf {
    uint4 w[kStepsPerSuper];
    uint4 s, b;  // SSG scales / biases (8-bit: only .x, .y used)
  };
  // item -> (row block, super-step); loads clamp to the last valid row / group
  auto issue = [&](Buf& bf, int blk, int ss) {
    const int row = min(blk * 32 + r, p.N - 1);
    const int g0 = min(g_begin + ss * SSG, p.G - SSG < 0 ? 0 : p.G - SSG);
    const uint32_t* wp = p.w + (size_t)row * p.wpr + (size_t)g0 * WPG + kq * 4;
#pragma unroll
    for (int i = 0; i < kStepsPerSuper; ++i) {
      // steps past the row end re-read its last step (never consumed)
      const int off = min(i * 8, p.wpr - g0 * WPG - 8);
      bf.w[i] = *reinterpret_cast<const uint4*>(wp + off);
    }
    const bf16_t* sp = p.s + (size_t)row * p.G + g0;
    const bf16_t* bp = p.b + (size_t)row * p.G + g0;
    if (SSG == 8) {
      bf.s = *reinterpret_cast<const uint4*>(sp);
      bf.b = *reinterpret_cast<const uint4*>(bp);
    } else {
      const uint2 sv = *reinterpret_cast<const uint2*>(sp);
      const uint2 bv = *reinterpret_cast<const uint2*>(bp);
      bf.s = make_uint4(sv.x, sv.y, 0, 0);
      bf.b = make_uint4(bv.x, bv.y, 0, 0);
    }
  };

  float acc[MR];
#pragma unroll
  for (int q = 0; q < MR; ++q) acc[q] = 0.f;

  auto consume = [&](const Buf& bf, int ss) {
    const int g0 = min(g_begin + ss * SSG, p.G - SSG < 0 ? 0 : p.G - SSG);
    const int g_first = g_begin + ss * SSG;  // groups [g_first, g_first+SSG) are due
    const uint32_t* sw = reinterpret_cast<const uint32_t*>(&bf.s);
    const uint32_t* bw = reinterpret_cast<const uint32_t*>(&bf.b);
#pragma unroll
    for (int gi = 0; gi < SSG; ++gi) {
      const int g = g0 + gi;
      // a clamped super-step overlaps groups already done: consume only the due ones
      if (g >= g_first && g < g_end) {
        floatx16 d;
#pragma unroll
        for (int e = 0; e < 16; ++e) d[e] = 0.f;
#pragma unroll
        for (int sp = 0; sp < SPG; ++sp) {
          const int i = gi * SPG + sp;
          const int step = g * SPG + sp;
          const uint32_t* wd = reinterpret_cast<const uint32_t*>(&bf.w[i]);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            uint4 bq;
            bq.x = (wd[t] & kmask) | kmagic;
            bq.y = ((wd[t] >> 4) & kmask) | kmagic;
            bq.z = ((wd[t] >> 8) & kmask) | kmagic;
            bq.w = ((wd[t] >> 12) & kmask) | kmagic;
            const uint4 av = xs[((step * 4 + t) * 2 + kq) * MT + a_lane];
            d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                        __builtin_bit_cast(bf16x8_t, bq), d, 0, 0, 0);
          }
        }
        const uint32_t sraw = sw[gi >> 1], braw = bw[gi >> 1];
        const float sc = (gi & 1) ? bf_hi(sraw) : bf_lo(sraw);
        const float bi = (gi & 1) ? bf_hi(braw) : bf_lo(braw);
#pragma unroll
        for (int q = 0; q < MR; ++q) {
          const float2 sm = sxs[g * MT + a_of[q]];
          acc[q] = fmaf(sc, d[q] - sm.x, acc[q]);
          acc[q] = fmaf(bi, sm.y, acc[q]);
        }
      }
    }
  };

  // flat sequence of (row block, super-step) items with two buffers in ping-pong
  const int my_blocks = (NB - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const int n_items = my_blocks * n_super;
  if (n_items <= 0) return;
  auto blk_of = [&](int it) { return (int)blockIdx.x + (it / n_super) * (int)gridDim.x; };

  auto finish_block = [&](int blk) {
    __syncthreads();  // wave 0 has finished reading the previous block's partials
#pragma unroll
    for (int q = 0; q < MR; ++q) {
      red[(wave * MR + q) * 64 + lane] = acc[q];
      acc[q] = 0.f;
    }
    __syncthreads();
    if (wave == 0) {
      const int row = blk * 32 + r;
#pragma unroll
      for (int q = 0; q < MR; ++q) {
        const int m = 8 * (q >> 2) + 4 * Rg + (q & 3);
        float v = red[q * 64 + lane] + red[(MR + q) * 64 + lane] + red[(2 * MR + q) * 64 + lane] +
                  red[(3 * MR + q) * 64 + lane];
        if (m < p.M && row < p.N) {
          const size_t o = (size_t)m * p.N + row;
          if (p.residual) v = bf2f(f2bf(v)) + bf2f(p.residual[o]);
          p.y[o] = f2bf(v);
        }
      }
    }
  };

  Buf b0, b1;
  issue(b0, blk_of(0), 0);
  int it = 0;
  for (;;) {
    if (it + 1 < n_items) issue(b1, blk_of(it + 1), (it + 1) % n_super);
    consume(b0, it % n_super);
    if (it % n_super == n_super - 1) finish_block(blk_of(it));
    if (++it >= n_items) break;
    if (it + 1 < n_items) issue(b0, blk_of(it + 1), (it + 1) % n_super);
    consume(b1, it % n_super);
    if (it % n_super == n_super - 1) finish_block(blk_of(it));
    if (++it >= n_items) break;
  }
}

template <int BITS, int MR>
int launch(const MfmaParams& p, size_t lds, hipStream_t st) {
  auto kern = qmv_mfma_kernel<BITS, MR>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 1024);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  const int NB = (p.N + 31) / 32;
  const int per_cu = lds <= 72 * 1024 ? 2 : 1;
  int grid = NB < 256 * per_cu ? NB : 256 * per_cu;
  kern<<<dim3(grid), dim3(kThreads), lds, st>>>(p);
  return EXO_OK;
}

}  // namespace

// rows of x that fit one launch (LDS holds their whole K), 0 if not even one
int exo_qmv_mfma_max_rows(int K, int bits) {
  if (K % (bits == 4 ? 512 : 256) != 0) return 0;
  const size_t per_row = (size_t)K * bits / 32 * 16 + (size_t)(K / 64) * 8;
  const size_t budget = 150 * 1024 - kWaves * 8 * 64 * 4;
  size_t m = budget / per_row;
  return m > 16 ? 16 : (int)m;
}

// y[M,N] for 2 <= M <= exo_qmv_mfma_max_rows(K, bits)
int exo_qmv_mfma_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const bf16_t* residual, bf16_t* y,
                        int M, int N, int K, int bits, hipStream_t st) {
  MfmaParams p;
  p.x = x;
  p.w = w;
  p.s = s;
  p.b = b;
  p.residual = residual;
  p.y = y;
  p.norm_w = norm_w;
  p.eps = eps;
  p.M = M;
  p.N = N;
  p.K = K;
  p.wpr = K * bits / 32;
  p.G = K / 64;
  const int ssg = bits == 4 ? 8 : 4;
  int gw = (p.G + kWaves - 1) / kWaves;
  gw = (gw + ssg - 1) / ssg * ssg;
  p.gw = gw;
  const int MR = M <= 8 ? 4 : 8;
  const size_t lds = (size_t)p.wpr * 16 * M + (size_t)p.G * 8 * M + (size_t)kWaves * MR * 64 * 4;
  if (bits == 4)
    return MR == 4 ? launch<4, 4>(p, lds, st) : launch<4, 8>(p, lds, st);
  return MR == 4 ? launch<8, 4>(p, lds, st) : launch<8, 8>(p, lds, st);
}
