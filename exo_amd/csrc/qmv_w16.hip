// Fused dequant-GEMV for up to 16 activation rows on v_mfma_f32_16x16x32_bf16 (4-bit codes).
//
// The instruction multiplies A[16][32] by B[32][16]: lane l holds A[l%16][8*(l/16) .. +8],
// B[8*(l/16) .. +8][l%16], and D[4*(l/16) + r][l%16] in register r.  Here A is the activations
// (row = activation row m), B a block of 16 weight rows (column = weight row j), so a lane's
// four results belong to ONE weight row: scale and bias of a quantisation group are one value
// per lane.
//  * a wave instruction loads 16 rows x 64 contiguous bytes (128 codes = two groups of a row):
//    lane (lane/4, lane%4) takes 16-byte chunk lane%4 of row lane/4, so that the four lanes of
//    a quad read 64 contiguous bytes.  A product wants 8 codes (one word) of row j in lane
//    (j, kg): the words change lanes through the LDS crossbar (ds_bpermute_b32, no LDS memory)
//    when the block is consumed - two permutes and one select per product, because the four
//    K slots of a product must come from one group (= two chunks x four words).
//  * a wave owns SL such 64-byte slices of every row block of its workgroup; the matching
//    activations stay in registers in operand order for the whole launch.  The waves of a
//    workgroup together cover K; their partial sums meet in LDS once per phase of row blocks.
//  * codes become (128+nibble) bf16 pairs with one v_and_or_b32 each (exact).  Per group:
//      acc += s * D + (b - 128 s) * Sx        D = sum (128+q) x,  Sx = sum x   (float32)
//  * DEPTH row blocks of weights are in flight per wave (register buffers in rotation); every
//    refill is issued whether or not a block is left (past the end it is out of the buffer's
//    range and moves no data), so that the number of loads in flight at each wait is a constant.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "qmv_internal.h"

namespace {

#ifndef EXO_W16_PAIR8
#define EXO_W16_PAIR8 1  // the (gate, up) pair in blocks of 8 rows of both matrices where that fits
#endif
#ifndef EXO_W16_ABL
#define EXO_W16_ABL 0  // timing-only ablations (wrong results): 1 no products, 2 no lane permutation, 4 no group epilogue, 8 no unpacking
#endif

struct W16Params {
  const bf16_t* x;       // [M, K]
  const bf16_t* norm_w;  // [K] or null: fused RMSNorm of x
  float eps;
  const uint32_t* w[2];  // packed [N, K/8]   ([1]: the up matrix of a (gate, up) pair)
  const bf16_t* s[2];    // [N, K/64]
  const bf16_t* b[2];
  const bf16_t* residual;  // [M, N] or null
  bf16_t* y;               // [M, N]
  int M, N, K;
  int row_bytes;  // K / 2
  int G;          // K / 64
  int blocks;     // N / 16
  int ph;         // row blocks per workgroup at most (LDS holds their partial sums)
  int lw;         // lanes of a wave that hold results: 16 * ceil(M / 4)
  int red_bytes;  // LDS bytes of the partial sums; the staged scales and biases follow
  // K split over `kparts` workgroups per group of row blocks (long rows: the activations of
  // a whole row would not fit the registers): workgroup i takes part i % kparts, Gp groups
  // of every row; float32 partial results meet in `part`, the last workgroup of a group to
  // arrive adds them in part order
  int kparts, Gp;
  float* part;    // [kparts][M][N]
  int* counters;  // [block groups], zero between launches
};

__device__ __forceinline__ void st_dev(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_dev(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float sumsq8(const uint4& v) {
  return bf_lo(v.x) * bf_lo(v.x) + bf_hi(v.x) * bf_hi(v.x) + bf_lo(v.y) * bf_lo(v.y) +
         bf_hi(v.y) * bf_hi(v.y) + bf_lo(v.z) * bf_lo(v.z) + bf_hi(v.z) * bf_hi(v.z) +
         bf_lo(v.w) * bf_lo(v.w) + bf_hi(v.w) * bf_hi(v.w);
}
__device__ __forceinline__ void norm8(uint4& xv, const uint4& wv, float inv) {
  xv.x = pack_bf2(bf_lo(xv.x) * inv * bf_lo(wv.x), bf_hi(xv.x) * inv * bf_hi(wv.x));
  xv.y = pack_bf2(bf_lo(xv.y) * inv * bf_lo(wv.y), bf_hi(xv.y) * inv * bf_hi(wv.y));
  xv.z = pack_bf2(bf_lo(xv.z) * inv * bf_lo(wv.z), bf_hi(xv.z) * inv * bf_hi(wv.z));
  xv.w = pack_bf2(bf_lo(xv.w) * inv * bf_lo(wv.w), bf_hi(xv.w) * inv * bf_hi(wv.w));
}
// the 8 activations of one packed word in the order of the unpacked nibble pairs:
// (x0,x4),(x1,x5),(x2,x6),(x3,x7); `sum` = their sum
__device__ __forceinline__ uint4 pair_order(const uint4& xv, float& sum) {
  uint4 o;
  o.x = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);
  sum = (bf_lo(o.x) + bf_hi(o.x)) + (bf_lo(o.y) + bf_hi(o.y)) + (bf_lo(o.z) + bf_hi(o.z)) +
        (bf_lo(o.w) + bf_hi(o.w));
  return o;
}

template <int SL>
struct SbWord;  // (scale or bias) of the 2*SL groups of a wave's slices: SL words of two bf16
template <>
struct SbWord<1> {
  uint32_t v[1];
  __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, int vo, int so) {
    v[0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(r, vo, so, 0);
  }
};
template <>
struct SbWord<2> {
  uint32_t v[2];
  __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t r, int vo, int so) {
    const auto t = __builtin_amdgcn_raw_buffer_load_b64(r, vo, so, 0);
    const uint2 u = __builtin_bit_cast(uint2, t);
    v[0] = u.x;
    v[1] = u.y;
  }
};

// NMAT matrices (2: the (gate, up) pair with SwiGLU), SL 64-byte slices of K per wave, DEPTH
// row blocks in flight per wave.
// NORM: fused RMSNorm of the activations.
// SBLDS: the scales and biases of ALL the workgroup's rows are staged in LDS in front of the
// loop, with whole-line loads (one 16-byte chunk per thread and array).  Loaded per block by
// the lanes that need them - 8 bytes each out of 16 different lines per instruction, every
// line touched again by each of the 16 waves - they cost 4.5 of the 24 us of the 14336x4096
// pair (measured with the loads taken out).  Needs K a multiple of 512 and LDS for them beside
// the partial sums (up to 8 activation rows).
// KSPLIT: K split over several workgroups (single matrix, no fused norm).  An instance of its
// own: compiled into the others, the hand-over code costs them 0.5 us per launch untaken.
// P8 (the (gate, up) pair as ONE operand block: NMAT == 1, staged scales): the 16 columns of a
// product are 8 rows of the gate matrix and the same 8 rows of the up matrix.  A workgroup's
// share is then counted in blocks of 8 rows of both - 14336 rows are 1792 blocks, seven for each
// of 256 workgroups, where blocks of 16 rows leave half the workgroups with four and half with
// three.  Per-lane addresses (two matrices in one load instruction), clamped to the
// workgroup's last block instead of range-checked.
template <int NMAT, int SL, int DEPTH, bool NORM, bool SBLDS, bool KSPLIT = false, bool P8 = false>
__global__ __launch_bounds__(1024) void qmv_w16_kernel(const W16Params p) {
  static_assert(!P8 || (NMAT == 1 && SBLDS && !KSPLIT), "pair-of-8 mode: one operand block, staged scales");
  constexpr bool KSPLIT_OK = KSPLIT && NMAT == 1 && !NORM;
  constexpr int RPB = P8 ? 8 : 16;     // rows of a matrix per block
  constexpr int NS = P8 ? 2 : NMAT;    // matrices with scales to stage
  extern __shared__ float red[];  // [ph][NMAT][nw][4][lw]
  __shared__ float s_part[16][16];
  __shared__ int s_last;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = blockDim.x >> 6;
  const int j = lane & 15, kg = lane >> 4;  // operand layout: weight row (or activation row), K slot
  const int lr = lane >> 2, lc = lane & 3;  // load layout: row of the block, chunk of the slice

  // contiguous, balanced range of row blocks of this workgroup
  const int kparts = KSPLIT_OK ? p.kparts : 1;
  const int kpart = (int)blockIdx.x % kparts, bgroup = (int)blockIdx.x / kparts;
  const int ngroups = (int)gridDim.x / kparts;
  const int qbase = p.blocks / ngroups, qrem = p.blocks - qbase * ngroups;
  const int q0 = bgroup * qbase + min(bgroup, qrem);
  const int nq = qbase + (bgroup < qrem ? 1 : 0);
  if (nq <= 0) return;
  const int g_first = kpart * p.Gp;  // first quantisation group of this workgroup's part of K

  struct Buf {
    uint4 w[NMAT][SL];
    SbWord<SL> s[NMAT], b[NMAT];
  };
  // buffer resources over exactly this workgroup's rows (a refill past them returns zeros)
  __amdgpu_buffer_rsrc_t rw[NMAT], rs[NS], rb[NS];
#pragma unroll
  for (int a = 0; a < NMAT; ++a)
    rw[a] = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(p.w[a]) + (size_t)q0 * RPB * p.row_bytes), 0,
        nq * RPB * p.row_bytes, 0x00020000);
#pragma unroll
  for (int a = 0; a < NS; ++a) {
    rs[a] = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.s[a] + (size_t)q0 * RPB * p.G), 0,
                                              nq * RPB * p.G * 2, 0x00020000);
    rb[a] = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.b[a] + (size_t)q0 * RPB * p.G), 0,
                                              nq * RPB * p.G * 2, 0x00020000);
  }
  const int wofs = lr * p.row_bytes + g_first * 32 + wave * (SL * 64) + lc * 16;
  // P8: this lane's row of its matrix (lanes of block rows 0..7: gate, 8..15: up), first block
  const uint32_t* const w_mine = (P8 && lr >= 8) ? p.w[1] : p.w[0];
  const char* const w_lane = reinterpret_cast<const char*>(w_mine) +
                             (size_t)(q0 * RPB + (lr & (RPB - 1))) * p.row_bytes + wave * (SL * 64) + lc * 16;
  const int sofs = (j * p.G + g_first + wave * (SL * 2)) * 2;  // this lane's weight row, the wave's groups
  // PIN (the issues in front of the loop): the loads leave in program order - weights, then
  // scales and biases, buffer by buffer, as in the loop.  The compiler counts the loads still
  // in flight at each wait; where the order in front of the loop differs from the order in the
  // loop it has to assume the worse of the two and waits for a whole buffer too many.
  auto issue_w = [&](Buf& bf, int q, bool pin) {  // q: row block of this workgroup's range (past it: zeros)
    const int wq = q * 16 * p.row_bytes;  // uniform: scalar offset
    if (pin) __builtin_amdgcn_sched_barrier(0);
    if constexpr (P8) {
      const char* src = w_lane + (size_t)min(q, nq - 1) * (8 * p.row_bytes);
#pragma unroll
      for (int sl = 0; sl < SL; ++sl) bf.w[0][sl] = *reinterpret_cast<const uint4*>(src + sl * 64);
    } else {
#pragma unroll
      for (int sl = 0; sl < SL; ++sl)
#pragma unroll
        for (int a = 0; a < NMAT; ++a)
          bf.w[a][sl] = __builtin_bit_cast(
              uint4, __builtin_amdgcn_raw_buffer_load_b128(rw[a], wofs + sl * 64, wq, 0));
    }
    if (pin) __builtin_amdgcn_sched_barrier(0);
  };
  auto issue_sb = [&](Buf& bf, int q, bool pin) {
    const int sq = q * 16 * p.G * 2;
#if (EXO_W16_ABL & 64)  // timing only: no scale / bias loads
#pragma unroll
    for (int a = 0; a < NMAT; ++a)
#pragma unroll
      for (int sl = 0; sl < SL; ++sl) bf.s[a].v[sl] = bf.b[a].v[sl] = 0x3c003c00u + sq;
#else
#pragma unroll
    for (int a = 0; a < NMAT; ++a) {
      bf.s[a].load(rs[a], sofs, sq);
      bf.b[a].load(rb[a], sofs, sq);
    }
#endif
    if (pin) __builtin_amdgcn_sched_barrier(0);
  };
  auto issue = [&](Buf& bf, int q, bool pin) {
    issue_w(bf, q, pin);
    if (!SBLDS) issue_sb(bf, q, pin);
  };
  // staged scales / biases: array (matrix a, scale|bias) x local row x (G + 4) bf16 (rows
  // padded by 8 bytes: the 16 rows a wave reads at once then sit in different banks)
  char* const sb_lds = reinterpret_cast<char*>(red) + p.red_bytes;
  const int sb_row = p.Gp * 2 + 8, sb_arr = p.ph * RPB * sb_row;
  char* const nw_lds = sb_lds + (SBLDS ? NS * 2 * sb_arr : 0);  // the norm weights, K bf16

  // ---- activations: lane (m = j, kg) holds, for product (sl, g, h), the 8 elements of row m
  // that the weight word of lane (., kg) covers: word 4*(2g + kg%2) + 2h + kg/2 of the slice
  uint4 xa[SL][2][2];
  float sx[SL][2][4];  // group sums of the activation rows 4*kg + r of this lane's results
  Buf buf[DEPTH];
  {
    // range-checked loads: lanes of rows m >= M get zeros
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.x), 0, p.M * p.K * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16_t*>(NORM ? p.norm_w : p.x), 0, p.K * 2, 0x00020000);
    const int lane_word = 4 * (kg & 1) + (kg >> 1);  // + 8g + 2h: the word of product (g, h)
    const int xofs = (j * p.K + lane_word * 8) * 2, nofs = lane_word * 16;
    // bytes of activations in front of the wave's slices
    const int wave_ofs = g_first * 128 + wave * (SL * 256);
    // staging: chunk tid of each array (past the workgroup's rows: out of range, no traffic)
    // (the norm weights too: chunk tid; every lane reads its words back after the barrier -
    // loaded per lane they are 16 times the bytes, one copy per activation row, and their
    // registers are live across the barrier beside everything else)
    uint4 nstg = make_uint4(0, 0, 0, 0);
    if (NORM) nstg = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rn, tid * 16, 0, 0));
    uint4 stg[NS][2];
    if (SBLDS) {
      // thread -> (local row, 16-byte chunk of the row's part); past the rows: out of range
      const int cpr = p.Gp >> 3, row = tid / cpr, col = tid - row * cpr;
      const int so = row < nq * RPB ? (row * p.G + g_first) * 2 + col * 16 : 0x7ffffff0;
#pragma unroll
      for (int a = 0; a < NS; ++a) {
        stg[a][0] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs[a], so, 0, 0));
        stg[a][1] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rb[a], so, 0, 0));
      }
    }
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int wo = (sl * 16 + 8 * g + 2 * h) * 16;
          xa[sl][g][h] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rx, xofs + wo, wave_ofs, 0));
        }
    // the activation loads go first (they are waited for first), then the weights - with the
    // fused norm only the first block: beside the raw words and the staging registers every
    // buffer at once does not fit, and a spilled value is reloaded behind a wait for ALL
    // outstanding loads
#pragma unroll
    for (int d = 0; d < (NORM ? 1 : DEPTH); ++d) issue(buf[d], d, true);
    auto stage_sb = [&](const uint4 (&v)[NS][2]) {
      const int cpr = p.Gp >> 3;  // 16-byte chunks per row
      const int row = tid / cpr, col = tid - row * cpr;
      if (row < nq * RPB) {
#pragma unroll
        for (int a = 0; a < NS; ++a)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            uint2* dst = reinterpret_cast<uint2*>(sb_lds + (a * 2 + t) * sb_arr + row * sb_row + col * 16);
            dst[0] = make_uint2(v[a][t].x, v[a][t].y);
            dst[1] = make_uint2(v[a][t].z, v[a][t].w);
          }
      }
    };
    if (SBLDS && !NORM) {
      stage_sb(stg);
      __syncthreads();
    }
    if (NORM) {
      // rows past the waves of this workgroup count as zero in the fixed-order sum below
      if (wave + nw < 16 && lane < 16) {
        for (int w2 = wave + nw; w2 < 16; w2 += nw) s_part[w2][lane] = 0.f;
      }
    }
    if (NORM) {  // fused RMSNorm: every wave holds its slices of every row
      float ss = 0.f;
#pragma unroll
      for (int sl = 0; sl < SL; ++sl)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int h = 0; h < 2; ++h) ss += sumsq8(xa[sl][g][h]);
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      if (lane < 16) s_part[wave][lane] = ss;
      if (SBLDS) stage_sb(stg);
      if (tid * 16 < p.K * 2) *reinterpret_cast<uint4*>(nw_lds + tid * 16) = nstg;
      __syncthreads();
      // the waves' sums of row m in wave order: lane (m, kg) adds waves kg, kg+4, kg+8, kg+12
      float t = (s_part[kg][j] + s_part[kg + 4][j]) + (s_part[kg + 8][j] + s_part[kg + 12][j]);
      t += __shfl_xor(t, 16, 64);
      t += __shfl_xor(t, 32, 64);
      const float inv = rsqrtf(t / (float)p.K + p.eps);
#pragma unroll
      for (int sl = 0; sl < SL; ++sl)
#pragma unroll
        for (int g = 0; g < 2; ++g)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int wo = (sl * 16 + 8 * g + 2 * h) * 16;
            norm8(xa[sl][g][h], *reinterpret_cast<const uint4*>(nw_lds + wave_ofs + nofs + wo), inv);
          }
    }
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        float gs = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float s1;
          xa[sl][g][h] = pair_order(xa[sl][g][h], s1);
          gs += s1;
        }
        gs += __shfl_xor(gs, 16, 64);
        gs += __shfl_xor(gs, 32, 64);  // every lane (m, .) holds the group sum of row m
#pragma unroll
        for (int r = 0; r < 4; ++r) sx[sl][g][r] = __shfl(gs, 4 * kg + r, 64);
      }
    if (NORM) {
#pragma unroll
      for (int d = 1; d < DEPTH; ++d) issue(buf[d], d, true);
    }
  }

  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));
  // The lane's coordinates once more, from the hardware lane count: values derived from the
  // first copy would have to live through the register-tight set-up above, and the compiler
  // spilled one of them - a spilled value is reloaded behind a wait for ALL outstanding loads.
  const int lane_l = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  const int jl = lane_l & 15, kgl = lane_l >> 4;
  const bool hi_half = kgl >= 2;
  const int lw = p.lw;

  // one row block of this wave's slices; leaves the wave's partial sums in LDS slot `slot`
  auto consume = [&](const Buf& bf, int slot) {
    floatx4 acc[NMAT];
#pragma unroll
    for (int a = 0; a < NMAT; ++a) acc[a] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int a = 0; a < NMAT; ++a)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          // lane (j, kg) takes its words from the lane that loaded chunk 2g + kg%2 of row j
          const int src = (4 * jl + 2 * g + (kgl & 1)) * 4;
#if (EXO_W16_ABL & 2)
          const uint32_t q0w = bf.w[a][sl].x + src, q1w = bf.w[a][sl].y, q2w = bf.w[a][sl].z, q3w = bf.w[a][sl].w;
#else
          const uint32_t q0w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bf.w[a][sl].x);
          const uint32_t q1w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bf.w[a][sl].y);
          const uint32_t q2w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bf.w[a][sl].z);
          const uint32_t q3w = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bf.w[a][sl].w);
#endif
          floatx4 dq = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t wd = h == 0 ? (hi_half ? q1w : q0w) : (hi_half ? q3w : q2w);
            uint4 bw;
#if (EXO_W16_ABL & 8)
            bw.x = wd; bw.y = wd ^ kmagic; bw.z = wd | kmagic; bw.w = wd & kmagic;
#else
            bw.x = (wd & kmask) | kmagic;
            bw.y = ((wd >> 4) & kmask) | kmagic;
            bw.z = ((wd >> 8) & kmask) | kmagic;
            bw.w = ((wd >> 12) & kmask) | kmagic;
#endif
#if (EXO_W16_ABL & 1)
            dq[0] += __builtin_bit_cast(float, bw.x ^ bw.y ^ bw.z ^ bw.w ^ xa[sl][g][h].x);
#else
            dq = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[sl][g][h]),
                                                        __builtin_bit_cast(bf16x8_t, bw), dq, 0, 0, 0);
#endif
          }
          uint32_t sw, bwd;
          if (P8) {  // this lane's column: row jl % 8 of the gate (jl < 8) or the up matrix
            const char* base = sb_lds + (slot * 8 + (jl & 7)) * sb_row + (wave * SL + sl) * 4 + (jl >> 3) * 2 * sb_arr;
            sw = *reinterpret_cast<const uint32_t*>(base);
            bwd = *reinterpret_cast<const uint32_t*>(base + sb_arr);
          } else if (SBLDS) {
            const char* base = sb_lds + (slot * 16 + jl) * sb_row + (wave * SL + sl) * 4;
            sw = *reinterpret_cast<const uint32_t*>(base + (a * 2) * sb_arr);
            bwd = *reinterpret_cast<const uint32_t*>(base + (a * 2 + 1) * sb_arr);
          } else {
            sw = bf.s[a].v[sl];
            bwd = bf.b[a].v[sl];
          }
          const float sc = g == 0 ? bf_lo(sw) : bf_hi(sw);
          const float bi = g == 0 ? bf_lo(bwd) : bf_hi(bwd);
#if (EXO_W16_ABL & 4)
          acc[a][0] += dq[0] * sc + dq[1] + dq[2] + dq[3] + bi;
#else
          const float t = fmaf(-128.f, sc, bi);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            acc[a][r] = fmaf(sc, dq[r], acc[a][r]);
            acc[a][r] = fmaf(t, sx[sl][g][r], acc[a][r]);
          }
#endif
        }
    if (lane_l < lw) {
#pragma unroll
      for (int a = 0; a < NMAT; ++a)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          red[((((size_t)slot * NMAT + a) * nw + wave) * 4 + r) * lw + lane_l] = acc[a][r];
    }
  };

  // the phase's results: sum over the waves in a fixed order, epilogue, store
  auto finish_phase = [&](int q_first, int n, bool res) {
    __syncthreads();
    if constexpr (P8) {
      for (int idx = tid; idx < n * p.M * 8; idx += (int)blockDim.x) {
        const int jj = idx & 7, m = (idx >> 3) % p.M, slot = (idx >> 3) / p.M;
        const float* src = &red[(((size_t)slot * nw * 4) + (m & 3)) * lw + (m >> 2) * 16 + jj];
        float tg = 0.f, tu = 0.f;
        for (int w = 0; w < nw; ++w) {
          tg += src[(size_t)w * 4 * lw];
          tu += src[(size_t)w * 4 * lw + 8];
        }
        // SwiGLU on the bf16-rounded projections
        const float g = bf2f(f2bf(tg)), up = bf2f(f2bf(tu));
        p.y[(size_t)m * p.N + (q0 + q_first + slot) * 8 + jj] = f2bf(g / (1.f + __expf(-g)) * up);
      }
      __syncthreads();
      return;
    }
    for (int idx = tid; idx < n * p.M * 16; idx += (int)blockDim.x) {
      const int jj = idx & 15, m = (idx >> 4) % p.M, slot = (idx >> 4) / p.M;
      const int src_lane = (m >> 2) * 16 + jj, r = m & 3;
      float tot[NMAT];
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        const float* src = &red[(((size_t)slot * NMAT + a) * nw * 4 + r) * lw + src_lane];
        float t = 0.f;
        for (int w = 0; w < nw; ++w) t += src[(size_t)w * 4 * lw];
        tot[a] = t;
      }
      const int row = (q0 + q_first + slot) * 16 + jj;
      const size_t o = (size_t)m * p.N + row;
      if (KSPLIT_OK && p.kparts > 1) {  // (single matrices only) this part's share of the sum
        st_dev(&p.part[(size_t)kpart * p.M * p.N + o], tot[0]);
        continue;
      }
      float out;
      if (NMAT == 2) {  // SwiGLU on the bf16-rounded projections
        const float g = bf2f(f2bf(tot[0])), up = bf2f(f2bf(tot[NMAT - 1]));
        out = g / (1.f + __expf(-g)) * up;
      } else {
        out = tot[0];
        if (res && p.residual) out = bf2f(f2bf(out)) + bf2f(p.residual[o]);
      }
      p.y[o] = f2bf(out);
    }
    __syncthreads();
  };
  // Split K: the last of a group's workgroups to arrive adds the parts in part order (the result
  // does not depend on arrival order) and writes y; the counter returns to zero.
  auto merge_parts = [&](int n) {
    wait_own_stores_done();  // this wave's device-scope partial stores have completed
    __syncthreads();
    if (tid == 0) {
      int* cnt = &p.counters[bgroup];
      const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      s_last = (old == p.kparts - 1);
      if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    for (int idx = tid; idx < n * p.M * 16; idx += (int)blockDim.x) {
      const int jj = idx & 15, m = (idx >> 4) % p.M, slot = (idx >> 4) / p.M;
      const size_t o = (size_t)m * p.N + (q0 + slot) * 16 + jj;
      float t = 0.f;
      for (int kp = 0; kp < p.kparts; ++kp) t += ld_dev(&p.part[(size_t)kp * p.M * p.N + o]);
      if (p.residual) t = bf2f(f2bf(t)) + bf2f(p.residual[o]);
      p.y[o] = f2bf(t);
    }
  };

  int slot = 0, q_first = 0;
  for (int base = 0;; base += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (base + d < nq) {
        consume(buf[d], slot);
        ++slot;
      }
      issue(buf[d], base + d + DEPTH, false);
    }
    if (base + DEPTH >= nq) break;
  }
  // (One phase: the launcher gives a workgroup no more row blocks than the LDS holds partial
  // sums for.  A reduction inside the streaming loop - even an empty conditional block that
  // resets `slot` - makes the compiler wait for a whole buffer too many at the first block of
  // every round.)
  finish_phase(q_first, slot, true);
  if (KSPLIT_OK && p.kparts > 1) merge_parts(slot);
}

constexpr size_t kLdsBudget = 144 * 1024;  // LDS for partial sums and staged scales (the norm weights: 8 KB more)

template <int NMAT, int SL, int DEPTH, bool NORM, bool SBLDS, bool KSPLIT = false, bool P8 = false>
int launch_w16s(W16Params p, int nw, hipStream_t st) {
  auto kern = qmv_w16_kernel<NMAT, SL, DEPTH, NORM, SBLDS, KSPLIT, P8>;
  constexpr int RPB = P8 ? 8 : 16, NS = P8 ? 2 : NMAT;
  p.blocks = p.N / RPB;
  p.lw = 16 * ((p.M + 3) / 4);
  const size_t per_block = (size_t)NMAT * nw * 4 * p.lw * sizeof(float);
  const size_t sb_block = SBLDS ? (size_t)NS * 2 * RPB * (p.Gp * 2 + 8) : 0;
  int ph = (int)(kLdsBudget / (per_block + sb_block));  // row blocks a workgroup can hold
  // staging: one 16-byte chunk per thread and array
  const int stage_max = 64 * nw / (RPB * (p.Gp / 8));
  if (SBLDS && ph > stage_max) ph = stage_max;
  if (ph < 1) {
    exo_set_error("exo_qmv: internal: no LDS for one row block (M=%d K=%d)", p.M, p.K);
    return EXO_ERR_ARG;
  }
  // one workgroup per CU (kparts workgroups per group of row blocks); more rounds where a
  // workgroup's share would not fit the LDS
  const int round = 256 / p.kparts;
  int groups = round;
  while ((p.blocks + groups - 1) / groups > ph) groups += round;
  if (groups > p.blocks) groups = p.blocks;
  const int grid = groups * p.kparts;
  const int nq = (p.blocks + groups - 1) / groups;
  p.ph = nq;
  p.red_bytes = (int)(per_block * nq);
  const size_t lds = (per_block + sb_block) * nq + (NORM ? (size_t)p.K * 2 : 0);
  static bool attr_done = false;
  if (!attr_done && lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  exo_note_variant("qmv_w16<%d,%d,%d,%s,%s> grid=%d waves=%d blocks=%d kparts=%d", P8 ? 2 : NMAT, SL, DEPTH,
                   NORM ? "norm" : "plain", P8 ? "pair8" : (SBLDS ? "staged" : "direct"), grid, nw, nq, p.kparts);
  kern<<<dim3(grid), dim3(64 * nw), lds, st>>>(p);
  return EXO_OK;
}
template <int NMAT, int SL, int DEPTH>
int launch_w16(const W16Params& p, int nw, hipStream_t st) {
  // staged scales where they fit the LDS beside the partial sums of one round of 256 workgroups
  // (the 14336-row pair: up to 12 activation rows) and one chunk per thread covers them
  const int round = 256 / p.kparts;
  const int groups1 = p.blocks < round ? p.blocks : round, nq1 = (p.blocks + groups1 - 1) / groups1;
  const size_t need1 = ((size_t)NMAT * nw * 4 * 16 * ((p.M + 3) / 4) * sizeof(float) +
                        (size_t)NMAT * 2 * 16 * (p.Gp * 2 + 8)) * nq1;
  const bool staged = p.Gp % 8 == 0 && need1 <= kLdsBudget && nq1 <= 32 * nw / p.Gp && !(EXO_W16_ABL & 128);
  if constexpr (NMAT == 2) {
    // the pair in blocks of 8 rows of both matrices where their share of one round of 256
    // workgroups fits the LDS with staged scales: 14336 rows are seven such blocks per
    // workgroup, against four or three blocks of 16 rows (8 activation rows: 20.4 -> us)
    const int blocks8 = p.N / 8, g8 = blocks8 < 256 ? blocks8 : 256, nq8 = (blocks8 + g8 - 1) / g8;
    const size_t need8 = ((size_t)nw * 4 * 16 * ((p.M + 3) / 4) * sizeof(float) +
                          (size_t)2 * 2 * 8 * (p.Gp * 2 + 8)) * nq8;
    if (p.N % 8 == 0 && p.Gp % 8 == 0 && need8 <= kLdsBudget && nq8 <= 64 * nw / (8 * (p.Gp / 8)) &&
        EXO_W16_PAIR8) {
      return p.norm_w ? launch_w16s<1, SL, DEPTH, true, true, false, true>(p, nw, st)
                      : launch_w16s<1, SL, DEPTH, false, true, false, true>(p, nw, st);
    }
  }
  if (p.kparts > 1) {
    if constexpr (NMAT == 1)
      return staged ? launch_w16s<1, SL, DEPTH, false, true, true>(p, nw, st)
                    : launch_w16s<1, SL, DEPTH, false, false, true>(p, nw, st);
    exo_set_error("exo_qmv: internal: split K with a matrix pair");
    return EXO_ERR_ARG;
  }
  if (p.norm_w)
    return staged ? launch_w16s<NMAT, SL, DEPTH, true, true>(p, nw, st)
                  : launch_w16s<NMAT, SL, DEPTH, true, false>(p, nw, st);
  return staged ? launch_w16s<NMAT, SL, DEPTH, false, true>(p, nw, st)
                : launch_w16s<NMAT, SL, DEPTH, false, false>(p, nw, st);
}

// 64-byte slices per wave and waves per workgroup for rows of `row_bytes`
bool w16_shape(int row_bytes, int* sl_out, int* nw_out) {
  if (row_bytes % 64) return false;
  const int slices = row_bytes / 64;
  for (int sl = 1; sl <= 2; sl *= 2) {
    if (slices % sl) continue;
    const int nw = slices / sl;
    if (nw > 16 || nw < 4) continue;
    *sl_out = sl;
    *nw_out = nw;
    return true;
  }
  return false;
}

// parts of K (workgroups per group of row blocks) for rows of `row_bytes`: 1 where a row's
// activations fit the registers of one workgroup, else - with a workspace, without a fused norm
// or a second matrix - the smallest split into equal parts of whole 16-byte scale chunks
int w16_parts(int row_bytes, bool can_split, int* sl_out, int* nw_out) {
  if (w16_shape(row_bytes, sl_out, nw_out)) return 1;
  if (!can_split || row_bytes % 64) return 0;
  const int slices = row_bytes / 64;  // one slice = two quantisation groups
  for (int kp = 2; kp <= 8; ++kp)
    if (slices % kp == 0 && (2 * slices / kp) % 8 == 0 && w16_shape(row_bytes / kp, sl_out, nw_out))
      return kp;
  return 0;
}

}  // namespace

bool exo_qmv_w16_ok(int M, int N, int K, int bits, bool norm, bool pair, bool has_workspace) {
  int sl, nw;
  if (M < 1 || M > 16 || N % 16 || N < 16 || bits != 4 || K % 128) return false;
  if ((int64_t)N * K / 2 >= (1ll << 31)) return false;
  const int kp = w16_parts(K / 2, has_workspace && !norm && !pair, &sl, &nw);
  if (kp == 0) return false;
  if (kp > 1 && (N / 16) * 4 > 64 * 1024) return false;  // counters: one per group of row blocks
  return true;
}

int exo_qmv_w16_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                       const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                       const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                       void* workspace, hipStream_t st) {
  W16Params p;
  p.x = x;
  p.norm_w = norm_w;
  p.eps = eps;
  p.w[0] = w;
  p.s[0] = s;
  p.b[0] = b;
  p.w[1] = w2 ? w2 : w;
  p.s[1] = s2 ? s2 : s;
  p.b[1] = b2 ? b2 : b;
  p.residual = residual;
  p.y = y;
  p.M = M;
  p.N = N;
  p.K = K;
  p.row_bytes = K / 2;
  p.G = K / 64;
  p.blocks = N / 16;  // (the launcher sets the count for its block size)
  p.ph = 1;
  p.lw = 64;
  p.red_bytes = 0;
  const bool pair = w2 != nullptr;
  int sl = 0, nw = 0;
  const int kp = exo_qmv_w16_ok(M, N, K, 4, norm_w != nullptr, pair, workspace != nullptr)
                     ? w16_parts(p.row_bytes, workspace && !norm_w && !pair, &sl, &nw)
                     : 0;
  if (kp == 0) {
    exo_set_error("exo_qmv: shape M=%d N=%d K=%d not covered by the 16x16x32 kernel", M, N, K);
    return EXO_ERR_ARG;
  }
  p.kparts = kp;
  p.Gp = p.G / kp;
  // the workspace of the split-K GEMV: counters (64 KiB), then the float32 partial results
  p.counters = reinterpret_cast<int*>(workspace);
  p.part = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + 64 * 1024) : nullptr;
#ifndef EXO_W16_DEPTH
#define EXO_W16_DEPTH 2
#endif
  if (sl == 1) return pair ? launch_w16<2, 1, EXO_W16_DEPTH>(p, nw, st) : launch_w16<1, 1, EXO_W16_DEPTH>(p, nw, st);
  return pair ? launch_w16<2, 2, 2>(p, nw, st) : launch_w16<1, 2, EXO_W16_DEPTH>(p, nw, st);
}
