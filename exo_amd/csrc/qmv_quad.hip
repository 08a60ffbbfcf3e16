// Fused dequant-GEMV for 1..16 activation rows on v_mfma_f32_4x4x4_16b_bf16.
//
// The instruction multiplies sixteen independent 4x4 blocks: block b takes A[i][k] from lane
// 4b+i and B[k][j] from lane 4b+j (k = the 4 bf16 of the lane's 64-bit operand) and leaves
// D[i][j] in register i of lane 4b+j.  Here a block is (4 weight rows) x (4 activation rows)
// x (4 elements of K), and the K elements of consecutive products of a lane are consecutive
// elements of ITS OWN 16-byte chunk of a packed row - the sum over K never crosses lanes
// inside the loop, exactly as in the dot2 kernel, but four activation rows cost one
// instruction of the matrix pipe instead of four times the vector work.
//  * a wave instruction loads 4 rows x 256 contiguous bytes: lane (lane/16, lane%16) takes chunk
//    lane%16 of row lane/16, so that the four lanes of a quad read 64 contiguous bytes (a quad
//    whose lanes touch four rows costs four times the address cycles).  The instruction wants
//    chunk b of row j in lane 4b+j: the loaded registers change lanes through the LDS crossbar
//    (ds_bpermute_b32, no LDS memory, no vector-ALU work) when the batch is consumed.
//  * a wave owns SL such slices of K for every row quad q of its workgroup; the matching
//    activations (row i = lane%4 of each set of four, elements of chunk b) stay in registers
//    in operand order for the whole launch - no LDS traffic in the loop.  The waves of a
//    workgroup together cover K; their partial sums meet in LDS once per phase of row quads.
//  * codes become (128+nibble) bf16 pairs with one v_and_or_b32 each (exact); the 128 offset
//    is removed by starting every chunk's accumulator at -128 * (sum of the chunk's
//    activations); per chunk: acc += s * D + beta * Sx, float32, s and beta of the chunk's
//    quantisation group.  8-bit codes are two nibbles against (x, 16x).
//  * D row-quad batches of weights are in flight per wave (register buffers in rotation).
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "qmv_internal.h"

namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#ifndef EXO_QUAD_ABL
#define EXO_QUAD_ABL 0  // timing-only ablations (wrong results): 1 no products, 2 no lane permutation
#endif
#ifndef EXO_QMV_QUAD_MAX_DEPTH
#define EXO_QMV_QUAD_MAX_DEPTH 6
#endif
constexpr int kQuadMaxDepth = EXO_QMV_QUAD_MAX_DEPTH;  // row quads in flight per wave, at most

struct QuadParams {
  const bf16_t* x;       // [M, K]
  const bf16_t* norm_w;  // [K] or null: fused RMSNorm of x
  float eps;
  const uint32_t* w[2];  // packed [N, K*bits/32]   ([1]: the up matrix of a (gate, up) pair)
  const bf16_t* s[2];    // [N, K/64]
  const bf16_t* b[2];
  const bf16_t* residual;  // [M, N] or null
  bf16_t* y;               // [M, N]
  int M, N, K;
  int row_bytes;  // K * bits / 8
  int G;          // K / 64
  int quads;      // N / 4
  int ph;         // row quads per reduction phase (LDS holds their partial sums)
};

template <int BITS>
__device__ __forceinline__ uint4 load_word_x(const bf16_t* base, int wi) {
  if (BITS == 4) return *reinterpret_cast<const uint4*>(base + (size_t)wi * 8);
  const uint2 v = *reinterpret_cast<const uint2*>(base + (size_t)wi * 4);
  return make_uint4(v.x, v.y, 0, 0);
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
template <int BITS>
__device__ __forceinline__ void norm_word(uint4& xv, const uint4& wv, float inv) {
  xv.x = pack_bf2(bf_lo(xv.x) * inv * bf_lo(wv.x), bf_hi(xv.x) * inv * bf_hi(wv.x));
  xv.y = pack_bf2(bf_lo(xv.y) * inv * bf_lo(wv.y), bf_hi(xv.y) * inv * bf_hi(wv.y));
  if (BITS == 4) {
    xv.z = pack_bf2(bf_lo(xv.z) * inv * bf_lo(wv.z), bf_hi(xv.z) * inv * bf_hi(wv.z));
    xv.w = pack_bf2(bf_lo(xv.w) * inv * bf_lo(wv.w), bf_hi(xv.w) * inv * bf_hi(wv.w));
  }
}
// The activations of one packed word in the order of the unpacked nibble pairs: 4-bit
// (x0,x4),(x1,x5) | (x2,x6),(x3,x7); 8-bit (x0,x2),(16x0,16x2) | (x1,x3),(16x1,16x3) - the
// two 64-bit operands of the word's two products.  `stored` = sum of the operand values,
// `truesum` = sum of the activations.
template <int BITS>
__device__ __forceinline__ uint4 permute_word(const uint4& xv, float& stored, float& truesum) {
  uint4 o;
  if (BITS == 4) {
    o.x = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);
    o.y = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);
    o.z = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);
    o.w = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);
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

__device__ __forceinline__ short4_t as_s4(uint32_t lo, uint32_t hi) {
  return __builtin_bit_cast(short4_t, make_uint2(lo, hi));
}

// sum over the lanes of a row of 16 that share lane % 4 (the 4 blocks of the row), in every lane
__device__ __forceinline__ float sum_blocks_row16(float v) {
  v += dpp_get<0x124, 0xf>(v);  // row_ror:4
  v += dpp_get<0x128, 0xf>(v);  // row_ror:8
  return v;
}
// value of lane 4*(lane/4) + I of the same block
template <int I>
__device__ __forceinline__ float quad_bcast(float v) {
  return dpp_get<I | (I << 2) | (I << 4) | (I << 6), 0xf>(v);
}

// MSETS sets of four activation rows; MU = rows of the (single) set that are real when
// MSETS == 1 (1, 2 or 4: the chunk epilogue touches only those accumulator registers).
// SL = 256-byte slices of K per wave.
// (Sixteen activation rows hold 64 operand registers per slice: those instances run 8 waves per
// workgroup at most, one workgroup per CU, and may use 256 registers.)
template <int BITS, int NMAT, int MSETS, int MU, int SL>
__global__ __launch_bounds__(MSETS == 4 ? 512 : 1024) void qmv_quad_kernel(const QuadParams p) {
  constexpr int MROWS = (MSETS - 1) * 4 + MU;  // activation rows with a result
  // row quads in flight per wave.  With 16 waves per CU the depth hardly matters (gate/up pair
  // at two | four rows, us: depth 1 17.6 | 20.0, 2 17.3 | 19.8, 3 18.4 | 21.0, 4 18.6 | 21.4,
  // 5 19.9 | 22.2; 4096x4096: depth 1 4.9 | 6.3, 2 5.2 | 6.3, 4 5.3 | 6.6, 6 5.8 | 7.1): two
  // buffers, and no spill (a spilled load result is waited for on the spot)
#ifndef EXO_QUAD_DEPTH_ONE
#define EXO_QUAD_DEPTH_ONE 2
#endif
#ifndef EXO_QUAD_DEPTH_PAIR
#define EXO_QUAD_DEPTH_PAIR 2
#endif
  constexpr int DEPTH0 = NMAT * SL == 1 ? EXO_QUAD_DEPTH_ONE
                                        : ((NMAT * SL == 2 && SL == 1 && MSETS == 1) ? EXO_QUAD_DEPTH_PAIR : 2);
  constexpr int DEPTH = DEPTH0 > kQuadMaxDepth ? kQuadMaxDepth : DEPTH0;
  constexpr int CHUNK_EL = 128 / BITS;            // elements of a 16-byte chunk: 32 / 16
  constexpr int CPG = 64 / CHUNK_EL;              // chunks per quantisation group: 2 / 4
  extern __shared__ float red[];  // [ph][NMAT][MROWS][nw][16]
  __shared__ float s_part[16][16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = blockDim.x >> 6;
  const int j = lane & 3, b = lane >> 2;      // operand layout: row of the quad, chunk of the slice
  const int lj = lane >> 4, lb = lane & 15;   // load layout
  const int perm_src = (16 * j + b) * 4;      // ds_bpermute address: lane 4b+j takes lane 16j+b

  // contiguous, balanced range of row quads of this workgroup
  const int qbase = p.quads / (int)gridDim.x, qrem = p.quads - qbase * (int)gridDim.x;
  const int q0 = (int)blockIdx.x * qbase + min((int)blockIdx.x, qrem);
  const int nq = qbase + ((int)blockIdx.x < qrem ? 1 : 0);
  if (nq <= 0) return;

  // ---- weights: register buffers of one row quad each
  struct Buf {
    uint4 w[NMAT][SL];
    // (scale, bias) of the chunk's group.  One register each: packing the two 16-bit loads into
    // one register makes the compiler wait for them on the spot.
    bf16_t s[NMAT][SL], b[NMAT][SL];
  };
  // Buffer resources over exactly this workgroup's rows: a refill past the last row quad is
  // out of range, returns zeros and moves no data, yet counts as a load in flight - the
  // number of loads outstanding at every wait stays a compile-time constant.
  __amdgpu_buffer_rsrc_t rw[NMAT], rs[NMAT], rb[NMAT];
#pragma unroll
  for (int a = 0; a < NMAT; ++a) {
    rw[a] = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(p.w[a]) + (size_t)q0 * 4 * p.row_bytes), 0,
        nq * 4 * p.row_bytes, 0x00020000);
    rs[a] = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.s[a] + (size_t)q0 * 4 * p.G), 0,
                                              nq * 4 * p.G * 2, 0x00020000);
    rb[a] = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.b[a] + (size_t)q0 * 4 * p.G), 0,
                                              nq * 4 * p.G * 2, 0x00020000);
  }
  // this lane's byte offsets inside a row quad (load layout)
  const int wofs = lj * p.row_bytes + wave * (SL * 256) + lb * 16;
  // group of this lane's chunk: 256 bytes hold 16 chunks = 16 / CPG groups
  const int sofs = (lj * p.G + wave * (SL * (16 / CPG)) + lb / CPG) * 2;
  // PIN (the issues in front of the loop): the loads leave in program order, buffer by buffer,
  // as in the loop.  The compiler counts the loads still in flight at each wait; where the
  // order in front of the loop differs from the order in the loop it assumes the worse of the
  // two and waits for a whole buffer too many.
  auto issue = [&](Buf& bf, int q, bool pin = false) {  // q: row quad of this workgroup's range (past it: zeros)
    const int wq = q * 4 * p.row_bytes, sq = q * 4 * p.G * 2;  // uniform: scalar offsets
    if (pin) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        bf.w[a][sl] = __builtin_bit_cast(
            uint4, __builtin_amdgcn_raw_buffer_load_b128(rw[a], wofs + sl * 256, wq, 0));
#if (EXO_QUAD_ABL & 4)
        bf.s[a][sl] = 0x3c00;
        bf.b[a][sl] = 0x3c00;
#else
        bf.s[a][sl] = (bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rs[a], sofs + sl * (16 / CPG) * 2, sq, 0);
        bf.b[a][sl] = (bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rb[a], sofs + sl * (16 / CPG) * 2, sq, 0);
#endif
        if (pin) __builtin_amdgcn_sched_barrier(0);
      }
  };
  Buf buf[DEPTH];
  // operands: xa[set][sl][t][h] = the 64-bit A operand of product h of word t
  short4_t xa[MSETS][SL][4][2];
  float4_t cinit[MSETS][SL];  // -128 * (sum of the stored operand values) per activation row
  float sxv[MSETS][SL][4];    // sum of the activations of the chunk per activation row
  const int wi0 = wave * (SL * 64) + b * 4;  // first packed word of this lane's chunk, slice 0
  // words of one slice -> operands and chunk sums
  auto to_operands = [&](const uint4 (&xw)[4], int set, int sl) {
    float stored = 0.f, truesum = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float st_, ts_;
      const uint4 o = permute_word<BITS>(xw[t], st_, ts_);
      xa[set][sl][t][0] = as_s4(o.x, o.y);
      xa[set][sl][t][1] = as_s4(o.z, o.w);
      stored += st_;
      truesum += ts_;
    }
    // lane (b, j) needs the sums of activation row i for every accumulator register i
    cinit[set][sl][0] = -128.f * quad_bcast<0>(stored);
    sxv[set][sl][0] = quad_bcast<0>(truesum);
    if (MU > 1 || MSETS > 1) {
      cinit[set][sl][1] = -128.f * quad_bcast<1>(stored);
      sxv[set][sl][1] = quad_bcast<1>(truesum);
    } else {
      cinit[set][sl][1] = 0.f;
      sxv[set][sl][1] = 0.f;
    }
    if (MU > 2 || MSETS > 1) {
      cinit[set][sl][2] = -128.f * quad_bcast<2>(stored);
      sxv[set][sl][2] = quad_bcast<2>(truesum);
      cinit[set][sl][3] = -128.f * quad_bcast<3>(stored);
      sxv[set][sl][3] = quad_bcast<3>(truesum);
    } else {
      cinit[set][sl][2] = cinit[set][sl][3] = 0.f;
      sxv[set][sl][2] = sxv[set][sl][3] = 0.f;
    }
  };
  if constexpr (SL == 1) {
    // the activation loads go first (they are waited for first), then the weights
    uint4 xraw[MSETS][4], nraw[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int set = 0; set < MSETS; ++set) {
        const int m = set * 4 + j;
        xraw[set][t] = make_uint4(0, 0, 0, 0);
        if (m < p.M) xraw[set][t] = load_word_x<BITS>(p.x + (size_t)m * p.K, wi0 + t);
      }
      nraw[t] = make_uint4(0, 0, 0, 0);
      if (p.norm_w) nraw[t] = load_word_x<BITS>(p.norm_w, wi0 + t);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(buf[d], d, true);
    if (p.norm_w) {  // fused RMSNorm: every wave holds its slice of every row
#pragma unroll
      for (int set = 0; set < MSETS; ++set) {
        float ss = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t) ss += sumsq_word<BITS>(xraw[set][t]);
        ss = sum_blocks_row16(ss);
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        if (lane < 4) s_part[wave][set * 4 + lane] = ss;
      }
      __syncthreads();
#pragma unroll
      for (int set = 0; set < MSETS; ++set) {
        // the per-wave sums of this lane's row, added in wave order (lanes 0..nw-1 hold one each)
        float tot_j = 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          float v = lane < nw ? s_part[lane][set * 4 + jj] : 0.f;
          v = wave_sum_to_lane63(v);
          v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
          if (j == jj) tot_j = v;
        }
        const float inv = rsqrtf(tot_j / (float)p.K + p.eps);
#pragma unroll
        for (int t = 0; t < 4; ++t) norm_word<BITS>(xraw[set][t], nraw[t], inv);
      }
    }
#pragma unroll
    for (int set = 0; set < MSETS; ++set) to_operands(xraw[set], set, 0);
  } else {
    // several slices per wave (long rows; the launcher sends no fused norm here): one slice at
    // a time, so that the raw words of a slice are dead before the next ones arrive
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(buf[d], d, true);
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int set = 0; set < MSETS; ++set) {
        const int m = set * 4 + j;
        uint4 xw[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          xw[t] = make_uint4(0, 0, 0, 0);
          if (m < p.M) xw[t] = load_word_x<BITS>(p.x + (size_t)m * p.K, wi0 + sl * 64 + t);
        }
        to_operands(xw, set, sl);
      }
  }

  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));

  float acc[NMAT][MSETS][4];
#pragma unroll
  for (int a = 0; a < NMAT; ++a)
#pragma unroll
    for (int set = 0; set < MSETS; ++set)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[a][set][i] = 0.f;

  constexpr int RU = (MSETS > 1) ? 4 : MU;  // accumulator registers in use per set

  // one row quad of this wave's slices; leaves the wave's partial sums in LDS slot `slot`
  auto consume = [&](const Buf& bf, int slot) {
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        // load layout -> operand layout
        uint32_t wd[4];
#if (EXO_QUAD_ABL & 2)
        wd[0] = bf.w[a][sl].x; wd[1] = bf.w[a][sl].y; wd[2] = bf.w[a][sl].z; wd[3] = bf.w[a][sl].w;
        const uint32_t sbw = (uint32_t)bf.s[a][sl] | ((uint32_t)bf.b[a][sl] << 16);
#else
        wd[0] = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_src, (int)bf.w[a][sl].x);
        wd[1] = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_src, (int)bf.w[a][sl].y);
        wd[2] = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_src, (int)bf.w[a][sl].z);
        wd[3] = (uint32_t)__builtin_amdgcn_ds_bpermute(perm_src, (int)bf.w[a][sl].w);
        // (pinned here: packed any earlier - the compiler moves the two cheap operations in
        // front of the branch around this block, to the end of the previous round - the wait
        // for the scale loads drains the buffers that were just refilled)
        uint32_t s_raw = bf.s[a][sl], b_raw = bf.b[a][sl];
        asm volatile("" : "+v"(s_raw), "+v"(b_raw));
        const uint32_t sbw =
            (uint32_t)__builtin_amdgcn_ds_bpermute(perm_src, (int)(s_raw | (b_raw << 16)));
#endif
        const float sc = bf_lo(sbw), bi = bf_hi(sbw);
        float4_t dq[MSETS];
#pragma unroll
        for (int set = 0; set < MSETS; ++set) dq[set] = cinit[set][sl];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t p0 = (wd[t] & kmask) | kmagic;
          const uint32_t p1 = ((wd[t] >> 4) & kmask) | kmagic;
          const uint32_t p2 = ((wd[t] >> 8) & kmask) | kmagic;
          const uint32_t p3 = ((wd[t] >> 12) & kmask) | kmagic;
          const short4_t b0 = as_s4(p0, p1), b1 = as_s4(p2, p3);
#if (EXO_QUAD_ABL & 1)
          for (int set = 0; set < MSETS; ++set)
            dq[set][0] += __builtin_bit_cast(float, p0 ^ p1 ^ p2 ^ p3);
          (void)b0; (void)b1;
#else
#pragma unroll
          for (int set = 0; set < MSETS; ++set) {
            dq[set] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[set][sl][t][0], b0, dq[set], 0, 0, 0);
            dq[set] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[set][sl][t][1], b1, dq[set], 0, 0, 0);
          }
#endif
        }
#pragma unroll
        for (int set = 0; set < MSETS; ++set)
#pragma unroll
          for (int i = 0; i < RU; ++i) {
            acc[a][set][i] = fmaf(sc, dq[set][i], acc[a][set][i]);
            acc[a][set][i] = fmaf(bi, sxv[set][sl][i], acc[a][set][i]);
          }
      }
    // the wave's partial sums of this row quad: over its 16 chunk lanes per row of 16 lanes
#pragma unroll
    for (int a = 0; a < NMAT; ++a)
#pragma unroll
      for (int set = 0; set < MSETS; ++set)
#pragma unroll
        for (int i = 0; i < RU; ++i) {
          const int m = set * 4 + i;
          const float v = sum_blocks_row16(acc[a][set][i]);
          acc[a][set][i] = 0.f;
          if (m < MROWS && (lane & 15) < 4)
            red[((((size_t)slot * NMAT + a) * MROWS + m) * nw + wave) * 16 + (lane >> 4) * 4 + j] = v;
        }
  };

  // the phase's results: sum over waves and lane rows in a fixed order, epilogue, store.
  // RES: add the residual (its loads would sit inside the streaming loop otherwise, where a
  // conditional load makes every later wait a wait for all outstanding loads; the launcher
  // gives a launch with a residual a single phase)
  auto finish_phase = [&](int q_first, int n, bool res) {
    __syncthreads();
    for (int idx = tid; idx < n * MROWS * 4; idx += (int)blockDim.x) {
      const int jj = idx & 3, m = (idx >> 2) % MROWS, slot = (idx >> 2) / MROWS;
      if (m >= p.M) continue;
      float tot[NMAT];
#pragma unroll
      for (int a = 0; a < NMAT; ++a) {
        const float* src = &red[(((size_t)slot * NMAT + a) * MROWS + m) * nw * 16 + jj];
        float t = 0.f;
        for (int w = 0; w < nw; ++w)
          t += (src[w * 16] + src[w * 16 + 4]) + (src[w * 16 + 8] + src[w * 16 + 12]);
        tot[a] = t;
      }
      const int row = (q0 + q_first + slot) * 4 + jj;
      const size_t o = (size_t)m * p.N + row;
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

  // Every refill is issued whether or not a row quad is left (past the end it is out of the
  // buffer's range: no data moves), so that the number of loads in flight at each wait is a
  // constant the compiler knows; only the products are skipped past the end.
  int slot = 0, q_first = 0;
  for (int base = 0;; base += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (base + d < nq) {
        consume(buf[d], slot);
        ++slot;
      }
      issue(buf[d], base + d + DEPTH);
    }
    if (base + DEPTH >= nq) break;
  }
  // (One phase: the launcher gives a workgroup no more row quads than the LDS holds partial
  // sums for.  A reduction inside the streaming loop - even an empty conditional block that
  // resets `slot` - makes the compiler wait for a whole buffer too many at the first quad of
  // every round.)
  finish_phase(q_first, slot, true);
}

constexpr size_t kRedBudget = 48 * 1024;  // LDS for the partial sums of a phase

template <int BITS, int NMAT, int MSETS, int MU, int SL>
int launch_quad(QuadParams p, int nw, hipStream_t st) {
  auto kern = qmv_quad_kernel<BITS, NMAT, MSETS, MU, SL>;
  constexpr int MROWS = (MSETS - 1) * 4 + MU;
  // one round of workgroups: two per CU up to 8 waves, one beyond; more rounds where a
  // workgroup's row quads would not fit the LDS with their partial sums
  const int per_cu = (nw <= 8 && MSETS < 4) ? 2 : 1;
  const size_t per_quad = (size_t)NMAT * MROWS * nw * 16 * sizeof(float);
  const size_t budget = per_cu == 2 ? kRedBudget : 2 * kRedBudget;
  const int ph = (int)(budget / per_quad);
  int grid = 256 * per_cu;
  while ((p.quads + grid - 1) / grid > ph) grid += 256 * per_cu;
  if (grid > p.quads) grid = p.quads;
  const int nq = (p.quads + grid - 1) / grid;
  p.ph = nq;
  const size_t lds = per_quad * nq;
  static bool attr_done = false;
  if (!attr_done && lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  exo_note_variant("qmv_quad<%d,%d,%d,%d,%d> grid=%d waves=%d phase=%d", BITS, NMAT, MSETS, MU, SL,
                   grid, nw, ph);
  kern<<<dim3(grid), dim3(64 * nw), lds, st>>>(p);
  return EXO_OK;
}

template <int BITS, int NMAT, int SL>
int launch_quad_m(const QuadParams& p, int nw, hipStream_t st) {
  if (p.M == 1) return launch_quad<BITS, NMAT, 1, 1, SL>(p, nw, st);
  if (p.M == 2) return launch_quad<BITS, NMAT, 1, 2, SL>(p, nw, st);
  if (p.M <= 4) return launch_quad<BITS, NMAT, 1, 4, SL>(p, nw, st);
  if (p.M <= 8) return launch_quad<BITS, NMAT, 2, 4, SL>(p, nw, st);
  if (SL == 1) return launch_quad<BITS, NMAT, 4, 4, 1>(p, nw, st);
  exo_set_error("exo_qmv: no 4x4x4 instance for %d rows with %d slices per wave", p.M, SL);
  return EXO_ERR_ARG;
}

// slices of 256 bytes per wave and waves per workgroup for rows of `row_bytes`
bool quad_shape(int row_bytes, int M, bool norm, int* sl_out, int* nw_out) {
  if (row_bytes % 256) return false;
  const int slices = row_bytes / 256;
  for (int sl = 1; sl <= 2; sl *= 2) {
    if (slices % sl) continue;
    const int nw = slices / sl;
    if (nw > (M > 8 ? 8 : 16)) continue;
    if (M > 8 && sl > 1) return false;   // 16 rows: one slice per wave (registers)
    if (norm && sl > 1) return false;    // the fused norm keeps a row's words in registers
    *sl_out = sl;
    *nw_out = nw;
    return true;
  }
  return false;
}

}  // namespace

bool exo_qmv_quad_ok(int M, int N, int K, int bits, bool norm) {
  int sl, nw;
  if (M < 1 || M > 16 || N % 4 || N < 4 || (bits != 4 && bits != 8) || K % 64) return false;
  return quad_shape(K * bits / 8, M, norm, &sl, &nw);
}

int exo_qmv_quad_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                        const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                        int bits, hipStream_t st) {
  QuadParams p;
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
  p.row_bytes = K * bits / 8;
  p.G = K / 64;
  p.quads = N / 4;
  p.ph = 1;
  int sl = 0, nw = 0;
  if (!exo_qmv_quad_ok(M, N, K, bits, norm_w != nullptr) ||
      !quad_shape(p.row_bytes, M, norm_w != nullptr, &sl, &nw)) {
    exo_set_error("exo_qmv: shape M=%d N=%d K=%d bits=%d not covered by the 4x4x4 kernel", M, N, K, bits);
    return EXO_ERR_ARG;
  }
  const bool pair = w2 != nullptr;
#define EXO_QUAD_CASE(B_, SL_)                                             \
  if (bits == B_ && sl == SL_)                                             \
    return pair ? launch_quad_m<B_, 2, SL_>(p, nw, st) : launch_quad_m<B_, 1, SL_>(p, nw, st);
  EXO_QUAD_CASE(4, 1)
  EXO_QUAD_CASE(4, 2)
  EXO_QUAD_CASE(8, 1)
  EXO_QUAD_CASE(8, 2)
#undef EXO_QUAD_CASE
  exo_set_error("exo_qmv: internal: no 4x4x4 instance");
  return EXO_ERR_ARG;
}
