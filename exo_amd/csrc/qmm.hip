// Quantised matmul for prefill (any M): y[M,N] = x[M,K] @ dq(W)[N,K]^T.
//
// Matrix-core design for gfx950.  A 256-thread workgroup (2 x 2 waves) computes a
// 256x128 output tile (128x128 for M <= 128); one 64-wide K step per iteration = exactly
// one quantisation group, so a packed row segment needs a single (scale, bias).
//  * Activations go from global memory straight into LDS (buffer_load_dwordx4 ... lds: no
//    registers, no LDS store instructions), two tile buffers, one barrier per K step.  The
//    tile rows are 128 bytes apart without padding (the loads write in lane order); chunk c
//    of row r sits at slot c ^ (r % 8), so the operand reads of 16 rows spread over the
//    banks.  LDS bandwidth, not the matrix cores, limited the first version of this kernel,
//    so the weights do NOT go through LDS:
//  * every wave loads the packed words of its own 64 weight rows straight into registers
//    in the MFMA B-operand layout - lane (row, half) takes 16 B (4-bit) or 32 B (8-bit) =
//    32 consecutive codes - and dequantises them there to bf16(fma(s, q, b)) with
//    v_cvt_f32_ubyteN.  MFMA step t of a K step then covers k = 32*half + 8*t .. +8, and
//    the A operand is read from the activation tile at that same offset.  The two waves
//    that share weight rows dequantise them twice; in exchange the LDS carries a third less
//    traffic.
//  * All global loads are buffer loads: workgroup-uniform descriptors, 32-bit lane offsets
//    that never change, the K step as the scalar offset - no address arithmetic in the
//    loop.  (scale, bias) of four K steps come in one 8-byte load when K % 256 == 0.
//  * v_mfma_f32_32x32x16_bf16, float32 accumulators (128x64 per wave); the tile and the
//    weights of the next K step are requested before the current one is multiplied.
//  * grouped mode (MoE prefill): blockIdx.y is a tile of one expert's sorted rows.
//  * 128-row tiles over K ranges of 768 or more: weights and activation chunks of four K
//    steps in flight in registers (DEEP, below) instead of one step.
//  * up to 128 rows and few column tiles: blockIdx.z splits K; float32 partial tiles and a
//    small reduce launch.
//  * up to 32 rows (64 on matrices of 8192 rows or more): the four waves sit side by side on
//    a (32 or 64) x 256 tile, so no weight row is dequantised twice, and K is split until the
//    launch has up to two workgroups per CU (14336x4096 4-bit at 32 rows: 31 -> 21 us,
//    4096x14336: 32.5 -> 23 us; at 96 rows and more the 128-row tile is level or faster).
//    Where that launch's time goes (14336x4096 4-bit, 32 rows, 22 us with the reduce launch):
//    the weights alone, requested as they are, take 10 us (what the one-row GEMV takes for the
//    same matrix); the dequantisation and products add 5 us that do not overlap (all
//    workgroups run in step: one round of 448 workgroups, two K ranges of loads each); the
//    float32 partial tiles 3.4 us to store and 4 us to reduce; the activation tiles 1 us.
//    Requesting the weights as whole 128-byte lines (8 rows x 128 B per wave instruction
//    instead of 32 rows x 32 B) gained 8 %, re-reading one weight block from L2 nothing, a ring
//    of eight register stages nothing, four K steps per barrier nothing: none was kept.
#include "../../include/exo_mi355x.h"
#include "common.h"

#include <algorithm>
#include <type_traits>

namespace {

#ifndef EXO_QMM_RING8
#define EXO_QMM_RING8 1
#endif
constexpr bool kRing8 = EXO_QMM_RING8 != 0;  // the ring for 8-bit weights too
constexpr int BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row

struct QmmParams {
  const bf16_t* x;
  const uint32_t* w;
  const bf16_t* s;
  const bf16_t* b;
  const bf16_t* residual;
  bf16_t* y;
  int M, N, K;
  // grouped mode (MoE experts, rows sorted by expert): blockIdx.y is a tile of
  // tiles[]; row r of the tile is pair sorted[start + r]; it reads activation row
  // pair / x_div and writes output row pair; the tile multiplies by expert e's matrix
  const int32_t* sorted;  // [pairs]
  const int32_t* tiles;   // [max_tiles][3] = expert (-1: unused), start, rows
  int x_div;
  size_t w_stride, s_stride;  // elements between consecutive experts
  // split-K (few row tiles): blockIdx.z owns K steps [z*kc, (z+1)*kc) and writes a
  // float32 partial tile; qmm_reduce_kernel adds them
  int ksplit, kc;
  float* part;  // [ksplit][M][N]
  bool wide = false;  // host only: launch the (32*MI) x 256 tile (up to 128 rows)
  // pair mode (Llama MLP, prefill): w/s/b is the gate matrix, w2/s2/b2 the up matrix, both
  // [N, K]; y[M,N] = silu(x gate^T) * (x up^T) with both projections rounded to bf16 first
  const uint32_t* w2 = nullptr;
  const bf16_t* s2 = nullptr;
  const bf16_t* b2 = nullptr;
};

// byte I of v as float.  Written as the instruction: the compiler otherwise extracts
// bytes 1 and 2 with a v_bfe_u32 first.
template <int I>
__device__ __forceinline__ float ubyte_f(uint32_t v) {
  float f;
  if (I == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
  if (I == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
  if (I == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
  if (I == 3) asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
  return f;
}

// buffer descriptor over memory that starts at `base`: raw (stride 0) 32-bit data, no
// range check (every offset the kernel forms is in range by construction)
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}

// 16 bytes per lane from a buffer straight into LDS: lane l of the wave writes
// lds_base + 16*l (buffer_load_dwordx4 ... lds); completion is counted by vmcnt
__device__ __forceinline__ void load_to_lds16(__amdgpu_buffer_rsrc_t rsrc, void* lds_base,
                                              uint32_t voffset, uint32_t soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(
      rsrc, (__attribute__((address_space(3))) void*)lds_base, 16, voffset, soffset, 0, 0);
}

// elements between the partial tiles of consecutive K ranges (16-byte aligned rows of 4)
__host__ __device__ inline size_t part_stride(int M, int N) {
  return ((size_t)M * N + 3) / 4 * 4;
}

// packed codes of one (weight row, half of a K step): 32 codes
template <int BITS>
struct WRaw {
  uint4 q[BITS / 4];
  bf16_t s, b;
};

// 8 codes -> the bf16x8 B operand of one MFMA step
template <int BITS>
__device__ __forceinline__ bf16x8_t dequant8(const WRaw<BITS>& r, int t, float s, float b) {
  uint4 o;
  if (BITS == 4) {
    const uint32_t v = reinterpret_cast<const uint32_t*>(&r.q[0])[t];
    const uint32_t ev = v & 0x0f0f0f0fu, od = (v >> 4) & 0x0f0f0f0fu;
    o.x = pack_bf2(fmaf(s, ubyte_f<0>(ev), b), fmaf(s, ubyte_f<0>(od), b));
    o.y = pack_bf2(fmaf(s, ubyte_f<1>(ev), b), fmaf(s, ubyte_f<1>(od), b));
    o.z = pack_bf2(fmaf(s, ubyte_f<2>(ev), b), fmaf(s, ubyte_f<2>(od), b));
    o.w = pack_bf2(fmaf(s, ubyte_f<3>(ev), b), fmaf(s, ubyte_f<3>(od), b));
  } else {
    const uint32_t v0 = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t];
    const uint32_t v1 = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t + 1];
    o.x = pack_bf2(fmaf(s, ubyte_f<0>(v0), b), fmaf(s, ubyte_f<1>(v0), b));
    o.y = pack_bf2(fmaf(s, ubyte_f<2>(v0), b), fmaf(s, ubyte_f<3>(v0), b));
    o.z = pack_bf2(fmaf(s, ubyte_f<0>(v1), b), fmaf(s, ubyte_f<1>(v1), b));
    o.w = pack_bf2(fmaf(s, ubyte_f<2>(v1), b), fmaf(s, ubyte_f<3>(v1), b));
  }
  return __builtin_bit_cast(bf16x8_t, o);
}

// One 32-bit register (two bf16) of that operand: piece P = 0..3.  `lo`, `hi` are the two
// source words prepared by dequant_words().
template <int BITS>
__device__ __forceinline__ void dequant_words(const WRaw<BITS>& r, int t, uint32_t& lo, uint32_t& hi) {
  if (BITS == 4) {
    const uint32_t v = reinterpret_cast<const uint32_t*>(&r.q[0])[t];
    lo = v & 0x0f0f0f0fu;         // even codes, one per byte
    hi = (v >> 4) & 0x0f0f0f0fu;  // odd codes
  } else {
    lo = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t];
    hi = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t + 1];
  }
}
template <int BITS, int P>
__device__ __forceinline__ uint32_t dequant_piece(uint32_t lo, uint32_t hi, float s, float b) {
  if (BITS == 4) return pack_bf2(fmaf(s, ubyte_f<P>(lo), b), fmaf(s, ubyte_f<P>(hi), b));
  const uint32_t v = P < 2 ? lo : hi;
  return pack_bf2(fmaf(s, ubyte_f<(2 * P) & 3>(v), b), fmaf(s, ubyte_f<((2 * P) & 3) + 1>(v), b));
}

// MI = 32-row MFMA tiles per wave along M: the workgroup tile is (64*MI) x 128.
// SB4: rows of scales / biases are 8-byte aligned (K a multiple of 256), so the (scale,
// bias) of four consecutive K steps come in one 8-byte load each instead of four 2-byte
// ones - a 2-byte load that touches 32 rows costs the memory pipeline as much as a
// 16-byte one.
// PAIR: the workgroup's 128 weight rows are 64 rows of the gate matrix and the same 64 rows
// of the up matrix - a wave's two column tiles are (gate, up) of the same 32 output columns,
// so the SwiGLU happens in the epilogue and neither projection is written to memory.
// WIDE: the four waves sit side by side - the workgroup tile is (32*MI) x 256 weight rows,
// every wave owns 64 of them, so nothing is dequantised twice.  Plain GEMM (inputs of up to
// 64 rows): blockIdx.z always owns a K range and the tile leaves as a float32 partial.
// Grouped GEMM (MI = 4: the expert's 128-row tile against 256 weight rows, the wave tile of
// the 256-row kernel): whole K, the usual epilogue.  The same tile for the plain (gate, up)
// pair of a long input: per product it stages half the activation bytes of the 256 x 64 tile
// (the weights, re-read twice as often, are the smaller stream there).
// DEEP (128-row tiles with SB4): four K steps of weights and three of activations in flight
// instead of one.  A 128-row tile holds half the arithmetic per K step of the 256-row one, so
// with one step in flight a workgroup spends most of a step waiting for the next one's loads,
// and the whole launch moves (bytes in flight) / (memory latency): 8 KB per workgroup and
// step, 512 workgroups, 2 us = 2 TB/s, which is what the grouped expert GEMMs of a MoE prompt
// ran at.
// KH (the 256-row tile of the plain GEMM): eight waves, two teams of four that each run the
// kernel's loop over one half of K on tiles of their own; at the end the second team's
// accumulators pass through LDS and are added to the first's, which writes the tile out.  A
// launch of one such tile per CU has two waves per SIMD where four-wave workgroups would leave
// one, without partial tiles in memory.
template <int BITS, int MI, bool GROUPED = false, bool SB4 = false, bool PAIR = false,
          bool WIDE = false, bool DEEP = false, bool KH = false>
__global__ __launch_bounds__(KH ? 512 : 256, KH ? 1 : 2) void qmm_kernel(const QmmParams p) {
  static_assert(!WIDE || GROUPED || !PAIR || MI == 4, "the wide pair tile has 128 rows");
  static_assert(!DEEP || (SB4 && ((MI == 2 && !WIDE) || (WIDE && MI < 4))),
                "the deep pipeline is for 128-row tiles; on the 32- and 64-row wide tiles the flag "
                "selects the ring (K ranges long enough to fill it)");
  static_assert(!KH || (MI == 4 && SB4 && !GROUPED && !DEEP && !(WIDE && PAIR)),
                "two K halves per workgroup: the 256-row tile of the plain and the pair GEMM, "
                "the wide tile of the plain GEMM");
  constexpr int kThreads = 256;  // of a team
  constexpr int BM = WIDE ? 32 * MI : 64 * MI;
  constexpr int WN = PAIR ? 32 : 64;              // output columns per wave
  constexpr int BN = WIDE ? 4 * WN : 2 * WN;      // output columns per workgroup
  constexpr int XR = BM * 8 / kThreads;  // 16-byte x loads per thread and K step
  constexpr int SLOTS = 2;  // activation tiles in LDS
  // (the grouped wide tile leaves through the staging epilogue: four waves x 32*MI rows)
  constexpr int XS_ROWS = WIDE ? 2 * BM : BM;  // (wide: room for the ring's four tiles)
  __shared__ __attribute__((aligned(16))) bf16_t xs[KH ? 2 * SLOTS : SLOTS][XS_ROWS * LDS_STRIDE];

  const int tid = threadIdx.x & (kThreads - 1), lane = tid & 63;  // within the team
  const int team = KH ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * BN;
  const int wm = WIDE ? 0 : (wave >> 1) * (32 * MI), wn = WIDE ? wave * WN : (wave & 1) * WN;
  const int G = p.K >> 6;
  const int wpr = p.K * BITS / 32;
  int m0 = blockIdx.y * BM, m_end = p.M;
  size_t w_off = 0, s_off = 0;
  __shared__ int row_pair[GROUPED ? BM : 1];  // pair index of every row of the tile
  if (GROUPED) {
    const int32_t* ti = p.tiles + 3 * (size_t)blockIdx.y;
    const int e = ti[0];
    if (e < 0) return;  // whole workgroup: tile slot not in use
    m0 = 0;
    m_end = ti[2];
    for (int r = tid; r < BM; r += kThreads) row_pair[r] = r < m_end ? p.sorted[ti[1] + r] : -1;
    w_off = (size_t)e * p.w_stride;
    s_off = (size_t)e * p.s_stride;
    __syncthreads();
  }

  // weight rows of this lane: column tile j -> row n0 + wn + 32*j + lane%32, half lane/32.
  // Addresses are a workgroup-uniform base plus a 32-bit lane offset (the tile spans at
  // most 128 rows), so the loop carries no 64-bit address arithmetic.
  // a wave whose rows all lie past the end of the input (the lower half of a last, short row
  // tile) requests no weights and multiplies nothing: it only helps to load the activation
  // tiles and keeps the barriers, and leaves the CU's vector and matrix pipes to the others
  const bool idle = m0 + wm >= m_end;
  const int frow = lane & 31, kq = lane >> 5;
  const uint32_t* wbase = p.w + w_off + (size_t)n0 * wpr;
  const bf16_t* sbase = p.s + s_off + (size_t)n0 * G;
  const bf16_t* bbase = p.b + s_off + (size_t)n0 * G;
  uint32_t woff[2], soff[2];
  bool w_ok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn + (PAIR ? 0 : j * 32) + frow;
    w_ok[j] = n < p.N;
    const uint32_t rel = (uint32_t)(min(n, p.N - 1) - n0);  // rows past N re-read the last one
    woff[j] = (rel * (uint32_t)wpr + kq * BITS) * 4;  // bytes; 32 codes = BITS words per half K step
    soff[j] = rel * (uint32_t)G * 2;
  }
  // Loads go through buffer instructions: a workgroup-uniform descriptor, a 32-bit lane
  // offset that never changes, and the K step as the scalar offset.
  // (pair mode: a second set of descriptors for the up matrix, column tile 1)
  constexpr int ND = PAIR ? 2 : 1;
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x);
  __amdgpu_buffer_rsrc_t rw[ND], rs[ND], rb[ND];
  rw[0] = make_rsrc(wbase);
  rs[0] = make_rsrc(sbase);
  rb[0] = make_rsrc(bbase);
  if (PAIR) {
    rw[ND - 1] = make_rsrc(p.w2 + w_off + (size_t)n0 * wpr);
    rs[ND - 1] = make_rsrc(p.s2 + s_off + (size_t)n0 * G);
    rb[ND - 1] = make_rsrc(p.b2 + s_off + (size_t)n0 * G);
  }
  // activation rows of this thread: rows past the end re-read the last valid row (their
  // products are never written)
  uint32_t xoff[XR];
#pragma unroll
  for (int r = 0; r < XR; ++r) {
    // 16-byte chunk `id` of the LDS tile (row id/8, slot id%8) holds chunk slot ^ (row%8) of
    // that activation row: rows are 128 bytes apart without padding (the loads write LDS in
    // lane order), and the XOR keeps the operand reads of 16 rows off each other's banks
    const int id = tid + kThreads * r;
    const int trow = id >> 3, kp = (id & 7) ^ (trow & 7);
    const int row = min(trow, m_end - 1 - m0);
    const uint32_t src = GROUPED ? (uint32_t)(row_pair[row] / p.x_div) : (uint32_t)(m0 + row);
    xoff[r] = (src * (uint32_t)p.K + kp * 8) * 2;  // bytes
  }

  struct WStage {
    WRaw<BITS> w[2];
  };

  // the activation tile goes from global memory straight into LDS (no registers, no LDS
  // store instructions): wave instruction r writes chunks [wave*64 + 256*r, +64) in lane
  // order.  Completion is counted by vmcnt.
  constexpr int TILE_BYTES = BM * 128;
  // (a team's tiles: two, or the four of the ring)
  char* const tiles = reinterpret_cast<char*>(&xs[0][0]) + team * ((KH && WIDE ? 4 : SLOTS) * TILE_BYTES);
  auto load_x = [&](int buf, int k0) {
#pragma unroll
    for (int r = 0; r < XR; ++r)
      load_to_lds16(rx, tiles + buf * TILE_BYTES + (wave * 64 + kThreads * r) * 16, xoff[r], k0 * 2);
  };
  // s_waitcnt vmcnt(n) alone (the other counters at "no wait")
  auto wait_vm = [](auto n) {
    constexpr int N = decltype(n)::value;
    __builtin_amdgcn_s_waitcnt((N & 15) | 0x0F70 | ((N >> 4) << 14));
  };
  auto load_w = [&](WStage& st, int k0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int i = 0; i < BITS / 4; ++i)
        st.w[j].q[i] = __builtin_bit_cast(
            uint4, __builtin_amdgcn_raw_buffer_load_b128(rw[PAIR ? j : 0], woff[j] + i * 16, k0 * BITS / 8, 0));
      if (!SB4) {
        st.w[j].s = (bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rs[PAIR ? j : 0], soff[j], (k0 >> 6) * 2, 0);
        st.w[j].b = (bf16_t)__builtin_amdgcn_raw_buffer_load_b16(rb[PAIR ? j : 0], soff[j], (k0 >> 6) * 2, 0);
      }
    }
  };
  // SB4: (scale, bias) of K steps [4*blk, 4*blk+4) for both column tiles
  struct SBlock {
    uint2 s[2], b[2];
  };
  auto load_sb = [&](SBlock& sb, int blk) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      sb.s[j] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(rs[PAIR ? j : 0], soff[j], blk * 8, 0));
      sb.b[j] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(rb[PAIR ? j : 0], soff[j], blk * 8, 0));
    }
  };
  auto pick = [&](const uint2& v, int e) {  // element e (uniform) of four bf16
    const uint32_t w = (e & 2) ? v.y : v.x;
    return (e & 1) ? bf_hi(w) : bf_lo(w);
  };

  // byte offset of this lane's operand chunk of MFMA step t inside its tile row
  int aoff[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) aoff[t] = ((kq * 4 + t) ^ (frow & 7)) * 16;

  floatx16 acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // multiply tile `buf` by the weights held (packed) in `st`
  auto multiply = [&](const WStage& st, int buf, const SBlock& sb, int e) {
    float sc[2], bi[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      sc[j] = SB4 ? pick(sb.s[j], e) : bf2f(st.w[j].s);
      bi[j] = SB4 ? pick(sb.b[j], e) : bf2f(st.w[j].b);
      if (!w_ok[j]) sc[j] = bi[j] = 0.f;
    }
    // MFMA step t covers k = 32*kq + 8*t .. +8 of the K step.  Software pipeline: the A
    // operands and the dequantised B operands of step t+1 are produced while the products
    // of step t run - a 32x32x16 MFMA occupies the matrix core for 8 passes, time for about
    // seven vector instructions of the same wave.  The order is pinned slot by slot (one
    // MFMA, one register of the next B operand, one LDS read) with scheduling barriers;
    // left alone, the compiler clumps the MFMAs behind all the vector work.
    static_assert(MI == 2 || MI == 4 || (WIDE && MI == 1),
                  "eight operand registers are spread over 2*MI slots");
    const char* arow = tiles + buf * TILE_BYTES + (wm + frow) * 128;
    bf16x8_t a[2][MI];
    uint4 bq[2][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
      a[0][i] = *reinterpret_cast<const bf16x8_t*>(arow + i * 32 * 128 + aoff[0]);
#pragma unroll
    for (int j = 0; j < 2; ++j) bq[0][j] = __builtin_bit_cast(uint4, dequant8<BITS>(st.w[j], 0, sc[j], bi[j]));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int cur = t & 1, nxt = cur ^ 1;
      uint32_t lo[2], hi[2];
      if (t < 3) {
#pragma unroll
        for (int j = 0; j < 2; ++j) dequant_words<BITS>(st.w[j], t + 1, lo[j], hi[j]);
      }
#pragma unroll
      for (int m = 0; m < 2 * MI; ++m) {
        const int i = m >> 1, j = m & 1;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            a[cur][i], __builtin_bit_cast(bf16x8_t, bq[cur][j]), acc[i][j], 0, 0, 0);
        if (t < 3) {
          // 8 registers of the next B operands over the 2*MI slots
          constexpr int PER = 8 / (2 * MI);
#pragma unroll
          for (int u = 0; u < PER; ++u) {
            const int r8 = m * PER + u, jj = r8 >> 2;
            uint32_t* dst = reinterpret_cast<uint32_t*>(&bq[nxt][jj]);
            switch (r8 & 3) {
              case 0: dst[0] = dequant_piece<BITS, 0>(lo[jj], hi[jj], sc[jj], bi[jj]); break;
              case 1: dst[1] = dequant_piece<BITS, 1>(lo[jj], hi[jj], sc[jj], bi[jj]); break;
              case 2: dst[2] = dequant_piece<BITS, 2>(lo[jj], hi[jj], sc[jj], bi[jj]); break;
              default: dst[3] = dequant_piece<BITS, 3>(lo[jj], hi[jj], sc[jj], bi[jj]); break;
            }
          }
          if (m < MI)
            a[nxt][m] = *reinterpret_cast<const bf16x8_t*>(arow + m * 32 * 128 + aoff[t + 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // At K step k: the x tile of k is in LDS buffer k&1, the x tile of k+1 in registers
  // (xr), the packed weights of k and k+1 in w0 / w1.  Per step: the next x tile goes to
  // the other LDS buffer and its registers are refilled two steps ahead, the current tile
  // is multiplied, the freed weight stage is refilled two steps ahead; one barrier.
  // this workgroup's K range (all of K unless split; a multiple of four K steps)
  // (two teams: the halves of the workgroup's range - all of K unless the launch splits it)
  const int kr0 = GROUPED ? 0 : (int)blockIdx.z * p.kc;
  const int klen = GROUPED ? p.K : min(p.K, kr0 + p.kc) - kr0;
  const int kb = KH ? kr0 + team * (klen >> 1) : kr0;
  const int ke = KH ? kb + (klen >> 1) : kr0 + klen;
  if (DEEP && !WIDE) {
    // Four register stages each of weights and of activation chunks, requested four steps
    // ahead; the activations pass through registers into the two LDS tiles one step ahead
    // (no LDS-direct loads here: the compiler makes every LDS read wait for ALL outstanding
    // LDS-direct loads, which would drain the pipeline in every step), so every wait count is
    // the compiler's own and exact - the loop is straight-line, its last block of four steps
    // peeled, no request conditional.
    // Step s: barrier (tile s complete, tile s-1 no longer read); store the chunks of step
    // s+1 into the other tile; request the chunks of step s+4; multiply; request the weights
    // of step s+4 into the stage just used.
    WStage wq[4];
    uint4 xq[4][XR];
    SBlock sbc, sbn;
    auto fetch_x = [&](uint4(&dst)[XR], int k0) {
#pragma unroll
      for (int r = 0; r < XR; ++r)
        dst[r] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rx, xoff[r], k0 * 2, 0));
    };
    auto store_x = [&](int buf, const uint4(&src)[XR]) {
#pragma unroll
      for (int r = 0; r < XR; ++r)
        *reinterpret_cast<uint4*>(tiles + buf * TILE_BYTES + (tid + kThreads * r) * 16) = src[r];
    };
    load_sb(sbc, kb >> 8);
    sbn = sbc;
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // (a K range is a multiple of four steps)
      fetch_x(xq[u], kb + u * BK);
      if (!idle) load_w(wq[u], kb + u * BK);
    }
    store_x(0, xq[0]);
    int k0 = kb;
    for (; k0 + 4 * BK < ke; k0 += 4 * BK) {
      load_sb(sbn, (k0 >> 8) + 1);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int k = k0 + u * BK;
        __syncthreads();
        store_x((u + 1) & 1, xq[(u + 1) & 3]);
        fetch_x(xq[u], k + 4 * BK);
        if (!idle) {
          multiply(wq[u], u & 1, sbc, u);
          load_w(wq[u], k + 4 * BK);
        }
      }
      sbc = sbn;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // the last block: everything it needs is under way
      __syncthreads();
      if (u < 3) store_x((u + 1) & 1, xq[(u + 1) & 3]);
      if (!idle) multiply(wq[u], u & 1, sbc, u);
    }
  }
  // RING (the 128-row wide tiles: the plain pair's and the grouped GEMM's): the activation tile is a quarter of the
  // staging area, so four tiles fit; activations (straight into LDS) and weights (four
  // register stages) are requested three K steps ahead.  Every request is unconditional
  // (past the end of K the last step again, never multiplied) and the loop body is four steps
  // long with static stage indices, so that the wait at the end of a step is an exact count:
  // the two youngest steps' requests may still be out.
  constexpr bool RING = WIDE && SB4 && (BITS == 4 || kRing8) && (MI == 4 || DEEP);
  // (8-bit: two steps ahead - three live stages of 16 registers; four spill)
  constexpr int AHEAD = BITS == 4 ? 3 : 2;
  static_assert(RING || !(WIDE && DEEP), "a wide tile with the pipeline flag runs the ring");
  if (RING) {
    constexpr int NW = 2 * (BITS / 4);  // weight requests per step
    WStage wq[4];
    SBlock sbc, sbn;
    const int last = ke - BK;
    load_sb(sbn, kb >> 8);
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      load_x(u, min(kb + u * BK, last));
      load_w(wq[u], min(kb + u * BK, last));
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    for (int k0 = kb; k0 < ke; k0 += 4 * BK) {
      sbc = sbn;  // this block's scales: requested a block ago (the first: above)
      load_sb(sbn, min((k0 >> 8) + 1, (ke >> 8) - 1));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int kn = min(k0 + (u + AHEAD) * BK, last);
        load_x((u + AHEAD) & 3, kn);
        load_w(wq[(u + AHEAD) & 3], kn);
        multiply(wq[u], u, sbc, u);
        wait_vm(std::integral_constant<int, (AHEAD - 1) * (XR + NW)>{});
        __syncthreads();
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the repeats requested past the end: landed before
  }                                      // the staging below reuses this memory
  WStage w0, w1;
  SBlock sb0, sb1;  // current block of four K steps, next block
  if (SB4 && !DEEP && !RING) {
    load_sb(sb0, kb >> 8);
    sb1 = sb0;
  }
  if (!DEEP && !RING) {
    load_x(0, kb);
    if (!idle) load_w(w0, kb);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the tile is in LDS
  __syncthreads();
  // At K step k: the x tile of k is in LDS buffer k&1 and the packed weights of k in w0.
  // The tile and the weights of k+1 are requested first, then tile k is multiplied; every
  // load of the step has landed before the one barrier that ends it.
  int buf = 0;
  for (int k0 = kb; !DEEP && !RING && k0 < ke; k0 += BK) {
    const int ks = k0 >> 6;
    if (SB4 && (ks & 3) == 0) {  // a new block: its values arrived during the previous one
      sb0 = sb1;
      if (k0 + 4 * BK < ke) load_sb(sb1, (ks >> 2) + 1);
    }
    if (k0 + BK < ke) {
      load_x(buf ^ 1, k0 + BK);
      if (!idle) load_w(w1, k0 + BK);
    }
    if (!idle) multiply(w0, buf, sb0, ks & 3);
    w0 = w1;
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    buf ^= 1;
  }

  if (KH) {
    // the second team's sums: through LDS (lane-contiguous floats per accumulator register),
    // added to the first team's, which goes on alone
    float* ex = reinterpret_cast<float*>(&xs[0][0]);
    __syncthreads();  // both teams have finished reading their activation tiles
    if (team == 1) {
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            ex[(((wave * MI + i) * 2 + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (team == 0) {
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[i][j][r] += ex[(((wave * MI + i) * 2 + j) * 16 + r) * 64 + lane];
          asm volatile("" ::: "memory");  // one accumulator's reads at a time: no extra registers
        }
    }
    __syncthreads();  // the sums have been read: the staging below overwrites this memory
    if (team == 1) return;  // (no workgroup barrier after this point)
  }

  if ((WIDE && MI < 4) || (!GROUPED && p.ksplit > 1)) {
    // Split-K: the float32 partial tile of this K range goes to the workspace; a second,
    // small launch adds the ranges in a fixed order (qmm_reduce_kernel).  Pair mode: a range
    // holds the gate partials followed by the up partials (qmm_reduce_swiglu_kernel).
    const size_t one = part_stride(p.M, p.N);
    float* mine = p.part + (size_t)blockIdx.z * (PAIR ? 2 * one : one);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = PAIR ? n0 + wn + frow : n0 + wn + j * 32 + frow;
        float* dst = mine + ((PAIR && j) ? one : 0);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm + i * 32 + (r >> 2) * 8 + kq * 4 + (r & 3);
          if (m < m_end && n < p.N) dst[(size_t)m * p.N + n] = acc[i][j][r];
        }
      }
    return;
  }


  // Epilogue through LDS.  D[i][j] holds column lane%32 (W row n) and rows
  // 8*(r/4) + 4*(lane/32) + r%4 (token m): a wave first writes its (32*MI) x 64 tile as bf16
  // into its own slice of the (now idle) activation buffers - 2-byte LDS stores at constant
  // offsets from one base, so no address lives in registers next to the accumulators -
  // and then copies whole rows out with 16-byte stores (residual added on the way).
  if (!KH) __syncthreads();  // every wave has finished reading the last activation tile
  constexpr int TS = 64 + 8;  // row stride of the staging tile (bf16)
  bf16_t* stage = &xs[0][0] + (size_t)wave * (32 * MI) * TS;
  if (PAIR) {
    // SwiGLU of the bf16-rounded projections (the rounding points of two GEMMs followed by
    // the elementwise kernel), then rows of 32 columns out
    bf16_t* sp = stage + (kq * 4) * TS + frow;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float g = bf2f(f2bf(acc[i][0][r])), u = bf2f(f2bf(acc[i][1][r]));
        sp[(i * 32 + (r >> 2) * 8 + (r & 3)) * TS] = f2bf(g / (1.f + __expf(-g)) * u);
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    const bool vec_ok = (p.N & 7) == 0;
    const int c8 = (lane & 3) * 8;
    for (int it = 0; it < 2 * MI; ++it) {
      const int row = it * 16 + (lane >> 2);
      const int m = m0 + wm + row, n = n0 + wn + c8;
      if (m >= m_end || n >= p.N) continue;
      const size_t o = (size_t)(GROUPED ? row_pair[m] : m) * p.N + n;
      const uint4 v = *reinterpret_cast<const uint4*>(stage + row * TS + c8);
      if (vec_ok) {
        *reinterpret_cast<uint4*>(p.y + o) = v;
      } else {
        const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          if (n + c >= p.N) break;
          p.y[o + c] = f2bf((c & 1) ? bf_hi(w4[c >> 1]) : bf_lo(w4[c >> 1]));
        }
      }
    }
    return;
  }
  {
    bf16_t* sp = stage + (kq * 4) * TS + frow;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          sp[(i * 32 + (r >> 2) * 8 + (r & 3)) * TS + j * 32] = f2bf(acc[i][j][r]);
  }
  // the slice is private to the wave: its own LDS writes are complete before its reads
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_wave_barrier();
  const bool vec_ok = (p.N & 7) == 0;
  const int c8 = (lane & 7) * 8;  // first of this lane's 8 columns
  for (int it = 0; it < 4 * MI; ++it) {
    const int row = it * 8 + (lane >> 3);  // row of the wave's tile
    const int m = m0 + wm + row, n = n0 + wn + c8;
    if (m >= m_end || n >= p.N) continue;
    const size_t o = (size_t)(GROUPED ? row_pair[m] : m) * p.N + n;
    uint4 v = *reinterpret_cast<const uint4*>(stage + row * TS + c8);
    if (vec_ok) {
      if (p.residual) {
        const uint4 rv = *reinterpret_cast<const uint4*>(p.residual + o);
        v.x = pack_bf2(bf_lo(v.x) + bf_lo(rv.x), bf_hi(v.x) + bf_hi(rv.x));
        v.y = pack_bf2(bf_lo(v.y) + bf_lo(rv.y), bf_hi(v.y) + bf_hi(rv.y));
        v.z = pack_bf2(bf_lo(v.z) + bf_lo(rv.z), bf_hi(v.z) + bf_hi(rv.z));
        v.w = pack_bf2(bf_lo(v.w) + bf_lo(rv.w), bf_hi(v.w) + bf_hi(rv.w));
      }
      *reinterpret_cast<uint4*>(p.y + o) = v;
    } else {  // N not a multiple of 8: rows are not 16-byte aligned
      const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        if (n + c >= p.N) break;
        float f = (c & 1) ? bf_hi(w4[c >> 1]) : bf_lo(w4[c >> 1]);
        if (p.residual) f += bf2f(p.residual[o + c]);
        p.y[o + c] = f2bf(f);
      }
    }
  }
}

constexpr int kQmmMaxSplit = 16;  // K ranges the reduce kernel adds
#ifndef EXO_QMM_GROUPED_WIDE
#define EXO_QMM_GROUPED_WIDE 1
#endif
constexpr bool kGroupedWide = EXO_QMM_GROUPED_WIDE != 0;
#ifndef EXO_QMM_DEEP_MIN_K
#define EXO_QMM_DEEP_MIN_K 768
#endif
// K range per workgroup from which the 128-row tile runs the four-stage pipeline (shorter
// ranges never reach its steady state)
constexpr int kDeepMinK = EXO_QMM_DEEP_MIN_K;

// y = bf16(sum over the K ranges, in order) (+ residual): four outputs per thread
__global__ __launch_bounds__(256) void qmm_reduce_kernel(const float* __restrict__ part,
                                                         const bf16_t* __restrict__ residual,
                                                         bf16_t* __restrict__ y, int64_t total,
                                                         int64_t stride, int ksplit, int vec_ok) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  if (vec_ok && i + 4 <= total) {
    float4 v[kQmmMaxSplit];
#pragma unroll
    for (int z = 0; z < kQmmMaxSplit; ++z)
      if (z < ksplit) v[z] = *reinterpret_cast<const float4*>(part + (size_t)z * stride + i);
    float4 t = v[0];
#pragma unroll
    for (int z = 1; z < kQmmMaxSplit; ++z)
      if (z < ksplit) {
        t.x += v[z].x;
        t.y += v[z].y;
        t.z += v[z].z;
        t.w += v[z].w;
      }
    float o[4] = {bf2f(f2bf(t.x)), bf2f(f2bf(t.y)), bf2f(f2bf(t.z)), bf2f(f2bf(t.w))};
    if (residual) {
      const uint2 rv = *reinterpret_cast<const uint2*>(residual + i);
      o[0] += bf_lo(rv.x);
      o[1] += bf_hi(rv.x);
      o[2] += bf_lo(rv.y);
      o[3] += bf_hi(rv.y);
    }
    uint2 w;
    w.x = pack_bf2(o[0], o[1]);
    w.y = pack_bf2(o[2], o[3]);
    *reinterpret_cast<uint2*>(y + i) = w;
  } else {
    for (int64_t e = i; e < min(i + 4, total); ++e) {
      float t = 0.f;
      for (int z = 0; z < ksplit; ++z) t += part[(size_t)z * stride + e];
      t = bf2f(f2bf(t));
      if (residual) t += bf2f(residual[e]);
      y[e] = f2bf(t);
    }
  }
}

// Pair mode: sums of the gate and of the up partials, each rounded to bf16 as the projections
// of two GEMMs would be, then SwiGLU.  `stride` floats between K ranges, `half` between the
// gate and the up partials of one range.
__global__ __launch_bounds__(256) void qmm_reduce_swiglu_kernel(const float* __restrict__ part,
                                                                bf16_t* __restrict__ y,
                                                                int64_t total, int64_t stride,
                                                                int64_t half, int ksplit) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  const int cnt = (int)min((int64_t)4, total - i);
  float g[4] = {0.f, 0.f, 0.f, 0.f}, u[4] = {0.f, 0.f, 0.f, 0.f};
  if (cnt == 4) {  // (rows of partials start at multiples of four floats)
    float4 gv[8], uv[8];
#pragma unroll
    for (int z = 0; z < 8; ++z)
      if (z < ksplit) {
        gv[z] = *reinterpret_cast<const float4*>(part + (size_t)z * stride + i);
        uv[z] = *reinterpret_cast<const float4*>(part + (size_t)z * stride + half + i);
      }
#pragma unroll
    for (int z = 0; z < 8; ++z)
      if (z < ksplit) {
        g[0] += gv[z].x; g[1] += gv[z].y; g[2] += gv[z].z; g[3] += gv[z].w;
        u[0] += uv[z].x; u[1] += uv[z].y; u[2] += uv[z].z; u[3] += uv[z].w;
      }
  } else {
    for (int e = 0; e < cnt; ++e)
      for (int z = 0; z < ksplit; ++z) {
        g[e] += part[(size_t)z * stride + i + e];
        u[e] += part[(size_t)z * stride + half + i + e];
      }
  }
  for (int e = 0; e < cnt; ++e) {
    const float gb = bf2f(f2bf(g[e])), ub = bf2f(f2bf(u[e]));
    y[i + e] = f2bf(gb / (1.f + __expf(-gb)) * ub);
  }
}

// launches of fewer than this many 128 x 128 output tiles may split K (one tile per CU and
// less: 2048x4096 under 1023 rows, 128 tiles, 65 -> 38 us with two K ranges)
constexpr int kQmmSplitTiles = 256;

// K split of a launch: when its 128 x 128 output tiles cover less than half the chip (a
// short input, or a narrow matrix such as a MoE router under a long prompt); chunks of whole
// blocks of four K steps, at least two blocks
void plan_split(int M, int N, int K, bool have_ws, int* ksplit, int* kc) {
  *ksplit = 1;
  *kc = K;
  if (!have_ws || K % 256 != 0) return;
  const int tiles = exo_ceil_div(N, 128) * exo_ceil_div(M, 128);
  if (tiles >= kQmmSplitTiles) return;
  int ks = 1;
  while (ks < 8 && tiles * ks < 256 && K / (ks * 2) >= 256) ks *= 2;
  if (ks == 1) return;
  int c = exo_ceil_div(K, ks);
  c = (c + 255) / 256 * 256;
  *kc = c;
  *ksplit = exo_ceil_div(K, c);
}

// The wide tile (no weight row dequantised twice), K split so that the launch has up to two
// workgroups per CU.  Matrices of more than kQmmWideMaxN rows have enough column tiles for
// the 128-column tile without partials.
constexpr int kQmmWideMaxN = 32768;

int wide_max_split(int N) {
  const int tiles = exo_ceil_div(N, 256);
  int ks = 1;
  while (ks < kQmmMaxSplit && tiles * ks * 2 <= 512) ks *= 2;
  return ks;
}

bool plan_wide(int M, int N, int K, const QmmParams& p, bool have_ws, int* ksplit, int* kc) {
  if (!have_ws || M > 64 || (M > 32 && N < 8192) || N > kQmmWideMaxN || K % 256 != 0) return false;
  if ((((uintptr_t)p.s | (uintptr_t)p.b) & 7) != 0) return false;
  const int cap = wide_max_split(N);
  int ks = 1;
  while (ks < cap && K / (ks * 2) >= 256) ks *= 2;
  int c = exo_ceil_div(K, ks);
  c = (c + 255) / 256 * 256;
  *kc = c;
  *ksplit = exo_ceil_div(K, c);
  return true;
}

// The wide tile is 128 rows tall: it streams the weights once per 128 input rows where the
// 256-row tile streams them once per 256.  That is the smaller stream as long as the matrix
// stays in the 256 MB last-level cache between passes; a vocabulary-sized one (128256x4096:
// 295 MB) does not, and ran 10 % slower through the wide tile (2338 -> 2572 us under 2048 rows).
inline bool weights_stay_cached(int64_t rows, int K, int bits) {
  return rows * K * bits / 8 <= (int64_t)128 << 20;
}

#ifndef EXO_QMM_WIDE_HALVES
#define EXO_QMM_WIDE_HALVES 1
#endif
constexpr bool kWideHalves = EXO_QMM_WIDE_HALVES != 0;
#ifndef EXO_QMM_WIDE_HALVES_MAX_TILES
#define EXO_QMM_WIDE_HALVES_MAX_TILES 256
#endif
constexpr int kWideHalvesMaxTiles = EXO_QMM_WIDE_HALVES_MAX_TILES;
#ifndef EXO_QMM_WIDE_RING_MIN_TILES
#define EXO_QMM_WIDE_RING_MIN_TILES 257
#endif
constexpr int kWideRingMinTiles = EXO_QMM_WIDE_RING_MIN_TILES;

#ifndef EXO_QMM_WIDE_SPLIT
#define EXO_QMM_WIDE_SPLIT 1
#endif
#ifndef EXO_QMM_WIDE_SPLIT_MIN_K
#define EXO_QMM_WIDE_SPLIT_MIN_K 1024
#endif
constexpr bool kWideSplit = EXO_QMM_WIDE_SPLIT != 0;
constexpr int kWideSplitMinK = EXO_QMM_WIDE_SPLIT_MIN_K;
constexpr int kWideSplitMinWgs = 160;
#ifndef EXO_QMM_WIDE_RING_MIN_K
#define EXO_QMM_WIDE_RING_MIN_K 768
#endif
constexpr int kWideRingMinK = EXO_QMM_WIDE_RING_MIN_K;

template <int BITS>
void launch_qmm(const QmmParams& p, hipStream_t st) {
  const int M = p.M, N = p.N;
  if (p.wide) {
    const dim3 g(exo_ceil_div(N, 256), 1, p.ksplit);
    // K ranges of twelve steps or more fill the ring (4096x14336 4-bit at 17 rows 22.3 -> 19.3
    // us); on short ranges its start-up costs more than it returns (14336x4096: 20.5 -> 21.4)
    const bool ring = p.kc >= kWideRingMinK;
    if (M <= 32 && ring)
      exo_note_variant("qmm_kernel<%d, 1, false, true, false, true, true>", BITS), qmm_kernel<BITS, 1, false, true, false, true, true><<<g, 256, 0, st>>>(p);
    else if (M <= 32)
      exo_note_variant("qmm_kernel<%d, 1, false, true, false, true>", BITS), qmm_kernel<BITS, 1, false, true, false, true><<<g, 256, 0, st>>>(p);
    else if (ring)
      exo_note_variant("qmm_kernel<%d, 2, false, true, false, true, true>", BITS), qmm_kernel<BITS, 2, false, true, false, true, true><<<g, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 2, false, true, false, true>", BITS), qmm_kernel<BITS, 2, false, true, false, true><<<g, 256, 0, st>>>(p);
    const int64_t total = (int64_t)M * N;
    const int vec_ok = (((uintptr_t)p.y | (uintptr_t)p.residual) & 7) == 0;
    qmm_reduce_kernel<<<dim3(exo_ceil_div(exo_ceil_div(total, 4), 256)), 256, 0, st>>>(
        p.part, p.residual, p.y, total, (int64_t)part_stride(M, N), p.ksplit, vec_ok);
    return;
  }
  // taller inputs: 256-row tiles halve the dequantisation work and the LDS reads per output
  const dim3 g2(exo_ceil_div(N, 128), exo_ceil_div(M, 128), p.ksplit), g4(exo_ceil_div(N, 128), exo_ceil_div(M, 256));
  const bool sb4 = p.K % 256 == 0 && (((uintptr_t)p.s | (uintptr_t)p.b) & 7) == 0;
  // a grid of up to 128 of the tall tiles leaves at least half of the CUs idle: twice as
  // many 128-row tiles are faster there (1024x4096 at 2046 rows: 89 -> 70 us; 4096x4096 at
  // 1023 rows, exactly 128 tall tiles: 93 -> 77 us), not beyond (192 tall tiles: 88 vs 97 us)
  const bool small_grid = (int64_t)g4.x * g4.y <= 128;
  if (M <= 128 || small_grid || p.ksplit > 1) {  // (only the 128-row tile splits K)
    // K ranges of 1024 or more, all of one length: the wide tile with eight waves, the two
    // teams on the halves of the workgroup's range (no weight row dequantised twice, the ring,
    // as many partial tiles as before): 4096x14336 4-bit under 600 rows 145 -> 104 us, 4096x4096
    // 52 -> 43, 6144x4096 under 300 rows 48 -> 40, 14336x4096 under 128 rows 41 -> 37; launches
    // that would have fewer than 160 such workgroups lose (2048x4096 under 1022 rows, 128
    // workgroups: 37 -> 42 us)
    if (kWideSplit && sb4 && (BITS == 4 || kRing8) && p.ksplit > 1 && M > 64 && p.kc >= kWideSplitMinK &&
        p.kc % 512 == 0 && p.K % p.kc == 0 &&
        (int64_t)exo_ceil_div(N, 256) * exo_ceil_div(M, 128) * p.ksplit >= kWideSplitMinWgs)
      exo_note_variant("qmm_kernel<%d, 4, false, true, false, true, false, true>", BITS), qmm_kernel<BITS, 4, false, true, false, true, false, true>
          <<<dim3(exo_ceil_div(N, 256), exo_ceil_div(M, 128), p.ksplit), 512, 0, st>>>(p);
    else if (sb4 && p.kc >= kDeepMinK)
      exo_note_variant("qmm_kernel<%d, 2, false, true, false, false, true>", BITS), qmm_kernel<BITS, 2, false, true, false, false, true><<<g2, 256, 0, st>>>(p);
    else if (sb4)
      exo_note_variant("qmm_kernel<%d, 2, false, true>", BITS), qmm_kernel<BITS, 2, false, true><<<g2, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 2, false, false>", BITS), qmm_kernel<BITS, 2, false, false><<<g2, 256, 0, st>>>(p);
    if (p.ksplit > 1) {
      const int64_t total = (int64_t)M * N;
      const int vec_ok = (((uintptr_t)p.y | (uintptr_t)p.residual) & 7) == 0;
      qmm_reduce_kernel<<<dim3(exo_ceil_div(exo_ceil_div(total, 4), 256)), 256, 0, st>>>(
          p.part, p.residual, p.y, total, (int64_t)part_stride(M, N), p.ksplit, vec_ok);
    }
  } else {
    // up to one tall tile per CU: eight waves per tile, K in two halves (four-wave workgroups
    // leave one wave per SIMD there).  4096x4096 under 2046 rows, 256 tiles: 95.0 -> 89.7 us,
    // 4096x14336: 279 -> 266 us, 6144x4096 under 1022 rows, 192 tiles: 82.0 -> 77.5 us; more
    // tiles than CUs lose (384: 127 -> 144 us, 512: 155 -> 171 us)
    const int64_t tall = (int64_t)g4.x * g4.y;
    // 4-bit, up to one WIDE tile (128 x 256) per CU: the two K halves on that tile instead,
    // with the ring of four - half the staged activation bytes per product and the weights
    // three steps ahead (4096x4096 under 2046 rows 89.5 -> 84.8 us, 4096x14336 280 -> 239,
    // 6144x4096 under 1022 rows 87 -> 78, 8192x8192 under 600 rows 138 -> 122; with up to 512
    // such tiles it wins on some shapes and loses on others, so 256 it is)
    const dim3 gw(exo_ceil_div(N, 256), exo_ceil_div(M, 128));
    if (kWideHalves && sb4 && (BITS == 4 || kRing8) && (int64_t)gw.x * gw.y <= kWideHalvesMaxTiles && p.K % 512 == 0 && p.K >= 1024)
      exo_note_variant("qmm_kernel<%d, 4, false, true, false, true, false, true>", BITS), qmm_kernel<BITS, 4, false, true, false, true, false, true><<<gw, 512, 0, st>>>(p);
    else if (sb4 && tall <= 256 && p.K % 512 == 0 && p.K >= 1024)
      exo_note_variant("qmm_kernel<%d, 4, false, true, false, false, false, true>", BITS), qmm_kernel<BITS, 4, false, true, false, false, false, true><<<g4, 512, 0, st>>>(p);
    // more wide tiles than CUs: the wide tile with the ring, four waves (6144x4096 under 2046
    // rows 144 -> 126 us, 4096x14336 under 4094 rows 523 -> 472, 8192x8192 under 2046 rows
    // 292 -> 270)
    else if (sb4 && (BITS == 4 || kRing8) && (int64_t)gw.x * gw.y >= kWideRingMinTiles && weights_stay_cached(N, p.K, BITS))
      exo_note_variant("qmm_kernel<%d, 4, false, true, false, true>", BITS), qmm_kernel<BITS, 4, false, true, false, true><<<gw, 256, 0, st>>>(p);
    else if (sb4)
      exo_note_variant("qmm_kernel<%d, 4, false, true>", BITS), qmm_kernel<BITS, 4, false, true><<<g4, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 4, false, false>", BITS), qmm_kernel<BITS, 4, false, false><<<g4, 256, 0, st>>>(p);
  }
}

template <int BITS>
void launch_grouped(const QmmParams& p, int row_tiles, hipStream_t st) {
  const bool sb4 = p.K % 256 == 0 &&
                   (((uintptr_t)p.s | (uintptr_t)p.b | (uintptr_t)p.s2 | (uintptr_t)p.b2) & 7) == 0;
  const bool pair = p.w2 != nullptr;  // (gate, up) with the SwiGLU in the epilogue
  // Four waves side by side on 256 weight rows per workgroup and K step instead of 2 x 2 on
  // 128: the expert matrices are streamed once per 128-row tile whatever the tile's width, and
  // a wave of the 2 x 2 layout dequantises the same 64 weight rows as its neighbour.
  if (sb4 && kGroupedWide) {
    const dim3 grid(exo_ceil_div(p.N, pair ? 128 : 256), row_tiles);
    if (pair)
      exo_note_variant("qmm_kernel<%d, 4, true, true, true, true>", BITS), qmm_kernel<BITS, 4, true, true, true, true><<<grid, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 4, true, true, false, true>", BITS), qmm_kernel<BITS, 4, true, true, false, true><<<grid, 256, 0, st>>>(p);
    return;
  }
  const dim3 grid(exo_ceil_div(p.N, pair ? 64 : 128), row_tiles);
  if (pair) {
    if (sb4 && p.K >= kDeepMinK)
      exo_note_variant("qmm_kernel<%d, 2, true, true, true, false, true>", BITS), qmm_kernel<BITS, 2, true, true, true, false, true><<<grid, 256, 0, st>>>(p);
    else if (sb4)
      exo_note_variant("qmm_kernel<%d, 2, true, true, true>", BITS), qmm_kernel<BITS, 2, true, true, true><<<grid, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 2, true, false, true>", BITS), qmm_kernel<BITS, 2, true, false, true><<<grid, 256, 0, st>>>(p);
  } else if (sb4 && p.K >= kDeepMinK) {
    exo_note_variant("qmm_kernel<%d, 2, true, true, false, false, true>", BITS), qmm_kernel<BITS, 2, true, true, false, false, true><<<grid, 256, 0, st>>>(p);
  } else if (sb4) {
    exo_note_variant("qmm_kernel<%d, 2, true, true>", BITS), qmm_kernel<BITS, 2, true, true><<<grid, 256, 0, st>>>(p);
  } else {
    exo_note_variant("qmm_kernel<%d, 2, true, false>", BITS), qmm_kernel<BITS, 2, true, false><<<grid, 256, 0, st>>>(p);
  }
}

constexpr int kGroupBM = 128;  // rows per tile of the grouped GEMM
constexpr int kGroupMaxE = 256;

// Sort the (token, slot) pairs by expert and cut every expert's run into tiles of
// kGroupBM rows.  One workgroup: counts in LDS, a wave's scan over the experts, a second
// pass that scatters the pair indices.  The order inside an expert's run depends on
// atomic arrival order; every output row is computed independently of its tile position,
// so results do not.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* __restrict__ idx, int P,
                                                         int E, int32_t* __restrict__ sorted,
                                                         int32_t* __restrict__ tiles,
                                                         int max_tiles) {
  __shared__ int cnt[kGroupMaxE], off[kGroupMaxE], cur[kGroupMaxE], tile0[kGroupMaxE + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int i = tid; i < P; i += 1024) {
    const int e = idx[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (tid < 64) {
    // exclusive scans of the counts and of the tile counts over the experts by one wave:
    // lane l owns experts [4l, 4l+4) (E <= 256); a scan over one thread's loop of dependent
    // LDS accesses took 5 of this launch's 10.8 us at 128 experts
    int c[4], o = 0, t = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 4 * tid + j;
      c[j] = e < E ? cnt[e] : 0;
      o += c[j];
      t += (c[j] + kGroupBM - 1) / kGroupBM;
    }
    int po = o, pt = t;  // inclusive prefix over the lanes
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int uo = __shfl_up(po, d, 64), ut = __shfl_up(pt, d, 64);
      if (tid >= d) {
        po += uo;
        pt += ut;
      }
    }
    o = po - o;  // exclusive
    t = pt - t;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 4 * tid + j;
      if (e < E) {
        off[e] = o;
        cur[e] = o;
        tile0[e] = t;
      }
      o += c[j];
      t += (c[j] + kGroupBM - 1) / kGroupBM;
    }
    if (tid == 63) tile0[E] = pt;
  }
  __syncthreads();
  for (int i = tid; i < P; i += 1024) {
    const int e = idx[i];
    if (e >= 0 && e < E) sorted[atomicAdd(&cur[e], 1)] = i;
  }
  for (int e = tid; e < E; e += 1024) {
    const int nt = tile0[e + 1] - tile0[e];
    for (int j = 0; j < nt; ++j) {
      int32_t* t = tiles + 3 * (size_t)(tile0[e] + j);
      t[0] = e;
      t[1] = off[e] + j * kGroupBM;
      t[2] = min(kGroupBM, cnt[e] - j * kGroupBM);
    }
  }
  for (int t = tile0[E] + tid; t < max_tiles; t += 1024) tiles[3 * (size_t)t] = -1;
}

int group_max_tiles(int64_t pairs, int E) { return (int)((pairs + kGroupBM - 1) / kGroupBM) + E; }

}  // namespace

extern "C" int64_t exo_moe_group_workspace(int T, int topk, int E) {
  if (T <= 0 || topk <= 0 || E <= 0) return 0;
  const int64_t pairs = (int64_t)T * topk;
  return (pairs + 3 * (int64_t)group_max_tiles(pairs, E)) * 4;
}

extern "C" int exo_moe_group(const int32_t* idx, int T, int topk, int E, void* workspace,
                             int64_t workspace_bytes, exo_stream_t stream) {
  EXO_REQUIRE(idx && workspace, "exo_moe_group: null pointer");
  EXO_REQUIRE(T > 0 && topk > 0 && E > 0 && E <= kGroupMaxE && (int64_t)T * topk < (1ll << 30),
              "exo_moe_group: need T>0, topk>0, 0<E<=%d; got T=%d topk=%d E=%d", kGroupMaxE, T,
              topk, E);
  EXO_REQUIRE(workspace_bytes >= exo_moe_group_workspace(T, topk, E),
              "exo_moe_group: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)exo_moe_group_workspace(T, topk, E));
  const int P = T * topk;
  int32_t* sorted = reinterpret_cast<int32_t*>(workspace);
  moe_group_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(idx, P, E, sorted, sorted + P,
                                                       group_max_tiles(P, E));
  EXO_CHECK_LAUNCH("exo_moe_group");
  return EXO_OK;
}

static int gather_qmm_impl(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, const uint32_t* w2, const uint16_t* s2,
                           const uint16_t* b2, const void* workspace, uint16_t* y, int T, int topk,
                           int x_rows, int E, int N, int K, int bits, int group_size,
                           exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_gather_qmm: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_gather_qmm: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(N > 0 && K > 0 && K % 64 == 0, "exo_gather_qmm: bad shape N=%d K=%d", N, K);
  EXO_REQUIRE(T > 0 && topk > 0 && E > 0 && E <= kGroupMaxE && (int64_t)T * topk < (1ll << 30),
              "exo_gather_qmm: bad T=%d topk=%d E=%d", T, topk, E);
  EXO_REQUIRE(x_rows == 1 || x_rows == topk, "exo_gather_qmm: x_rows must be 1 or topk, got %d",
              x_rows);
  EXO_REQUIRE(x && w && scales && biases && workspace && y, "exo_gather_qmm: null pointer");
  const int P = T * topk;
  const int max_tiles = group_max_tiles(P, E);
  EXO_REQUIRE(max_tiles <= 65535, "exo_gather_qmm: %d row tiles exceed the grid limit", max_tiles);
  EXO_REQUIRE((int64_t)T * topk * K < (1ll << 31),
              "exo_gather_qmm: T*topk*K=%lld exceeds 32-bit byte offsets",
              (long long)T * topk * K);
  QmmParams p{x, w, scales, biases, nullptr, y, P, N, K};
  p.sorted = reinterpret_cast<const int32_t*>(workspace);
  p.tiles = p.sorted + P;
  p.x_div = x_rows == 1 ? topk : 1;
  p.w_stride = (size_t)N * (K * bits / 32);
  p.s_stride = (size_t)N * (K / 64);
  p.ksplit = 1;
  p.kc = K;
  p.part = nullptr;
  p.w2 = w2;
  p.s2 = s2;
  p.b2 = b2;
  if (bits == 4)
    launch_grouped<4>(p, max_tiles, (hipStream_t)stream);
  else
    launch_grouped<8>(p, max_tiles, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_gather_qmm");
  return EXO_OK;
}

extern "C" int exo_gather_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const void* workspace, uint16_t* y, int T,
                              int topk, int x_rows, int E, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
  return gather_qmm_impl(x, w, scales, biases, nullptr, nullptr, nullptr, workspace, y, T, topk,
                         x_rows, E, N, K, bits, group_size, stream);
}

extern "C" int exo_gather_qmm_swiglu(const uint16_t* x, const uint32_t* w_gate,
                                     const uint16_t* s_gate, const uint16_t* b_gate,
                                     const uint32_t* w_up, const uint16_t* s_up,
                                     const uint16_t* b_up, const void* workspace, uint16_t* y,
                                     int T, int topk, int x_rows, int E, int N, int K, int bits,
                                     int group_size, exo_stream_t stream) {
  EXO_REQUIRE(w_up && s_up && b_up, "exo_gather_qmm_swiglu: null pointer");
  return gather_qmm_impl(x, w_gate, s_gate, b_gate, w_up, s_up, b_up, workspace, y, T, topk,
                         x_rows, E, N, K, bits, group_size, stream);
}

// K ranges of a pair launch of up to 128 rows whose 128 x 64 output tiles (of the pair) leave
// half of the chip or more idle - the MLP of a small model under a short prompt (8192 x 2048
// pair at 126 rows: 128 tiles): ranges of four K steps or more until the launch has up to
// one workgroup per CU; a second launch adds the ranges and applies the SwiGLU.
int pair_max_split(int M, int N) {
  if (M > 128) return 1;
  const int64_t tiles = (int64_t)exo_ceil_div(N, 64) * exo_ceil_div(M, 128);
  int ks = 1;
  while (ks < 8 && tiles * ks * 2 <= 256) ks *= 2;
  return ks;
}

void plan_pair_split(const QmmParams& p, bool have_ws, int* ksplit, int* kc) {
  *ksplit = 1;
  *kc = p.K;
  if (!have_ws || p.K % 256 != 0) return;
  const int cap = pair_max_split(p.M, p.N);
  int ks = 1;
  while (ks < cap && p.K / (ks * 2) >= 256) ks *= 2;
  if (ks == 1) return;
  int c = exo_ceil_div(p.K, ks);
  c = (c + 255) / 256 * 256;
  *kc = c;
  *ksplit = exo_ceil_div(p.K, c);
}

#ifndef EXO_QMM_PAIR_WIDE_MIN_M
#define EXO_QMM_PAIR_WIDE_MIN_M 129
#endif
// rows from which the (gate, up) pair takes the 128 x 128 tile with the four waves side by
// side instead of the 256 x 64 one: ahead at every length measured (14336x4096 pair 4-bit:
// 600 rows 216 -> 205 us, 1022 rows 303 -> 288, 2046 rows 504 -> 487, 4094 rows 954 -> 919;
// 12288x4096 8-bit at 600 rows, whose third 256-row tile is mostly empty, 195 -> 139 us)
constexpr int kPairWideMinM = EXO_QMM_PAIR_WIDE_MIN_M;

template <int BITS>
void launch_pair(const QmmParams& p, hipStream_t st) {
  const dim3 g2(exo_ceil_div(p.N, 64), exo_ceil_div(p.M, 128), p.ksplit),
      g4(exo_ceil_div(p.N, 64), exo_ceil_div(p.M, 256));
  const bool sb4 = p.K % 256 == 0 &&
                   (((uintptr_t)p.s | (uintptr_t)p.b | (uintptr_t)p.s2 | (uintptr_t)p.b2) & 7) == 0;
  const bool small_grid = (int64_t)g4.x * g4.y <= 128;
  if (p.M <= 128 || small_grid) {
    if (sb4 && p.kc >= kDeepMinK)
      exo_note_variant("qmm_kernel<%d, 2, false, true, true, false, true>", BITS), qmm_kernel<BITS, 2, false, true, true, false, true><<<g2, 256, 0, st>>>(p);
    else if (sb4)
      exo_note_variant("qmm_kernel<%d, 2, false, true, true>", BITS), qmm_kernel<BITS, 2, false, true, true><<<g2, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 2, false, false, true>", BITS), qmm_kernel<BITS, 2, false, false, true><<<g2, 256, 0, st>>>(p);
    if (p.ksplit > 1) {
      const int64_t total = (int64_t)p.M * p.N, one = (int64_t)part_stride(p.M, p.N);
      qmm_reduce_swiglu_kernel<<<dim3(exo_ceil_div(exo_ceil_div(total, 4), 256)), 256, 0, st>>>(
          p.part, p.y, total, 2 * one, one, p.ksplit);
    }
  } else {
    // (up to one tall tile per CU: eight waves per tile, as in launch_qmm)
    if (sb4 && (int64_t)g4.x * g4.y <= 256 && p.K % 512 == 0 && p.K >= 1024)
      exo_note_variant("qmm_kernel<%d, 4, false, true, true, false, false, true>", BITS), qmm_kernel<BITS, 4, false, true, true, false, false, true><<<g4, 512, 0, st>>>(p);
    else if (sb4 && p.M >= kPairWideMinM && weights_stay_cached(2 * (int64_t)p.N, p.K, BITS))
      exo_note_variant("qmm_kernel<%d, 4, false, true, true, true>", BITS), qmm_kernel<BITS, 4, false, true, true, true><<<dim3(exo_ceil_div(p.N, 128), exo_ceil_div(p.M, 128)), 256, 0, st>>>(p);
    else if (sb4)
      exo_note_variant("qmm_kernel<%d, 4, false, true, true>", BITS), qmm_kernel<BITS, 4, false, true, true><<<g4, 256, 0, st>>>(p);
    else
      exo_note_variant("qmm_kernel<%d, 4, false, false, true>", BITS), qmm_kernel<BITS, 4, false, false, true><<<g4, 256, 0, st>>>(p);
  }
}

extern "C" int64_t exo_qmm_swiglu_workspace(int M, int N) {
  if (M <= 0 || N <= 0) return 0;
  const int ks = pair_max_split(M, N);
  return ks > 1 ? (int64_t)ks * 2 * (int64_t)part_stride(M, N) * 4 : 0;
}

extern "C" int exo_qmm_swiglu_ws(const uint16_t* x, const uint32_t* w_gate,
                                 const uint16_t* s_gate, const uint16_t* b_gate,
                                 const uint32_t* w_up, const uint16_t* s_up,
                                 const uint16_t* b_up, uint16_t* y, void* workspace,
                                 int64_t workspace_bytes, int M, int N, int K, int bits,
                                 int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_qmm_swiglu: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_qmm_swiglu: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 64 == 0, "exo_qmm_swiglu: bad shape M=%d N=%d K=%d",
              M, N, K);
  EXO_REQUIRE(x && w_gate && s_gate && b_gate && w_up && s_up && b_up && y,
              "exo_qmm_swiglu: null pointer");
  if (M == 0) return EXO_OK;
  EXO_REQUIRE(exo_ceil_div(M, 128) <= 65535, "exo_qmm_swiglu: M=%d too large", M);
  EXO_REQUIRE((int64_t)M * K < (1ll << 31),
              "exo_qmm_swiglu: M*K=%lld exceeds 32-bit byte offsets", (long long)M * K);
  if (exo_qmm_swiglu_workspace(M, N) == 0) workspace = nullptr;
  EXO_REQUIRE(!workspace || (workspace_bytes >= exo_qmm_swiglu_workspace(M, N) &&
                             ((uintptr_t)workspace & 255) == 0),
              "exo_qmm_swiglu_ws: workspace of %lld bytes, need %lld (256-byte aligned)",
              (long long)workspace_bytes, (long long)exo_qmm_swiglu_workspace(M, N));
  QmmParams p{x, w_gate, s_gate, b_gate, nullptr, y, M, N, K};
  p.sorted = nullptr;
  p.tiles = nullptr;
  p.x_div = 1;
  p.w_stride = p.s_stride = 0;
  p.w2 = w_up;
  p.s2 = s_up;
  p.b2 = b_up;
  const bool sb4 = K % 256 == 0 &&
                   (((uintptr_t)s_gate | (uintptr_t)b_gate | (uintptr_t)s_up | (uintptr_t)b_up) & 7) == 0;
  plan_pair_split(p, workspace != nullptr && sb4, &p.ksplit, &p.kc);
  p.part = reinterpret_cast<float*>(workspace);
  if (bits == 4)
    launch_pair<4>(p, (hipStream_t)stream);
  else
    launch_pair<8>(p, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_qmm_swiglu");
  return EXO_OK;
}

extern "C" int exo_qmm_swiglu(const uint16_t* x, const uint32_t* w_gate, const uint16_t* s_gate,
                              const uint16_t* b_gate, const uint32_t* w_up, const uint16_t* s_up,
                              const uint16_t* b_up, uint16_t* y, int M, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
  return exo_qmm_swiglu_ws(x, w_gate, s_gate, b_gate, w_up, s_up, b_up, y, nullptr, 0, M, N, K,
                           bits, group_size, stream);
}

extern "C" int64_t exo_qmm_workspace(int M, int N) {
  if (M <= 0 || N <= 0) return 0;
  int64_t ranges = 0;
  const int64_t tiles = (int64_t)exo_ceil_div(N, 128) * exo_ceil_div(M, 128);
  if (tiles < kQmmSplitTiles) {
    ranges = 1;
    while (ranges < 8 && tiles * ranges < 256) ranges *= 2;  // as plan_split
  }
  if (M <= 64 && N <= kQmmWideMaxN) ranges = std::max<int64_t>(ranges, wide_max_split(N));
  return ranges * (int64_t)part_stride(M, N) * 4;
}

extern "C" int exo_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M,
                       int N, int K, int bits, int group_size, exo_stream_t stream) {
  return exo_qmm_ws(x, w, scales, biases, residual, y, nullptr, 0, M, N, K, bits, group_size,
                    stream);
}

extern "C" int exo_qmm_ws(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, const uint16_t* residual, uint16_t* y,
                          void* workspace, int64_t workspace_bytes, int M, int N, int K,
                          int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_qmm: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_qmm: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 64 == 0, "exo_qmm: bad shape M=%d N=%d K=%d", M, N,
              K);
  EXO_REQUIRE(x && w && scales && biases && y, "exo_qmm: null pointer");
  if (M == 0) return EXO_OK;
  if (exo_qmm_workspace(M, N) == 0) workspace = nullptr;
  EXO_REQUIRE(!workspace || (workspace_bytes >= exo_qmm_workspace(M, N) &&
                             ((uintptr_t)workspace & 255) == 0),
              "exo_qmm_ws: workspace of %lld bytes, need %lld (256-byte aligned)",
              (long long)workspace_bytes, (long long)exo_qmm_workspace(M, N));
  QmmParams p{x, w, scales, biases, residual, y, M, N, K};
  p.sorted = nullptr;
  p.tiles = nullptr;
  p.x_div = 1;
  p.w_stride = p.s_stride = 0;
  p.wide = plan_wide(M, N, K, p, workspace != nullptr, &p.ksplit, &p.kc);
  if (!p.wide) plan_split(M, N, K, workspace != nullptr, &p.ksplit, &p.kc);
  p.part = reinterpret_cast<float*>(workspace);
  EXO_REQUIRE(exo_ceil_div(M, 128) <= 65535, "exo_qmm: M=%d too large", M);
  EXO_REQUIRE((int64_t)M * K < (1ll << 31), "exo_qmm: M*K=%lld exceeds 32-bit byte offsets",
              (long long)M * K);
  if (bits == 4)
    launch_qmm<4>(p, (hipStream_t)stream);
  else
    launch_qmm<8>(p, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_qmm");
  return EXO_OK;
}
