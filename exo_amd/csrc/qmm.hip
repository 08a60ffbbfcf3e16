// Quantised matmul for prefill (any M): y[M,N] = x[M,K] @ dq(W)[N,K]^T.
//
// Matrix-core design for gfx950.  A 256-thread workgroup (2 x 2 waves) computes a
// 256x128 output tile (128x128 for M <= 128); one 64-wide K step per iteration = exactly
// one quantisation group, so a packed row segment needs a single (scale, bias).
//  * Activations go through LDS (two buffers: the next tile is stored while the current
//    one is multiplied, one barrier per K step).  LDS bandwidth, not the matrix cores, is
//    what limits this kernel, so the weights do NOT go through LDS:
//  * every wave loads the packed words of its own 64 weight rows straight into registers
//    in the MFMA B-operand layout - lane (row, half) takes 16 B (4-bit) or 32 B (8-bit) =
//    32 consecutive codes - and dequantises them there to bf16(fma(s, q, b)) with
//    v_cvt_f32_ubyteN.  MFMA step t of a K step then covers k = 32*half + 8*t .. +8, and
//    the A operand is read from the activation tile at that same offset, so no data is
//    rearranged.  The two waves that share weight rows dequantise them twice; in exchange
//    the LDS carries a third less traffic and its writes are plain copies.
//  * v_mfma_f32_32x32x16_bf16, float32 accumulators (128x64 per wave), global loads two
//    K steps ahead in registers.  LDS rows are padded by 16 bytes: conflict-free b128.
//  * grouped mode (MoE prefill): blockIdx.y is a tile of one expert's sorted rows.
#include "../../include/exo_mi355x.h"
#include "common.h"

namespace {

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
};

__device__ __forceinline__ float ubyte_f(uint32_t v, int i) {
  return (float)((v >> (8 * i)) & 0xffu);  // v_cvt_f32_ubyteN
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
    o.x = pack_bf2(fmaf(s, ubyte_f(ev, 0), b), fmaf(s, ubyte_f(od, 0), b));
    o.y = pack_bf2(fmaf(s, ubyte_f(ev, 1), b), fmaf(s, ubyte_f(od, 1), b));
    o.z = pack_bf2(fmaf(s, ubyte_f(ev, 2), b), fmaf(s, ubyte_f(od, 2), b));
    o.w = pack_bf2(fmaf(s, ubyte_f(ev, 3), b), fmaf(s, ubyte_f(od, 3), b));
  } else {
    const uint32_t v0 = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t];
    const uint32_t v1 = reinterpret_cast<const uint32_t*>(&r.q[0])[2 * t + 1];
    o.x = pack_bf2(fmaf(s, ubyte_f(v0, 0), b), fmaf(s, ubyte_f(v0, 1), b));
    o.y = pack_bf2(fmaf(s, ubyte_f(v0, 2), b), fmaf(s, ubyte_f(v0, 3), b));
    o.z = pack_bf2(fmaf(s, ubyte_f(v1, 0), b), fmaf(s, ubyte_f(v1, 1), b));
    o.w = pack_bf2(fmaf(s, ubyte_f(v1, 2), b), fmaf(s, ubyte_f(v1, 3), b));
  }
  return __builtin_bit_cast(bf16x8_t, o);
}

// MI = 32-row MFMA tiles per wave along M: the workgroup tile is (64*MI) x 128.
template <int BITS, int MI, bool GROUPED = false>
__global__ __launch_bounds__(256, 2) void qmm_kernel(const QmmParams p) {
  constexpr int kThreads = 256;
  constexpr int BM = 64 * MI, BN = 128;
  constexpr int XR = BM * 8 / kThreads;  // 16-byte x loads per thread and K step
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][BM * LDS_STRIDE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * BN;
  const int wm = (wave >> 1) * (32 * MI), wn = (wave & 1) * 64;
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

  // weight rows of this lane: column tile j -> row n0 + wn + 32*j + lane%32, half lane/32
  const int frow = lane & 31, kq = lane >> 5;
  const uint32_t* wsrc[2];
  const bf16_t* ssrc[2];
  const bf16_t* bsrc[2];
  bool w_ok[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn + j * 32 + frow;
    w_ok[j] = n < p.N;
    const size_t row = (size_t)(w_ok[j] ? n : 0);
    wsrc[j] = p.w + w_off + row * wpr + kq * BITS;  // 32 codes = BITS words per half K step
    ssrc[j] = p.s + s_off + row * G;
    bsrc[j] = p.b + s_off + row * G;
  }

  struct XStage {
    uint4 xa[XR];
  };
  struct WStage {
    WRaw<BITS> w[2];
  };

  auto load_x = [&](XStage& st, int k0) {
#pragma unroll
    for (int r = 0; r < XR; ++r) {
      const int id = tid + kThreads * r;
      const int row = id >> 3, kp = id & 7;
      if (m0 + row < m_end) {
        const size_t src = GROUPED ? (size_t)(row_pair[row] / p.x_div) : (size_t)(m0 + row);
        st.xa[r] = *reinterpret_cast<const uint4*>(p.x + src * p.K + k0 + kp * 8);
      } else {
        st.xa[r] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto load_w = [&](WStage& st, int k0) {
    const int kw = k0 * BITS / 32;  // word offset of this K step
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int i = 0; i < BITS / 4; ++i)
        st.w[j].q[i] = *reinterpret_cast<const uint4*>(wsrc[j] + kw + i * 4);
      st.w[j].s = ssrc[j][k0 >> 6];
      st.w[j].b = bsrc[j][k0 >> 6];
    }
  };

  auto store_x = [&](const XStage& st, int buf) {
#pragma unroll
    for (int r = 0; r < XR; ++r) {
      const int id = tid + kThreads * r;
      const int row = id >> 3, kp = id & 7;
      *reinterpret_cast<uint4*>(&xs[buf][row * LDS_STRIDE + kp * 8]) = st.xa[r];
    }
  };

  floatx16 acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // multiply tile `buf` by the weights held (packed) in `st`
  auto multiply = [&](const WStage& st, int buf) {
    float sc[2], bi[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      sc[j] = w_ok[j] ? bf2f(st.w[j].s) : 0.f;
      bi[j] = w_ok[j] ? bf2f(st.w[j].b) : 0.f;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {  // MFMA step t covers k = 32*kq + 8*t .. +8 of the K step
      bf16x8_t a[MI], bq[2];
#pragma unroll
      for (int i = 0; i < MI; ++i)
        a[i] = *reinterpret_cast<const bf16x8_t*>(
            &xs[buf][(wm + i * 32 + frow) * LDS_STRIDE + kq * 32 + t * 8]);
#pragma unroll
      for (int j = 0; j < 2; ++j) bq[j] = dequant8<BITS>(st.w[j], t, sc[j], bi[j]);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], bq[j], acc[i][j], 0, 0, 0);
    }
  };

  // At K step k: the x tile of k is in LDS buffer k&1, the x tile of k+1 in registers
  // (xr), the packed weights of k and k+1 in w0 / w1.  Per step: the next x tile goes to
  // the other LDS buffer and its registers are refilled two steps ahead, the current tile
  // is multiplied, the freed weight stage is refilled two steps ahead; one barrier.
  XStage xr;
  WStage w0, w1;
  load_x(xr, 0);
  load_w(w0, 0);
  store_x(xr, 0);
  if (BK < p.K) {
    load_x(xr, BK);
    load_w(w1, BK);
  }
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < p.K; k0 += BK) {
    if (k0 + BK < p.K) store_x(xr, buf ^ 1);
    if (k0 + 2 * BK < p.K) load_x(xr, k0 + 2 * BK);
    multiply(w0, buf);
    w0 = w1;  // a few register moves keep the loop body single (no unrolled twin)
    if (k0 + 2 * BK < p.K) load_w(w1, k0 + 2 * BK);
    __syncthreads();
    buf ^= 1;
  }

  // Epilogue through LDS.  D[i][j] holds column lane%32 (W row n) and rows
  // 8*(r/4) + 4*(lane/32) + r%4 (token m): a wave first writes its (32*MI) x 64 tile as bf16
  // into its own slice of the (now idle) activation buffers - 2-byte LDS stores at constant
  // offsets from one base, so no address lives in registers next to the accumulators -
  // and then copies whole rows out with 16-byte stores (residual added on the way).
  __syncthreads();  // every wave has finished reading the last activation tile
  constexpr int TS = 64 + 8;  // row stride of the staging tile (bf16)
  bf16_t* stage = &xs[0][0] + (size_t)wave * (32 * MI) * TS;
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

template <int BITS>
void launch_qmm(const QmmParams& p, hipStream_t st) {
  const int M = p.M, N = p.N;
  // taller inputs: 256-row tiles halve the dequantisation work and the LDS reads per output
  if (M <= 128)
    qmm_kernel<BITS, 2><<<dim3(exo_ceil_div(N, 128), exo_ceil_div(M, 128)), 256, 0, st>>>(p);
  else
    qmm_kernel<BITS, 4><<<dim3(exo_ceil_div(N, 128), exo_ceil_div(M, 256)), 256, 0, st>>>(p);
}

constexpr int kGroupBM = 128;  // rows per tile of the grouped GEMM
constexpr int kGroupMaxE = 256;

// Sort the (token, slot) pairs by expert and cut every expert's run into tiles of
// kGroupBM rows.  One workgroup: counts in LDS, a serial scan over the experts, a second
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
  if (tid == 0) {
    int o = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o;
      cur[e] = o;
      tile0[e] = t;
      o += cnt[e];
      t += (cnt[e] + kGroupBM - 1) / kGroupBM;
    }
    tile0[E] = t;
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

extern "C" int exo_gather_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const void* workspace, uint16_t* y, int T,
                              int topk, int x_rows, int E, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
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
  QmmParams p{x, w, scales, biases, nullptr, y, P, N, K};
  p.sorted = reinterpret_cast<const int32_t*>(workspace);
  p.tiles = p.sorted + P;
  p.x_div = x_rows == 1 ? topk : 1;
  p.w_stride = (size_t)N * (K * bits / 32);
  p.s_stride = (size_t)N * (K / 64);
  const dim3 grid(exo_ceil_div(N, 128), max_tiles);
  if (bits == 4)
    qmm_kernel<4, 2, true><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  else
    qmm_kernel<8, 2, true><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  EXO_CHECK_LAUNCH("exo_gather_qmm");
  return EXO_OK;
}

extern "C" int exo_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M,
                       int N, int K, int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_qmm: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_qmm: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 64 == 0, "exo_qmm: bad shape M=%d N=%d K=%d", M, N,
              K);
  EXO_REQUIRE(x && w && scales && biases && y, "exo_qmm: null pointer");
  if (M == 0) return EXO_OK;
  QmmParams p{x, w, scales, biases, residual, y, M, N, K};
  p.sorted = nullptr;
  p.tiles = nullptr;
  p.x_div = 1;
  p.w_stride = p.s_stride = 0;
  EXO_REQUIRE(exo_ceil_div(M, 128) <= 65535, "exo_qmm: M=%d too large", M);
  if (bits == 4)
    launch_qmm<4>(p, (hipStream_t)stream);
  else
    launch_qmm<8>(p, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_qmm");
  return EXO_OK;
}
