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
//  * KW waves (4, 8 or 16) split the K range of one block of 32 rows; their partial sums
//    meet in LDS once per block.  Few row blocks: many waves per block, so that the
//    grid is wide without a merge through memory.  Many row blocks: KW = 4 and NG such
//    wave teams per workgroup, which share the staged activations;
//  * with a workspace, K is also split over workgroups (blockIdx.y): 16 rows then fit
//    the LDS at any K and a short N still fills the chip; the last workgroup of a row
//    block to arrive adds the float32 partials in a fixed order.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "qmv_internal.h"

namespace {

struct MfmaParams {
  const bf16_t* x;         // [M,K]
  const uint32_t* w;       // [N, wpr]
  const bf16_t* s;         // [N, K/64]
  const bf16_t* b;
  // second matrix of the (gate, up) pair with the SwiGLU epilogue, or null
  const uint32_t* w2;
  const bf16_t* s2;
  const bf16_t* b2;
  const bf16_t* residual;  // [M,N] or null
  bf16_t* y;               // [M,N]
  const bf16_t* norm_w;    // [K] or null (fused RMSNorm of x)
  float eps;
  int M, N, K, wpr, G;
  int gw;  // groups per wave (multiple of the groups per super-step)
  // split-K: blockIdx.y owns groups [y*gc, (y+1)*gc); partial sums meet in `part`
  int ksplit, gc;
  float* part;    // [ksplit][1 or 2 matrices][M][N] float32
  int* counters;  // [row blocks], zero between launches
};

__device__ __forceinline__ void st_dev(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_dev(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int BITS>
__device__ __forceinline__ uint4 load_word_x(const bf16_t* base, int wi) {
  if (BITS == 4) return *reinterpret_cast<const uint4*>(base + (size_t)wi * 8);
  const uint2 v = *reinterpret_cast<const uint2*>(base + (size_t)wi * 4);
  return make_uint4(v.x, v.y, 0, 0);
}
template <int BITS>
__device__ __forceinline__ float sumsq_word(const uint4& v, float acc) {
  acc = dot2_bf16(v.x, v.x, dot2_bf16(v.y, v.y, acc));
  if (BITS == 4) acc = dot2_bf16(v.z, v.z, dot2_bf16(v.w, v.w, acc));
  return acc;
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
// activations of one packed word in the register order of the unpacked nibble pairs;
// `sum` = sum of the word's activations.  (8-bit: the operand holds every activation twice,
// as x against the low nibble and 16x against the high one, so the sum of the stored
// values is exactly 17 times the sum of the activations.)
template <int BITS>
__device__ __forceinline__ uint4 permute_word(const uint4& xv, float& sum) {
  constexpr uint32_t kOnes = 0x3F803F80u;  // bf16 (1, 1)
  uint4 o;
  if (BITS == 4) {
    o.x = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);  // (x0,x4)
    o.y = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);  // (x1,x5)
    o.z = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);  // (x2,x6)
    o.w = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);  // (x3,x7)
    sum = dot2_bf16(o.x, kOnes, dot2_bf16(o.y, kOnes, dot2_bf16(o.z, kOnes, dot2_bf16(o.w, kOnes, 0.f))));
  } else {  // byte codes as two nibbles against (x, 16x)
    const uint32_t a = __builtin_amdgcn_perm(xv.y, xv.x, 0x05040100u);   // (x0,x2)
    const uint32_t c2 = __builtin_amdgcn_perm(xv.y, xv.x, 0x07060302u);  // (x1,x3)
    o.x = a;
    o.y = pack_bf2(bf_lo(a) * 16.f, bf_hi(a) * 16.f);
    o.z = c2;
    o.w = pack_bf2(bf_lo(c2) * 16.f, bf_hi(c2) * 16.f);
    sum = dot2_bf16(a, kOnes, dot2_bf16(c2, kOnes, 0.f));
  }
  return o;
}

// MR = D registers in use: 4 covers M <= 8, 8 covers M <= 16.  KW = waves that split K
// for one row block, NG = such wave teams per workgroup.  SPS = 16-byte loads in flight
// per lane and buffer (a "super-step").
// SBLK (4-bit, a wave's share of a row = 8 or 16 whole groups, no ragged chunks): the
// (scale, bias) of a wave's whole share come in ONE 16-byte load each per row block - the
// two lane halves take 8 groups each when the share is 16 - instead of an 8-byte load per
// super-step: a row's scales are one 128-byte line at K = 4096, and every load instruction
// that touches 32 rows costs 32 line requests whatever it brings back (measured with the
// same loads and no arithmetic: 73 -> 54 us on 128256 x 4096).
template <int BITS, int MR, int KW, int NG, int SPS, bool SBLK = false>
__global__ __launch_bounds__(64 * KW * NG) void qmv_mfma_kernel(const MfmaParams p) {
  constexpr int kThreads = 64 * KW * NG;
  constexpr int WPG = 64 * BITS / 32;  // words per group: 8 / 16
  constexpr int SPG = WPG / 8;         // load steps per group: 1 / 2
  constexpr int SSG = SPS / SPG;       // groups per super-step
  static_assert(SSG >= 2 && SSG <= 8, "scale vector of 2..8 bf16");
  extern __shared__ uint4 smem[];
  const int MT = p.M;
  constexpr int MROWS = MR * 2;  // activation rows this instantiation covers
  // this workgroup's share of K: groups [gbase, gbase+Gc), words [wbase, wbase+wcount)
  const int gbase = (int)blockIdx.y * p.gc;
  const int Gc = min(p.gc, p.G - gbase);
  const int wbase = gbase * WPG, wcount = Gc * WPG;
  // activations by row, slot (step, t, kq) inside; the row stride is padded by two slots
  // so that the rows a wave reads together (same slot, rows 0..MT-1) fall into different
  // banks, while the staging threads of one row write consecutive slots
  const int XS = p.gc * WPG + 2;
  uint4* xs = smem;                                                   // [MT][XS]
  float2* sxs = reinterpret_cast<float2*>(smem + (size_t)XS * MT);    // [gc][MT]
  float* red_all = reinterpret_cast<float*>(sxs + (size_t)p.gc * MT);       // [NG][KW][MR][64]
  __shared__ float s_red[KW * NG * 16];
  __shared__ float s_inv[16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int quartet = wave_all / KW, wave = wave_all % KW;
  float* red = red_all + quartet * (KW * MR * 64);
  const int r = lane & 31, kq = lane >> 5;
  const int NB = (p.N + 31) >> 5;

  const int g_begin = wave * p.gw;  // this wave's share of the chunk
  const int g_end = min(Gc, g_begin + p.gw);
  const int n_super = p.gw / SSG;   // same for every wave of the grid

  struct Buf {
    uint4 w[SPS];
    uint4 s, b;  // SSG scales / biases (unused with SBLK)
  };
  // SBLK: (scale, bias) of this wave's share of the row block in flight / in use.  With 16
  // groups per wave lane half kq holds groups [8kq, 8kq+8) of the share, with 8 both halves
  // hold all of them.
  uint4 s_next = make_uint4(0, 0, 0, 0), b_next = s_next, s_cur = s_next, b_cur = s_next;
  // item -> (row block, super-step); loads clamp to the last valid row / group
  auto issue = [&](Buf& bf, int blk, int mat, int ss) {
    const int row = min(blk * 32 + r, p.N - 1);
    const int g0 = min(g_begin + ss * SSG, Gc - SSG);
    const uint32_t* wp = (mat ? p.w2 : p.w) + (size_t)row * p.wpr + (size_t)(gbase + g0) * WPG + kq * 4;
#pragma unroll
    for (int i = 0; i < SPS; ++i) {
      // steps past the chunk end re-read its last step (never consumed)
      const int off = min(i * 8, wcount - g0 * WPG - 8);
      bf.w[i] = *reinterpret_cast<const uint4*>(wp + off);
    }
    const bf16_t* sp = (mat ? p.s2 : p.s) + (size_t)row * p.G + gbase + g0;
    const bf16_t* bp = (mat ? p.b2 : p.b) + (size_t)row * p.G + gbase + g0;
    if (SBLK) {
      if (ss == 0) {  // g0 == g_begin here
        const int half = p.gw == 16 ? kq * 8 : 0;
        s_next = *reinterpret_cast<const uint4*>(sp + half);
        b_next = *reinterpret_cast<const uint4*>(bp + half);
      }
    } else if (SSG == 8) {
      bf.s = *reinterpret_cast<const uint4*>(sp);
      bf.b = *reinterpret_cast<const uint4*>(bp);
    } else if (SSG == 4) {
      const uint2 sv = *reinterpret_cast<const uint2*>(sp);
      const uint2 bv = *reinterpret_cast<const uint2*>(bp);
      bf.s = make_uint4(sv.x, sv.y, 0, 0);
      bf.b = make_uint4(bv.x, bv.y, 0, 0);
    } else {
      bf.s = make_uint4(*reinterpret_cast<const uint32_t*>(sp), 0, 0, 0);
      bf.b = make_uint4(*reinterpret_cast<const uint32_t*>(bp), 0, 0, 0);
    }
  };

  // flat sequence of (row block, matrix, super-step) items; the teams of a workgroup take
  // neighbouring row blocks and run the same number of items (barriers are block-wide)
  const int nmat = p.w2 ? 2 : 1;
  const int NBq = (NB + NG - 1) / NG;
  const int my_blocks = (NBq - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const int n_items = my_blocks * nmat * n_super;
  if (n_items <= 0) return;
  auto blk_of = [&](int it) {
    return ((int)blockIdx.x + (it / (nmat * n_super)) * (int)gridDim.x) * NG + quartet;
  };
  auto mat_of = [&](int it) { return (it / n_super) & (nmat - 1); };

  Buf b0, b1;
  // weights do not depend on x: in flight while x is staged (where registers allow)
  constexpr bool kEarly = (MR == 4);
  if (kEarly) issue(b0, blk_of(0), 0, 0);

  // ---- stage the activations: optional RMSNorm, permute, group sums
  {
    // one pass over x when every thread sees at most one word of the row and the
    // workgroup stages the whole row: the words read for the norm stay in registers
    const bool keep = p.norm_w && p.ksplit == 1 && p.wpr <= kThreads;
    uint4 xkeep[MROWS];
    uint4 nwkeep = make_uint4(0, 0, 0, 0);
    if (keep && tid < p.wpr) nwkeep = load_word_x<BITS>(p.norm_w, tid);
    if (p.norm_w) {
      // rows are loaded in batches of 4 (clamped to the last real row) so that the loads
      // of a batch are in flight together instead of one latency per row
      float ss[MROWS];
#pragma unroll
      for (int m = 0; m < MROWS; ++m) ss[m] = 0.f;
      for (int wi = tid; wi < p.wpr; wi += kThreads)
#pragma unroll
        for (int m0 = 0; m0 < MROWS; m0 += 4) {
          if (m0 < MT) {
            uint4 xv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
              xv[j] = load_word_x<BITS>(p.x + (size_t)min(m0 + j, MT - 1) * p.K, wi);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              ss[m0 + j] = sumsq_word<BITS>(xv[j], ss[m0 + j]);
              if (keep) xkeep[m0 + j] = xv[j];
            }
          }
        }
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        const float t = wave_sum_to_lane63(ss[m]);
        if (lane == 63) s_red[wave_all * 16 + m] = t;
      }
      __syncthreads();
      if (tid < MROWS) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < KW * NG; ++w) t += s_red[w * 16 + tid];
        s_inv[tid] = rsqrtf(t / (float)p.K + p.eps);
      }
      __syncthreads();
    }
    for (int wl = tid; wl < wcount; wl += kThreads) {
      const int wi = wbase + wl;
      const int step = wl >> 3, q2 = (wl >> 2) & 1, t = wl & 3;
      const int dst = (step * 4 + t) * 2 + q2;
      uint4 nw = make_uint4(0, 0, 0, 0);
      if (keep)
        nw = nwkeep;
      else if (p.norm_w)
        nw = load_word_x<BITS>(p.norm_w, wi);
#pragma unroll
      for (int m0 = 0; m0 < MROWS; m0 += 4) {
        if (m0 < MT) {
          uint4 xr[4];
          if (keep) {
#pragma unroll
            for (int j = 0; j < 4; ++j) xr[j] = xkeep[m0 + j];
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              xr[j] = load_word_x<BITS>(p.x + (size_t)min(m0 + j, MT - 1) * p.K, wi);
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int m = m0 + j;
            uint4 xv = xr[j];
            if (p.norm_w) norm_word<BITS>(xv, nw, s_inv[m]);
            float sum;
            const uint4 pw = permute_word<BITS>(xv, sum);
            // the WPG consecutive words (lanes) of a group: wcount is a multiple of WPG,
            // so a run of WPG lanes is active or idle as a whole
            sum = run_sum<WPG>(sum);
            if (m < MT) {
              xs[m * XS + dst] = pw;
              if ((wl & (WPG - 1)) == 0)
                sxs[(wl / WPG) * MT + m] = make_float2((BITS == 4 ? 128.f : 128.f * 17.f) * sum, sum);
            }
          }
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
  const uint4* xa = xs + min(r, MT - 1) * XS + kq;  // A-operand row of this lane

  uint32_t kmask = 0x000F000Fu, kmagic = 0x43004300u;
  asm volatile("" : "+s"(kmask));
  asm volatile("" : "+v"(kmagic));

  float acc[MR];
#pragma unroll
  for (int q = 0; q < MR; ++q) acc[q] = 0.f;
  if (!kEarly) issue(b0, blk_of(0), 0, 0);

  auto consume = [&](const Buf& bf, int ss) {
    const int g0 = min(g_begin + ss * SSG, Gc - SSG);
    const int g_first = g_begin + ss * SSG;  // groups [g_first, g_first+SSG) are due
    uint32_t sblk[2] = {0, 0}, bblk[2] = {0, 0};  // SBLK: the two words of this super-step
    if (SBLK) {
      if (ss == 0) {
        s_cur = s_next;
        b_cur = b_next;
      }
      // groups [4ss, 4ss+4) of the share: words 2*(ss&1), +1 of the half that holds them
      const bool hi = ss & 1;
      sblk[0] = hi ? s_cur.z : s_cur.x;
      sblk[1] = hi ? s_cur.w : s_cur.y;
      bblk[0] = hi ? b_cur.z : b_cur.x;
      bblk[1] = hi ? b_cur.w : b_cur.y;
      if (p.gw == 16) {  // every lane takes them from the half that loaded them
        const int src = ((lane & 31) + 32 * ((ss >> 1) & 1)) * 4;
        sblk[0] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sblk[0]);
        sblk[1] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)sblk[1]);
        bblk[0] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bblk[0]);
        bblk[1] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)bblk[1]);
      }
    }
    const uint32_t* sw = SBLK ? sblk : reinterpret_cast<const uint32_t*>(&bf.s);
    const uint32_t* bw = SBLK ? bblk : reinterpret_cast<const uint32_t*>(&bf.b);
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
            const uint4 av = xa[(step * 4 + t) * 2];
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

  float vg[MR];  // the gate sums of this row block while the up matrix is under way
#pragma unroll
  for (int q = 0; q < MR; ++q) vg[q] = 0.f;

  auto finish_block = [&](int blk, int mat) {
    __syncthreads();  // the team's first wave has finished reading the previous partials
#pragma unroll
    for (int q = 0; q < MR; ++q) {
      red[(wave * MR + q) * 64 + lane] = acc[q];
      acc[q] = 0.f;
    }
    __syncthreads();
    if (wave == 0 && blk < NB) {
      const int row = blk * 32 + r;
      float v[MR];
#pragma unroll
      for (int q = 0; q < MR; ++q) v[q] = 0.f;
#pragma unroll 1
      for (int w0 = 0; w0 < KW; w0 += 4)
#pragma unroll
        for (int q = 0; q < MR; ++q)
          v[q] += (red[(w0 * MR + q) * 64 + lane] + red[((w0 + 1) * MR + q) * 64 + lane]) +
                  (red[((w0 + 2) * MR + q) * 64 + lane] + red[((w0 + 3) * MR + q) * 64 + lane]);
      const bool pair_open = nmat == 2 && mat == 0;  // the up matrix is still to come
      bool write = !pair_open;
      if (p.ksplit > 1) {
        // partial sums go out at device scope (the merging workgroup may sit on another
        // XCD) and are added up after the last row block, see the end of the kernel:
        // nothing here waits for them
#pragma unroll
        for (int q = 0; q < MR; ++q) {
          const int m = 8 * (q >> 2) + 4 * Rg + (q & 3);
          if (m < p.M && row < p.N)
            st_dev(&p.part[(((size_t)blockIdx.y * nmat + mat) * p.M + m) * p.N + row], v[q]);
        }
        write = false;
      } else if (pair_open) {
#pragma unroll
        for (int q = 0; q < MR; ++q) vg[q] = v[q];
      }
      if (write) {
#pragma unroll
        for (int q = 0; q < MR; ++q) {
          const int m = 8 * (q >> 2) + 4 * Rg + (q & 3);
          if (m < p.M && row < p.N) {
            const size_t o = (size_t)m * p.N + row;
            float t = v[q];
            if (nmat == 2) {  // SwiGLU on the bf16-rounded projections
              const float g = bf2f(f2bf(vg[q])), up = bf2f(f2bf(t));
              t = g / (1.f + __expf(-g)) * up;
            } else if (p.residual) {
              t = bf2f(f2bf(t)) + bf2f(p.residual[o]);
            }
            p.y[o] = f2bf(t);
          }
        }
      }
    }
  };

  int it = 0;
  for (;;) {
    if (it + 1 < n_items) issue(b1, blk_of(it + 1), mat_of(it + 1), (it + 1) % n_super);
    consume(b0, it % n_super);
    if (it % n_super == n_super - 1) finish_block(blk_of(it), mat_of(it));
    if (++it >= n_items) break;
    if (it + 1 < n_items) issue(b0, blk_of(it + 1), mat_of(it + 1), (it + 1) % n_super);
    consume(b1, it % n_super);
    if (it % n_super == n_super - 1) finish_block(blk_of(it), mat_of(it));
    if (++it >= n_items) break;
  }
  if (p.ksplit == 1) return;

  // Split K: the ksplit workgroups of one blockIdx.x have walked the same row blocks.  The
  // last of them to get here adds the float32 partials of all those blocks, in a fixed
  // order (the result does not depend on arrival order), and writes y.  One counter round
  // trip per workgroup, after the streaming, instead of one per row block inside it.
  __shared__ int s_last;
  wait_own_stores_done();  // this wave's device-scope partial stores have completed
  __syncthreads();
  if (tid == 0) {
    int* cnt = &p.counters[blockIdx.x];
    const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.ksplit - 1);
    if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  const int per_blk = 32 * p.M;
  const int total = my_blocks * NG * per_blk;
  const size_t mstride = (size_t)p.M * p.N;  // one matrix of one K chunk
  for (int e = tid; e < total; e += kThreads) {
    const int bq = e / per_blk, rem = e - bq * per_blk;
    const int m = rem >> 5;
    const int blk = ((int)blockIdx.x + (bq / NG) * (int)gridDim.x) * NG + bq % NG;
    const int row = blk * 32 + (rem & 31);
    if (blk >= NB || row >= p.N) continue;
    const size_t o = (size_t)m * p.N + row;
    float t = 0.f, tg = 0.f;
    for (int ks = 0; ks < p.ksplit; ++ks) {
      t += ld_dev(&p.part[((size_t)ks * nmat + (nmat - 1)) * mstride + o]);
      if (nmat == 2) tg += ld_dev(&p.part[(size_t)ks * nmat * mstride + o]);
    }
    if (nmat == 2) {  // SwiGLU on the bf16-rounded projections
      const float g = bf2f(f2bf(tg)), up = bf2f(f2bf(t));
      t = g / (1.f + __expf(-g)) * up;
    } else if (p.residual) {
      t = bf2f(f2bf(t)) + bf2f(p.residual[o]);
    }
    p.y[o] = f2bf(t);
  }
}

template <int BITS, int MR, int KW, int NG, int SPS, bool SBLK = false>
int launch(const MfmaParams& p, size_t lds, hipStream_t st) {
  auto kern = qmv_mfma_kernel<BITS, MR, KW, NG, SPS, SBLK>;
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 2048);
    if (e != hipSuccess) {
      exo_set_error("exo_qmv: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    attr_done = true;
  }
  const int NBq = ((p.N + 31) / 32 + NG - 1) / NG;
  int per_cu = lds <= 38 * 1024 ? 4 : (lds <= 51 * 1024 ? 3 : (lds <= 78 * 1024 ? 2 : 1));
  if (per_cu * KW * NG > 16) per_cu = 16 / (KW * NG);  // at most 16 waves per CU
  if (per_cu < 1) per_cu = 1;
  int gx = 256 * per_cu / p.ksplit;
  if (gx < 1) gx = 1;
  if (gx > NBq) gx = NBq;
  // several row blocks per workgroup: the same number for every workgroup (448 blocks at 16
  // rows: 256 workgroups of one or two blocks 25.2 us, 224 of two 21.7; the pair 44.7 -> 38.5)
  if (gx < NBq) {
    const int per = (NBq + gx - 1) / gx;
    gx = (NBq + per - 1) / per;
  }
  exo_note_variant("qmv_mfma<%d,%d,%d,%d,%d,%s> grid=%dx%d", BITS, MR, KW, NG, SPS, SBLK ? "true" : "false",
                   gx, p.ksplit);
  kern<<<dim3(gx, p.ksplit), dim3(64 * KW * NG), lds, st>>>(p);
  return EXO_OK;
}

constexpr int kMaxSplit = 8;
constexpr size_t kLdsBudget = 150 * 1024;

size_t lds_bytes(int M, int gc, int bits, int MR, int KW, int NG) {
  const size_t wpg = 64 * bits / 32;
  return (size_t)(gc * wpg + 2) * 16 * M + (size_t)gc * 8 * M + (size_t)NG * KW * MR * 64 * 4;
}

}  // namespace

// rows of x that fit one launch without split-K (LDS holds their whole K), 0 if the
// kernel does not take this K at all
int exo_qmv_mfma_max_rows(int K, int bits) {
  if (K % (bits == 4 ? 512 : 256) != 0) return 0;
  const size_t per_row = ((size_t)K * bits / 32 + 2) * 16 + (size_t)(K / 64) * 8;
  const size_t budget = kLdsBudget - 4 * 4 * 8 * 64 * 4;
  size_t m = budget / per_row;
  return m > 16 ? 16 : (int)m;
}

// bytes of split-K workspace for up to 16 rows: row-block counters, then the partials.
// The counter area has one size for every N, so that partials of one launch never land
// where another launch (of another N, sharing the workspace) keeps its counters.
constexpr size_t kCounterBytes = 64 * 1024;
size_t exo_qmv_mfma_workspace(int N) {
  return kCounterBytes + (size_t)kMaxSplit * 16 * N * 4;
}

// y[M,N] for 2 <= M <= 16; with a second matrix (w2, s2, b2: the up projection, w being
// the gate) y = silu(x W^T) * (x W2^T) and the workspace is sized for 2N rows.  Without a
// workspace M must not exceed
// exo_qmv_mfma_max_rows(K, bits); with one, K may be split over up to kMaxSplit workgroups
// per row block so that any M <= 16 fits and a short N still fills the chip.
int exo_qmv_mfma_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                        const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                        int bits, void* workspace, hipStream_t st) {
  MfmaParams p;
  p.x = x;
  p.w = w;
  p.s = s;
  p.b = b;
  p.w2 = w2;
  p.s2 = s2;
  p.b2 = b2;
  const int nmat = w2 ? 2 : 1;
  p.residual = residual;
  p.y = y;
  p.norm_w = norm_w;
  p.eps = eps;
  p.M = M;
  p.N = N;
  p.K = K;
  p.wpr = K * bits / 32;
  p.G = K / 64;
  const int MR = M <= 8 ? 4 : 8;
  const int NB = (N + 31) / 32;
  const int sps = 4;
  const int ssg = sps / (bits == 4 ? 1 : 2);
  const int n_steps = p.G / ssg;  // super-steps along K
  // waves per row block: as many as keep the grid at about 4096 waves per matrix with at
  // least one super-step each, 16 only where two remain (16 needs the 128-register kernels:
  // M <= 8 only).  Measured at 8 rows, K = 4096: 6144 rows 16 waves 12.5 us, 8 waves 12.0;
  // the 14336-row (gate, up) pair 4 waves 26.5 us, 8 waves 24.6.
  int KW = 4;
  if (MR == 4) {
    while (KW < 16 && NB * KW * 2 <= 4096 && n_steps >= KW * 2 && (KW < 8 || n_steps >= KW * 4))
      KW *= 2;
  } else if (NB <= 128 && n_steps <= 16) {
    KW = 8;  // more registers per wave: 8 waves, and only where both N and K are short
  }
  // many row blocks: teams of 4 waves share the staged x (2 teams for up to 8 rows, 3 for
  // up to 16)
  const int NG = (KW == 4 && NB >= 1024) ? (MR == 8 ? 3 : 2) : 1;
  const int NBq = (NB + NG - 1) / NG;
  // LDS the activations of a chunk may take: two workgroups per CU while a workgroup is
  // 4 or 8 waves, one beyond
  const size_t lds_cap = (KW * NG <= 8 ? 78u : 150u) * 1024;
  int ksplit = 1;
  if (workspace && (size_t)NB * 4 > kCounterBytes) workspace = nullptr;  // N beyond 524288
  if (workspace) {
    // split K until a chunk of x fits the LDS, and further while the grid stays within one
    // workgroup per CU (4096 rows at 8 waves: 128 workgroups 9.8 us, 256: 8.9; 6144 rows:
    // 192 workgroups 12.0 us, 384: 14.5); a chunk is at least one super-step per wave
    while (ksplit < kMaxSplit && (p.G + ksplit - 1) / ksplit > KW * ssg &&
           (lds_bytes(M, (p.G + ksplit - 1) / ksplit, bits, MR, KW, NG) > lds_cap ||
            NBq * (ksplit + 1) <= 256))
      ++ksplit;
  }
  int gc = (p.G + ksplit - 1) / ksplit;
  gc = (gc + ssg - 1) / ssg * ssg;  // chunks in whole super-steps
  if (gc > p.G) gc = p.G;
  ksplit = (p.G + gc - 1) / gc;
  p.ksplit = ksplit;
  p.gc = gc;
  int gw = (gc + KW - 1) / KW;
  p.gw = (gw + ssg - 1) / ssg * ssg;
  p.counters = reinterpret_cast<int*>(workspace);
  p.part = workspace ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + kCounterBytes)
                     : nullptr;
  const size_t lds = lds_bytes(M, gc, bits, MR, KW, NG);
  if (lds > kLdsBudget) {
    exo_set_error("exo_qmv: %d rows of K=%d need %zu bytes of LDS", M, K, lds);
    return EXO_ERR_ARG;
  }
  // whole-share (scale, bias) loads: 4-bit, 8 or 16 groups per wave that tile the row
  // exactly (no clamped super-steps, every 16-byte load aligned and inside its row)
  const bool sblk = bits == 4 && (p.gw == 8 || p.gw == 16) && p.gw * KW == gc && p.G % gc == 0 &&
                    gc % 8 == 0 && p.G % 8 == 0 &&
                    (((uintptr_t)s | (uintptr_t)b | (uintptr_t)s2 | (uintptr_t)b2) & 15) == 0;
#define EXO_MFMA_SBLK(MR_, KW_, NG_) \
  if (sblk && MR == MR_ && KW == KW_ && NG == NG_) return launch<4, MR_, KW_, NG_, 4, true>(p, lds, st);
  EXO_MFMA_SBLK(4, 4, 1)
  EXO_MFMA_SBLK(4, 4, 2)
  EXO_MFMA_SBLK(4, 8, 1)
  EXO_MFMA_SBLK(8, 4, 1)
  EXO_MFMA_SBLK(8, 4, 3)
#undef EXO_MFMA_SBLK
#define EXO_MFMA_CASE(B_, MR_, KW_, NG_) \
  if (bits == B_ && MR == MR_ && KW == KW_ && NG == NG_) return launch<B_, MR_, KW_, NG_, 4>(p, lds, st);
#define EXO_MFMA_BITS(B_)    \
  EXO_MFMA_CASE(B_, 4, 4, 1)  \
  EXO_MFMA_CASE(B_, 4, 4, 2)  \
  EXO_MFMA_CASE(B_, 4, 8, 1)  \
  EXO_MFMA_CASE(B_, 4, 16, 1) \
  EXO_MFMA_CASE(B_, 8, 4, 1)  \
  EXO_MFMA_CASE(B_, 8, 4, 3)  \
  EXO_MFMA_CASE(B_, 8, 8, 1)
  EXO_MFMA_BITS(4)
  EXO_MFMA_BITS(8)
#undef EXO_MFMA_BITS
#undef EXO_MFMA_CASE
  exo_set_error("exo_qmv: no kernel for bits=%d rows=%d", bits, M);
  return EXO_ERR_ARG;
}
