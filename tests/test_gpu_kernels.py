"""Parity of every HIP kernel, called through the C ABI, against the CPU oracle.

Bar: bit-exact for codes / dequantised weights / indices; rtol 2e-2 (+ atol =
rtol*rms) for bf16 activations.
"""

import numpy as np
import pytest
import torch

from oracle import affine
from oracle import ops as O
from tests.util import (
    assert_close, assert_close_stat, n_bits, n_f32, rand_bf16, rand_quantized, rng, t_bf16, t_qw, t_u32,
)

pytestmark = pytest.mark.gpu

from exo_amd import native, ops  # noqa: E402


def test_library_loads_and_reports_mode():
    lib = native.load()
    assert lib.exo_abi_version() == 1
    assert lib.exo_dequant_two_roundings() in (0, 1)


@pytest.mark.parametrize("bits", [4, 8])
def test_unpack_codes_bit_exact(device, bits):
    w = rng(1).integers(0, 2**32, size=(37, 96), dtype=np.uint64).astype(np.uint32)
    got = ops.unpack_codes(t_u32(w, device), bits).cpu().numpy()
    np.testing.assert_array_equal(got, affine.unpack_codes(w, bits))


@pytest.mark.parametrize("bits", [4, 8])
def test_dequantize_bit_exact(device, bits):
    trip = rand_quantized(50, 512, bits, seed=3)
    got = n_bits(ops.dequantize(t_qw(trip, bits, device)))
    mode = "M1" if native.load().exo_dequant_two_roundings() else "M2"
    want = affine.dequantize(*trip, 64, bits, mode)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("bits", [4, 8])
def test_dequantize_all_codes_extreme_scales(device, bits):
    # every code value at every slot, with scales/biases spanning magnitudes
    K = 256 if bits == 8 else 64
    per = 1 << bits
    codes = (np.arange(per * K).reshape(per, K) // 1 + np.arange(per)[:, None]) % per
    codes = np.tile(codes.astype(np.uint8), (1, 1))
    w = affine.pack_codes(codes, bits)
    G = K // 64
    s = affine.f32_to_bf16_bits((rng(5).standard_normal((per, G)) * 10.0 ** rng(6).integers(-6, 3, (per, G))).astype(np.float32))
    b = affine.f32_to_bf16_bits((rng(7).standard_normal((per, G)) * 10.0 ** rng(8).integers(-6, 3, (per, G))).astype(np.float32))
    got = n_bits(ops.dequantize(t_qw((w, s, b), bits, device)))
    mode = "M1" if native.load().exo_dequant_two_roundings() else "M2"
    np.testing.assert_array_equal(got, affine.dequantize(w, s, b, 64, bits, mode))


@pytest.mark.parametrize("bits", [4, 8])
def test_embed_bit_exact(device, bits):
    trip = rand_quantized(300, 256, bits, seed=9)
    ids = np.array([0, 299, 5, 5, 17, 128], np.int32)
    got = n_bits(ops.embed(torch.from_numpy(ids).to(device), t_qw(trip, bits, device)))
    mode = "M1" if native.load().exo_dequant_two_roundings() else "M2"
    want = affine.dequantize(trip[0][ids], trip[1][ids], trip[2][ids], 64, bits, mode)
    np.testing.assert_array_equal(got, want)


QMV_SHAPES = [  # (N, K)
    (256, 4096), (64, 2048), (128, 14336), (96, 768), (64, 1536), (200, 8192), (128, 64),
    (72, 192), (160, 7168),
]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("N,K", QMV_SHAPES)
@pytest.mark.parametrize("M", [1, 2, 3, 7, 16])
def test_qmv(device, bits, N, K, M):
    trip = rand_quantized(N, K, bits, seed=N + K + bits)
    x = rand_bf16((M, K), seed=M + K)
    got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device)))
    want = affine.qmm(x, *trip, 64, bits)
    assert_close(got, want, what=f"qmv {M}x{N}x{K} b{bits}")


@pytest.mark.parametrize("bits", [4, 8])
def test_qmv_is_accurate_beyond_bf16(device, bits):
    # float32 accumulation: before the final rounding the result should sit within
    # about one bf16 ulp of the float64 value.
    N, K, M = 512, 4096, 1
    trip = rand_quantized(N, K, bits, seed=77)
    x = rand_bf16((M, K), seed=78)
    got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device)))
    wd = affine.dequantize_f32(*trip, 64, bits).astype(np.float64)
    exact = x.astype(np.float64) @ wd.T
    err = np.abs(got - exact)
    assert np.all(err <= np.abs(exact) * 2.0**-8 + 1e-4), err.max()


@pytest.mark.parametrize("bits", [4, 8])
def test_qmv_residual(device, bits):
    N, K, M = 192, 2048, 3
    trip = rand_quantized(N, K, bits, seed=21)
    x = rand_bf16((M, K), seed=22)
    r = rand_bf16((M, N), seed=23)
    got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device), residual=t_bf16(r, device)))
    want = affine.bf16_round(affine.qmm(x, *trip, 64, bits) + r)
    assert_close(got, want, what="qmv+residual")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [1, 2, 4, 9, 16])
def test_qmv_swiglu(device, bits, M):
    N, K = 320, 2048
    g = rand_quantized(N, K, bits, seed=31)
    u = rand_quantized(N, K, bits, seed=32)
    x = rand_bf16((M, K), seed=33)
    got = n_f32(ops.qmv_swiglu(t_bf16(x, device), t_qw(g, bits, device), t_qw(u, bits, device)))
    want = O.swiglu(affine.qmm(x, *g, 64, bits), affine.qmm(x, *u, 64, bits))
    assert_close(got, want, what="qmv_swiglu")


W16_SHAPES = [  # (N, K): rows of 6 | 8 | 14 | 16 waves x 1 | 2 slices, K split 2 | 4 ways
    (4112, 768), (2064, 1024), (1008, 2560), (1040, 3584), (528, 4096), (272, 8192), (304, 14336),
]


@pytest.mark.parametrize("N,K", W16_SHAPES)
@pytest.mark.parametrize("M", [5, 8, 11, 16])
def test_qmv_16x16x32_kernel_shapes(device, N, K, M):
    """The 16x16x32 matrix-core GEMV (4-bit, 5..16 rows) over its wave /
    slice layouts: plain, with residual, with the fused RMSNorm (rows of up to 4096 elements),
    and the (gate, up) pair with SwiGLU; every result against the oracle, every launch asserted
    to have reached that kernel."""
    bits = 4
    trip = rand_quantized(N, K, bits, seed=N + K)
    qw = t_qw(trip, bits, device)
    x = rand_bf16((M, K), seed=M + K, scale=1.5)
    xt = t_bf16(x, device)
    want = affine.qmm(x, *trip, 64, bits)
    got = ops.quantized_matmul(xt, qw)
    assert native.last_variant().startswith("qmv_w16<1,"), native.last_variant()
    if K > 4096:
        assert "kparts=1" not in native.last_variant(), native.last_variant()
    assert_close(n_f32(got), want, what=f"w16 {M}x{N}x{K}")
    r = rand_bf16((M, N), seed=N + 3)
    got = ops.quantized_matmul(xt, qw, residual=t_bf16(r, device))
    assert native.last_variant().startswith("qmv_w16<1,"), native.last_variant()
    assert_close(n_f32(got), affine.bf16_round(affine.bf16_round(want) + r), what=f"w16 residual {M}x{N}x{K}")
    # the split-K workspace is left clean: the same launch again gives the same bits
    again = ops.quantized_matmul(xt, qw, residual=t_bf16(r, device))
    assert torch.equal(got.view(torch.int16), again.view(torch.int16))
    if K <= 4096:
        w = affine.bf16_round(rand_bf16((K,), seed=6) * 0.1 + 1.0)
        xn = O.rms_norm(x, w, 1e-5)
        got = ops.quantized_matmul(xt, qw, norm_weight=t_bf16(w, device), eps=1e-5)
        assert native.last_variant().startswith("qmv_w16<1,") and "norm" in native.last_variant(), native.last_variant()
        assert_close(n_f32(got), affine.qmm(xn, *trip, 64, bits), what=f"w16 norm {M}x{N}x{K}")
        up = rand_quantized(N, K, bits, seed=N + K + 1)
        got = ops.qmv_swiglu(xt, qw, t_qw(up, bits, device), norm_weight=t_bf16(w, device), eps=1e-5)
        assert native.last_variant().startswith("qmv_w16<2,"), native.last_variant()
        assert_close(n_f32(got), O.swiglu(affine.qmm(xn, *trip, 64, bits), affine.qmm(xn, *up, 64, bits)),
                     what=f"w16 pair {M}x{N}x{K}")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(8, 1000, 4096), (3, 96, 14336), (16, 2080, 2048), (5, 14336, 512)])
def test_qmv_swiglu_rows_equal_separate_launches(device, bits, M, N, K):
    """The one-launch (gate, up, SwiGLU) of 2..16 rows rounds each projection to bf16
    before the SwiGLU, so it equals the two GEMVs followed by the elementwise kernel bit
    for bit; with and without the fused RMSNorm, with K split over workgroups (short N)
    and not."""
    g = t_qw(rand_quantized(N, K, bits, seed=N + 1), bits, device)
    u = t_qw(rand_quantized(N, K, bits, seed=N + 2), bits, device)
    x = t_bf16(rand_bf16((M, K), seed=M + K, scale=2.0), device)
    w = t_bf16(affine.bf16_round(rand_bf16((K,), seed=6) * 0.1 + 1.0), device)
    for nw in (None, w):
        fused = ops.qmv_swiglu(x, g, u, norm_weight=nw, eps=1e-5)
        sep = ops.swiglu(ops.quantized_matmul(x, g, norm_weight=nw, eps=1e-5),
                         ops.quantized_matmul(x, u, norm_weight=nw, eps=1e-5))
        if (nw is None and M > 8 and bits == 8) or N * K * bits // 8 <= (1 << 20):
            # these single projections take the split-K GEMM, or (a matrix of up to 1 MiB)
            # one single-row launch set per row: another summation order
            assert_close(n_f32(fused), n_f32(sep), what="fused pair vs separate projections")
        else:
            assert torch.equal(fused.view(torch.int16), sep.view(torch.int16))
    # the shared workspace is left clean for a launch of another shape
    y = ops.quantized_matmul(x[:2], g)
    assert torch.equal(y.view(torch.int16), ops.quantized_matmul(x[:2], g).view(torch.int16))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [2, 4, 8, 16])
@pytest.mark.parametrize("N,K", [(128, 2048), (60, 4096), (256, 768)])
def test_small_matrix_rows_equal_single_row_launches(device, bits, M, N, K):
    """A matrix of up to 1 MiB (a MoE router) under 2..16 rows runs the single-row kernel once
    per row in one launch: every row equals its own single-row launch bit for bit, with and
    without the fused RMSNorm, and the oracle within tolerance."""
    trip = rand_quantized(N, K, bits, seed=N + K)
    x = rand_bf16((M, K), seed=M + 7, scale=2.0)
    qw, xt = t_qw(trip, bits, device), t_bf16(x, device)
    w = t_bf16(affine.bf16_round(rand_bf16((K,), seed=6) * 0.1 + 1.0), device)
    for nw in (None, w):
        got = ops.quantized_matmul(xt, qw, norm_weight=nw, eps=1e-5)
        for r in range(M):
            one = ops.quantized_matmul(xt[r:r + 1], qw, norm_weight=nw, eps=1e-5)
            assert torch.equal(got[r:r + 1].view(torch.int16), one.view(torch.int16)), (r, nw is None)
    assert_close(n_f32(ops.quantized_matmul(xt, qw)), affine.qmm(x, *trip, 64, bits), what="rows of a small matrix")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(300, 256, 512), (129, 100, 192), (513, 192, 1024), (40, 64, 256), (2046, 1000, 320),
                                   (300, 4100, 768), (700, 8200, 768), (260, 4104, 1280)])
def test_qmm_swiglu_pair(device, bits, M, N, K):
    """Gate and up projections with the SwiGLU in the GEMM's epilogue: the bits of the two
    GEMMs followed by the elementwise kernel (same products, same rounding points), and the
    oracle within tolerance.  Ragged M and N, N not a multiple of 8, K with and without the
    four-step scale blocks; the last three shapes are launches of more than 128 tall tiles,
    which take the 128 x 128 tile with the four waves side by side."""
    g = rand_quantized(N, K, bits, seed=N + 11)
    u = rand_quantized(N, K, bits, seed=N + 12)
    x = rand_bf16((M, K), seed=M + K)
    gq, uq, xt = t_qw(g, bits, device), t_qw(u, bits, device), t_bf16(x, device)
    got = ops.qmm_swiglu(xt, gq, uq)
    sep = ops.swiglu(ops.qmm(xt, gq), ops.qmm(xt, uq))
    assert torch.equal(got.view(torch.int16), sep.view(torch.int16))
    # two roundings in a row (projection, then SwiGLU): a flipped bf16 rounding of a
    # projection near zero can leave a handful of the elements outside the elementwise
    # bound, so a fraction of 1e-5 is allowed
    want = O.swiglu(affine.qmm(x, *g, 64, bits), affine.qmm(x, *u, 64, bits))
    assert_close_stat(n_f32(got), want, max_outlier_frac=1e-5, what="qmm_swiglu")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(126, 8192, 2048), (40, 256, 1024), (100, 100, 768), (128, 4100, 4096), (17, 64, 512)])
def test_qmm_swiglu_pair_split_k(device, bits, M, N, K):
    """The pair GEMM of a short input with K split over workgroups (partials of both
    projections, then one reduce + SwiGLU launch): against the oracle, and against the unsplit
    launch (same rounding points, the float32 sums in another order), twice in a row on the
    shared workspace."""
    g = rand_quantized(N, K, bits, seed=N + 21)
    u = rand_quantized(N, K, bits, seed=N + 22)
    x = rand_bf16((M, K), seed=M + K + 1)
    gq, uq, xt = t_qw(g, bits, device), t_qw(u, bits, device), t_bf16(x, device)
    assert native.load().exo_qmm_swiglu_workspace(M, N) > 0
    one = ops.qmm_swiglu(xt, gq, uq, split_k=False)
    want = O.swiglu(affine.qmm(x, *g, 64, bits), affine.qmm(x, *u, 64, bits))
    for _ in range(2):
        got = ops.qmm_swiglu(xt, gq, uq)
        assert_close_stat(n_f32(got), want, max_outlier_frac=1e-5, what="qmm_swiglu split-K")
        assert_close_stat(n_f32(got), n_f32(one), max_outlier_frac=1e-4, what="split-K vs one launch")
        ops.qmm(xt, gq)  # another user of the workspace pool in between


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(128, 256, 512), (33, 130, 192), (257, 128, 1024), (17, 64, 64)])
def test_qmm_mfma(device, bits, M, N, K):
    trip = rand_quantized(N, K, bits, seed=M + N)
    x = rand_bf16((M, K), seed=M * 3 + 1)
    got = n_f32(ops.qmm(t_bf16(x, device), t_qw(trip, bits, device)))
    want = affine.qmm(x, *trip, 64, bits)
    assert_close(got, want, what=f"qmm {M}x{N}x{K} b{bits}")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(100, 256, 4096), (33, 130, 14336), (128, 1000, 2048), (17, 64, 1024),
                                   (12, 256, 8192), (9, 96, 1024), (1023, 128, 2048), (300, 200, 4096),
                                   (32, 520, 512), (64, 600, 1024), (65, 300, 768), (20, 257, 256),
                                   (300, 10880, 1024), (1023, 2048, 1024), (300, 4100, 4096), (100, 14336, 4096),
                                   (600, 2052, 4096)])
def test_qmm_split_k(device, bits, M, N, K):
    """Few output tiles (a short input, or a narrow matrix under a long one): K is split
    over workgroups and the float32 partial tiles are added by a second launch.  Against
    the oracle, against the
    unsplit kernel (same products, another summation order: a few bf16 ulps at most),
    with the residual, and three times in a row with identical bits.  The last three
    shapes have K ranges of 1024 and take the wide tile with eight waves (two teams on the
    halves of a range)."""
    trip = rand_quantized(N, K, bits, seed=M + N)
    x = rand_bf16((M, K), seed=M * 3 + 1)
    r = rand_bf16((M, N), seed=M + 5)
    qw, xt, rt = t_qw(trip, bits, device), t_bf16(x, device), t_bf16(r, device)
    want = affine.qmm(x, *trip, 64, bits)
    first = None
    for _ in range(3):
        got = ops.quantized_matmul(xt, qw)
        assert_close(n_f32(got), want, what=f"qmm split-K {M}x{N}x{K} b{bits}")
        first = got.clone() if first is None else first
        assert torch.equal(got.view(torch.int16), first.view(torch.int16))
    unsplit = ops.qmm(xt, qw)
    assert_close(n_f32(got), n_f32(unsplit), rtol=1e-2, what="split vs unsplit")
    got_r = n_f32(ops.quantized_matmul(xt, qw, residual=rt))
    assert_close(got_r, affine.bf16_round(affine.bf16_round(want) + r), what="qmm split-K + residual")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K", [(1100, 4100, 1024), (1300, 2052, 1536), (700, 8192, 1024)])
def test_qmm_eight_wave_tiles(device, bits, M, N, K):
    """Launches of more than 128 tall tiles but at most one tile per CU run eight waves per
    tile, two teams on the two halves of K merged through LDS: the wide 128 x 256 tile with
    the ring of four (4-bit) or the 256 x 128 tile (8-bit).  Ragged M and N, with the residual."""
    trip = rand_quantized(N, K, bits, seed=M + N)
    x = rand_bf16((M, K), seed=M * 3 + 1)
    r = rand_bf16((M, N), seed=M + 5)
    qw, xt, rt = t_qw(trip, bits, device), t_bf16(x, device), t_bf16(r, device)
    want = affine.qmm(x, *trip, 64, bits)
    assert_close(n_f32(ops.qmm(xt, qw)), want, what=f"qmm {M}x{N}x{K} b{bits}")
    got_r = n_f32(ops.quantized_matmul(xt, qw, residual=rt))
    assert_close(got_r, affine.bf16_round(affine.bf16_round(want) + r), what="qmm + residual")


def test_qmm_residual_and_dispatch(device):
    M, N, K, bits = 40, 192, 256, 4
    trip = rand_quantized(N, K, bits, seed=5)
    x = rand_bf16((M, K), seed=6)
    r = rand_bf16((M, N), seed=7)
    got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device), residual=t_bf16(r, device)))
    want = affine.bf16_round(affine.qmm(x, *trip, 64, bits) + r)
    assert_close(got, want, what="qmm+residual")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("x_rows", ["one", "topk"])
def test_gather_qmv(device, bits, x_rows):
    E, N, K, T, topk = 6, 96, 768, 3, 4
    trip = rand_quantized(N, K, bits, seed=40, E=E)
    idx = rng(41).integers(0, E, size=(T, topk)).astype(np.int32)
    R = 1 if x_rows == "one" else topk
    x = rand_bf16((T, R, K), seed=42)
    got = n_f32(ops.gather_qmm(t_bf16(x, device), t_qw(trip, bits, device), torch.from_numpy(idx).to(device)))
    want = affine.gather_qmm(x, *trip, idx, 64, bits)
    assert_close(got, want, what="gather_qmv")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("x_rows", ["one", "topk"])
@pytest.mark.parametrize("E,N,K,T,topk", [(6, 96, 768, 40, 4), (128, 200, 128, 300, 8), (3, 64, 64, 1, 2)])
def test_grouped_qmm(device, bits, x_rows, E, N, K, T, topk):
    """Prefill-sized gather_qmm: pairs sorted by expert, one matrix-core tile row block per
    expert run (experts with no rows, with a partial tile and with several tiles), against
    the oracle's per-pair loop."""
    trip = rand_quantized(N, K, bits, seed=40 + E, E=E)
    idx = rng(41 + T).integers(0, E, size=(T, topk)).astype(np.int32)
    if E == 128:
        idx[: T // 2, 0] = 5  # one expert with more than a tile of rows
    R = 1 if x_rows == "one" else topk
    x = rand_bf16((T, R, K), seed=42)
    it = torch.from_numpy(idx).to(device)
    ws = ops.moe_group(it, E)
    P = T * topk
    sorted_pairs = ws[:P].cpu().numpy()
    assert sorted(sorted_pairs.tolist()) == list(range(P))          # a permutation of the pairs
    experts_in_order = idx.reshape(-1)[sorted_pairs]
    assert np.all(np.diff(experts_in_order) >= 0)                    # grouped by expert
    tiles = ws[P:].cpu().numpy().reshape(-1, 3)
    used = tiles[tiles[:, 0] >= 0]
    assert used[:, 2].sum() == P and used[:, 2].max() <= 128
    got = n_f32(ops.grouped_qmm(t_bf16(x, device), t_qw(trip, bits, device), ws, topk))
    want = affine.gather_qmm(x, *trip, idx, 64, bits)
    assert_close(got, want, what="grouped_qmm")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("E,N,K,T,topk", [(6, 96, 768, 40, 4), (128, 200, 256, 300, 8), (3, 60, 64, 1, 2)])
def test_grouped_qmm_swiglu(device, bits, E, N, K, T, topk):
    """SwitchGLU's gate and up projections with the SwiGLU in the grouped GEMM's epilogue:
    the bits of the two grouped GEMMs followed by the elementwise kernel (ragged tiles,
    N not a multiple of 64 or 8, K with and without the four-step scale blocks)."""
    g = rand_quantized(N, K, bits, seed=60 + E, E=E)
    u = rand_quantized(N, K, bits, seed=61 + E, E=E)
    idx = rng(62 + T).integers(0, E, size=(T, topk)).astype(np.int32)
    if E == 128:
        idx[: T // 2, 0] = 5
    x = t_bf16(rand_bf16((T, 1, K), seed=63), device)
    gq, uq = t_qw(g, bits, device), t_qw(u, bits, device)
    ws = ops.moe_group(torch.from_numpy(idx).to(device), E)
    got = ops.grouped_qmm_swiglu(x, gq, uq, ws, topk)
    sep = ops.swiglu(ops.grouped_qmm(x, gq, ws, topk), ops.grouped_qmm(x, uq, ws, topk))
    assert torch.equal(got.view(torch.int16), sep.view(torch.int16))


@pytest.mark.parametrize("bits", [4, 8])
def test_gather_qmv_swiglu(device, bits):
    E, N, K, T, topk = 5, 64, 2048, 2, 3
    g = rand_quantized(N, K, bits, seed=50, E=E)
    u = rand_quantized(N, K, bits, seed=51, E=E)
    idx = rng(52).integers(0, E, size=(T, topk)).astype(np.int32)
    x = rand_bf16((T, K), seed=53)
    got = n_f32(ops.gather_qmv_swiglu(t_bf16(x, device), t_qw(g, bits, device), t_qw(u, bits, device), torch.from_numpy(idx).to(device)))
    want = O.swiglu(affine.gather_qmm(x[:, None], *g, idx, 64, bits), affine.gather_qmm(x[:, None], *u, idx, 64, bits))
    assert_close(got, want, what="gather_qmv_swiglu")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("E,N,K,T,topk,renorm,norm", [(128, 768, 2048, 1, 8, True, True), (128, 768, 2048, 4, 8, True, True),
                                                      (60, 64, 2048, 3, 4, False, False), (256, 96, 512, 2, 16, True, True),
                                                      (7, 200, 768, 5, 3, True, False)])
def test_route_gather_qmv_swiglu_equals_topk_then_gather(device, bits, E, N, K, T, topk, renorm, norm):
    """The expert gate/up launch that routes by itself: the indices and scores it writes are
    those of exo_router_topk bit for bit, its output that of the gather launch given them
    (row-streaming and generic kernel, with and without the fused norm); indices also against
    the oracle."""
    g = rand_quantized(N, K, bits, seed=70 + E, E=E)
    u = rand_quantized(N, K, bits, seed=71 + E, E=E)
    logits = rand_bf16((T, E), seed=72 + E, scale=2.0)
    x = t_bf16(rand_bf16((T, K), seed=73), device)
    nw = t_bf16(affine.bf16_round(rand_bf16((K,), seed=74) + 1.0), device) if norm else None
    gq, uq, lt = t_qw(g, bits, device), t_qw(u, bits, device), t_bf16(logits, device)
    idx0, sc0 = ops.router_topk(lt, topk, renorm)
    want = ops.gather_qmv_swiglu(x, gq, uq, idx0, norm_weight=nw, eps=1e-5)
    for _ in range(2):
        idx, sc, got = ops.route_gather_qmv_swiglu(x, lt, topk, renorm, gq, uq, norm_weight=nw, eps=1e-5)
        assert torch.equal(idx, idx0)
        assert torch.equal(sc.view(torch.int16), sc0.view(torch.int16))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    np.testing.assert_array_equal(idx0.cpu().numpy(), O.router_topk(logits, topk, renorm)[0])


def test_bad_arguments_raise(device):
    trip = rand_quantized(64, 128, 4, seed=1)
    qw = t_qw(trip, 4, device)
    with pytest.raises(ValueError):
        ops.quantized_matmul(t_bf16(rand_bf16((1, 64), 1), device), qw)
    lib = native.load()
    assert lib.exo_qmv(None, None, None, None, None, None, 1, 64, 128, 5, 64, None) == -1
    assert b"bits" in lib.exo_last_error()
    assert lib.exo_qmv(None, None, None, None, None, None, 1, 64, 128, 4, 32, None) == -1
    assert lib.exo_qmv(None, None, None, None, None, None, 17, 64, 128, 4, 64, None) == -1


@pytest.mark.parametrize("H", [2048, 4096, 64, 8192])
@pytest.mark.parametrize("with_res", [False, True])
def test_add_rmsnorm(device, H, with_res):
    rows = 5
    x = rand_bf16((rows, H), seed=H)
    r = rand_bf16((rows, H), seed=H + 1) if with_res else None
    w = rand_bf16((H,), seed=H + 2) + 1.0
    w = affine.bf16_round(w)
    h, n = ops.add_rms_norm(t_bf16(x, device), t_bf16(r, device) if with_res else None, t_bf16(w, device), 1e-5)
    hh = affine.bf16_round(x + r) if with_res else x
    np.testing.assert_array_equal(n_f32(h), hh)
    assert_close(n_f32(n), O.rms_norm(hh, w, 1e-5), rtol=1e-2, what="rmsnorm")


@pytest.mark.parametrize("D,Hq,Hkv", [(64, 8, 2), (128, 4, 4), (128, 16, 2)])
@pytest.mark.parametrize("qk_norm", [False, True])
def test_rope_kv_append(device, D, Hq, Hkv, qk_norm):
    B, T, S_max = 2, 3, 40
    pos = np.array([5, 17], np.int32)
    qkv = rand_bf16((B * T, (Hq + 2 * Hkv) * D), seed=D + Hq)
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
    inv = O.rope_inv_freq(D, 5e5, scaling)
    qn = affine.bf16_round(rand_bf16((D,), 3) + 1.0) if qk_norm else None
    kn = affine.bf16_round(rand_bf16((D,), 4) + 1.0) if qk_norm else None
    kc = torch.zeros(B, Hkv, S_max, D, dtype=torch.bfloat16, device=device)
    vc = torch.zeros_like(kc)
    q_out = torch.empty(B * T, Hq * D, dtype=torch.bfloat16, device=device)
    ops.rope_kv_append(
        t_bf16(qkv, device), q_out, kc, vc, torch.from_numpy(pos).to(device),
        torch.from_numpy(inv).to(device), B, T, Hq, Hkv, D,
        t_bf16(qn, device) if qk_norm else None, t_bf16(kn, device) if qk_norm else None, 1e-6,
    )
    x = qkv.reshape(B, T, Hq + 2 * Hkv, D)
    q, k, v = x[:, :, :Hq], x[:, :, Hq:Hq + Hkv], x[:, :, Hq + Hkv:]
    if qk_norm:
        q = O.rms_norm(q, qn, 1e-6)
        k = O.rms_norm(k, kn, 1e-6)
    for b in range(B):
        qr = O.rope(q[b:b + 1].transpose(0, 2, 1, 3), inv, int(pos[b]))  # [1,H,T,D]
        kr = O.rope(k[b:b + 1].transpose(0, 2, 1, 3), inv, int(pos[b]))
        got_q = n_f32(q_out).reshape(B, T, Hq, D)[b].transpose(1, 0, 2)
        assert_close(got_q, qr[0], rtol=1e-2, what="rope q")
        got_k = n_f32(kc)[b, :, pos[b]:pos[b] + T]
        assert_close(got_k, kr[0], rtol=1e-2, what="rope k")
        np.testing.assert_array_equal(n_f32(vc)[b, :, pos[b]:pos[b] + T], v[b].transpose(1, 0, 2))
    # nothing outside the appended window was written
    assert float(n_f32(kc)[0, :, :5].sum()) == 0.0 and float(n_f32(kc)[0, :, 8:].sum()) == 0.0
    # with the angle table (long enough; too short for the second sequence): the same bits
    inv_t = torch.from_numpy(inv).to(device)
    for rows in (S_max, 12):
        kc2, vc2, q2 = torch.zeros_like(kc), torch.zeros_like(vc), torch.empty_like(q_out)
        ops.rope_kv_append(
            t_bf16(qkv, device), q2, kc2, vc2, torch.from_numpy(pos).to(device), inv_t, B, T, Hq, Hkv, D,
            t_bf16(qn, device) if qk_norm else None, t_bf16(kn, device) if qk_norm else None, 1e-6,
            rope_tab=ops.rope_table(inv_t, rows, D),
        )
        for a, b_ in ((q2, q_out), (kc2, kc), (vc2, vc)):
            assert torch.equal(a.view(torch.int16), b_.view(torch.int16))


@pytest.mark.parametrize("D,Hq,Hkv", [(64, 32, 8), (128, 32, 8), (128, 32, 4), (128, 64, 4), (128, 4, 4)])
@pytest.mark.parametrize("lens", [[1, 2], [100, 37], [513, 1024]])
def test_sdpa_decode(device, D, Hq, Hkv, lens):
    B, S_max = len(lens), 1024
    q = rand_bf16((B, Hq * D), seed=D + Hq + lens[0])
    k = rand_bf16((B, Hkv, S_max, D), seed=11)
    v = rand_bf16((B, Hkv, S_max, D), seed=12)
    pos = np.array([n - 1 for n in lens], np.int32)
    out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=device)
    ws = ops.sdpa_decode_workspace(B, Hq, D, device)
    ops.sdpa_decode(t_bf16(q, device), t_bf16(k, device), t_bf16(v, device), torch.from_numpy(pos).to(device), out, ws, D ** -0.5, B, Hq, Hkv, D)
    for b in range(B):
        want = O.sdpa(q[b].reshape(1, Hq, 1, D), k[b:b + 1, :, :lens[b]], v[b:b + 1, :, :lens[b]], D ** -0.5, None)
        assert_close(n_f32(out)[b].reshape(Hq, D), want[0, :, 0], what=f"sdpa decode len {lens[b]}")


@pytest.mark.parametrize("D,Hq,Hkv", [(64, 8, 2), (128, 8, 2), (128, 4, 4), (128, 4, 2), (128, 16, 2), (64, 16, 1)])
@pytest.mark.parametrize("T,pos", [(19, (0, 30)), (5, (0, 3)), (100, (0, 77)), (64, (64, 1)), (161, (0, 200))])
def test_sdpa_prefill_causal(device, D, Hq, Hkv, T, pos):
    """Chunks shorter than 8 tokens run the per-token kernel, longer ones the matrix-core
    flash kernel: 1, 2, 4, 8 and 16 query heads per kv head, chunk lengths on and off the
    32-token tile, caches that start empty and part-filled, several key tiles."""
    B, S_max = 2, 384
    pos = np.array(pos, np.int32)
    q = rand_bf16((B * T, Hq * D), seed=D + T)
    k = rand_bf16((B, Hkv, S_max, D), seed=13)
    v = rand_bf16((B, Hkv, S_max, D), seed=14)
    out = torch.empty(B * T, Hq * D, dtype=torch.bfloat16, device=device)
    ops.sdpa_prefill(t_bf16(q, device), t_bf16(k, device), t_bf16(v, device), torch.from_numpy(pos).to(device), out, D ** -0.5, B, T, Hq, Hkv, D)
    for b in range(B):
        S = int(pos[b]) + T
        qq = q.reshape(B, T, Hq, D)[b:b + 1].transpose(0, 2, 1, 3)
        want = O.sdpa(qq, k[b:b + 1, :, :S], v[b:b + 1, :, :S], D ** -0.5, S - T)
        got = n_f32(out).reshape(B, T, Hq, D)[b].transpose(1, 0, 2)
        assert_close(got, want[0], what=f"sdpa prefill T={T} pos={pos[b]}")


def test_sdpa_prefill_cache_exactly_full(device):
    """The last key tile ends at the end of the cache allocation (no reads past it)."""
    B, T, Hq, Hkv, D, S_max = 1, 40, 8, 2, 128, 100
    pos = np.array([60], np.int32)
    q = rand_bf16((B * T, Hq * D), seed=3)
    k = rand_bf16((B, Hkv, S_max, D), seed=4)
    v = rand_bf16((B, Hkv, S_max, D), seed=5)
    out = torch.empty(B * T, Hq * D, dtype=torch.bfloat16, device=device)
    ops.sdpa_prefill(t_bf16(q, device), t_bf16(k, device), t_bf16(v, device), torch.from_numpy(pos).to(device), out, D ** -0.5, B, T, Hq, Hkv, D)
    qq = q.reshape(B, T, Hq, D).transpose(0, 2, 1, 3)
    want = O.sdpa(qq, k, v, D ** -0.5, S_max - T)
    assert_close(n_f32(out).reshape(T, Hq, D).transpose(1, 0, 2), want[0], what="sdpa prefill full cache")


def test_swiglu(device):
    g = rand_bf16((3, 1001), seed=1, scale=3.0)
    u = rand_bf16((3, 1001), seed=2)
    got = n_f32(ops.swiglu(t_bf16(g, device), t_bf16(u, device)))
    assert_close(got, O.swiglu(g, u), rtol=1e-2, what="swiglu")


@pytest.mark.parametrize("E,k,renorm", [(128, 8, True), (128, 8, False), (60, 4, True), (256, 16, True)])
def test_router_topk(device, E, k, renorm):
    rows = 9
    logits = rand_bf16((rows, E), seed=E + k, scale=2.0)
    idx, sc = ops.router_topk(t_bf16(logits, device), k, renorm)
    widx, wsc = O.router_topk(logits, k, renorm)
    np.testing.assert_array_equal(idx.cpu().numpy(), widx)
    assert_close(n_f32(sc), wsc, rtol=2.0**-7, what="router scores")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("E,N,K,T,topk", [(6, 200, 768, 3, 8), (5, 96, 1536, 2, 4), (4, 64, 2048, 1, 2),
                                          (3, 72, 192, 2, 3), (9, 64, 768, 2, 9)])
def test_gather_qmv_combine(device, bits, E, N, K, T, topk):
    """Down projection of SwitchGLU + weighted sum over the experts + residual in one
    launch: against the oracle, and against the two separate launches it replaces
    (same rounding points; the dot products are summed in another order).  The last two
    shapes take the fallback through the scratch buffer (rows that share a wave by
    threes; more than 8 experts per token)."""
    trip = rand_quantized(N, K, bits, seed=E + N, E=E)
    idx = rng(43).integers(0, E, size=(T, topk)).astype(np.int32)
    x = rand_bf16((T, topk, K), seed=44)
    sc = affine.bf16_round(np.abs(rand_bf16((T, topk), seed=45)) / 8)
    r = rand_bf16((T, N), seed=46)
    qw, xt, it = t_qw(trip, bits, device), t_bf16(x, device), torch.from_numpy(idx).to(device)
    st, rt = t_bf16(sc, device), t_bf16(r, device)
    scratch = torch.empty(T, topk, N, dtype=torch.bfloat16, device=device)
    got = ops.gather_qmv_combine(xt, qw, it, st, residual=rt, scratch=scratch)
    eo = affine.gather_qmm(x, *trip, idx, 64, bits)
    acc = affine.bf16_round(affine.bf16_round(eo * sc[..., None]).sum(1, dtype=np.float32))
    assert_close(n_f32(got), affine.bf16_round(acc + r), what="gather_qmv_combine")
    sep = ops.moe_combine(ops.gather_qmm(xt, qw, it), st, rt)
    assert_close(n_f32(got), n_f32(sep), rtol=1e-2, what="fused vs separate")
    no_res = ops.gather_qmv_combine(xt, qw, it, st, scratch=scratch)
    assert_close(n_f32(no_res), acc, what="gather_qmv_combine without residual")


@pytest.mark.parametrize("T,topk,H", [(3, 8, 2048), (5, 6, 4096), (2, 3, 100), (4, 9, 264)])
def test_moe_combine(device, T, topk, H):
    """Rows of 8-element multiples take the 16-byte kernel (slots in groups of four, the
    last group partial), the others the scalar one."""
    y = rand_bf16((T, topk, H), seed=1)
    s = affine.bf16_round(np.abs(rand_bf16((T, topk), seed=2)) / 8)
    r = rand_bf16((T, H), seed=3)
    got = n_f32(ops.moe_combine(t_bf16(y, device), t_bf16(s, device), t_bf16(r, device)))
    acc = affine.bf16_round(affine.bf16_round(y * s[..., None]).sum(1, dtype=np.float32))
    assert_close(got, affine.bf16_round(acc + r), rtol=1e-2, what="moe_combine")


@pytest.mark.parametrize("V", [128256, 1000, 64])
def test_argmax_logsumexp(device, V):
    rows = 3
    logits = rand_bf16((rows, V), seed=V, scale=2.0)
    logits[1, 7] = logits[1].max()  # a tie: lowest index must win
    tok = torch.empty(rows, dtype=torch.int32, device=device)
    lse = torch.empty(rows, dtype=torch.float32, device=device)
    lp = torch.empty(rows, dtype=torch.float32, device=device)
    pos = torch.tensor([4, 5, 6], dtype=torch.int32, device=device)
    ops.argmax_logsumexp(t_bf16(logits, device), tok, lse, lp, ops.argmax_workspace(rows, device), pos)
    np.testing.assert_array_equal(tok.cpu().numpy(), np.argmax(logits, -1))
    want_lse = O.logsumexp(logits)[:, 0]
    np.testing.assert_allclose(lse.cpu().numpy(), want_lse, rtol=1e-5)
    np.testing.assert_allclose(lp.cpu().numpy(), logits.max(-1) - want_lse, rtol=1e-4, atol=1e-5)
    assert pos.cpu().tolist() == [5, 6, 7]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("N,K,M", [(256, 4096, 1), (128, 14336, 2), (96, 768, 1), (64, 2048, 4), (72, 192, 3),
                                   (200, 4096, 2), (64, 8192, 2)])
def test_norm_qmv_fused(device, bits, N, K, M):
    trip = rand_quantized(N, K, bits, seed=N + K)
    x = rand_bf16((M, K), seed=K + M, scale=3.0)
    w = affine.bf16_round(rand_bf16((K,), seed=5) * 0.1 + 1.0)
    got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device), norm_weight=t_bf16(w, device), eps=1e-5))
    want = affine.qmm(O.rms_norm(x, w, 1e-5), *trip, 64, bits)
    assert_close(got, want, what="norm+qmv")
    g = rand_quantized(N, K, bits, seed=N + K + 1)
    got = n_f32(ops.qmv_swiglu(t_bf16(x, device), t_qw(trip, bits, device), t_qw(g, bits, device), norm_weight=t_bf16(w, device), eps=1e-5))
    xn = O.rms_norm(x, w, 1e-5)
    assert_close(got, O.swiglu(affine.qmm(xn, *trip, 64, bits), affine.qmm(xn, *g, 64, bits)), what="norm+qmv_swiglu")


@pytest.mark.parametrize("D,Hq,Hkv", [(64, 32, 8), (128, 32, 8), (128, 64, 4), (128, 4, 4), (128, 32, 4),
                                      (128, 16, 4)])
@pytest.mark.parametrize("qk_norm", [False, True])
@pytest.mark.parametrize("lens", [[1, 2], [100, 37], [513, 1000], [129, 33, 1024, 257]])
@pytest.mark.parametrize("table", [False, True])
def test_attn_decode_fused(device, D, Hq, Hkv, qk_norm, lens, table):
    """rope + head norm + cache append + attention in one launch == the three oracle ops."""
    B, S_max = len(lens), 1024
    pos = np.array([n - 1 for n in lens], np.int32)
    qkv = rand_bf16((B, (Hq + 2 * Hkv) * D), seed=D + Hq + lens[0])
    k = rand_bf16((B, Hkv, S_max, D), seed=11)
    v = rand_bf16((B, Hkv, S_max, D), seed=12)
    inv = O.rope_inv_freq(D, 5e5, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192})
    qn = affine.bf16_round(rand_bf16((D,), 3) * 0.1 + 1.0) if qk_norm else None
    kn = affine.bf16_round(rand_bf16((D,), 4) * 0.1 + 1.0) if qk_norm else None
    kc, vc = t_bf16(k, device), t_bf16(v, device)
    out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=device)
    ws = ops.sdpa_decode_workspace(B, Hq, D, device)
    inv_t = torch.from_numpy(inv).to(device)
    tab = ops.rope_table(inv_t, S_max, D) if table else None
    for _ in range(2):  # twice: the arrival counters must be back at zero
        ops.attn_decode(t_bf16(qkv, device), kc, vc, torch.from_numpy(pos).to(device),
                        inv_t, out, ws, D ** -0.5, B, Hq, Hkv, D,
                        t_bf16(qn, device) if qk_norm else None, t_bf16(kn, device) if qk_norm else None, 1e-6,
                        rope_tab=tab)
    x = qkv.reshape(B, 1, Hq + 2 * Hkv, D)
    q, kk, vv = x[:, :, :Hq], x[:, :, Hq:Hq + Hkv], x[:, :, Hq + Hkv:]
    if qk_norm:
        q, kk = O.rms_norm(q, qn, 1e-6), O.rms_norm(kk, kn, 1e-6)
    for b in range(B):
        p = int(pos[b])
        qr = O.rope(q[b:b + 1].transpose(0, 2, 1, 3), inv, p)
        kr = O.rope(kk[b:b + 1].transpose(0, 2, 1, 3), inv, p)
        kfull = np.concatenate([k[b:b + 1, :, :p], kr], axis=2)
        vfull = np.concatenate([v[b:b + 1, :, :p], vv[b:b + 1].transpose(0, 2, 1, 3)], axis=2)
        want = O.sdpa(qr, kfull, vfull, D ** -0.5, None)
        assert_close(n_f32(out)[b].reshape(Hq, D), want[0, :, 0], what=f"attn_decode len {lens[b]}")
        assert_close(n_f32(kc)[b, :, p], kr[0, :, 0], rtol=1e-2, what="appended k")
        np.testing.assert_array_equal(n_f32(vc)[b, :, p], vv[b, 0])
        np.testing.assert_array_equal(n_f32(kc)[b, :, p + 1:], k[b, :, p + 1:])  # nothing else touched
        np.testing.assert_array_equal(n_f32(kc)[b, :, :p], k[b, :, :p])


# ------------------------------------------------------------------ KV wire layout


@pytest.mark.parametrize("Hkv,S_max,D,start,n", [(8, 64, 128, 0, 64), (4, 300, 64, 7, 201),
                                                 (2, 16, 8, 15, 1), (3, 40, 128, 5, 0)])
def test_kv_export_import_nhd(device, Hkv, S_max, D, start, n):
    """Byte-exact against the transpose the reference ships
    (engines/mlx/disaggregated/adapter.py:74-83): wire[t,h,:] = cache[h,start+t,:]."""
    g = torch.Generator(device="cpu").manual_seed(5)
    row = torch.randn(Hkv, S_max, D, generator=g).bfloat16().to(device)
    wire = ops.kv_export_nhd(row, start, n)
    want = row[:, start:start + n].permute(1, 0, 2).contiguous()
    assert wire.shape == (n, Hkv, D) and torch.equal(wire.view(torch.int16), want.view(torch.int16))
    dst = torch.full_like(row, 7.0)
    ops.kv_import_nhd(wire, dst, start)
    ref = torch.full_like(row, 7.0)
    ref[:, start:start + n] = row[:, start:start + n]
    assert torch.equal(dst.view(torch.int16), ref.view(torch.int16))


def test_kv_wire_argument_errors(device):
    row = torch.zeros(2, 16, 8, dtype=torch.bfloat16, device=device)
    with pytest.raises(ValueError):
        ops.kv_export_nhd(row, 10, 7)            # beyond S_max
    with pytest.raises(ValueError):
        ops.kv_export_nhd(row, -1, 2)
    with pytest.raises(ValueError):
        ops.kv_import_nhd(torch.zeros(3, 2, 4, dtype=torch.bfloat16, device=device), row, 0)
    with pytest.raises(ValueError):
        ops.kv_export_nhd(torch.zeros(2, 16, 12, dtype=torch.bfloat16, device=device), 0, 1)


def test_qmv_workspace_shared_by_launches_of_different_shapes(device):
    """The split-K workspace is shared by all 2..16-row GEMVs of a device: a launch with a
    short N must not leave anything where a later launch with more row blocks keeps its
    arrival counters (the partial sums sit behind a counter area of fixed size)."""
    for bits, M, N, K in [(4, 3, 128, 4096), (4, 16, 4096, 14336), (8, 5, 64, 2048), (8, 8, 4096, 14336),
                          (4, 16, 4096, 14336)]:
        trip = rand_quantized(64, K, bits, seed=N + K + bits)
        reps = N // 64
        trip = tuple(np.concatenate([t] * reps) for t in trip)  # N rows from 64 distinct ones
        x = rand_bf16((M, K), seed=M + K)
        got = n_f32(ops.quantized_matmul(t_bf16(x, device), t_qw(trip, bits, device)))
        want = np.tile(affine.qmm(x, *(t[:64] for t in trip), 64, bits), (1, reps))
        assert_close(got, want, what=f"qmv {M}x{N}x{K} b{bits}")
