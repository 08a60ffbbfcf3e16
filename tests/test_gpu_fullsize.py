"""Parity at the benchmark configurations' real shapes.

The small-shape tests compare every element against the oracle; here the matrices are the
size the configurations name (up to 128256 x 4096), so the oracle checks a seeded
subsample of output rows and the whole result is held to properties that do not depend
on size: agreement with `dequantize` (bit-exact against the oracle elsewhere) followed
by a float32 library matmul, and embed(ids) == rows of dequantize(W).  One transformer
block of each model family at its real shape is compared with the oracle directly.
"""

import dataclasses

import numpy as np
import pytest
import torch

from oracle import affine
from oracle import models as OM
from tests.util import (assert_close, assert_close_stat, check_tokens, n_bits, n_f32, rand_bf16,
                        t_bf16, weights_to_numpy)

pytestmark = pytest.mark.gpu

from exo_amd import ops  # noqa: E402
from exo_amd.config import named_config  # noqa: E402
from exo_amd.model import ShardModel  # noqa: E402
from exo_amd.ops import QuantizedWeight  # noqa: E402
from exo_amd.synth import synth_weights  # noqa: E402

SWEEP_SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]


def _packed(N, K, bits, seed, device):
    """Already-packed random matrix: every code value occurs, scales ~ the magnitude
    N(0, 0.02) weights quantise to, biases near -half-range (signed weights)."""
    g = torch.Generator(device=device).manual_seed(seed)
    w = torch.randint(-2**31, 2**31 - 1, (N, K * bits // 32), dtype=torch.int32, device=device, generator=g)
    levels = float(2**bits - 1)
    s = (torch.rand(N, K // 64, device=device, generator=g) * 0.1 + 0.05) / levels
    b = -s * levels * (0.4 + 0.2 * torch.rand(N, K // 64, device=device, generator=g))
    return QuantizedWeight(w, s.bfloat16(), b.bfloat16(), bits)


def _rows_np(qw, rows):
    r = torch.as_tensor(rows, device=qw.weight.device)
    return (qw.weight[r].cpu().numpy().view(np.uint32), n_bits(qw.scales[r]), n_bits(qw.biases[r]))


# projections of the other configurations whose workgroup count is rounded to whole
# multiples of the CU count or to an even number of rows per wave: 5 and 3 rows per wave,
# a split of 9216 rows over 768 workgroups, one-unit rows of a 151936-row head
LAUNCH_SHAPES = [(5120, 2048, 4), (3072, 2048, 4), (6144, 4096, 4), (9216, 4096, 8),
                 (4096, 8192, 8), (6144, 4096, 8), (151936, 2048, 4)]


@pytest.mark.parametrize("N,K,bits", LAUNCH_SHAPES)
def test_qmv_launch_shapes(device, N, K, bits):
    """Single-row and 8-row GEMV with the fused RMSNorm and with the fused residual, every
    output against dequantize + float32 matmul, a row sample against the oracle."""
    qw = _packed(N, K, bits, seed=N + K + bits, device=device)
    rows = np.unique(np.concatenate([[0, 1, N - 2, N - 1], np.random.default_rng(N).integers(0, N, 124)]))
    sub = _rows_np(qw, rows)
    rt = torch.as_tensor(rows, device=device)
    wd = ops.dequantize(qw).float()
    nw = affine.bf16_round(rand_bf16((K,), seed=7) * 0.1 + 1.0)
    nwt = t_bf16(nw, device)
    for M in (1, 8):
        x = rand_bf16((M, K), seed=M + N)
        xt = t_bf16(x, device)
        res = rand_bf16((M, N), seed=M + K)
        y = ops.quantized_matmul(xt, qw, residual=t_bf16(res, device))
        want = affine.bf16_round(affine.qmm(x, *sub, 64, bits)) + res[:, rows]
        assert_close(n_f32(y[:, rt]), affine.bf16_round(want), what=f"residual, oracle rows, {M}x{N}x{K} b{bits}")
        full = (xt.float() @ wd.T).bfloat16().float() + t_bf16(res, device).float()
        assert_close(n_f32(y), n_f32(full), what=f"residual, all outputs, {M}x{N}x{K} b{bits}")
        yn = ops.quantized_matmul(xt, qw, norm_weight=nwt, eps=1e-5)
        xn = ops.rms_norm(xt, nwt, 1e-5)
        assert_close(n_f32(yn), n_f32(xn.float() @ wd.T), what=f"norm, all outputs, {M}x{N}x{K} b{bits}")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("N,K", SWEEP_SHAPES)
def test_qmatmul_sweep_shapes(device, bits, N, K):
    """Every (N,K) of the qmatmul sweep at M = 1, 2, 3, 4, 16 (GEMV kernels) and 128 (MFMA
    GEMM), plus M = 2048 where the output stays small."""
    qw = _packed(N, K, bits, seed=N + K + bits, device=device)
    rows = np.unique(np.concatenate([[0, 1, N - 2, N - 1], np.random.default_rng(N + K).integers(0, N, 188)]))
    sub = _rows_np(qw, rows)
    wd = ops.dequantize(qw).float()            # [N,K]; bit-exact vs the oracle in its own test
    for M in [1, 2, 3, 4, 16, 128] + ([2048] if N <= 14336 else []):
        x = rand_bf16((M, K), seed=M + K)
        xt = t_bf16(x, device)
        y = ops.quantized_matmul(xt, qw)
        assert y.shape == (M, N) and y.dtype == torch.bfloat16
        m_or = min(M, 16)                      # the oracle finishes 16 rows in about a second
        want = affine.qmm(x[:m_or], *sub, 64, bits)
        assert_close(n_f32(y[:m_or][:, torch.as_tensor(rows, device=device)]), want,
                     what=f"oracle rows, {M}x{N}x{K} b{bits}")
        full = xt.float() @ wd.T               # float32 library matmul over ALL outputs
        assert_close(n_f32(y), n_f32(full), what=f"all outputs vs dequantize+matmul, {M}x{N}x{K} b{bits}")


@pytest.mark.parametrize("bits", [4, 8])
def test_embedding_table_at_vocab_size(device, bits):
    """embed(ids) == dequantize(W)[ids] bit for bit at 128256 x 4096 and 151936 x 2048."""
    for V, H in ((128256, 4096), (151936, 2048)):
        qw = _packed(V, H, bits, seed=V + bits, device=device)
        ids = torch.from_numpy(np.random.default_rng(V).integers(0, V, 300).astype(np.int32))
        ids[:3] = torch.tensor([0, V - 1, V // 2], dtype=torch.int32)
        got = ops.embed(ids.to(device), qw)
        want = ops.dequantize(qw)[ids.long().to(device)]
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        sub = _rows_np(qw, ids[:16].numpy())
        ref = affine.dequantize(*sub, 64, bits, mode="M1")
        assert np.array_equal(n_bits(got[:16]), ref)  # the oracle returns bf16 bits
        del qw


def _one_layer(name, device, seed=5):
    """Layer 1 of a three-layer model with the named architecture's real shapes: a middle
    shard, so hidden state in, hidden state out."""
    cfg = dataclasses.replace(named_config(name), num_hidden_layers=3)
    w = synth_weights(cfg, 1, 2, seed=seed, device=device)
    gm = ShardModel(cfg, w, 1, 2, device)
    ocfg = OM.Config.from_json(cfg.to_dict())
    om = OM.ShardModel(ocfg, weights_to_numpy(w), 1, 2, gemm_rows=16, use_c=True)
    return cfg, gm, om


@pytest.mark.parametrize("name", ["llama-3.2-1b", "llama-3.1-8b"])
def test_llama_block_at_real_shape(device, name):
    """One block: a 24-token chunk (MFMA GEMM + causal attention) then three single-token
    steps (GEMV + decode attention) on the same cache, against the oracle."""
    cfg, gm, om = _one_layer(name, device)
    oc, gc = OM.make_kv_cache(1), gm.make_cache(1, 64)
    h = rand_bf16((1, 24, cfg.hidden_size), seed=24)
    assert_close(n_f32(gm(None, gc, input_embeddings=t_bf16(h, device))),
                 om(None, oc, input_hidden=h), what=f"{name} block T=24")
    for step in range(3):
        h1 = rand_bf16((1, 1, cfg.hidden_size), seed=100 + step)
        assert_close(n_f32(gm(None, gc, input_embeddings=t_bf16(h1, device))),
                     om(None, oc, input_hidden=h1), what=f"{name} block step {step}")
    assert gc[0].offset == 27 and oc[0].offset == 27


@pytest.mark.parametrize("name,T", [("qwen3-30b-a3b", 6), ("qwen3-235b-a22b", 3)])
def test_moe_block_at_real_shape(device, name, T):
    """128 experts, top-8, q/k-norm at the real expert shapes (768x2048 4-bit, 1536x4096
    8-bit): a short chunk and two single-token steps.  A token whose router decision is a
    near-tie in the oracle may pick another expert and is exempt (printed)."""
    cfg, gm, om = _one_layer(name, device)
    oc, gc = OM.make_kv_cache(1), gm.make_cache(1, 32)
    h = rand_bf16((1, T, cfg.hidden_size), seed=T)
    om.router_margins.clear()
    want = om(None, oc, input_hidden=h)
    got = n_f32(gm(None, gc, input_embeddings=t_bf16(h, device)))
    tied = check_tokens(got, want, om, f"{name} block T={T}")
    for step in range(2):
        if tied:
            break
        h1 = rand_bf16((1, 1, cfg.hidden_size), seed=200 + step)
        om.router_margins.clear()
        want = om(None, oc, input_hidden=h1)
        got = n_f32(gm(None, gc, input_embeddings=t_bf16(h1, device)))
        tied = check_tokens(got, want, om, f"{name} block step {step}")


@pytest.mark.parametrize("Hq,Hkv,S", [(32, 8, 2304), (32, 4, 1280), (64, 4, 4224)])
def test_decode_attention_at_config_lengths(device, Hq, Hkv, S):
    """Decode attention at the cache lengths the configurations reach (2048+256, 1024+256,
    4096+128) against float32 library attention over the same cache."""
    D, B = 128, 1
    g = torch.Generator(device=device).manual_seed(S)
    k = torch.randn(B, Hkv, S, D, device=device, generator=g).bfloat16()
    v = torch.randn(B, Hkv, S, D, device=device, generator=g).bfloat16()
    q = torch.randn(B, Hq * D, device=device, generator=g).bfloat16()
    pos = torch.tensor([S - 1], dtype=torch.int32, device=device)  # attends over pos+1 keys
    ws = ops.sdpa_decode_workspace(B, Hq, D, device)
    out = torch.empty_like(q)
    ops.sdpa_decode(q, k, v, pos, out, ws, D ** -0.5, B, Hq, Hkv, D)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.view(B, Hq, 1, D).float(), k.float(), v.float(), enable_gqa=True)
    assert_close(n_f32(out.view(B, Hq, D)), n_f32(ref.view(B, Hq, D)), what=f"decode sdpa S={S}")
