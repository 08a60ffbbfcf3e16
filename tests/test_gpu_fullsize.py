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
    """Every (N,K) of the qmatmul sweep at M = 1, 2, 3, 4, 5, 8, 12, 16 (GEMV kernels), 24, 32 and 64
    (the 256-column GEMM tile with K split up to 16 ways) and 128 (128-row tile), plus M = 2048
    where the output stays small."""
    qw = _packed(N, K, bits, seed=N + K + bits, device=device)
    rows = np.unique(np.concatenate([[0, 1, N - 2, N - 1], np.random.default_rng(N + K).integers(0, N, 188)]))
    sub = _rows_np(qw, rows)
    wd = ops.dequantize(qw).float()            # [N,K]; bit-exact vs the oracle in its own test
    for M in [1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 64, 128] + ([2048] if N <= 14336 else []):
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


# ------------------------------------------------------------------ workload-size attention


def _causal_ref(q, k, v, pos, T, heads, Hq, Hkv, D):
    """float32 library attention for a subset of query heads: q [T, Hq*D] of one sequence,
    k/v [Hkv, S_max, D], query t attends keys j <= pos + t."""
    S = pos + T
    G = Hq // Hkv
    qh = q.view(T, Hq, D)[:, heads].permute(1, 0, 2).float()              # [h, T, D]
    kv = torch.as_tensor([h // G for h in heads], device=q.device)
    kk, vv = k[kv, :S].float(), v[kv, :S].float()                          # [h, S, D]
    mask = torch.arange(S, device=q.device)[None, :] <= (pos + torch.arange(T, device=q.device))[:, None]
    return torch.nn.functional.scaled_dot_product_attention(qh, kk, vv, attn_mask=mask)  # [h, T, D]


@pytest.mark.parametrize("Hq,Hkv,T,pos,S_max", [
    (32, 8, 2046, 0, 2304),      # Llama-3.1-8B prompt chunk
    (32, 4, 1022, 0, 1280),      # Qwen3-30B-A3B prompt chunk
    (64, 4, 4094, 0, 4224),      # Qwen3-235B-A22B prompt chunk
    (32, 8, 2048, 1500, 8192),   # a later chunk of a long prompt in the engine's default cache
    (32, 8, 4096, 4096, 8192),   # a full-size chunk ending exactly at the end of the cache
    (32, 4, 1024, 39936, 40960),   # the last chunk of a prompt that fills Qwen3's 40960 positions
    (32, 8, 1024, 130048, 131072), # the same at Llama-3.1's 131072 positions
])
def test_prefill_attention_at_config_lengths(device, Hq, Hkv, T, pos, S_max):
    """The matrix-core flash kernel over thousands of keys (many key tiles, the causal edge
    inside the last tiles) against float32 library attention, on the first, a middle and the
    last query head of the first and the last kv head."""
    D = 128
    g = torch.Generator(device=device).manual_seed(T + pos)
    q = torch.randn(T, Hq * D, device=device, generator=g).bfloat16()
    k = torch.randn(1, Hkv, S_max, D, device=device, generator=g).bfloat16()
    v = torch.randn(1, Hkv, S_max, D, device=device, generator=g).bfloat16()
    out = torch.empty_like(q)
    ops.sdpa_prefill(q, k, v, torch.tensor([pos], dtype=torch.int32, device=device), out,
                     D ** -0.5, 1, T, Hq, Hkv, D)
    G = Hq // Hkv
    heads = sorted({0, G // 2, G - 1, Hq - G, Hq - 1})
    ref = _causal_ref(q, k[0], v[0], pos, T, heads, Hq, Hkv, D)
    got = out.view(T, Hq, D)[:, heads].permute(1, 0, 2)
    assert_close(n_f32(got), n_f32(ref), what=f"prefill sdpa T={T} pos={pos} {Hq}/{Hkv}")


@pytest.mark.parametrize("D,Hq,Hkv,T,pos,S_max", [
    (128, 32, 4, 1000, 37, 1280),   # ragged chunk behind cached tokens, odd tile count per workgroup
    (128, 16, 8, 300, 0, 512),      # 2 heads per kv head: a workgroup's waves are different token tiles
    (128, 4, 4, 257, 5, 384),       # 1 head per kv head, the shortest chunk that takes this layout
    (64, 8, 2, 260, 0, 320),        # head_dim 64
    (128, 64, 4, 512, 1536, 2048),  # 16 heads per kv head, a later chunk
])
def test_prefill_attention_two_team_layout(device, D, Hq, Hkv, T, pos, S_max):
    """Launches of at most 256 workgroups and 256 or more tokens run eight waves per workgroup,
    two teams on the two halves of the key tiles, merged through LDS: every query head against
    float32 library attention."""
    g = torch.Generator(device=device).manual_seed(T + pos + D)
    q = torch.randn(T, Hq * D, device=device, generator=g).bfloat16()
    k = torch.randn(1, Hkv, S_max, D, device=device, generator=g).bfloat16()
    v = torch.randn(1, Hkv, S_max, D, device=device, generator=g).bfloat16()
    out = torch.empty_like(q)
    ops.sdpa_prefill(q, k, v, torch.tensor([pos], dtype=torch.int32, device=device), out,
                     D ** -0.5, 1, T, Hq, Hkv, D)
    heads = list(range(Hq))
    ref = _causal_ref(q, k[0], v[0], pos, T, heads, Hq, Hkv, D)
    got = out.view(T, Hq, D).permute(1, 0, 2)
    assert_close(n_f32(got), n_f32(ref), what=f"two-team prefill sdpa T={T} pos={pos} {Hq}/{Hkv} D={D}")


def _fused_decode_case(device, B, Hq, Hkv, lens, S_max, seed, keys_hint=0):
    """exo_attn_decode (rope + append + attention) for B sequences at the given lengths,
    against: rope by the oracle, float32 library attention over the cache."""
    from oracle import ops as O
    D = 128
    g = torch.Generator(device=device).manual_seed(seed)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, device=device, generator=g).bfloat16()
    kc = torch.randn(B, Hkv, S_max, D, device=device, generator=g).bfloat16()
    vc = torch.randn(B, Hkv, S_max, D, device=device, generator=g).bfloat16()
    k0, v0 = kc.clone(), vc.clone()
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=device)
    inv = O.rope_inv_freq(D, 5e5, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192})
    inv_t = torch.from_numpy(inv).to(device)
    out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=device)
    ws = ops.sdpa_decode_workspace(B, Hq, D, device)
    tab = ops.rope_table(inv_t, S_max, D)
    for _ in range(2):  # twice: the arrival counters must be back at zero
        ops.attn_decode(qkv, kc, vc, pos, inv_t, out, ws, D ** -0.5, B, Hq, Hkv, D, rope_tab=tab,
                        keys_hint=keys_hint)
    x = n_f32(qkv).reshape(B, 1, Hq + 2 * Hkv, D)
    for b in range(B):
        p = lens[b] - 1
        qr = O.rope(x[b:b + 1, :, :Hq].transpose(0, 2, 1, 3), inv, p)               # [1,Hq,1,D]
        kr = O.rope(x[b:b + 1, :, Hq:Hq + Hkv].transpose(0, 2, 1, 3), inv, p)       # [1,Hkv,1,D]
        vn = x[b, 0, Hq + Hkv:]                                                     # [Hkv,D]
        kk = torch.cat([k0[b, :, :p].float(), t_bf16(kr[0], device).float()], dim=1)  # [Hkv,p+1,D]
        vv = torch.cat([v0[b, :, :p].float(), t_bf16(vn, device).float()[:, None]], dim=1)
        ref = torch.nn.functional.scaled_dot_product_attention(
            t_bf16(qr[0], device).float()[None], kk[None], vv[None], enable_gqa=True)[0, :, 0]
        assert_close(n_f32(out[b].view(Hq, D)), n_f32(ref), what=f"attn_decode B={B} len {lens[b]}")
        assert torch.equal(kc[b, :, :p], k0[b, :, :p]) and torch.equal(kc[b, :, p + 1:], k0[b, :, p + 1:])
        assert_close(n_f32(kc[b, :, p]), kr[0, :, 0], rtol=1e-2, what="appended k")


@pytest.mark.parametrize("B,Hq,Hkv,lens,S_max", [
    (8, 32, 8, [2304, 2050, 2049, 2048, 1999, 1025, 130, 1], 2304),   # Llama-8B batch 8: matrix-core kernel
    (4, 32, 4, [1280, 1026, 1025, 513], 1280),                        # Qwen3-30B batch 4: matrix-core kernel
    (1, 32, 8, [2050], 8192),                                         # batch 1 in the engine's default cache
    (1, 32, 8, [8191], 8192),
    (4, 32, 8, [8191, 2050, 4097, 3], 8192),
    (8, 32, 8, [8192, 8191, 2050, 2049, 4097, 4096, 65, 64], 8192),
    (2, 64, 4, [4224, 4097], 4224),                                   # Qwen3-235B shard heads
    (2, 32, 4, [40960, 32769], 40960),                                # Qwen3's longest context
    (1, 32, 8, [131072], 131072),                                     # Llama-3.1's longest context
    (4, 32, 8, [131072, 65537, 2050, 1], 131072),                     # 2 GiB of keys: byte offsets past 2^31
])
def test_fused_decode_attention_at_config_lengths(device, B, Hq, Hkv, lens, S_max):
    _fused_decode_case(device, B, Hq, Hkv, lens, S_max, seed=B * 1000 + lens[0])


@pytest.mark.parametrize("hint", [ops.ATTN_LONG_KEYS, ops.ATTN_VERY_LONG_KEYS])
@pytest.mark.parametrize("B,Hq,Hkv,lens,S_max", [
    (1, 32, 8, [6144], 8192),                          # the first step of the long layout
    (1, 32, 8, [1], 16384),                            # a hint may be wrong: one key
    (2, 32, 4, [12288, 130], 16384),                   # splits of 128 keys, most empty for row 1
    (1, 64, 4, [16383], 16384),                        # 16 query heads per kv head
    (2, 32, 4, [40960, 32769], 40960),
    (1, 32, 8, [131072], 131072),
    (4, 32, 8, [131072, 65537, 2050, 1], 131072),      # the layout the head count takes anyway
    (1, 16, 8, [9000], 16384),                         # 2 heads per kv head: stays on the scalar kernel
])
def test_fused_decode_attention_long_context_layout(device, B, Hq, Hkv, lens, S_max, hint):
    """exo_attn_decode_hint with the hint at the two long-context thresholds: the matrix-core
    kernel for any head count, up to 16 or 32 key splits merged by the last workgroup; run
    twice on one workspace (the arrival counters return to zero)."""
    _fused_decode_case(device, B, Hq, Hkv, lens, S_max, seed=B * 1000 + lens[0] + 7, keys_hint=hint)


@pytest.mark.parametrize("B,Hq,Hkv,lens,S_max", [
    (2, 32, 8, [3072, 2000], 4096),                    # the first step of the layout
    (2, 32, 8, [6000, 1], 8192),
    (3, 32, 8, [4500, 3071, 8192], 8192),
    (1, 32, 8, [4000], 8192),                          # one sequence: stays on the scalar kernel
])
def test_fused_decode_attention_mid_context_layout(device, B, Hq, Hkv, lens, S_max):
    """exo_attn_decode_hint with the hint at the middle threshold: the matrix-core kernel
    already from 3072 keys when the step has 16 or more (sequence, kv head) pairs."""
    _fused_decode_case(device, B, Hq, Hkv, lens, S_max, seed=B * 1000 + lens[0] + 9,
                       keys_hint=ops.ATTN_MID_KEYS)


def test_attention_layouts_share_a_workspace(device):
    """One workspace, zeroed once, taken in turn by the three layouts (their counters sit at
    the same place, the partials of one never reach the counters)."""
    from oracle import ops as O
    B, Hq, Hkv, D, S_max, n = 1, 32, 8, 128, 16384, 13000
    g = torch.Generator(device=device).manual_seed(11)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, device=device, generator=g).bfloat16()
    kc = torch.randn(B, Hkv, S_max, D, device=device, generator=g).bfloat16()
    vc = torch.randn(B, Hkv, S_max, D, device=device, generator=g).bfloat16()
    pos = torch.tensor([n - 1], dtype=torch.int32, device=device)
    inv_t = torch.from_numpy(O.rope_inv_freq(D, 1e6, None)).to(device)
    ws = ops.sdpa_decode_workspace(B, Hq, D, device)
    outs = []
    hints = (0, ops.ATTN_LONG_KEYS, ops.ATTN_VERY_LONG_KEYS)
    for hint in hints + hints:
        out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=device)
        ops.attn_decode(qkv, kc, vc, pos, inv_t, out, ws, D ** -0.5, B, Hq, Hkv, D, keys_hint=hint)
        outs.append(out)
    assert all(torch.equal(outs[i], outs[i + 3]) for i in range(3))
    assert_close(n_f32(outs[1]), n_f32(outs[0]), what="long against short layout")
    assert_close(n_f32(outs[2]), n_f32(outs[0]), what="very long against short layout")


# ------------------------------------------------------------------ batched decode blocks


@pytest.mark.parametrize("name,B,T0", [("llama-3.1-8b", 8, 24), ("qwen3-30b-a3b", 4, 6)])
def test_block_batched_decode_at_real_shape(device, name, B, T0):
    """One block at the real shapes with B sequences decoded together (8 rows: matrix-core
    GEMV and matrix-core decode attention; MoE at 4 rows: gather kernels over 32 (token,
    slot) pairs): a chunk per sequence, then three single-token steps, against the oracle."""
    cfg, gm, om = _one_layer(name, device)
    oc, gc = OM.make_kv_cache(1), gm.make_cache(B, 64)
    h = rand_bf16((B, T0, cfg.hidden_size), seed=B + T0)
    om.router_margins.clear()
    want = om(None, oc, input_hidden=h)
    got = n_f32(gm(None, gc, input_embeddings=t_bf16(h, device)))
    tied = False
    if cfg.is_moe:
        tied = check_tokens(got, want, om, f"{name} B={B} chunk")
    else:
        assert_close(got, want, what=f"{name} B={B} chunk", tail_frac=1e-5)  # 786432 elements
    for step in range(3):
        if tied:
            break
        h1 = rand_bf16((B, 1, cfg.hidden_size), seed=300 + step)
        om.router_margins.clear()
        want = om(None, oc, input_hidden=h1)
        got = n_f32(gm(None, gc, input_embeddings=t_bf16(h1, device)))
        if cfg.is_moe:
            tied = check_tokens(got, want, om, f"{name} B={B} step {step}")
        else:
            assert_close(got, want, what=f"{name} B={B} step {step}")
    assert gc[0].offset == oc[0].offset


# ------------------------------------------------------------------ configs[0], whole


def _config0(device):
    from exo_amd.synth import synth_weights as sw
    cfg = named_config("llama-3.2-1b")
    w = sw(cfg, seed=0, device=device)
    om = OM.ShardModel(OM.Config.from_json(cfg.to_dict()), weights_to_numpy(w), use_c=True)  # exact mode
    prompt = torch.randint(0, cfg.vocab_size, (128,), generator=torch.Generator().manual_seed(1234)).tolist()
    return cfg, w, om, prompt


@pytest.mark.timeout(900)
def test_llama_1b_every_layer_at_depth(device):
    """Every one of the 16 layers of the first benchmark configuration at its real shape and
    on the activations it really sees at its depth: the oracle (exact mode: un-rounded float32
    weights for every row count) walks the model layer by layer, each GPU layer is fed the
    ORACLE's input of that layer - the 126-token prompt chunk (matrix-core GEMM + flash
    attention), then three single-token steps (GEMV + decode attention on the cache the chunk
    left).  Errors cannot compound across layers here.  The single-token steps (un-rounded
    weights on both sides) are held to the single-layer elementwise bound at every depth.
    The chunk goes through the matrix-core GEMM, whose operands are the weights rounded to
    bf16; against the exact oracle that alone moves a layer's output by about 1e-2 relative
    RMS with 0.4 % of the elements past the elementwise bound (the oracle differs from ITSELF
    by that much when told to round its weights: 9.6e-3 and 0.38 % on layer 0), so the chunk
    is held to relative RMS <= 2e-2 and <= 1 % outliers; the mirrored oracle (weights rounded
    where the GEMM rounds them) holds the chunk to the elementwise bound in
    test_llama_block_at_real_shape.  Then the final norm + tied 128256-row head."""
    from oracle import ops as O
    cfg, w, om, prompt = _config0(device)
    L = cfg.num_hidden_layers
    toks = np.array(prompt[:126])[None]
    steps = [prompt[126], prompt[127], 4242]
    ocache = OM.make_kv_cache(L)
    emb = lambda t: affine.embed(np.asarray(t).reshape(-1), om.weights["model.embed_tokens.weight"],  # noqa: E731
                                 om.weights["model.embed_tokens.scales"], om.weights["model.embed_tokens.biases"],
                                 64, 4, "M1").reshape(1, -1, cfg.hidden_size)
    # oracle pass: inputs[i][c] = hidden state entering layer i for call c (chunk, 3 steps)
    inputs = [[] for _ in range(L + 1)]
    for call in [toks] + [np.array([[t]]) for t in steps]:
        h = emb(call)
        for i in range(L):
            inputs[i].append(h)
            h = om.layer(h, i, ocache[i])
        inputs[L].append(h)
    worst, worst_chunk = 0.0, 0.0
    for i in range(L):
        gl = ShardModel(cfg, w, i, i + 1, device)

        def run(gc, c, lo=0, hi=None):
            if i == 0:
                ids = toks[:, lo:hi] if c == 0 else np.array([[steps[c - 1]]])
                return n_f32(gl(torch.from_numpy(ids.astype(np.int32)), gc))
            x = inputs[i][c][:, lo:hi]
            return n_f32(gl(None, gc, input_embeddings=t_bf16(x, device), logits="none"))

        # the chunk in one call: matrix-core GEMM (bf16-rounded weights) + flash attention
        rel, _ = assert_close_stat(run(gl.make_cache(1, 160), 0), inputs[i + 1][0], max_outlier_frac=1e-2,
                                   what=f"config0 layer {i}, 126-token chunk through the GEMM")
        worst_chunk = max(worst_chunk, rel)
        # the same chunk in slices of 16 rows (matrix-core GEMV, un-rounded weights, short
        # causal attention chunks), then the single-token steps on that cache: elementwise
        gc = gl.make_cache(1, 160)
        got = np.concatenate([run(gc, 0, lo, min(lo + 16, 126)) for lo in range(0, 126, 16)], axis=1)
        e, atol = assert_close(got, inputs[i + 1][0], tail_frac=2e-4,
                               what=f"config0 layer {i}, chunk in slices of 16 rows")
        worst = max(worst, e / atol)
        for c in range(1, 4):
            e, atol = assert_close(run(gc, c), inputs[i + 1][c], what=f"config0 layer {i} step {c}")
            worst = max(worst, e / atol)
        del gl, gc
    print(f"[config0] 16 layers: GEMV-path calls worst |err| = {worst:.2f} x atol; 126-token GEMM chunk worst "
          f"relative RMS {worst_chunk:.2e}", flush=True)
    head = ShardModel(cfg, w, L - 1, L, device)
    hc = head.make_cache(1, 160)
    for c in range(1, 4):
        if c == 1:
            head(None, hc, input_embeddings=t_bf16(inputs[L - 1][0], device), logits="none")
        got = head(None, hc, input_embeddings=t_bf16(inputs[L - 1][c], device))
        hn = O.rms_norm(inputs[L][c], om._norm_w("model.norm.weight"), cfg.rms_norm_eps)
        want = om.linear(hn, "model.embed_tokens")
        assert_close_stat(n_f32(got), want, what=f"config0 last layer + norm + head, call {c}")


@pytest.mark.timeout(900)
def test_llama_1b_whole_model_greedy_64_tokens(device):
    """The first benchmark configuration end to end: the 16-layer Llama-3.2-1B architecture
    (tied 128256-row head, llama3 rope factor 32), seeded 128-token prompt, 64 greedy tokens
    through generate(), against the oracle in its EXACT mode.

    1. free running: tokens identical up to the first step where they differ; that step must
       be a near-tie of the oracle's own top two logits: their margin within the sum of the
       two logits' tolerances, each rtol * |logit| + rtol * rms(logits) with rtol = 2e-2 (the
       top logits of this random-weight model sit near 4, where one bf16 step is 0.031; the
       margin of every step is printed);
    2. teacher forced on the oracle's tokens for all 64 steps: the argmax agrees wherever the
       oracle's margin is not a near-tie, and the logits agree to a relative RMS of 4e-2.
       That is twice the single-op tolerance: through 16 layers of bf16-rounded ops two
       correct evaluation orders drift apart by that much on their own (the same prompt
       prefilled through this engine's GEMV path in chunks of 16 and of 1 token - identical
       un-rounded weights, different summation order - gives logits 2.2e-2 apart); the
       per-layer test above holds every layer to the tight bound."""
    from exo_amd.generate import generate, prefill
    from exo_amd.types import TextGenerationTaskParams
    cfg, w, om, prompt = _config0(device)
    gm = ShardModel(cfg, w, device=device)
    del w
    N, n_new = 128, 64
    print(f"[config0] oracle: prefill {N - 1} + {n_new} greedy steps", flush=True)
    want, wl = OM.greedy_generate(om, prompt, n_new)
    rms = np.sqrt(np.mean(wl.astype(np.float64) ** 2, axis=1))
    top2 = np.sort(wl, axis=1)[:, -2:]
    margin = top2[:, 1] - top2[:, 0]
    tol = 2e-2 * (np.abs(top2[:, 0]) + np.abs(top2[:, 1])) + 2 * 2e-2 * rms
    near_tie = margin <= tol
    task = TextGenerationTaskParams(model="llama-3.2-1b", max_output_tokens=n_new, temperature=0.0)
    got = [r.token for r in generate(gm, None, task, prompt)]
    assert len(got) == n_new
    first_bad = next((i for i in range(n_new) if got[i] != want[i]), None)
    for i in range(n_new):
        print(f"[config0] step {i:2d}: oracle {want[i]:6d} gpu {got[i]:6d} margin {margin[i]:.4f} "
              f"(tolerance {tol[i]:.4f}){' near-tie' if near_tie[i] else ''}"
              f"{'  <- first difference' if i == first_bad else ''}", flush=True)
    if first_bad is not None:
        assert near_tie[first_bad], (f"free-running tokens differ at step {first_bad} where the oracle's "
                                     f"margin {margin[first_bad]:.4f} is clear")
    print(f"[config0] free running: identical for {n_new if first_bad is None else first_bad} steps; "
          f"{int(near_tie[:32].sum())} near-ties among the first 32 oracle steps", flush=True)
    # teacher forced: the GPU follows the oracle's token sequence
    cache = gm.make_cache(1, N + n_new + 8)
    prefill(gm, prompt[:-1], cache)
    gm(torch.tensor([[prompt[-2]]], dtype=torch.int32), cache, logits="none")
    fed = [prompt[-1]] + want[:-1]
    agree, clear = 0, 0
    for i in range(n_new):
        bufs = gm._buffers(1, 1)
        bufs.tokens[0] = fed[i]
        bufs = gm.decode_step(cache, 1)
        lg = n_f32(bufs.logits[0])
        assert_close_stat(lg, wl[i], max_rel_rms=4e-2, max_outlier_frac=0.5,
                          what=f"config0 teacher-forced logits step {i}")
        tok = int(bufs.next_token[0])
        if i == first_bad:
            a, b = want[i], got[i]
            print(f"[config0] step {i}: oracle logits ({wl[i][a]:.4f}, {wl[i][b]:.4f}) for tokens ({a}, {b}); "
                  f"gpu logits ({lg[a]:.4f}, {lg[b]:.4f})", flush=True)
        if not near_tie[i]:
            clear += 1
            assert tok == want[i], f"step {i}: argmax {tok} vs oracle {want[i]} at margin {margin[i]:.4f}"
        agree += tok == want[i]
    print(f"[config0] teacher forced: argmax agrees on {agree}/{n_new} steps ({clear} with a clear margin)", flush=True)
    if first_bad is None or first_bad >= 32:
        return
    pytest.xfail(f"free-running tokens identical for {first_bad} < 32 steps: the oracle's own top-2 margin at "
                 f"step {first_bad} is {margin[first_bad]:.4f}, inside the tolerance {tol[first_bad]:.4f}; every "
                 f"teacher-forced step passed")
