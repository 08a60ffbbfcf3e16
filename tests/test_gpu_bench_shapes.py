"""Parity at the launch shapes the benchmark times (bench.py, configs[2] to configs[4]).

The kernel tests cover every instance on small shapes and the full-size tests cover single
launches; here the shapes, row counts and contexts are the ones of the timed workloads:
the whole 32-layer Llama-3.1-8B decode step at the benchmark's context, the gate/up pair
GEMM under a 2046-row prompt chunk, the grouped expert GEMMs at the real expert shapes and
prompt sizes, and several-layer MoE stacks.  Every shape-targeted test also asserts (through
exo_last_variant) that the launch reached the kernel instance it was written for.
"""

import dataclasses

import numpy as np
import pytest
import torch

from oracle import affine
from oracle import models as OM
from oracle import ops as O
from tests.util import (assert_close, assert_close_stat, check_tokens, n_bits, n_f32, rand_bf16,
                        t_bf16, weights_to_numpy)

pytestmark = pytest.mark.gpu

from exo_amd import native, ops  # noqa: E402
from exo_amd.config import named_config  # noqa: E402
from exo_amd.model import ShardModel  # noqa: E402
from exo_amd.ops import QuantizedWeight  # noqa: E402
from exo_amd.synth import synth_weights  # noqa: E402


def _packed(N, K, bits, seed, device, E=None):
    """Already-packed random matrix (every code value occurs), scales and biases of the
    magnitude N(0, 0.02) weights quantise to."""
    g = torch.Generator(device=device).manual_seed(seed)
    lead = () if E is None else (E,)
    w = torch.randint(-2**31, 2**31 - 1, lead + (N, K * bits // 32), dtype=torch.int32, device=device, generator=g)
    levels = float(2**bits - 1)
    s = (torch.rand(lead + (N, K // 64), device=device, generator=g) * 0.1 + 0.05) / levels
    b = -s * levels * (0.4 + 0.2 * torch.rand(lead + (N, K // 64), device=device, generator=g))
    return QuantizedWeight(w, s.bfloat16(), b.bfloat16(), bits)


def _np_rows(qw, rows, e=None):
    r = torch.as_tensor(rows, device=qw.weight.device)
    w, s, b = (qw.weight, qw.scales, qw.biases) if e is None else (qw.weight[e], qw.scales[e], qw.biases[e])
    return (w[r].cpu().numpy().view(np.uint32), n_bits(s[r]), n_bits(b[r]))


# ------------------------------------------------------------------ the headline step


@pytest.mark.timeout(900)
def test_llama_8b_decode_step_at_bench_context(device):
    """configs[2] as bench.py times it: all 32 layers + head of the Llama-3.1-8B architecture,
    4-bit g64, one sequence, a context of 2052 cached tokens (seeded synthetic K/V written
    into both caches, as the benchmark's CPU baseline does), three graph-replayed decode
    steps.  Logits against the C oracle in its exact mode: relative RMS <= 4e-2 (32 layers of
    bf16-rounded operations; two valid summation orders drift apart by 2e-2 over 16 layers),
    arg max equal wherever the oracle's own top-two margin is not a near-tie."""
    cfg = named_config("llama-3.1-8b")
    ctx, steps = 2052, 3
    w = synth_weights(cfg, seed=0, device=device)
    gm = ShardModel(cfg, w, device=device)
    om = OM.ShardModel(OM.Config.from_json(cfg.to_dict()), weights_to_numpy(w), use_c=True)
    del w
    L, Hkv, D = cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.head_dim
    gc = gm.make_cache(1, ctx + steps + 60)
    oc = OM.make_kv_cache(L)
    rng = np.random.default_rng(2052)
    for li in range(L):
        k = affine.bf16_round(rng.standard_normal((1, Hkv, ctx, D)).astype(np.float32))
        v = affine.bf16_round(rng.standard_normal((1, Hkv, ctx, D)).astype(np.float32))
        oc[li].k, oc[li].v, oc[li].offset = k, v, ctx
        gc.k[li][:, :, :ctx].copy_(t_bf16(k, device))
        gc.v[li][:, :, :ctx].copy_(t_bf16(v, device))
    gc.offsets[0] = ctx
    gc.sync_pos()
    tok = 1
    for step in range(steps):
        want = om(np.array([[tok]]), oc)[0, -1]
        bufs = gm._buffers(1, 1)
        bufs.tokens[0] = tok
        bufs = gm.decode_step(gc, 1)
        got = n_f32(bufs.logits[0])
        assert_close_stat(got, want, max_rel_rms=4e-2, max_outlier_frac=0.5,
                          what=f"llama-3.1-8b step {step} at context {ctx + step}")
        top2 = np.sort(want)[-2:]
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        margin = float(top2[1] - top2[0])
        tol = 2e-2 * float(abs(top2[0]) + abs(top2[1])) + 2 * 2e-2 * rms
        g_tok, o_tok = int(bufs.next_token[0]), int(np.argmax(want))
        print(f"[bench-shape] step {step}: oracle {o_tok} gpu {g_tok} margin {margin:.4f} tolerance {tol:.4f}",
              flush=True)
        if margin > tol:
            assert g_tok == o_tok, f"step {step}: arg max {g_tok} vs oracle {o_tok} at a clear margin {margin:.4f}"
        tok = o_tok  # both sides follow the oracle's token
    assert gc[0].offset == ctx + steps and oc[0].offset == ctx + steps


# ------------------------------------------------------------------ the prompt's dominant launches


@pytest.mark.parametrize("M,N,K,bits,variant", [
    (2046, 14336, 4096, 4, "qmm_kernel<4, 4, false, true, true, true>"),   # Llama-3.1-8B prompt chunk
    (2046, 12288, 4096, 8, "qmm_kernel<8, 4, false, true, true, true>"),   # an 8-bit MLP of that size
])
def test_gate_up_pair_gemm_at_prompt_size(device, M, N, K, bits, variant):
    """The (gate, up) pair GEMM with the SwiGLU epilogue under a 2046-row chunk - 44 % of the 8B
    prompt's time - on the wide tile with the ring: bit-equal to the two single GEMMs followed
    by the SwiGLU kernel; a sample of outputs against the oracle (weights rounded to bf16, as
    the matrix-core operand is), all outputs of both projections against dequantize + float32
    matmul."""
    g, u = _packed(N, K, bits, 11, device), _packed(N, K, bits, 12, device)
    x = rand_bf16((M, K), seed=M + N)
    xt = t_bf16(x, device)
    fused = ops.qmm_swiglu(xt, g, u)
    assert native.last_variant() == variant, native.last_variant()
    sep = ops.swiglu(ops.qmm(xt, g), ops.qmm(xt, u))
    assert torch.equal(fused.view(torch.int16), sep.view(torch.int16))
    rows = np.unique(np.random.default_rng(N).integers(0, N, 96))
    toks = np.unique(np.concatenate([[0, 127, 128, M - 1], np.random.default_rng(M).integers(0, M, 28)]))
    gw = affine.bf16_round(affine.dequantize_f32(*_np_rows(g, rows), 64, bits))
    uw = affine.bf16_round(affine.dequantize_f32(*_np_rows(u, rows), 64, bits))
    want = O.swiglu(affine.bf16_round(x[toks] @ gw.T), affine.bf16_round(x[toks] @ uw.T))
    got = n_f32(fused[torch.as_tensor(toks, device=device)][:, torch.as_tensor(rows, device=device)])
    assert_close(got, want, what=f"pair GEMM {M}x{N}x{K} b{bits}, oracle sample")
    # every output: the two projections the fused launch equals bit for bit, each against
    # dequantize + float32 matmul (a product of two rounded factors has no elementwise bound
    # of its own near a zero of either)
    for q, name in ((g, "gate"), (u, "up")):
        full = xt.float() @ ops.dequantize(q).float().T
        assert_close(n_f32(ops.qmm(xt, q)), n_f32(full), what=f"{name} GEMM {M}x{N}x{K} b{bits}, all outputs",
                     tail_frac=1e-5)


def test_head_matmul_under_a_full_prompt(device):
    """configs[1]'s largest cell, 128256 x 4096 at M = 2048 (4-bit): a row sample against the
    oracle, every output against dequantize + float32 matmul."""
    N, K, M, bits = 128256, 4096, 2048, 4
    qw = _packed(N, K, bits, 5, device)
    x = rand_bf16((M, K), seed=M)
    xt = t_bf16(x, device)
    y = ops.quantized_matmul(xt, qw)
    print(f"[bench-shape] 128256x4096 under 2048 rows: {native.last_variant()}", flush=True)
    rows = np.unique(np.concatenate([[0, 1, N - 2, N - 1], np.random.default_rng(N).integers(0, N, 60)]))
    toks = np.array([0, 1, 255, 256, 1023, 2047])
    wq = affine.bf16_round(affine.dequantize_f32(*_np_rows(qw, rows), 64, bits))
    want = affine.bf16_round(x[toks] @ wq.T)
    got = n_f32(y[torch.as_tensor(toks, device=device)][:, torch.as_tensor(rows, device=device)])
    assert_close(got, want, what="head GEMM, oracle sample")
    wd = ops.dequantize(qw).float()
    for lo in range(0, M, 512):  # in slices: the float32 reference of all outputs is 1 GB
        full = xt[lo:lo + 512].float() @ wd.T
        assert_close(n_f32(y[lo:lo + 512]), n_f32(full), what=f"head GEMM rows {lo}..", tail_frac=1e-5)


# ------------------------------------------------------------------ grouped expert GEMMs


@pytest.mark.parametrize("T,N,K,bits,pair,variant", [
    (1023, 768, 2048, 4, True, "qmm_kernel<4, 4, true, true, true, true>"),     # Qwen3-30B gate/up + SwiGLU
    (1023, 2048, 768, 4, False, "qmm_kernel<4, 4, true, true, false, true>"),   # Qwen3-30B down
    (300, 1536, 4096, 8, True, "qmm_kernel<8, 4, true, true, true, true>"),     # Qwen3-235B gate/up + SwiGLU
    (300, 4096, 1536, 8, False, "qmm_kernel<8, 4, true, true, false, true>"),   # Qwen3-235B down
])
def test_grouped_expert_gemm_at_real_shapes(device, T, N, K, bits, pair, variant):
    """128 experts, top-8, the token counts of the configurations' prompt chunks: every
    (token, slot) pair against dequantize + float32 matmul per expert, a seeded sample of
    pairs against the oracle (weights rounded to bf16, as the matrix-core operand is)."""
    E, topk = 128, 8
    g = _packed(N, K, bits, 21, device, E=E)
    u = _packed(N, K, bits, 22, device, E=E) if pair else None
    gen = torch.Generator(device=device).manual_seed(T + N)
    # distinct experts per token, skewed: expert 3 takes every token (several row tiles), the
    # low-numbered experts most of the rest, some experts few or none
    pri = torch.rand(T, E, device=device, generator=gen) + torch.linspace(0.6, 0.0, E, device=device)[None]
    pri[:, 3] += 2.0
    idx = pri.topk(topk, dim=1).indices.to(torch.int32).contiguous()
    ws = ops.moe_group(idx, E)
    if pair:
        x = rand_bf16((T, 1, K), seed=T)
        xt = t_bf16(x, device)
        y = ops.grouped_qmm_swiglu(xt, g, u, ws, topk)
    else:
        x = rand_bf16((T, topk, K), seed=T)
        xt = t_bf16(x, device)
        y = ops.grouped_qmm(xt, g, ws, topk)
    assert native.last_variant() == variant, native.last_variant()
    assert y.shape == (T, topk, N)
    counts = torch.bincount(idx.flatten().long(), minlength=E)
    assert int(counts.max()) > 128  # an expert with more than one row tile
    # the fused (gate, up, SwiGLU) launch has the bits of the two grouped GEMMs followed by the
    # elementwise kernel; every output of the single projections is then compared below (a
    # product of two rounded factors has no elementwise bound of its own near a zero of either)
    singles = [(g, y)]
    if pair:
        yg, yu = ops.grouped_qmm(xt, g, ws, topk), ops.grouped_qmm(xt, u, ws, topk)
        assert torch.equal(y.view(torch.int16), ops.swiglu(yg, yu).view(torch.int16))
        singles = [(g, yg), (u, yu)]
    # all pairs: per expert, dequantize + float32 matmul
    for q, yq in singles:
        for e in range(E):
            sel = (idx == e).nonzero()
            if sel.numel() == 0:
                continue
            t_i, s_i = sel[:, 0], sel[:, 1]
            xe = xt[t_i, 0 if pair else s_i].float()
            wd = ops.dequantize(QuantizedWeight(q.weight[e], q.scales[e], q.biases[e], bits)).float()
            assert_close(n_f32(yq[t_i, s_i]), n_f32(xe @ wd.T),
                         what=f"grouped GEMM expert {e} ({sel.shape[0]} rows)", tail_frac=1e-4)
    # oracle on a sample of pairs
    rng = np.random.default_rng(T)
    rows = np.unique(rng.integers(0, N, 48))
    idx_h = idx.cpu().numpy()
    for t in np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 10)])):
        for s in (0, topk - 1):
            e = int(idx_h[t, s])
            xr = x[t, 0 if pair else s]
            gw = affine.bf16_round(affine.dequantize_f32(*_np_rows(g, rows, e), 64, bits))
            if pair:
                uw = affine.bf16_round(affine.dequantize_f32(*_np_rows(u, rows, e), 64, bits))
                want = O.swiglu(affine.bf16_round(gw @ xr), affine.bf16_round(uw @ xr))
            else:
                want = affine.bf16_round(gw @ xr)
            got = n_f32(y[int(t), s][torch.as_tensor(rows, device=device)])
            assert_close(got, want, what=f"grouped GEMM pair ({t},{s}) expert {e}, oracle")


# ------------------------------------------------------------------ MoE stacks


def _token_errors(got, want):
    got, want = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2, axis=1))
    return np.sqrt(np.mean((got.astype(np.float64) - want) ** 2, axis=1)) / rms


@pytest.mark.timeout(1500)
@pytest.mark.parametrize("name,layers,T", [("qwen3-30b-a3b", 4, 200), ("qwen3-235b-a22b", 3, 200)])
def test_moe_stack_at_real_shape(device, name, layers, T):
    """Several MoE layers at the real shapes, as a middle pipeline shard (hidden state in,
    hidden state out - what configs[4] compares): a 200-token chunk through the grouped
    matrix-core GEMMs and the flash attention, then three single-token steps through the
    gather GEMVs, against the oracle (mirrored: weights rounded to bf16 where the GEMM rounds
    them).  Expert choice is discontinuous: a token whose 8th and 9th router logits are within
    bf16 noise in the oracle may take another expert (one expert of eight moves the token's
    output by about a tenth), and through the cache every later token sees it.  Required: every
    token up to the first such near-tie within relative RMS 2e-2; overall at least 80 % of
    the tokens within 2e-2 and none beyond 0.2; the single-token steps the same."""
    cfg = dataclasses.replace(named_config(name), num_hidden_layers=layers + 2)
    w = synth_weights(cfg, 1, 1 + layers, seed=3, device=device)
    gm = ShardModel(cfg, w, 1, 1 + layers, device)
    om = OM.ShardModel(OM.Config.from_json(cfg.to_dict()), weights_to_numpy(w), 1, 1 + layers,
                       gemm_rows=16, use_c=True)
    del w
    oc, gc = OM.make_kv_cache(layers), gm.make_cache(1, T + 8)
    h = rand_bf16((1, T, cfg.hidden_size), seed=T + layers)
    om.router_margins.clear()
    want = om(None, oc, input_hidden=h)
    got = n_f32(gm(None, gc, input_embeddings=t_bf16(h, device)))
    check_tokens(got, want, om, f"{name} {layers} layers, {T}-token chunk")  # strict up to the first near-tie
    err = _token_errors(got, want)
    print(f"[bench-shape] {name} chunk: {int((err <= 2e-2).sum())}/{T} tokens within 2e-2, worst {err.max():.3e}",
          flush=True)
    assert (err <= 2e-2).mean() >= 0.8 and err.max() <= 0.2, (float((err <= 2e-2).mean()), float(err.max()))
    for step in range(3):  # the gather GEMVs and the decode attention on the cache the chunk left
        h1 = rand_bf16((1, 1, cfg.hidden_size), seed=400 + step)
        om.router_margins.clear()
        want = om(None, oc, input_hidden=h1)
        got = n_f32(gm(None, gc, input_embeddings=t_bf16(h1, device)))
        e = float(_token_errors(got, want)[0])
        print(f"[bench-shape] {name} step {step}: relative RMS {e:.3e}", flush=True)
        check_tokens(got, want, om, f"{name} step {step}")  # 2e-2 unless this token's own routing is a near-tie
        assert e <= 0.2, e
    assert gc[0].offset == oc[0].offset == T + 3


# ------------------------------------------------------------------ which instance runs


def test_decode_launches_reach_their_instances(device):
    """The launches of the headline decode step report the instance they are tuned as."""
    bits, H, I = 4, 4096, 14336
    x = t_bf16(rand_bf16((1, H), seed=1), device)
    nw = t_bf16(affine.bf16_round(rand_bf16((H,), seed=2) * 0.1 + 1.0), device)
    g, u = _packed(I, H, bits, 1, device), _packed(I, H, bits, 2, device)
    ops.qmv_swiglu(x, g, u, norm_weight=nw, eps=1e-5)
    assert native.last_variant() == "qmv_rows<4,1,2,2,false> grid=1792x1", native.last_variant()
    ops.quantized_matmul(x, _packed(6144, H, bits, 3, device), norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_rows<4,1,1,2,false>"), native.last_variant()
    xa = t_bf16(rand_bf16((1, H), seed=6), device)
    ops.quantized_matmul(xa, _packed(H, H, bits, 5, device), residual=x)
    assert native.last_variant().startswith("qmv_rows<4,1,1,2,false>"), native.last_variant()
    ops.quantized_matmul(x, _packed(128256, H, bits, 6, device), norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_rows<4,1,1,2,false>"), native.last_variant()
    xi = t_bf16(rand_bf16((1, I), seed=3), device)
    ops.quantized_matmul(xi, _packed(H, I, bits, 4, device))
    assert native.last_variant().startswith("qmv_rows<4,1,1,7,false>"), native.last_variant()
    x4 = t_bf16(rand_bf16((4, H), seed=4), device)
    ops.qmv_swiglu(x4, g, u, norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_quad<4,2,1,4,1>"), native.last_variant()
    x8 = t_bf16(rand_bf16((8, H), seed=5), device)
    ops.qmv_swiglu(x8, g, u, norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_w16<2,2,2,norm,pair8> grid=256 waves=16 blocks=7"), native.last_variant()
    x16 = t_bf16(rand_bf16((16, H), seed=7), device)
    ops.qmv_swiglu(x16, g, u, norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_w16<2,2,2,norm,pair8> grid=256 waves=16 blocks=7"), native.last_variant()
    # the down projection under 8 rows: K split over four workgroups per group of row blocks
    xi8 = t_bf16(rand_bf16((8, I), seed=8), device)
    ops.quantized_matmul(xi8, _packed(H, I, bits, 4, device), residual=x8)
    assert native.last_variant().startswith("qmv_w16<1,2,2,plain,staged> grid=256 waves=14 blocks=4 kparts=4"), \
        native.last_variant()
    ops.quantized_matmul(x8, _packed(6144, H, bits, 3, device), norm_weight=nw, eps=1e-5)
    assert native.last_variant().startswith("qmv_w16<1,2,2,norm,staged>"), native.last_variant()
    # decode attention: one sequence of 32 / 8 heads on the scalar kernel, eight on the matrix cores
    D, Hq, Hkv, S = 128, 32, 8, 2304
    inv = torch.from_numpy(O.rope_inv_freq(D, 5e5, None)).to(device)
    for B, want in ((1, "sdpa_tiles<128,1,true> grid=8x32x1"), (8, "sdpa_decode_mfma<4>")):
        qkv = torch.randn(B, (Hq + 2 * Hkv) * D, device=device).bfloat16()
        kc = torch.randn(B, Hkv, S, D, device=device).bfloat16()
        vc = torch.randn(B, Hkv, S, D, device=device).bfloat16()
        pos = torch.full((B,), 2049, dtype=torch.int32, device=device)
        out = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=device)
        ops.attn_decode(qkv, kc, vc, pos, inv, out, ops.sdpa_decode_workspace(B, Hq, D, device), D ** -0.5,
                        B, Hq, Hkv, D)
        assert native.last_variant().startswith(want), native.last_variant()
