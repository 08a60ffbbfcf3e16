"""Pins of the CPU oracle (no GPU).

The reference holds no golden vectors for this path (its arithmetic is in the
un-vendored mlx / mlx_lm wheels), so each oracle function is pinned by something that
is NOT a retyping of its own formula: hand-packed words from the operator docstring,
hand-evaluated values, exhaustive round trips, library routines (transformers,
torch.nn.functional), closed-form invariants and a second independent implementation
(the C restatement).  What stays open is marked "parity unpinned" in oracle/__init__.py.
"""

import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import affine, cref
from oracle import models as OM
from oracle import ops as O
from tests.util import rand_bf16, rand_quantized, rng, tiny_config

# ------------------------------------------------------------------ packing (K0)


def test_pack_docstring_example():
    # "for 4-bit ... the 1st element occupies the 4 least significant bits, the 2nd
    # bits 4-7 etc."  (.typings/mlx/core/__init__.pyi:4180-4184)
    codes4 = np.array([[0, 1, 2, 3, 4, 5, 6, 7, 15, 0, 0, 0, 0, 0, 0, 9]], np.uint8)
    np.testing.assert_array_equal(affine.pack_codes(codes4, 4), [[0x76543210, 0x9000000F]])
    codes8 = np.array([[0, 1, 2, 3, 255, 0, 128, 7]], np.uint8)
    np.testing.assert_array_equal(affine.pack_codes(codes8, 8), [[0x03020100, 0x078000FF]])
    np.testing.assert_array_equal(affine.unpack_codes(np.array([[0x76543210]], np.uint32), 4)[0],
                                  np.arange(8))
    np.testing.assert_array_equal(cref.unpack_codes(np.array([[0x03020100]], np.uint32), 8)[0],
                                  np.arange(4))


@pytest.mark.parametrize("bits", [4, 8])
def test_pack_unpack_every_code_every_slot(bits):
    per, n = 32 // bits, 1 << bits
    for slot in range(per):
        codes = np.zeros((n, per), np.uint8)
        codes[:, slot] = np.arange(n)
        w = affine.pack_codes(codes, bits)
        assert np.all(w[:, 0] == (np.arange(n, dtype=np.uint64) << (bits * slot)))
        np.testing.assert_array_equal(affine.unpack_codes(w, bits), codes)
        np.testing.assert_array_equal(cref.unpack_codes(w, bits), codes)


# ------------------------------------------------------------------ dequantize


def _bf16_of_fraction(fr: Fraction) -> float:
    """Exact round-to-nearest-even of a rational to bf16 (8 significant bits)."""
    if fr == 0:
        return 0.0
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = math.floor(math.log2(fr))
    if Fraction(2) ** e > fr:
        e -= 1
    if Fraction(2) ** (e + 1) <= fr:
        e += 1
    ulp = Fraction(2) ** (e - 7)
    q, r = divmod(fr, ulp)
    if r > ulp / 2 or (r == ulp / 2 and q % 2 == 1):
        q += 1
    return float(sign * q * ulp)


@pytest.mark.parametrize("bits", [4, 8])
def test_dequantize_hand_evaluated_both_roundings(bits):
    # exact rational arithmetic of w = s*q + b, rounded once (M2) or per operation (M1)
    r = rng(3)
    n = 1 << bits
    K = 64
    codes = r.integers(0, n, size=(40, K)).astype(np.uint8)
    w = affine.pack_codes(codes, bits)
    s = affine.f32_to_bf16_bits((r.standard_normal((40, 1)) * 0.01).astype(np.float32))
    b = affine.f32_to_bf16_bits((r.standard_normal((40, 1)) * 0.1).astype(np.float32))
    m1 = affine.bf16_bits_to_f32(affine.dequantize(w, s, b, 64, bits, "M1"))
    m2 = affine.bf16_bits_to_f32(affine.dequantize(w, s, b, 64, bits, "M2"))
    sf, bf = affine.bf16_bits_to_f32(s), affine.bf16_bits_to_f32(b)
    differ = 0
    for i in range(40):
        S, B = Fraction(float(sf[i, 0])), Fraction(float(bf[i, 0]))
        for k in range(0, K, 7):
            q = int(codes[i, k])
            want2 = _bf16_of_fraction(S * q + B)
            want1 = _bf16_of_fraction(Fraction(_bf16_of_fraction(S * q)) + B)
            assert m2[i, k] == want2 and m1[i, k] == want1
            differ += want1 != want2
    assert differ > 0  # the two modes are genuinely different functions
    # the C restatement agrees bit for bit
    np.testing.assert_array_equal(cref.dequantize(w, s, b, bits, True), affine.dequantize(w, s, b, 64, bits, "M1"))
    np.testing.assert_array_equal(cref.dequantize(w, s, b, bits, False), affine.dequantize(w, s, b, 64, bits, "M2"))


def test_dequantize_simple_values():
    w = affine.pack_codes(np.tile(np.arange(16, dtype=np.uint8), (1, 4)), 4)
    s = affine.f32_to_bf16_bits(np.array([[0.5]], np.float32))
    b = affine.f32_to_bf16_bits(np.array([[-1.0]], np.float32))
    got = affine.bf16_bits_to_f32(affine.dequantize(w, s, b, 64, 4))
    np.testing.assert_array_equal(got[0, :16], 0.5 * np.arange(16) - 1.0)


# ------------------------------------------------------------------ quantize


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("rule", ["doc", "mlx"])
def test_quantize_reconstruction_bound_and_grid_recovery(bits, rule):
    w = (rng(bits).standard_normal((16, 256)) * 0.02).astype(np.float32)
    q, s, b = affine.quantize(w, 64, bits, rule)
    assert q.dtype == np.uint32 and q.shape == (16, 256 * bits // 32) and s.shape == (16, 4)
    wd = affine.dequantize_f32(q, s, b, 64, bits)
    step = np.abs(np.repeat(affine.bf16_bits_to_f32(s), 64, axis=-1))
    # "doc": every element lies inside the represented range: half a step (+ bf16 slack
    # of s, b).  "mlx": the scale is re-derived so that one edge is exact, which can
    # leave the far edge outside the grid by up to one more half step.
    half_steps = 1.05 if rule == "doc" else 2.1
    assert np.all(np.abs(wd - w) <= 0.5 * step * half_steps + 2e-4)
    # a matrix that already lies on a quantisation grid is recovered exactly
    codes = rng(9).integers(0, 1 << bits, size=(4, 128)).astype(np.uint8)
    codes[:, 0], codes[:, 1] = 0, (1 << bits) - 1
    codes[:, 64], codes[:, 65] = 0, (1 << bits) - 1
    grid = (0.0078125 * codes - 0.0625).astype(np.float32)  # s, b exact in bf16
    q2, s2, b2 = affine.quantize(grid, 64, bits, rule)
    np.testing.assert_array_equal(affine.dequantize_f32(q2, s2, b2, 64, bits), grid)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("rule", ["doc", "mlx"])
def test_product_quantizer_equals_oracle(bits, rule):
    from exo_amd.quantize import quantize as tq

    w = (rng(100 + bits).standard_normal((32, 192)) * 0.02).astype(np.float32)
    q, s, b = affine.quantize(w, 64, bits, rule)
    tq_, ts, tb = tq(torch.from_numpy(w), 64, bits, rule)
    np.testing.assert_array_equal(tq_.numpy().view(np.uint32), q)
    np.testing.assert_array_equal(ts.view(torch.int16).numpy().view(np.uint16), s)
    np.testing.assert_array_equal(tb.view(torch.int16).numpy().view(np.uint16), b)


# ------------------------------------------------------------------ qmm / gather_qmm


@pytest.mark.parametrize("bits", [4, 8])
def test_qmm_equals_dense_matmul_and_c(bits):
    trip = rand_quantized(48, 256, bits, seed=5)
    x = rand_bf16((5, 256), seed=6)
    wd = affine.bf16_bits_to_f32(affine.dequantize(*trip, 64, bits, "M2")).astype(np.float64)
    # library routine on the (bf16-rounded) dequantised matrix: differs from the fused
    # result only by the weight rounding, far below the output's bf16 ulp on average
    dense = x.astype(np.float64) @ affine.dequantize_f32(*trip, 64, bits).astype(np.float64).T
    got = affine.qmm(x, *trip, 64, bits, out_bf16=False)
    np.testing.assert_allclose(got, dense, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(x.astype(np.float64) @ wd.T, dense, rtol=0, atol=2e-2 * np.abs(dense).max())
    c = affine.bf16_bits_to_f32(cref.qmm_t(affine.f32_to_bf16_bits(x), *trip, bits))
    exact_bf16 = affine.bf16_round(dense.astype(np.float32))
    # C accumulates in another order: equal up to one bf16 ulp
    assert np.all(np.abs(c - exact_bf16) <= np.abs(exact_bf16) * 2.0**-7 + 1e-6)
    # linearity in x (a dropped bias term or a wrong group index would break it)
    x2 = rand_bf16((5, 256), seed=7)
    a = affine.qmm(x + x2, *trip, 64, bits, out_bf16=False)
    bsum = got + affine.qmm(x2, *trip, 64, bits, out_bf16=False)
    np.testing.assert_allclose(a, bsum, rtol=1e-4, atol=1e-5)


def test_qmm_constant_matrix_closed_form():
    # all codes = c, one scale/bias -> y = (s*c + b) * sum(x)
    codes = np.full((3, 128), 5, np.uint8)
    w = affine.pack_codes(codes, 4)
    s = affine.f32_to_bf16_bits(np.full((3, 2), 0.25, np.float32))
    b = affine.f32_to_bf16_bits(np.array([[1.0, -1.0]] * 3, np.float32))
    x = rand_bf16((2, 128), seed=1)
    want = (0.25 * 5 + 1.0) * x[:, :64].sum(-1) + (0.25 * 5 - 1.0) * x[:, 64:].sum(-1)
    got = affine.qmm(x, w, s, b, 64, 4, out_bf16=False)
    np.testing.assert_allclose(got, np.repeat(want[:, None], 3, 1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("bits", [4, 8])
def test_gather_qmm_brute_force(bits):
    E, N, K, T, topk = 4, 16, 128, 3, 2
    trip = rand_quantized(N, K, bits, seed=8, E=E)
    idx = rng(2).integers(0, E, size=(T, topk))
    x = rand_bf16((T, 1, K), seed=3)
    got = affine.gather_qmm(x, *trip, idx, 64, bits, out_bf16=False)
    for t in range(T):
        for j in range(topk):
            e = idx[t, j]
            want = affine.qmm(x[t], trip[0][e], trip[1][e], trip[2][e], 64, bits, out_bf16=False)[0]
            np.testing.assert_allclose(got[t, j], want, rtol=1e-6)


# ------------------------------------------------------------------ small ops vs libraries


def test_rms_norm_vs_transformers():
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    x = rand_bf16((4, 256), seed=1)
    w = rand_bf16((256,), seed=2) + 1
    m = LlamaRMSNorm(256, eps=1e-5)
    m.weight.data = torch.from_numpy(w)
    want = m(torch.from_numpy(x)).detach().numpy()
    with affine.exact_activations():
        got = O.rms_norm(x, w, 1e-5)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("factor,D", [(32.0, 64), (8.0, 128)])
def test_rope_llama3_frequencies_vs_transformers(factor, D):
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    rp = {"rope_type": "llama3", "rope_theta": 5e5, "factor": factor, "low_freq_factor": 1.0,
          "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
    cfg = LlamaConfig(hidden_size=D * 4, num_attention_heads=4, head_dim=D, rope_parameters=rp,
                      max_position_embeddings=131072)
    inv, _ = ROPE_INIT_FUNCTIONS["llama3"](cfg, "cpu")
    got = O.rope_inv_freq(D, 5e5, rp)
    np.testing.assert_allclose(got, inv.numpy(), rtol=1e-6)
    # default rope: closed form
    np.testing.assert_allclose(O.rope_inv_freq(D, 1e6, None), 1e6 ** (-np.arange(0, D, 2) / D), rtol=1e-6)
    # product model and oracle agree
    from exo_amd.config import ModelConfig
    from exo_amd.model import rope_inv_freq

    mc = ModelConfig("llama", D * 4, 1, 4, 4, D, 64, 10, rope_theta=5e5, rope_scaling=rp)
    np.testing.assert_array_equal(rope_inv_freq(mc).numpy(), got)


def test_rope_vs_transformers_and_invariants():
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    B, H, T, D, off = 1, 3, 5, 64, 11
    x = rand_bf16((B, H, T, D), seed=4)
    inv = O.rope_inv_freq(D, 5e5, None)
    with affine.exact_activations():
        got = O.rope(x, inv, off)
        got0 = O.rope(x[:, :, :1], inv, 0)
    pos = torch.arange(off, off + T, dtype=torch.float32)
    fr = torch.outer(pos, torch.from_numpy(inv))
    emb = torch.cat([fr, fr], -1)
    q, _ = apply_rotary_pos_emb(torch.from_numpy(x), torch.from_numpy(x), emb.cos()[None], emb.sin()[None])
    np.testing.assert_allclose(got, q.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(got0, x[:, :, :1])  # position 0 is the identity
    np.testing.assert_allclose((got**2).sum(-1), (x**2).sum(-1), rtol=1e-5)  # norm preserving
    # <R(p)a, R(q)b> depends on p - q only
    a, b = x[:, :, :1], x[:, :, 1:2]
    with affine.exact_activations():
        d1 = (O.rope(a, inv, 7) * O.rope(b, inv, 3)).sum()
        d2 = (O.rope(a, inv, 104) * O.rope(b, inv, 100)).sum()
    np.testing.assert_allclose(d1, d2, rtol=1e-3)


@pytest.mark.parametrize("T,S", [(1, 9), (6, 6), (4, 10)])
def test_sdpa_vs_torch(T, S):
    B, Hq, Hkv, D = 2, 8, 2, 32
    q, k, v = rand_bf16((B, Hq, T, D), 1), rand_bf16((B, Hkv, S, D), 2), rand_bf16((B, Hkv, S, D), 3)
    mask = torch.ones(T, S, dtype=torch.bool).tril(diagonal=S - T)
    want = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), attn_mask=mask,
        scale=D**-0.5, enable_gqa=True).numpy()
    with affine.exact_activations():
        got = O.sdpa(q, k, v, D**-0.5, S - T)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)


def test_swiglu_and_router_vs_torch():
    g, u = rand_bf16((3, 50), 1, 3.0), rand_bf16((3, 50), 2)
    with affine.exact_activations():
        got = O.swiglu(g, u)
    want = (torch.nn.functional.silu(torch.from_numpy(g)) * torch.from_numpy(u)).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    logits = rand_bf16((7, 16), 5, 2.0)
    with affine.exact_activations():
        idx, sc = O.router_topk(logits, 4, True)
    p = torch.softmax(torch.from_numpy(logits), -1)
    tv, ti = torch.topk(p, 4, dim=-1)
    np.testing.assert_array_equal(idx, ti.numpy())
    np.testing.assert_allclose(sc, (tv / tv.sum(-1, keepdim=True)).numpy(), rtol=1e-5)
    # ties go to the lower expert id
    tie = np.zeros((1, 8), np.float32)
    idx, _ = O.router_topk(tie, 3, False)
    np.testing.assert_array_equal(idx, [[0, 1, 2]])


# ------------------------------------------------------------------ whole models vs transformers


def _hf_from_oracle(kind):
    from exo_amd.synth import synth_weights

    cfg = tiny_config(kind, 4)
    w = synth_weights(cfg, seed=5, device="cpu")
    ow = {}
    for k, v in w.items():
        ow[k] = (v.numpy().view(np.uint32) if v.dtype == torch.int32
                 else v.view(torch.int16).numpy().view(np.uint16))
    ocfg = OM.Config.from_json(cfg.to_dict())
    om = OM.ShardModel(ocfg, ow)

    def dq(prefix, e=None):
        return torch.from_numpy(om._wd(prefix, e).copy())

    rp = dict(cfg.rope_scaling or {"rope_type": "default"}, rope_theta=cfg.rope_theta)
    common = dict(hidden_size=cfg.hidden_size, num_hidden_layers=cfg.num_hidden_layers,
                  num_attention_heads=cfg.num_attention_heads, num_key_value_heads=cfg.num_key_value_heads,
                  head_dim=cfg.head_dim, vocab_size=cfg.vocab_size, rms_norm_eps=cfg.rms_norm_eps,
                  tie_word_embeddings=cfg.tie_word_embeddings, rope_parameters=rp,
                  max_position_embeddings=131072, attention_bias=False)
    if kind.startswith("llama"):
        from transformers import LlamaConfig, LlamaForCausalLM

        hf = LlamaForCausalLM(LlamaConfig(intermediate_size=cfg.intermediate_size, mlp_bias=False, **common))
    else:
        from transformers import Qwen3MoeConfig, Qwen3MoeForCausalLM

        hf = Qwen3MoeForCausalLM(Qwen3MoeConfig(
            moe_intermediate_size=cfg.moe_intermediate_size, intermediate_size=cfg.moe_intermediate_size,
            num_experts=cfg.num_experts, num_experts_per_tok=cfg.num_experts_per_tok,
            norm_topk_prob=cfg.norm_topk_prob, decoder_sparse_step=1, mlp_only_layers=[], **common))
    sd = {}
    emb = affine.bf16_bits_to_f32(affine.dequantize(
        ow["model.embed_tokens.weight"], ow["model.embed_tokens.scales"], ow["model.embed_tokens.biases"], 64, 4, "M1"))
    sd["model.embed_tokens.weight"] = torch.from_numpy(emb)
    sd["model.norm.weight"] = torch.ones(cfg.hidden_size)
    # the head multiplies by the un-rounded dequantised table (fused GEMV semantics)
    sd["lm_head.weight"] = dq("model.embed_tokens" if cfg.tie_word_embeddings else "lm_head")
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        for n in ("q_proj", "k_proj", "v_proj", "o_proj"):
            sd[p + f"self_attn.{n}.weight"] = dq(p + f"self_attn.{n}")
        sd[p + "input_layernorm.weight"] = torch.ones(cfg.hidden_size)
        sd[p + "post_attention_layernorm.weight"] = torch.ones(cfg.hidden_size)
        if cfg.is_moe:
            sd[p + "self_attn.q_norm.weight"] = torch.ones(cfg.head_dim)
            sd[p + "self_attn.k_norm.weight"] = torch.ones(cfg.head_dim)
            sd[p + "mlp.gate.weight"] = dq(p + "mlp.gate")
            E = cfg.num_experts
            sd[p + "mlp.experts.gate_up_proj"] = torch.stack([
                torch.cat([dq(p + "mlp.switch_mlp.gate_proj", e), dq(p + "mlp.switch_mlp.up_proj", e)]) for e in range(E)])
            sd[p + "mlp.experts.down_proj"] = torch.stack([dq(p + "mlp.switch_mlp.down_proj", e) for e in range(E)])
        else:
            for n in ("gate_proj", "up_proj", "down_proj"):
                sd[p + f"mlp.{n}.weight"] = dq(p + f"mlp.{n}")
    missing, unexpected = hf.load_state_dict(sd, strict=False)
    assert not unexpected and all("rotary" in m or (cfg.tie_word_embeddings and m == "lm_head.weight") for m in missing), (missing, unexpected)
    if cfg.tie_word_embeddings:  # untie: embedding rows are bf16-rounded, the head is not
        hf.lm_head.weight = torch.nn.Parameter(sd["lm_head.weight"].clone())
        hf.model.embed_tokens.weight = torch.nn.Parameter(sd["model.embed_tokens.weight"].clone())
    return cfg, om, hf.eval().float()


@pytest.mark.parametrize("kind", ["llama", "llama_tied_d128", "qwen3_moe"])
def test_forward_structure_vs_transformers(kind):
    """The oracle's forward (embedding, norms, q/k-norm placement, RoPE with llama3
    scaling, causal GQA attention over the cache, SwiGLU / top-k routed experts,
    residuals, final norm, tied/untied head) equals the transformers implementation of
    the same architecture on the same (dequantised) weights, in exact-activation mode."""
    cfg, om, hf = _hf_from_oracle(kind)
    toks = rng(1).integers(0, cfg.vocab_size, size=(1, 12))
    with torch.no_grad():
        want = hf(torch.from_numpy(toks)).logits.numpy()
    with affine.exact_activations():
        cache = OM.make_kv_cache(cfg.num_hidden_layers)
        got_a = om(toks[:, :7], cache)
        got_b = om(toks[:, 7:], cache)  # second call continues from the cache
    got = np.concatenate([got_a, got_b], axis=1)
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-4 * np.abs(want).max())
    # with bf16 rounding between ops the oracle stays within the model-level tolerance
    cache = OM.make_kv_cache(cfg.num_hidden_layers)
    rounded = om(toks, cache)
    rel = np.sqrt(np.mean((rounded - want) ** 2)) / np.sqrt(np.mean(want**2))
    assert rel < 2e-2, rel


def test_generation_protocol_invariants():
    """Cache lengths the reference's tests state: prefill(n tokens) leaves n-1
    (test_kv_prefix_cache.py:157); generation starts from a cache of N-2 and re-feeds
    the last two prompt tokens (test_kv_prefix_cache.py:374, generate.py:710-733)."""
    cfg, om, _ = _hf_from_oracle("llama")
    prompt = [int(t) for t in rng(2).integers(0, cfg.vocab_size, size=9)]
    for faithful in (False, True):
        c = OM.make_kv_cache(cfg.num_hidden_layers)
        OM.prefill(om, prompt, c, faithful=faithful)
        assert all(x.offset == len(prompt) - 1 for x in c)
    c1, c2 = OM.make_kv_cache(cfg.num_hidden_layers), OM.make_kv_cache(cfg.num_hidden_layers)
    OM.prefill(om, prompt, c1, faithful=True)
    OM.prefill(om, prompt, c2, step=3)  # chunking does not change the cache
    np.testing.assert_allclose(c1[0].k, c2[0].k, rtol=0, atol=2e-2)
    toks, logits = OM.greedy_generate(om, prompt, 4)
    # greedy generation == argmax of a plain full forward over prompt + generated tokens
    full = om(np.array([prompt + toks[:-1]]), OM.make_kv_cache(cfg.num_hidden_layers))[0]
    for i, t in enumerate(toks):
        row = full[len(prompt) - 1 + i]
        top2 = np.sort(row)[-2:]
        assert int(np.argmax(row)) == t or top2[1] - top2[0] < 1e-2
    # the C-accelerated oracle produces the same tokens
    omc = OM.ShardModel(om.cfg, om.weights, use_c=True)
    toks_c, _ = OM.greedy_generate(omc, prompt, 4)
    assert toks_c == toks
