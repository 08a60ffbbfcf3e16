"""Pins of the sampling oracle (oracle/sampling.py) and of the host-side sampler record:
Philox against the published known-answer vectors, processors on hand-worked values,
the filter threshold against independent torch restatements (sort + cumsum, topk), the
inverse-CDF draw on hand-worked cases, top log-probabilities against torch.topk."""

import numpy as np
import pytest
import torch

from oracle import sampling as S
from oracle.affine import bf16_round


def test_philox_known_answers():
    """Random123 kat_vectors, philox4x32-10."""
    assert S.philox4x32_10((0, 0, 0, 0), (0, 0)) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert S.philox4x32_10((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2) == [
        0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert S.philox4x32_10((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0)) == [
        0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    u = S.uniform(0, 0)
    assert u == np.float32((0x6627E8D5 >> 8) * 2.0 ** -24) and 0.0 <= u < 1.0
    assert S.uniform(42, 0) != S.uniform(42, 1) != S.uniform(43, 1)


def test_processors_hand_values():
    x = np.array([2.0, -1.0, 0.5, 3.0, -4.0, 1.0], np.float32)
    hist = [5, 0, 1, 1, 3]  # oldest ... newest
    # ban
    got = S.apply_processors(x, hist, S.SamplerParams(banned=[2]))
    assert got[2] == bf16_round(np.array([-1e9], np.float32))[0] and list(got[[0, 1, 3, 4, 5]]) == [2.0, -1.0, 3.0, -4.0, 1.0]
    # repetition over the last 3 tokens (1, 1, 3): positive / 2, negative * 2, once per token
    got = S.apply_processors(x, hist, S.SamplerParams(repetition_penalty=2.0, repetition_context=3))
    assert list(got) == [2.0, -2.0, 0.5, 1.5, -4.0, 1.0]
    # presence over the last 4 (0, 1, 1, 3): -0.25 once each
    got = S.apply_processors(x, hist, S.SamplerParams(presence_penalty=0.25, presence_context=4))
    assert list(got) == [1.75, -1.25, 0.5, 2.75, -4.0, 1.0]
    # frequency over all 5: token 1 twice
    got = S.apply_processors(x, hist, S.SamplerParams(frequency_penalty=0.5, frequency_context=5))
    assert list(got) == [1.5, -2.0, 0.5, 2.5, -4.0, 0.5]
    # all of them, in order, on one token: token 1: -1 -> *2 = -2 -> -0.25 = -2.25 -> -2*0.5 = -3.25
    got = S.apply_processors(x, hist, S.SamplerParams(repetition_penalty=2.0, repetition_context=3,
                                                      presence_penalty=0.25, presence_context=4,
                                                      frequency_penalty=0.5, frequency_context=5))
    assert got[1] == -3.25 and got[3] == 3.0 / 2 - 0.25 - 0.5
    # results are rounded to bf16: 3.0 / 1.1 = 2.7272... -> 2.734375
    got = S.apply_processors(x, hist, S.SamplerParams(repetition_penalty=1.1, repetition_context=1))
    assert got[3] == np.float32(2.734375)
    # a context of zero or a penalty of 1 changes nothing
    assert list(S.apply_processors(x, hist, S.SamplerParams(repetition_penalty=1.0))) == list(x)
    assert list(S.apply_processors(x, [], S.SamplerParams(presence_penalty=1.0))) == list(x)


def _torch_keep_mask(x, top_p, min_p, top_k):
    """Independent restatement with library routines (sort / cumsum / topk)."""
    lp = torch.log_softmax(torch.from_numpy(x).double(), -1)
    keep = torch.ones_like(lp, dtype=torch.bool)
    if 0 < top_p < 1:
        sp, si = torch.sort(lp.exp())                 # ascending
        cum = sp.cumsum(-1)
        k = torch.zeros_like(keep)
        k[si] = cum > 1 - top_p
        # tokens of equal value stand or fall together (value threshold)
        thr = lp[k].min()
        keep &= lp >= thr
    if min_p > 0:
        keep &= lp >= lp.max() + np.log(np.float32(min_p))
    if top_k > 0:
        kth = lp.topk(min(top_k, lp.numel())).values[-1]
        keep &= lp >= kth
    return keep.numpy()


@pytest.mark.parametrize("top_p,min_p,top_k", [(0.9, 0.0, 0), (1.0, 0.05, 0), (1.0, 0.0, 7), (0.5, 0.02, 40),
                                               (0.999, 0.0, 0), (0.1, 0.0, 0), (1.0, 0.0, 0)])
def test_keep_threshold_matches_library_routines(top_p, min_p, top_k):
    r = np.random.default_rng(int(top_p * 1000) + top_k)
    for V, scale in ((1000, 2.0), (5000, 4.0), (300, 0.5)):
        x = bf16_round((r.standard_normal(V) * scale).astype(np.float32))
        p = S.SamplerParams(temperature=1.0, top_p=top_p, min_p=min_p, top_k=top_k)
        t = S.keep_threshold(x, p)
        np.testing.assert_array_equal(x >= t, _torch_keep_mask(x, top_p, min_p, top_k))
        assert (x >= t)[np.argmax(x)]


def test_inverse_cdf_hand_cases():
    x = np.log(np.array([1.0, 2.0, 1.0], np.float32))
    p = S.SamplerParams(temperature=1.0)
    assert [S.sample(x, p, u) for u in (0.0, 0.2, 0.26, 0.3, 0.74, 0.76, 0.99)] == [0, 0, 1, 1, 1, 2, 2]
    # temperature 0.5 squares the weights: 1 : 4 : 1
    p = S.SamplerParams(temperature=0.5)
    assert [S.sample(x, p, u) for u in (0.1, 0.17, 0.8, 0.84)] == [0, 1, 1, 2]
    # top_k = 1 leaves the most likely token whatever u is; temperature 0 is argmax
    assert S.sample(x, S.SamplerParams(temperature=1.0, top_k=1), 0.999) == 1
    assert S.sample(x, S.SamplerParams(temperature=0.0), 0.5) == 1
    # min_p = 0.6 drops the two tokens at half the top probability
    assert S.sample(x, S.SamplerParams(temperature=1.0, min_p=0.6), 0.01) == 1
    tok, lo, hi = S.sample(x, S.SamplerParams(temperature=1.0), 0.5, return_interval=True)
    assert tok == 1 and abs(lo - 0.25) < 1e-6 and abs(hi - 0.75) < 1e-6


def test_top_logprobs_matches_torch_topk():
    r = np.random.default_rng(3)
    x = bf16_round((r.standard_normal(4000) * 3).astype(np.float32))
    x[17] = x[901] = x.max()  # ties: lower id first
    ids, vals = S.top_logprobs(x, 20)
    lp = torch.log_softmax(torch.from_numpy(x).double(), -1)
    tv, _ = lp.topk(20)
    np.testing.assert_allclose(vals, tv.numpy(), rtol=0, atol=2e-6)
    assert ids[0] == 17 and ids[1] == 901 and len(set(ids.tolist())) == 20
    assert all(vals[i] >= vals[i + 1] for i in range(19))


def test_sampler_record_layout():
    """The host-side parameter block is the C struct of include/exo_mi355x.h, field by field."""
    from exo_amd.sampling import PARAMS_DTYPE, SamplerSettings
    from exo_amd.types import TextGenerationTaskParams
    s = SamplerSettings(temperature=0.7, top_p=0.9, min_p=0.05, top_k=40, repetition_penalty=1.1,
                        repetition_context=64, presence_penalty=0.5, frequency_penalty=0.25,
                        banned=[7, 9], seed=(5 << 32) | 6)
    raw = np.frombuffer(s.record().tobytes(), np.uint8)
    assert raw.size == 84
    f, i, u = raw.view(np.float32), raw.view(np.int32), raw.view(np.uint32)
    assert (f[0], f[1], f[2], i[3]) == (np.float32(0.7), np.float32(0.9), np.float32(0.05), 40)
    assert (f[4], i[5], f[6], i[7], f[8], i[9]) == (np.float32(1.1), 64, 0.5, 20, 0.25, 20)
    assert (u[10], u[11], i[12], list(i[13:21])) == (6, 5, 2, [7, 9, 0, 0, 0, 0, 0, 0])
    assert s.edits and s.draws and s.table and s.on_device()
    d = SamplerSettings.from_task(TextGenerationTaskParams(model="m"))
    assert (d.temperature, d.top_p, d.min_p, d.top_k, d.seed) == (0.7, 1.0, 0.05, 0, 42)
    assert d.draws and not d.table and not d.edits
    b = SamplerSettings.from_task(TextGenerationTaskParams(model="m", temperature=0.0, bench=True), [2, 3])
    assert b.banned == [2, 3] and b.edits and not b.draws
    assert not SamplerSettings(repetition_penalty=1.2, repetition_context=1000).on_device()
    # seed 0: 42 for the single-request generator (generate.py:547, `seed or 42`), 0 for the
    # batch generator (batch_generate.py:182, `is not None`)
    z = TextGenerationTaskParams(model="m", seed=0)
    assert SamplerSettings.from_task(z).seed == 42
    assert SamplerSettings.from_task(z, zero_seed_is_default=False).seed == 0
    assert SamplerSettings.from_task(TextGenerationTaskParams(model="m"),
                                     zero_seed_is_default=False).seed == 42
    assert PARAMS_DTYPE.names[-1] == "banned"


def test_filters_and_repetition_against_transformers():
    """The same definitions as implemented by another library: transformers' logits warpers
    (`TopPLogitsWarper`, `TopKLogitsWarper`, `MinPLogitsWarper`) and its
    `RepetitionPenaltyLogitsProcessor` - the kept set of every filter and of their composition,
    and the penalised values (penalty 2 and 0.5: results exact in bf16)."""
    from transformers.generation.logits_process import (
        MinPLogitsWarper, RepetitionPenaltyLogitsProcessor, TopKLogitsWarper, TopPLogitsWarper)
    rng = np.random.default_rng(5)
    for trial in range(40):
        V = int(rng.integers(5, 400))
        x = bf16_round((rng.standard_normal(V) * rng.uniform(0.5, 4.0)).astype(np.float32))
        if trial % 3 == 0:  # distinct values, so that no tie sits on a filter's edge
            x = bf16_round((np.argsort(np.argsort(x)) * 0.0625 - 3.0).astype(np.float32))
        xt = torch.from_numpy(x)[None].double()
        for top_p, min_p, top_k in [(0.9, 0.0, 0), (0.5, 0.0, 0), (1.0, 0.05, 0), (1.0, 0.3, 0),
                                    (1.0, 0.0, 1), (1.0, 0.0, 7), (0.8, 0.1, 0), (0.7, 0.0, 5), (0.95, 0.02, 40)]:
            y = xt.clone()
            if top_k > 0:
                y = TopKLogitsWarper(top_k=min(top_k, V))(None, y)
            if top_p < 1.0:
                y = TopPLogitsWarper(top_p=top_p)(None, xt.clone()).where(torch.isfinite(y), y)
            if min_p > 0.0:
                y = MinPLogitsWarper(min_p=min_p)(None, xt.clone()).where(torch.isfinite(y), y)
            want = torch.isfinite(y[0]).numpy()
            thr = S.keep_threshold(x, S.SamplerParams(temperature=1.0, top_p=top_p, min_p=min_p, top_k=top_k))
            got = x >= thr
            if len(np.unique(x)) == V:
                assert (got == want).all(), (trial, top_p, min_p, top_k)
            else:
                # values tied at a filter's edge: the library keeps some of them (by sort
                # position), this build all of them
                assert got[want].all() and (x[got & ~want] == x[want].min()).all(), (trial, top_p, min_p, top_k)
        hist = [int(t) for t in rng.integers(0, V, size=12)]
        for pen in (2.0, 0.5):
            want = RepetitionPenaltyLogitsProcessor(penalty=pen)(torch.tensor([hist]), torch.from_numpy(x)[None].clone())[0].numpy()
            got = S.apply_processors(x, hist, S.SamplerParams(repetition_penalty=pen, repetition_context=12))
            assert (got == want).all(), (trial, pen)
