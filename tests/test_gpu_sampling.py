"""The device sampling step (exo_sample through the C ABI) against the numpy oracle:
processors, log-normaliser, filter thresholds, the seeded draw, top-20 log-probabilities,
history ring and counters, on vocabularies of the benchmark sizes and small ragged ones."""

import numpy as np
import pytest
import torch

from oracle import sampling as S
from tests.util import rand_bf16, t_bf16

pytestmark = pytest.mark.gpu

from exo_amd.sampling import (MODE_DRAW, MODE_EDITS, MODE_TABLE, MODE_TOP, DeviceSampler,  # noqa: E402
                              SamplerSettings)


def _oracle_params(s: SamplerSettings) -> S.SamplerParams:
    return S.SamplerParams(
        temperature=s.temperature, top_p=s.top_p, min_p=s.min_p, top_k=s.top_k,
        repetition_penalty=s.repetition_penalty or 0.0, repetition_context=s.repetition_context,
        presence_penalty=s.presence_penalty or 0.0, presence_context=s.presence_context,
        frequency_penalty=s.frequency_penalty or 0.0, frequency_context=s.frequency_context,
        banned=list(s.banned), seed=s.seed)


def _check_rows(ds, logits, settings, histories, draws_before, want_top):
    """Outputs of one launch against the oracle, row by row."""
    tok = ds.token.cpu().numpy()
    lp = ds.logprob.cpu().numpy()
    lse = ds.lse.cpu().numpy()
    for r, (s, hist) in enumerate(zip(settings, histories)):
        p = _oracle_params(s)
        x = S.apply_processors(logits[r], hist, p)
        want_lse = S.logsumexp(x)
        assert abs(lse[r] - want_lse) <= 2e-5 * max(1.0, abs(want_lse)), (r, lse[r], want_lse)
        t = int(tok[r])
        assert 0 <= t < x.size
        if s.temperature == 0:
            assert t == int(np.argmax(x)), f"row {r}: greedy token {t} vs {int(np.argmax(x))}"
        else:
            u = S.uniform(s.seed, draws_before[r])
            thr = S.keep_threshold(x, p)
            assert x[t] >= thr, f"row {r}: token {t} (x={x[t]}) below the keep threshold {thr}"
            want, _, _ = S.sample(x, p, u, return_interval=True)
            if t != want:  # float32 sums in another order: u must sit at the edge of t's interval
                keep = x >= thr
                w = np.where(keep, np.exp(((x - x.max()) / np.float32(s.temperature)).astype(np.float64)), 0.0)
                cdf = np.cumsum(w) / w.sum()
                lo, hi = cdf[t] - w[t] / w.sum(), cdf[t]
                assert lo - 1e-5 <= u <= hi + 1e-5, f"row {r}: token {t} interval [{lo},{hi}) vs u={u}, oracle {want}"
        assert abs(lp[r] - (x[t] - want_lse)) <= 2e-5 * max(1.0, abs(x[t] - want_lse))
        if want_top:
            ids, vals = S.top_logprobs(x, 20)
            got_ids = ds.top_idx[r].cpu().numpy()[: len(ids)]
            got_vals = ds.top_val[r].cpu().numpy()[: len(ids)]
            np.testing.assert_array_equal(got_ids, ids, err_msg=f"row {r} top ids")
            np.testing.assert_allclose(got_vals, vals, rtol=0, atol=3e-5)


CASES = [
    SamplerSettings(temperature=0.0),
    SamplerSettings(),                                                  # the reference's defaults
    SamplerSettings(temperature=1.0, min_p=0.0),                        # no filter at all
    SamplerSettings(temperature=0.7, top_p=0.9, min_p=0.0),
    SamplerSettings(temperature=1.3, top_p=0.5, min_p=0.02, top_k=40),
    SamplerSettings(temperature=0.7, min_p=0.0, top_k=1),
    SamplerSettings(temperature=0.7, min_p=0.0, top_k=7, seed=(9 << 32) | 1234),
    SamplerSettings(temperature=0.0, banned=[0, 5], repetition_penalty=1.3, repetition_context=20),
    SamplerSettings(temperature=0.7, repetition_penalty=1.1, repetition_context=64,
                    presence_penalty=0.6, presence_context=30, frequency_penalty=0.4, frequency_context=50),
    SamplerSettings(temperature=0.9, top_p=0.95, frequency_penalty=1.5, frequency_context=256, banned=[3]),
]


@pytest.mark.parametrize("V", [128256, 151936, 1000, 777, 64, 19])
def test_sample_against_oracle(device, V):
    rows = len(CASES)
    logits = rand_bf16((rows, V), seed=V, scale=2.0)
    r = np.random.default_rng(V)
    ds = DeviceSampler(rows + 2, V, device)
    settings, histories = [], []
    for i, s in enumerate(CASES):
        s = SamplerSettings(**{**s.__dict__, "banned": [b % V for b in s.banned]})
        # histories of various lengths around the ring size, favouring likely tokens so the
        # penalties move tokens that matter
        n = [0, 3, 20, 100, 255, 256, 257, 700, 40, 300][i]
        hist = [int(t) for t in r.integers(0, V, size=n)]
        top = np.argsort(-logits[i])[:4]
        for j in range(0, n, 3):
            hist[j] = int(top[j % 4])
        ds.set_row(i, s, hist)
        settings.append(s)
        histories.append(hist)
    lt = t_bf16(logits, device)
    fb = torch.full((rows,), -7, dtype=torch.int32, device=device)
    pos = torch.arange(rows, dtype=torch.int32, device=device)
    mode = ds.mode(rows, want_top=True)
    assert mode == MODE_EDITS | MODE_DRAW | MODE_TABLE | MODE_TOP
    for step in range(3):
        draws_before = ds.draws.cpu().numpy().astype(np.uint32).tolist()
        ds.sample(lt, rows, mode, feedback=fb, pos_inc=pos)
        torch.cuda.synchronize()
        _check_rows(ds, logits, settings, histories, draws_before, want_top=True)
        tok = ds.token.cpu().numpy()[:rows]
        assert fb.cpu().tolist() == tok.tolist()
        assert pos.cpu().tolist() == [i + step + 1 for i in range(rows)]
        draws_after = ds.draws.cpu().numpy().astype(np.uint32).tolist()
        for i, s in enumerate(settings):
            assert draws_after[i] == draws_before[i] + (1 if s.temperature != 0 else 0)
            histories[i].append(int(tok[i]))  # the ring took the sampled token
            ring = ds.history[i].cpu().numpy()
            n = len(histories[i])
            assert int(ds.hist_len[i]) == n
            for a in range(max(0, n - 256), n):
                assert ring[a % 256] == histories[i][a]


def test_sample_modes_and_reuse(device):
    """Rows that do not ask for a stage pass through it untouched; the key tables are left
    zero (the same launch twice gives the same result); launches of different row counts
    share one workspace; the greedy mode equals the argmax entry point."""
    from exo_amd import ops
    V, rows = 128256, 4
    logits = rand_bf16((rows, V), seed=5, scale=3.0)
    logits[2, 11] = logits[2, 99] = logits[2].max()  # a tie at the top: lowest id wins
    lt = t_bf16(logits, device)
    ds = DeviceSampler(8, V, device)
    sets = [SamplerSettings(temperature=0.0), SamplerSettings(temperature=0.8, top_p=0.7, min_p=0.0),
            SamplerSettings(temperature=0.0), SamplerSettings(temperature=0.8, top_k=5)]
    for i, s in enumerate(sets):
        ds.set_row(i, s, [1, 2, 3])
    assert ds.mode(rows) == MODE_DRAW | MODE_TABLE and ds.mode(1) == 0
    hist = [[1, 2, 3] for _ in sets]
    ds.sample(lt, rows, ds.mode(rows))
    torch.cuda.synchronize()
    first = ds.token.cpu().numpy()[:rows].copy()
    _check_rows(ds, logits, sets, hist, [0] * rows, want_top=False)
    for i, s in enumerate(sets):  # same draw index again: identical tokens
        ds.set_row(i, s, [1, 2, 3])
    ds.sample(lt, rows, ds.mode(rows))
    ds.sample(lt, 1, ds.mode(1))  # a one-row launch on the same workspace
    torch.cuda.synchronize()
    assert int(ds.token[0]) == first[0]
    for i, s in enumerate(sets):
        ds.set_row(i, s, [1, 2, 3])
    ds.sample(lt, rows, ds.mode(rows) | MODE_TOP)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(ds.token.cpu().numpy()[:rows], first)
    _check_rows(ds, logits, sets, hist, [0] * rows, want_top=True)
    tok = torch.empty(rows, dtype=torch.int32, device=device)
    lse = torch.empty(rows, dtype=torch.float32, device=device)
    ops.argmax_logsumexp(lt, tok, lse, None, ops.argmax_workspace(rows, device))
    assert int(tok[0]) == first[0] and int(tok[2]) == first[2] == 11
    np.testing.assert_allclose(ds.lse.cpu().numpy()[:rows], lse.cpu().numpy(), rtol=1e-6)


def test_top_logprobs_of_flat_and_tied_rows(device):
    """Rows with thousands of tokens at the 20th largest value: an all-equal row (a zeroed or
    saturated head), a row of three distinct values, a row with 12 tokens above a plateau that
    spans several slices of the row. The lowest ids among the equals are reported, whatever
    order the workgroups of the launch arrive in; checked on repeated launches."""
    V, rows = 128256, 4
    logits = np.zeros((rows, V), np.float32)
    logits[1] = np.repeat(np.array([1.0, -2.0, 0.5], np.float32), V // 3)[:V]
    logits[2, :] = -1.0
    logits[2, 5000:90000] = 0.25                      # plateau over slices 2..44
    logits[2, [7, 120000, 64000, 3, 99999, 2049, 2048, 4095, 4096, 70001, 11, 128255]] = \
        np.array([5, 5, 4, 4, 3, 3, 3, 2, 2, 1, 1, 0.5], np.float32)
    logits[3] = rand_bf16((1, V), seed=3, scale=2.0)[0]
    logits[3, 100000:100040] = logits[3].max() + 1   # 40 equal maxima in one slice
    lt = t_bf16(logits, device)
    ds = DeviceSampler(rows, V, device)
    sets = [SamplerSettings(temperature=0.0) for _ in range(rows)]
    for rep in range(3):
        for i, s in enumerate(sets):
            ds.set_row(i, s, [])
        ds.top_idx.fill_(-7)
        ds.sample(lt, rows, MODE_TOP)
        torch.cuda.synchronize()
        _check_rows(ds, logits, sets, [[] for _ in sets], [0] * rows, want_top=True)
    assert ds.top_idx[0].cpu().tolist() == list(range(20))
    assert ds.top_idx[3].cpu().tolist() == list(range(100000, 100020))


def test_sample_with_no_token_kept_falls_back_to_the_argmax(device):
    """min_p above 1 keeps no token (the threshold lies above the maximum): the step returns the
    arg max of the processed logits, never an id outside the vocabulary."""
    V = 1000
    logits = rand_bf16((2, V), seed=21, scale=2.0)
    lt = t_bf16(logits, device)
    ds = DeviceSampler(2, V, device)
    ds.set_row(0, SamplerSettings(temperature=0.7, min_p=1.5), [])
    ds.set_row(1, SamplerSettings(temperature=0.7, min_p=1.5, top_k=5, banned=[int(np.argmax(logits[1]))]), [])
    ds.sample(lt, 2, ds.mode(2))
    torch.cuda.synchronize()
    x1 = logits[1].copy()
    x1[int(np.argmax(logits[1]))] = -np.inf
    assert ds.token[:2].cpu().tolist() == [int(np.argmax(logits[0])), int(np.argmax(x1))]


def test_sample_draws_follow_the_distribution(device):
    """4000 draws of one row (counter 0..3999) against the exact probabilities of its kept
    tokens: a chi-square bound that a wrong weight, threshold or CDF order would break."""
    V = 1000
    logits = rand_bf16((1, V), seed=77, scale=2.5)
    lt = t_bf16(logits, device)
    s = SamplerSettings(temperature=0.8, top_p=1.0, min_p=0.02, top_k=12, seed=99)
    p = _oracle_params(s)
    x = logits[0]
    keep = x >= S.keep_threshold(x, p)
    w = np.where(keep, np.exp((x - x.max()) / 0.8), 0.0)
    prob = w / w.sum()
    ds = DeviceSampler(1, V, device)
    ds.set_row(0, s, [])
    n = 4000
    counts = np.zeros(V)
    toks = []
    for _ in range(n):
        ds.sample(lt, 1, ds.mode(1))
        toks.append(ds.token[:1].clone())
    for t in torch.cat(toks).cpu().tolist():
        counts[t] += 1
    assert counts[~keep].sum() == 0 and int(keep.sum()) == 12
    chi2 = float((((counts - n * prob) ** 2)[keep] / (n * prob[keep])).sum())
    assert chi2 < 40.0, chi2  # 11 degrees of freedom: P(chi2 > 40) < 1e-4
    want = [S.sample(x, p, S.uniform(99, i)) for i in range(50)]
    assert torch.cat(toks).cpu().tolist()[:50] == want


def test_sample_argument_errors(device):
    ds = DeviceSampler(2, 1000, device)
    ds.set_row(0, SamplerSettings(), [])
    with pytest.raises(ValueError):
        ds.sample(torch.zeros(1, 999, dtype=torch.bfloat16, device=device), 1, 0)
    with pytest.raises(ValueError):
        ds.set_row(1, SamplerSettings(repetition_penalty=1.2, repetition_context=300), [])
    from exo_amd import native
    lib = native.load()
    assert lib.exo_sample(1, 1, None, None, None, 1, None, None, None, None, None, None, 1, 0, 1, 1000, 0, 0, None) == -1
    assert lib.exo_sample(1, 1, None, None, None, 1, None, None, None, None, None, None, 256, 1 << 30, 1, 300000, 0, 0, None) == -1
    assert b"exceeds" in lib.exo_last_error()
    # a history ring without entries
    lg = torch.zeros(1, 1000, dtype=torch.bfloat16, device=device)
    assert lib.exo_sample(lg.data_ptr(), ds.params.data_ptr(), ds.history.data_ptr(),
                          ds.hist_len.data_ptr(), ds.draws.data_ptr(), ds.token.data_ptr(),
                          ds.logprob.data_ptr(), ds.lse.data_ptr(), None, None, None, None,
                          ds.workspace.data_ptr(), ds.workspace.numel(), 1, 1000, 0, MODE_EDITS,
                          None) == -1
    assert b"hist_cap" in lib.exo_last_error()
