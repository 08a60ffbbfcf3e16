"""End-to-end parity of the shard forward and the generation protocol on the GPU
against the CPU oracle, on tiny random-weight checkpoints shared through safetensors."""

import time

import numpy as np
import pytest
import torch

from oracle import models as OM
from tests.util import (assert_close, assert_close_stat, check_tokens as _check_tokens,
                        load_checkpoint_numpy, n_f32, rng, tiny_config, t_bf16)

pytestmark = pytest.mark.gpu

from exo_amd.config import ModelConfig  # noqa: E402
from exo_amd.engine import Mi355xBuilder, ShardBatchGenerator  # noqa: E402
from exo_amd.generate import generate, prefill  # noqa: E402
from exo_amd.loader import load_shard_weights  # noqa: E402
from exo_amd.model import ShardModel  # noqa: E402
from exo_amd.synth import write_checkpoint  # noqa: E402
from exo_amd.types import BoundInstance, GenerationTask, ShardMetadata, TextGenerationTaskParams  # noqa: E402

KINDS = [("llama", 4), ("llama_tied_d128", 8), ("qwen3_moe", 4), ("qwen3_moe", 8),
         ("qwen3_moe_router8", 4)]


def _load(path, cfg, start, end, device):
    it = load_shard_weights(path, cfg, start, end, device)
    progress = []
    try:
        while True:
            progress.append(next(it))
    except StopIteration as s:
        return s.value, progress


@pytest.fixture(scope="module", params=KINDS, ids=lambda k: f"{k[0]}-b{k[1]}")
def ckpt(request, tmp_path_factory, device):
    kind, bits = request.param
    cfg = tiny_config(kind, bits)
    path = write_checkpoint(tmp_path_factory.mktemp(f"{kind}{bits}"), cfg, seed=3, device="cpu")
    ocfg, ow = load_checkpoint_numpy(path)
    w, progress = _load(path, cfg, 0, cfg.num_hidden_layers, device)
    assert progress == [(i + 1, cfg.num_hidden_layers) for i in range(cfg.num_hidden_layers)]
    # gemm_rows=16: inputs of more than 16 rows go through the matrix-core GEMM, which
    # multiplies by bf16-rounded weights; the oracle mirrors that arithmetic mode.
    return dict(cfg=cfg, path=path, oracle=OM.ShardModel(ocfg, ow, gemm_rows=16),
                model=ShardModel(cfg, w, device=device), ocfg=ocfg, ow=ow, w=w)


def test_logits_match_oracle_in_exact_mode(ckpt, device):
    """The same prefill + single-token steps against the oracle's own arithmetic mode:
    un-rounded float32 weights for every matmul, whatever its row count (gemm_rows=None),
    i.e. without telling the oracle where the matrix-core GEMM rounds its weights to bf16.
    Bound: relative RMS <= 2e-2 and at most 1 % of the elements past the elementwise bound,
    as for the real-shape layers against this mode (the oracle differs from itself by 0.4 %
    such elements when it rounds its weights; the 8-bit toy model, whose bf16 operand drops
    the most bits, measures 0.43-0.51 % depending on how K is split, the others <= 0.1 %)."""
    cfg, gm = ckpt["cfg"], ckpt["model"]
    om = OM.ShardModel(ckpt["ocfg"], ckpt["ow"])
    prompt = rng(12).integers(0, cfg.vocab_size, size=40)
    oc, gc = OM.make_kv_cache(om.n_local_layers), gm.make_cache(1, 128)
    want = om(prompt[None], oc)
    got = gm(torch.from_numpy(prompt[None].astype(np.int32)), gc)
    if cfg.is_moe:
        tied = _check_tokens(n_f32(got), want, om, "prefill logits, exact oracle")
    else:
        assert_close_stat(n_f32(got), want, max_outlier_frac=1e-2, what="prefill logits, exact oracle")
        tied = False
    for step in range(6):
        if tied:
            break
        t = int(rng(50 + step).integers(0, cfg.vocab_size))
        om.router_margins.clear()
        want = om(np.array([[t]]), oc)
        got = gm(torch.tensor([[t]], dtype=torch.int32), gc)
        if cfg.is_moe:
            tied = _check_tokens(n_f32(got), want, om, f"decode step {step}, exact oracle")
        else:
            assert_close_stat(n_f32(got), want, max_outlier_frac=1e-2,
                              what=f"decode logits step {step}, exact oracle")


def test_prefill_and_decode_logits_match_oracle(ckpt, device):
    cfg, om, gm = ckpt["cfg"], ckpt["oracle"], ckpt["model"]
    prompt = rng(11).integers(0, cfg.vocab_size, size=40)
    oc = OM.make_kv_cache(om.n_local_layers)
    gc = gm.make_cache(1, 128)
    om.router_margins.clear()
    want = om(prompt[None], oc)  # [1,40,V]
    got = gm(torch.from_numpy(prompt[None].astype(np.int32)), gc)  # T=40 -> MFMA + prefill sdpa
    assert gc[0].offset == 40 and oc[0].offset == 40
    if cfg.is_moe:
        tied = _check_tokens(n_f32(got), want, om, "prefill logits")
    else:
        assert_close_stat(n_f32(got), want, what="prefill logits")
        tied = False
    # teacher-forced single-token steps (GEMV + decode sdpa)
    for step in range(6):
        t = int(rng(step).integers(0, cfg.vocab_size))
        om.router_margins.clear()
        want = om(np.array([[t]]), oc)
        got = gm(torch.tensor([[t]], dtype=torch.int32), gc)
        if cfg.is_moe:
            # once a token was routed differently its KV entries differ: later steps exempt
            tied = _check_tokens(n_f32(got), want, om, f"decode step {step}") or tied
            if tied:
                break
        else:
            assert_close_stat(n_f32(got), want, what=f"decode logits step {step}")


@pytest.mark.parametrize("T", [1, 40])
def test_single_layer_elementwise(ckpt, device, T):
    """One transformer block fed the oracle's own input: no cross-layer accumulation
    of rounding flips, so the elementwise rtol 2e-2 bound applies."""
    cfg, path = ckpt["cfg"], ckpt["path"]
    if cfg.is_moe:
        pytest.skip("a router near-tie flips an expert for a whole token; covered statistically")
    w1, _ = _load(path, cfg, 1, 2, device)
    g1 = ShardModel(cfg, w1, 1, 2, device)
    o1 = OM.ShardModel(ckpt["ocfg"], ckpt["ow"], 1, 2, gemm_rows=16)
    from tests.util import rand_bf16
    h = rand_bf16((1, T, cfg.hidden_size), seed=T)
    want = o1(None, OM.make_kv_cache(1), input_hidden=h)
    got = g1(None, g1.make_cache(1, 64), input_embeddings=t_bf16(h, device))
    assert_close(n_f32(got), want, what=f"layer-1 hidden T={T}")


def test_short_multi_token_forward_uses_gemv_path(ckpt, device):
    cfg, om, gm = ckpt["cfg"], ckpt["oracle"], ckpt["model"]
    toks = rng(5).integers(0, cfg.vocab_size, size=(1, 7))
    oc, gc = OM.make_kv_cache(om.n_local_layers), gm.make_cache(1, 64)
    assert_close_stat(n_f32(gm(torch.from_numpy(toks.astype(np.int32)), gc)), om(toks, oc), what="T=7")


def test_greedy_tokens_identical_32_steps(ckpt, device):
    cfg, om, gm = ckpt["cfg"], ckpt["oracle"], ckpt["model"]
    prompt = [int(t) for t in rng(21).integers(0, cfg.vocab_size, size=24)]
    om.router_margins.clear()
    want, wl = OM.greedy_generate(om, prompt, 32)
    min_gap = min((float(g.min()) for _, g in om.router_margins), default=np.inf)
    task = TextGenerationTaskParams(model="tiny", max_output_tokens=32, temperature=0.0)
    got = [r.token for r in generate(gm, None, task, prompt)]
    assert len(got) == 32
    for i, (a, b) in enumerate(zip(got, want)):
        if a != b:
            top2 = np.sort(wl[i])[-2:]
            margin = float(top2[1] - top2[0])
            atol = 2e-2 * float(np.sqrt(np.mean(wl[i] ** 2)))
            if min_gap <= 2.0 ** -6:
                pytest.xfail(f"token mismatch at step {i} after a router near-tie (gap {min_gap:.2e})")
            assert margin <= 2 * atol, f"step {i}: got {a} want {b}, margin {margin} > {2 * atol}"
            pytest.xfail(f"near-tie at step {i} (margin {margin:.3e}); sequences diverge after it")
    assert got == want


def test_prefill_protocol_cache_lengths(ckpt, device):
    gm = ckpt["model"]
    cache = gm.make_cache(1, 64)
    tps, n = prefill(gm, list(range(10)), cache)
    assert n == 10 and cache[0].offset == 9  # len-1 after prefill
    cache2 = gm.make_cache(1, 64)
    prefill(gm, list(range(10)), cache2, faithful_extra_steps=False)
    assert cache2[0].offset == 9
    k1 = n_f32(cache.k[0][0, :, :9])
    k2 = n_f32(cache2.k[0][0, :, :9])
    np.testing.assert_array_equal(k1, k2)
    c3 = gm.make_cache(1, 64)
    assert prefill(gm, [], c3) == (0.0, 0) and c3[0].offset == 0
    prefill(gm, [5], c3)
    assert c3[0].offset == 0


def test_pipeline_shards_compose(ckpt, device):
    """shard [0,k) -> hidden -> shard [k,L) equals the full model (what config 5
    compares: the hidden state leaving the last local layer)."""
    cfg, om, gm, path = ckpt["cfg"], ckpt["oracle"], ckpt["model"], ckpt["path"]
    L = cfg.num_hidden_layers
    k = 1
    w0, _ = _load(path, cfg, 0, k, device)
    w1, _ = _load(path, cfg, k, L, device)
    assert not any(n.startswith("lm_head") or n.startswith("model.norm") for n in w0)
    s0, s1 = ShardModel(cfg, w0, 0, k, device), ShardModel(cfg, w1, k, L, device)
    toks = rng(8).integers(0, cfg.vocab_size, size=(1, 20))
    tt = torch.from_numpy(toks.astype(np.int32))
    c0, c1, cf = s0.make_cache(1, 64), s1.make_cache(1, 64), gm.make_cache(1, 64)
    assert len(c0) == k and len(c1) == L - k
    hidden = s0(tt, c0)
    assert hidden.shape == (1, 20, cfg.hidden_size)
    o0 = OM.ShardModel(ckpt["ocfg"], ckpt["ow"], 0, k, gemm_rows=16)
    want0 = o0(toks, OM.make_kv_cache(k))
    if cfg.is_moe:  # a router near-tie may send a token to another expert (exempt, printed)
        _check_tokens(n_f32(hidden), want0, o0, "shard-0 hidden")
    else:
        assert_close_stat(n_f32(hidden), want0, what="shard-0 hidden")
    logits = s1(None, c1, input_embeddings=hidden)
    full = gm(tt, cf)
    np.testing.assert_array_equal(n_f32(logits), n_f32(full))


def test_decode_step_first_replay_matches_call(ckpt, device):
    """The graph-replayed single-token step, from its very first replay after a capture,
    gives the bits of the plain forward: on a later shard (hidden state in, residuals
    added in place) and on the whole model with the sampled token fed back on the device."""
    cfg, gm, path = ckpt["cfg"], ckpt["model"], ckpt["path"]
    L = cfg.num_hidden_layers
    w0, _ = _load(path, cfg, 0, 1, device)
    w1, _ = _load(path, cfg, 1, L, device)
    s0, s1 = ShardModel(cfg, w0, 0, 1, device), ShardModel(cfg, w1, 1, L, device)
    toks = torch.from_numpy(rng(13).integers(0, cfg.vocab_size, size=(1, 12)).astype(np.int32))
    c0, ca, cb = s0.make_cache(1, 64), s1.make_cache(1, 64), s1.make_cache(1, 64)
    h = s0(toks, c0)
    s1(None, ca, input_embeddings=h, logits="none")
    s1(None, cb, input_embeddings=h, logits="none")
    for step in range(3):
        t = torch.tensor([[int(rng(100 + step).integers(0, cfg.vocab_size))]], dtype=torch.int32)
        h1 = s0(t, c0)
        want = s1(None, ca, input_embeddings=h1)
        bufs = s1._buffers(1, 1)
        bufs.h.copy_(h1.view(1, -1))
        bufs = s1.decode_step(cb, 1)
        assert torch.equal(bufs.logits.view(-1), want.view(-1)), f"later shard, step {step}"
        assert cb.offsets[0] == ca.offsets[0] and cb.pos.tolist() == ca.pos.tolist()
    # whole model, device-side token feedback: eager steps against graph replays
    ce, cg = gm.make_cache(1, 64), gm.make_cache(1, 64)
    for c in (ce, cg):
        gm(toks, c, logits="none")
    first = int(rng(14).integers(0, cfg.vocab_size))
    bufs = gm._buffers(1, 1)
    bufs.tokens[0] = first
    want_toks = []
    for _ in range(4):
        want_toks.append(int(gm.decode_step(ce, 1, use_graph=False, feedback=True).next_token[0]))
    bufs.tokens[0] = first
    got_toks = []
    for _ in range(4):
        got_toks.append(int(gm.decode_step(cg, 1, feedback=True).next_token[0]))
    assert got_toks == want_toks


def test_graph_capture_keeps_the_garbage_collector_out(device):
    """Recording a step into a graph with garbage waiting to be collected - cycles that own
    pinned host memory and events, as a finished batch engine leaves behind: nothing is
    collected while the stream records (a collection there aborted the process), the
    collector is back afterwards, and the replays give the eager result."""
    import gc
    from exo_amd.model import capture_graph

    class Node:
        pass

    def litter():
        for _ in range(50):
            a, b = Node(), Node()
            a.other, b.other = b, a
            a.buf = torch.empty(1024, dtype=torch.int32).pin_memory()
            a.ev = torch.cuda.Event()
            a.buf.copy_(torch.zeros(1024, dtype=torch.int32, device=device), non_blocking=True)
            a.ev.record()
    assert gc.isenabled()
    x = torch.arange(4096, dtype=torch.float32, device=device)
    y = torch.empty_like(x)
    litter()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with capture_graph(g):
        assert not gc.isenabled()
        litter_in_capture = [dict(k=i) for i in range(5000)]  # allocations that would trigger a collection
        torch.mul(x, 2.0, out=y)
        del litter_in_capture
    assert gc.isenabled()
    for rep in range(3):
        y.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, x * 2.0), rep


def test_decode_step_recaptures_when_the_context_regime_changes(ckpt, device):
    """The attention launch of a decode step is laid out per context regime (the host's count
    of the longest sequence against ATTN_LONG_KEYS): graph replays across the threshold give
    the tokens of eager steps, and the step is captured once per regime."""
    from exo_amd import ops
    cfg, gm = ckpt["cfg"], ckpt["model"]
    start = ops.ATTN_LONG_KEYS - 4
    ce, cg = gm.make_cache(1, ops.ATTN_LONG_KEYS + 64), gm.make_cache(1, ops.ATTN_LONG_KEYS + 64)
    g = torch.Generator(device=device).manual_seed(5)
    for li in range(len(ce.k)):
        for t in (ce.k[li], ce.v[li]):
            t[:, :, :start] = (0.5 * torch.randn(t[:, :, :start].shape, device=device, generator=g)).bfloat16()
        cg.k[li].copy_(ce.k[li])
        cg.v[li].copy_(ce.v[li])
    for c in (ce, cg):
        c.offsets[0] = start
        c.sync_pos()
    bufs = gm._buffers(1, 1)
    first = int(rng(21).integers(0, cfg.vocab_size))
    bufs.tokens[0] = first
    want = [int(gm.decode_step(ce, 1, use_graph=False, feedback=True).next_token[0]) for _ in range(8)]
    bufs.tokens[0] = first
    got = [int(gm.decode_step(cg, 1, feedback=True).next_token[0]) for _ in range(8)]
    assert got == want
    assert cg.offsets[0] == start + 8 and cg.pos.tolist() == [start + 8]
    for hint in (ops.ATTN_MID_KEYS, ops.ATTN_LONG_KEYS):  # one capture per regime, both on this cache
        assert gm._graphs[(1, True, False, 0, 0, hint)][1] is cg


def test_batch_generator_b2_equals_b1(ckpt, device):
    """Port of the reference's B=2 vs B=1 criterion
    (src/exo/worker/engines/mlx/tests/test_batch_generate.py:164-268): same greedy
    tokens whether a request runs alone or next to another one."""
    cfg, gm = ckpt["cfg"], ckpt["model"]
    p1 = [int(t) for t in rng(31).integers(0, cfg.vocab_size, size=12)]
    p2 = [int(t) for t in rng(32).integers(0, cfg.vocab_size, size=19)]
    params = TextGenerationTaskParams(model="tiny", max_output_tokens=12, temperature=0.0)

    def run(prompts):
        g = ShardBatchGenerator(gm, None, max_batch=4, max_seq=128)
        uids = [g.submit(params, p) for p in prompts]
        toks = {u: [] for u in uids}
        while g.has_work:
            for u, r in g.step():
                toks[u].append(r.token)
        return [toks[u] for u in uids]

    a1, = run([p1])
    a2, = run([p2])
    b1, b2 = run([p1, p2])
    assert len(a1) == 12 and a1 == b1 and a2 == b2


def _run_batch(gm, reqs, max_batch=4, force_host=False, stagger=0):
    """reqs = [(params, prompt)]; returns per request the list of responses.  ``stagger``:
    the second and later requests join after that many steps."""
    g = ShardBatchGenerator(gm, None, max_batch=max_batch, max_seq=256)
    out, uids = {}, []

    def submit(params, prompt):
        u = g.submit(params, prompt)
        if force_host:  # pretend the kernels do not take this request's settings
            from exo_amd.generate import make_sampler, processors_for
            seq = g.rows[-1]
            gen = torch.Generator(device=gm.device)
            gen.manual_seed(seq.settings.seed)
            seq.processors = processors_for(params, [])
            seq.sampler = make_sampler(seq.settings.temperature, seq.settings.top_p, seq.settings.min_p,
                                       seq.settings.top_k, gen)
        uids.append(u)
        out[u] = []

    submit(*reqs[0])
    pending = list(reqs[1:])
    steps = 0
    while g.has_work or pending:
        if pending and (steps >= stagger or not g.has_work):
            submit(*pending.pop(0))
        for u, r in g.step():
            out[u].append(r)
        steps += 1
        if not force_host and g.rows and all(q.on_device for q in g.rows):
            # the device-side state of every row belongs to the request that sits there now:
            # its seed, and a draw counter at the request's token count (or one step ahead
            # of it, while the next replay is in flight)
            from exo_amd.sampling import PARAMS_DTYPE
            torch.cuda.synchronize()
            n = len(g.rows)
            recs = np.frombuffer(g.sampler.params[: n * PARAMS_DTYPE.itemsize].cpu().numpy().tobytes(), PARAMS_DTYPE)
            draws = g.sampler.draws[:n].tolist()
            hist_len, ring = g.sampler.hist_len[:n].tolist(), g.sampler.history[:n].tolist()
            for r, q in enumerate(g.rows):
                assert int(recs[r]["seed_lo"]) == q.settings.seed & 0xFFFFFFFF, (steps, r)
                if g._sampler_stale:
                    continue
                if q.settings.draws:
                    assert draws[r] - q.stream.n_gen in (0, 1), (steps, r, draws[r], q.stream.n_gen)
                toks, cap = [int(t) for t in q.tokens], g.sampler.hist_cap
                assert hist_len[r] - len(toks) in (0, 1), (steps, r, hist_len[r], len(toks))
                for a in range(max(0, len(toks) - cap + 1), len(toks)):
                    assert ring[r][a % cap] == toks[a], (steps, r, a)
    return [out[u] for u in uids]


def test_device_sampling_is_per_request_and_survives_compaction(ckpt, device):
    """Sampled requests (temperature, min-p, top-k, top-p, penalties; different seeds) give
    the same tokens whether they run alone, together, or join a running batch, and whichever
    row they are moved to when another request finishes: the sampling state (parameters,
    history ring, draw counter) travels with the request."""
    cfg, gm = ckpt["cfg"], ckpt["model"]
    P = TextGenerationTaskParams
    reqs = [
        (P(model="t", max_output_tokens=5, temperature=0.9, seed=7), [int(t) for t in rng(101).integers(0, cfg.vocab_size, size=11)]),
        (P(model="t", max_output_tokens=14, temperature=0.7, top_k=20, seed=8, repetition_penalty=1.3,
           frequency_penalty=0.5), [int(t) for t in rng(102).integers(0, cfg.vocab_size, size=17)]),
        (P(model="t", max_output_tokens=9, temperature=1.1, top_p=0.8, min_p=0.0, seed=9, presence_penalty=0.7),
         [int(t) for t in rng(103).integers(0, cfg.vocab_size, size=9)]),
    ]
    solo = [[r.token for r in _run_batch(gm, [q])[0]] for q in reqs]
    assert [len(s) for s in solo] == [5, 14, 9]
    assert len(set(solo[1])) > 3  # it does sample
    together = [[r.token for r in rs] for rs in _run_batch(gm, reqs)]
    assert [len(t) for t in together] == [5, 14, 9]
    # Alone, a request runs the single-row kernels, and in another row of a batch its sums
    # are formed in another order (log-probabilities move by a few 1e-3): a draw that falls
    # on the edge between two tokens may then go the other way, so sampled tokens are only
    # compared between runs of the SAME placement (exactly); that the state travels with the
    # request (seed, draw counter, history ring) is checked row by row after every step
    # (_run_batch).
    flipped = [[r.token for r in rs] for rs in _run_batch(gm, reqs[::-1])][::-1]
    assert [len(t) for t in flipped] == [5, 14, 9]
    staggered = [[r.token for r in rs] for rs in _run_batch(gm, reqs, stagger=3)]
    assert [len(t) for t in staggered] == [5, 14, 9]
    assert staggered == [[r.token for r in rs] for rs in _run_batch(gm, reqs, stagger=3)]
    again = [[r.token for r in rs] for rs in _run_batch(gm, reqs)]
    assert again == together  # same seeds, same tokens
    other_seed = _run_batch(gm, [(P(model="t", max_output_tokens=14, temperature=0.7, top_k=20, seed=88,
                                    repetition_penalty=1.3, frequency_penalty=0.5), reqs[1][1])])[0]
    assert [r.token for r in other_seed] != solo[1]
    # sequential generate() runs the same kernels with the same seed
    assert [r.token for r in generate(gm, None, reqs[1][0], reqs[1][1])] == solo[1]


def test_device_logprobs_match_host_path(ckpt, device):
    """Greedy requests with log-probabilities: the device step (top-20 table, selected
    log-probability) against the same requests stepped with the processors and torch.topk on
    the host; a request whose settings the kernels do not take switches the whole batch to the
    host for as long as it runs and the others carry on unchanged."""
    cfg, gm = ckpt["cfg"], ckpt["model"]
    P = TextGenerationTaskParams
    reqs = [(P(model="t", max_output_tokens=6, temperature=0.0, logprobs=True, top_logprobs=5),
             [int(t) for t in rng(111).integers(0, cfg.vocab_size, size=13)]),
            (P(model="t", max_output_tokens=9, temperature=0.0, logprobs=True, top_logprobs=20,
               repetition_penalty=1.5), [int(t) for t in rng(112).integers(0, cfg.vocab_size, size=8)])]
    dev = _run_batch(gm, reqs)
    host = _run_batch(gm, reqs, force_host=True)
    for d, h in zip(dev, host):
        assert [r.token for r in d] == [r.token for r in h]
        assert len(d[0].top_logprobs) == len(h[0].top_logprobs)
        for rd, rh in zip(d, h):
            assert abs(rd.logprob - rh.logprob) < 2e-2  # a penalised logit is rounded to bf16 on the device
            # bf16 processors on the device, float32 on the host: the order of near-equal
            # entries may differ, the values may not
            np.testing.assert_allclose([i.logprob for i in rd.top_logprobs],
                                       [i.logprob for i in rh.top_logprobs], atol=2e-2)
            assert rd.top_logprobs[0].token == rh.top_logprobs[0].token
        assert d[-1].finish_reason == "length" and d[-1].stats.generation_tokens == len(d)
    # a context the history ring does not hold: that request samples on the host
    wide = (P(model="t", max_output_tokens=4, temperature=0.0, repetition_penalty=1.2,
              repetition_context_size=1000), reqs[0][1])
    mixed = _run_batch(gm, [reqs[1], wide], stagger=2)
    assert [r.token for r in mixed[0]] == [r.token for r in dev[1]]
    assert len(mixed[1]) == 4


def test_batch_generator_slot_compaction_and_cancel(ckpt, device):
    cfg, gm = ckpt["cfg"], ckpt["model"]
    short = TextGenerationTaskParams(model="tiny", max_output_tokens=3, temperature=0.0)
    long = TextGenerationTaskParams(model="tiny", max_output_tokens=9, temperature=0.0)
    pa = [int(t) for t in rng(41).integers(0, cfg.vocab_size, size=9)]
    pb = [int(t) for t in rng(42).integers(0, cfg.vocab_size, size=14)]
    solo = ShardBatchGenerator(gm, None, 4, 128)
    solo.submit(long, pb)
    want = []
    while solo.has_work:
        want += [r.token for _, r in solo.step()]
    g = ShardBatchGenerator(gm, None, 4, 128)
    ua, ub = g.submit(short, pa), g.submit(long, pb)  # a finishes first; b moves to row 0
    got, fin = [], {}
    while g.has_work:
        for u, r in g.step():
            if u == ub:
                got.append(r.token)
            if r.finish_reason:
                fin[u] = r.finish_reason
                assert r.stats is not None and r.usage.completion_tokens in (3, 9)
    assert got == want and fin == {ua: "length", ub: "length"}
    uc = g.submit(long, pb)
    g.step()
    g.cancel([uc])
    assert not g.has_work


@pytest.mark.parametrize("no_batch", [False, True])
def test_builder_engine_contract(ckpt, device, monkeypatch, no_batch):
    """Runner-side sequence of src/exo/worker/runner/runner.py:250-386: load (progress
    events) -> build -> warmup -> submit -> step until Finished; for the batched engine and
    for the sequential one the reference's builder returns under EXO_NO_BATCH
    (src/exo/worker/engines/mlx/builder.py:86-99)."""
    cfg, path = ckpt["cfg"], ckpt["path"]
    if no_batch:
        monkeypatch.setenv("EXO_NO_BATCH", "1")
    else:
        monkeypatch.delenv("EXO_NO_BATCH", raising=False)

    class Sender:
        def __init__(self):
            self.sent = []

        def send(self, e):
            self.sent.append(e)

    class Receiver:
        def __init__(self):
            self.pending = []

        def collect(self):
            p, self.pending = self.pending, []
            return p

    sender, recv = Sender(), Receiver()
    b = Mi355xBuilder("tiny/model", sender, recv, device=str(device), max_seq=256)
    shard = ShardMetadata("tiny/model", 0, cfg.num_hidden_layers, cfg.num_hidden_layers)
    inst = BoundInstance(shard, str(path))
    prog = list(b.load(inst))
    assert [(p.layers_loaded, p.total) for p in prog] == [
        (i + 1, cfg.num_hidden_layers) for i in range(cfg.num_hidden_layers)]
    eng = b.build()
    assert type(eng).__name__ == ("SequentialGenerator" if no_batch else "BatchGenerator")
    eng.warmup()
    assert eng.check_for_cancel_every >= 1
    prompt = [int(t) for t in rng(51).integers(0, cfg.vocab_size, size=20)]
    params = TextGenerationTaskParams(model="tiny/model", input=prompt, max_output_tokens=5,
                                      temperature=0.0, bench=True)
    eng.submit(GenerationTask("task-1", "cmd-1", params))
    events = []
    for _ in range(20):
        events += list(eng.step())
        if events and type(events[-1][1]).__name__ == "FinishedResponse":
            break
    kinds = [type(e).__name__ for _, e in events]
    assert kinds == ["TokenChunk"] * 5 + ["FinishedResponse"]
    assert events[4][1].finish_reason == "length" and events[4][1].stats.generation_tokens == 5
    assert all(tid == "task-1" for tid, _ in events)
    want = [r.token for r in generate(b.inference_model, None, params, prompt)]
    assert [e.token_id for _, e in events[:5]] == want
    # two queued requests: the sequential engine finishes the first before the second starts
    for name in ("task-a", "task-b"):
        eng.submit(GenerationTask(name, "cmd-" + name, params))
    events = []
    for _ in range(40):
        events += list(eng.step())
        if [type(e).__name__ for _, e in events].count("FinishedResponse") == 2:
            break
    per = {n: [e.token_id for t, e in events if t == n and type(e).__name__ == "TokenChunk"]
           for n in ("task-a", "task-b")}
    assert per == {"task-a": want, "task-b": want}
    if no_batch:
        assert [t for t, _ in events] == ["task-a"] * 6 + ["task-b"] * 6
    # cancellation of a running task
    eng.submit(GenerationTask("task-2", "cmd-2", TextGenerationTaskParams(
        model="tiny/model", input=prompt, max_output_tokens=500, temperature=0.0)))
    list(eng.step())
    recv.pending.append("task-2")
    eng.check_for_cancel_every = 1
    out = []
    for _ in range(5):
        out += list(eng.step())
    assert ("task-2", "CancelledResponse") in [(t, type(e).__name__) for t, e in out]
    # an error inside step is reported as an ErrorChunk before it propagates
    eng.submit(GenerationTask("task-3", "cmd-3", TextGenerationTaskParams(model="tiny/model", input=[])))
    with pytest.raises(ValueError):
        list(eng.step())
    assert type(sender.sent[-1][1]).__name__ == "ErrorChunk" and sender.sent[-1][0] == "cmd-3"
    eng.close()
    b.close()


def _run_requests(gm, prompts, params, pc, max_seq=2048):
    """Submit the prompts one after the other (each runs to completion) through one
    generator; returns the token lists and the per-request prefix-hit labels."""
    g = ShardBatchGenerator(gm, None, max_batch=2, max_seq=max_seq, kv_prefix_cache=pc)
    outs, hits = [], []
    for p in prompts:
        g.submit(params, p)
        toks = []
        while g.has_work:
            for _, r in g.step():
                toks.append(r.token)
                if r.stats is not None:
                    hits.append(r.stats.prefix_cache_hit)
        outs.append(toks)
    return outs, hits


def test_prefix_cache_generation_invariants(ckpt, device):
    """The generation-level invariants of the reference's prefix-cache tests
    (src/exo/worker/tests/unittests/test_mlx/test_kv_prefix_cache.py:345-412,495-532):
    a request stores N-2 positions; the same prompt again is an exact hit with exactly
    the last two tokens left to feed and produces the same tokens; the stored entry is
    not touched by the generation that used it."""
    from exo_amd.prefix_cache import KVPrefixCache, cache_length
    cfg, gm = ckpt["cfg"], ckpt["model"]
    prompt = [int(t) for t in rng(61).integers(0, cfg.vocab_size, size=40)]
    params = TextGenerationTaskParams(model="tiny", max_output_tokens=8, temperature=0.0)
    (cold,), _ = _run_requests(gm, [prompt], params, None)
    pc = KVPrefixCache(None, device)
    (first, second), hits = _run_requests(gm, [prompt, prompt], params, pc)
    assert first == cold and second == cold and hits == ["none", "exact"]
    assert len(pc.prompts) == 2  # short prompts add entries (hit < 1000 tokens)
    assert cache_length(pc.caches[0]) == len(prompt) - 2
    before = [t.clone() for t in pc.caches[0].layers]
    probe = gm.make_cache(1, 256)
    _, remaining, idx, exact = pc.get_kv_cache(probe, prompt)
    assert idx == 0 and exact and remaining == prompt[-2:]
    assert all(torch.equal(a, b) for a, b in zip(before, pc.caches[0].layers))
    # partial hit: same first 25 tokens, different tail -> same tokens as a cold run
    other = prompt[:25] + [int(t) for t in rng(62).integers(0, cfg.vocab_size, size=9)]
    (cold_other,), _ = _run_requests(gm, [other], params, None)
    pc2 = KVPrefixCache(None, device)
    (_, warm_other), hits = _run_requests(gm, [prompt, other], params, pc2)
    assert warm_other == cold_other and hits == ["none", "partial"]


def test_prefix_cache_long_prompt_updates_in_place(ckpt, device):
    """test_kv_prefix_cache.py:414-493: a second prompt sharing more than 1000 tokens
    (and more than half) with a stored one replaces that entry with the longer cache."""
    from exo_amd.prefix_cache import KVPrefixCache, cache_length
    cfg, gm = ckpt["cfg"], ckpt["model"]
    base = [int(t) for t in rng(71).integers(0, cfg.vocab_size, size=1100)]
    longer = base[:1080] + [int(t) for t in rng(72).integers(0, cfg.vocab_size, size=60)]
    params = TextGenerationTaskParams(model="tiny", max_output_tokens=4, temperature=0.0)
    (cold,), _ = _run_requests(gm, [longer], params, None)
    pc = KVPrefixCache(None, device)
    (_, warm), hits = _run_requests(gm, [base, longer], params, pc)
    assert hits == ["none", "partial"] and len(pc.prompts) == 1
    assert cache_length(pc.caches[0]) == len(longer) - 2 and len(pc.prompts[0]) == len(longer)
    # the restored prefix went through the same kernels as the cold prefill's first 1080
    # positions did only if both used the GEMM path; tokens must still agree
    assert warm == cold


def test_sequential_generate_with_prefix_cache(ckpt, device):
    from exo_amd.prefix_cache import KVPrefixCache, cache_length
    cfg, gm = ckpt["cfg"], ckpt["model"]
    prompt = [int(t) for t in rng(81).integers(0, cfg.vocab_size, size=30)]
    params = TextGenerationTaskParams(model="tiny", max_output_tokens=6, temperature=0.0)
    cold = [r.token for r in generate(gm, None, params, prompt, max_seq=128)]
    pc = KVPrefixCache(None, device)
    first = list(generate(gm, None, params, prompt, max_seq=128, kv_prefix_cache=pc))
    assert cache_length(pc.caches[0]) == len(prompt) - 2
    second = list(generate(gm, None, params, prompt, max_seq=128, kv_prefix_cache=pc))
    assert [r.token for r in first] == cold and [r.token for r in second] == cold
    assert first[-1].stats.prefix_cache_hit == "none" and second[-1].stats.prefix_cache_hit == "exact"
    bench = TextGenerationTaskParams(model="tiny", max_output_tokens=2, temperature=0.0, bench=True)
    third = list(generate(gm, None, bench, prompt, max_seq=128, kv_prefix_cache=pc))
    assert third[-1].stats.prefix_cache_hit == "none"   # bench requests opt in explicitly


# ------------------------------------------------------- disaggregated prefill


def test_send_and_ingest_kv_cache(ckpt, device):
    """Port of the reference's adapter tests
    (engines/mlx/disaggregated/tests/test_mlx_adapter.py:115-180): a cache sent and
    ingested is bit-identical; start_pos ships only the suffix; a fill level at or below
    start_pos ships nothing."""
    import io
    from exo_amd import disaggregated as D
    gm = ckpt["model"]
    src = gm.make_cache(2, 64)
    for t in src.k + src.v:
        t.copy_(torch.randn(t.shape, device=device).bfloat16())
    src.offsets[1] = 37
    src.sync_pos()
    buf = io.BytesIO()
    sent = D.write_cache_to_wire(buf, src, row=1, request_id="r", model_id="m")
    assert sent == 37
    buf.seek(0)
    res = D.read_result(buf)
    assert res.header.num_layers == len(src) and res.total_tokens == 37
    assert sorted(res.kv_chunks) == list(range(len(src)))
    c0 = res.kv_chunks[0][0]
    assert c0.shape == (37, src.k[0].shape[1], src.k[0].shape[3]) and c0.dtype == "bfloat16"
    dst = gm.make_cache(1, 48)
    assert D.ingest_into_cache(res, dst, row=0) == 37 and dst.offsets[0] == 37
    assert dst.pos.tolist() == [37]
    for i in range(len(src)):
        assert torch.equal(dst.k[i][0, :, :37], src.k[i][1, :, :37])
        assert torch.equal(dst.v[i][0, :, :37], src.v[i][1, :, :37])
    # suffix only
    buf = io.BytesIO()
    assert D.write_cache_to_wire(buf, src, row=1, start_pos=30) == 7
    buf.seek(0)
    res = D.read_result(buf)
    assert res.header.start_pos == 30 and res.kv_chunks[0][0].num_tokens == 7
    dst.k[0][0, :, 30:37].zero_()
    assert D.ingest_into_cache(res, dst, row=0, start_pos=30) == 37
    assert torch.equal(dst.k[0][0, :, :37], src.k[0][1, :, :37])
    # nothing to send
    buf = io.BytesIO()
    assert D.write_cache_to_wire(buf, src, row=1, start_pos=40) == 0
    buf.seek(0)
    res = D.read_result(buf)
    assert res.kv_chunks == {} and res.total_tokens == 0


@pytest.mark.parametrize("engine_cls", ["BatchGenerator", "SequentialGenerator"])
def test_serve_prefill_over_tcp_then_decode(ckpt, device, engine_cls):
    """The engine (batched or sequential) as prefill server: a request over the TCP front is resolved by
    Engine.serve_prefill; the KV that arrives is bit-identical to a local prefill of the
    same tokens and a decoder continuing from it produces the local tokens.  The server
    stops three positions short of the tokens it is given (serve.py:43-58: target n-2,
    and the prefill routine leaves one more out), so the client asks with one padding
    token to receive N-2 positions."""
    from exo_amd import disaggregated as D
    import exo_amd.engine as E
    from exo_amd.prefix_cache import KVPrefixCache
    BatchGenerator = getattr(E, engine_cls)
    cfg, gm = ckpt["cfg"], ckpt["model"]
    prompt = [int(t) for t in rng(91).integers(0, cfg.vocab_size, size=45)]
    params = TextGenerationTaskParams(model="tiny", max_output_tokens=6, temperature=0.0)
    want = [r.token for r in generate(gm, None, params, prompt, max_seq=128)]
    local = gm.make_cache(1, 128)
    prefill(gm, prompt[:-1], local)

    eng = BatchGenerator(model=gm, tokenizer=None, model_id="tiny", max_seq=128,
                         kv_prefix_cache=KVPrefixCache(None, device))
    served = []

    def resolve(job, wfile):  # the runner would queue this for the engine thread
        eng.serve_prefill(job, wfile)
        served.append(job.request_id)
        return True

    srv = D.PrefillServer(resolve, "127.0.0.1", 0)
    try:
        ep = f"127.0.0.1:{srv.server_address[1]}"
        dec = gm.make_cache(1, 128)
        progress = []
        tps, n = D.remote_prefill(prompt + [0], dec, lambda d, t: progress.append((d, t)),
                                  endpoint=ep, request_id="req-1", model_id="tiny")
        for _ in range(500):  # the handler thread notes the job after the client has its reply
            if served:
                break
            time.sleep(0.01)
        assert served == ["req-1"] and n == len(prompt) - 2 and dec.offsets[0] == n and tps > 0
        assert progress and progress[-1][1] == len(prompt) + 1
        for i in range(len(dec)):
            assert torch.equal(dec.k[i][0, :, :n], local.k[i][0, :, :n])
            assert torch.equal(dec.v[i][0, :, :n], local.v[i][0, :, :n])
        # the same request again is served from the server's prefix cache
        dec2 = gm.make_cache(1, 128)
        D.remote_prefill(prompt + [0], dec2, None, endpoint=ep, request_id="req-2", model_id="tiny")
        assert torch.equal(dec2.k[0][0, :, :n], local.k[0][0, :, :n])
        assert len(eng.kv_prefix_cache.prompts) == 1  # hit ratio >= 0.5: updated in place
    finally:
        srv.stop()
    # decode from the ingested cache: feed prompt[-2], then generate from prompt[-1]
    gm(torch.tensor([[prompt[-2]]], dtype=torch.int32), dec, logits="none")
    tok, got = prompt[-1], []
    for _ in range(6):
        bufs = gm._buffers(1, 1)
        bufs.tokens[0] = tok
        bufs = gm.decode_step(dec, 1)
        tok = int(bufs.next_token[0])
        got.append(tok)
    assert got == want
    eng.close()


def test_submit_fetches_long_prompts_from_a_prefill_server(ckpt, device):
    """A task that names a prefill endpoint and has more than 1000 uncached prompt tokens is
    prefilled over the wire (src/exo/worker/engines/mlx/generator/batch_generate.py:205-246):
    the generated tokens equal those of a local prefill, the server was asked once, short
    prompts stay local, and a dead endpoint falls back to the local path."""
    from exo_amd import disaggregated as D
    from exo_amd.engine import BatchGenerator
    from exo_amd.prefix_cache import KVPrefixCache
    cfg, gm = ckpt["cfg"], ckpt["model"]
    prompt = [int(t) for t in rng(121).integers(0, cfg.vocab_size, size=1203)]
    P = TextGenerationTaskParams
    local = [r.token for r in _run_batch_seq(gm, P(model="tiny", max_output_tokens=6, temperature=0.0), prompt)]
    server_engine = BatchGenerator(model=gm, tokenizer=None, model_id="tiny", max_seq=2048,
                                   kv_prefix_cache=KVPrefixCache(None, device))
    served = []

    def resolve(job, wfile):
        server_engine.serve_prefill(job, wfile)
        served.append((len(job.token_ids), job.start_pos))
        return True

    srv = D.PrefillServer(resolve, "127.0.0.1", 0)
    try:
        ep = f"127.0.0.1:{srv.server_address[1]}"
        remote = _run_batch_seq(gm, P(model="tiny", max_output_tokens=6, temperature=0.0, prefill_endpoint=ep), prompt)
        for _ in range(500):
            if served:
                break
            time.sleep(0.01)
        # the few positions the server's reply stops short of are computed here as a short
        # chunk (GEMV kernels) where the local path has them inside its one long GEMM chunk:
        # last-bit differences there may turn a near-tie, so the tokens are compared at the
        # start and the shipped KV bit for bit
        assert [r.token for r in remote][:3] == local[:3] and served == [(len(prompt) - 1, 0)]
        assert remote[-1].stats.prompt_tps > 0
        ga, gb = ShardBatchGenerator(gm, None, 1, 2048), ShardBatchGenerator(gm, None, 1, 2048)
        ga.submit(P(model="tiny", max_output_tokens=2, temperature=0.0), prompt)
        gb.submit(P(model="tiny", max_output_tokens=2, temperature=0.0, prefill_endpoint=ep), prompt)
        n_ship = len(prompt) - 1 - 3
        assert ga.cache.offsets[0] == gb.cache.offsets[0] == len(prompt) - 1
        for li in range(len(ga.cache)):
            assert torch.equal(ga.cache.k[li][0, :, :n_ship], gb.cache.k[li][0, :, :n_ship])
            assert torch.equal(ga.cache.v[li][0, :, :n_ship], gb.cache.v[li][0, :, :n_ship])
        # (layer 0's keys of the locally filled positions depend on the tokens alone)
        assert_close_stat(n_f32(gb.cache.k[0][0, :, n_ship:len(prompt) - 2]),
                          n_f32(ga.cache.k[0][0, :, n_ship:len(prompt) - 2]), what="gap positions, layer 0 keys")
        short = _run_batch_seq(gm, P(model="tiny", max_output_tokens=3, temperature=0.0, prefill_endpoint=ep), prompt[:50])
        assert len(short) == 3 and len(served) == 2  # 50 tokens: not worth the trip (2 = the fetches above)
    finally:
        srv.stop()
    dead = _run_batch_seq(gm, P(model="tiny", max_output_tokens=6, temperature=0.0,
                                prefill_endpoint="127.0.0.1:9"), prompt)
    assert [r.token for r in dead] == local
    server_engine.close()
    ga.close()
    gb.close()


def _run_batch_seq(gm, params, prompt):
    g = ShardBatchGenerator(gm, None, max_batch=2, max_seq=2048)
    g.submit(params, prompt)
    out = []
    while g.has_work:
        out += [r for _, r in g.step()]
    return out


def test_generate_with_persistent_state_equals_fresh_state(ckpt, device):
    """generate() on a cache row and sampler that outlive the request (what the sequential
    engine keeps, so that its HIP graphs are captured once): the same tokens as with fresh
    ones, request after request, also after a request that was abandoned half way, greedy and
    sampled."""
    from exo_amd.generate import GenerateState
    cfg, gm = ckpt["cfg"], ckpt["model"]
    P = TextGenerationTaskParams
    reqs = [(P(model="t", max_output_tokens=7, temperature=0.0), 23),
            (P(model="t", max_output_tokens=9, temperature=0.8, top_k=12, seed=5, repetition_penalty=1.2), 9),
            (P(model="t", max_output_tokens=5, temperature=0.0, logprobs=True, top_logprobs=3), 31)]
    st = GenerateState(gm, 128)
    for i, (params, n) in enumerate(reqs):
        prompt = [int(t) for t in rng(300 + i).integers(0, cfg.vocab_size, size=n)]
        want = [(r.token, r.finish_reason) for r in generate(gm, None, params, prompt)]
        got = [(r.token, r.finish_reason) for r in generate(gm, None, params, prompt, state=st)]
        assert got == want, i
        it = generate(gm, None, params, prompt, state=st)  # abandoned after two tokens
        next(it), next(it)
        it.close()
    with pytest.raises(ValueError):
        list(generate(gm, None, reqs[0][0], list(range(1, 128)), state=st))
