"""Host-side logic that needs no GPU: C-ABI surface, loader, config, cache bookkeeping,
Engine event ordering with a faked inner generator, samplers."""

import ctypes
import json
import re
from pathlib import Path

import numpy as np
import ctypes as C

import pytest
import torch

from exo_amd import native
from exo_amd.config import ModelConfig, named_config
from exo_amd.engine import BatchGenerator, build_model_path
from exo_amd.generate import PrefillCancelled, ban_token_ids, extract_top_logprobs, make_sampler
from exo_amd.loader import layer_index_of, load_shard_weights, wanted
from exo_amd.synth import synth_weights, write_checkpoint
from exo_amd.tokenizer import IdTokenizer, load_tokenizer
from exo_amd.types import GenerationResponse, GenerationTask, TextGenerationTaskParams
from tests.util import tiny_config

ROOT = Path(__file__).resolve().parent.parent


# ------------------------------------------------------------------ C ABI


def _declared_symbols():
    text = (ROOT / "include" / "exo_mi355x.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(exo_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    syms = _declared_symbols()
    assert len(syms) >= 20
    assert native.LIB_PATH.exists(), "build with `python -m exo_amd.build`"
    lib = ctypes.CDLL(str(native.LIB_PATH))  # loads without a GPU
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/exo_mi355x.h but not exported"
    assert sorted(native.SIGNATURES) == syms  # the ctypes table covers the header one to one


def test_argument_errors_without_gpu():
    lib = native.load()
    assert lib.exo_abi_version() == 1
    # argument validation happens before any HIP call
    assert lib.exo_qmv(None, None, None, None, None, None, 1, 64, 128, 3, 64, None) == -1
    assert b"bits must be 4 or 8" in lib.exo_last_error()
    assert lib.exo_qmm(None, None, None, None, None, None, 1, 64, 100, 4, 64, None) == -1
    assert lib.exo_sdpa_decode(None, None, None, None, None, None, 1.0, 1, 8, 3, 128, 64, None) == -1
    assert lib.exo_router_topk(None, None, None, 1, 300, 8, 1, None) == -1
    # the no-allocation decode attention rejects sizes beyond its static scratch
    assert lib.exo_sdpa_decode_static(None, None, None, None, None, 1.0, 9, 32, 8, 128, 64, None) == -1
    assert b"exceed the static scratch" in lib.exo_last_error()
    # decode attention workspace: a counter per query head (whole 256-byte lines), then the
    # partials of 16 key splits per head, or of the long-context layout's up to 32 splits on
    # at most 256 workgroups where that is more
    assert lib.exo_sdpa_decode_workspace(2, 32, 128) == (64 + 64 * 32 * 130) * 4
    assert lib.exo_sdpa_decode_workspace(8, 32, 128) == (256 + 256 * 16 * 130) * 4
    assert lib.exo_sdpa_decode_workspace(64, 32, 128) == (2048 + 2048 * 16 * 130) * 4
    one = C.c_void_p(1)  # any non-null pointer: rejected before it is ever used
    assert lib.exo_attn_decode_hint(one, one, one, one, one, None, None, None, 0.0, one, one, 1.0, 1, 32, 8,
                                    128, 8192, -5, None) == -1
    assert b"keys_hint" in lib.exo_last_error()
    # the expert launch that routes by itself: the limits of exo_router_topk
    rc = lib.exo_norm_route_gather_qmv_swiglu(one, None, 0.0, one, 1, one, one, one, one, one, one, one, one,
                                              one, 1, 8, 300, 64, 2048, 4, 64, None)
    assert rc == -1 and b"E<=256" in lib.exo_last_error()
    # RoPE with a table but no rows; head_dim outside {64, 128}
    assert lib.exo_rope_kv_append_tab(one, one, one, one, one, one, one, 0, None, None, 0.0, 1, 1, 8, 2, 128,
                                      16, None) == -1
    assert b"table without rows" in lib.exo_last_error()
    assert lib.exo_rope_kv_append_tab(one, one, one, one, one, one, None, 0, None, None, 0.0, 1, 1, 8, 2, 96,
                                      16, None) == -1
    # pair GEMM: the K-split workspace is sized per shape, 0 where the launch never splits
    assert lib.exo_qmm_swiglu_workspace(126, 8192) == 2 * 2 * 126 * 8192 * 4
    assert lib.exo_qmm_swiglu_workspace(126, 4096) == 4 * 2 * 126 * 4096 * 4  # 64 tiles: four ranges
    assert lib.exo_qmm_swiglu_workspace(129, 8192) == 0 and lib.exo_qmm_swiglu_workspace(126, 14336) == 0
    rc = lib.exo_qmm_swiglu_ws(one, one, one, one, one, one, one, one, C.c_void_p(256), 16, 126, 8192, 2048,
                               4, 64, None)
    assert rc == -1 and b"workspace of 16 bytes" in lib.exo_last_error()
    with pytest.raises(ValueError):
        native.check(-1, "x")


def test_bench_reads_the_committed_counter_summary():
    """roofline.traffic of the bench line comes from the committed rocprofv3 --pmc summary:
    the launch names bench.py asks for must be the ones that file lists."""
    import importlib.util
    import pathlib
    root = pathlib.Path(__file__).resolve().parents[1]
    spec = importlib.util.spec_from_file_location("bench_module", root / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    traffic, src = bench.pmc_traffic("norm_gate_up_swiglu")
    assert traffic is not None and 0.95 < traffic / 66105344 < 1.10, (traffic, src)
    assert "commit" in src


def test_decode_context_regimes():
    """The decode step's attention layout follows the host's count of the longest sequence of
    the rows it serves: below 3072 keys, from 3072, from 6144, from 12288 (one captured graph
    each)."""
    from types import SimpleNamespace
    from exo_amd import ops
    from exo_amd.model import ShardModel
    cache = SimpleNamespace(offsets=[10, 6142, 6143, 12286, 12287, 40000])
    hint = ShardModel._keys_hint
    assert hint(cache, slice(0, 1)) == 0 and hint(cache, slice(0, 2)) == ops.ATTN_MID_KEYS
    assert hint(SimpleNamespace(offsets=[3070]), slice(0, 1)) == 0
    assert hint(SimpleNamespace(offsets=[3071]), slice(0, 1)) == ops.ATTN_MID_KEYS
    assert hint(cache, slice(0, 3)) == ops.ATTN_LONG_KEYS          # 6143 cached + the new key
    assert hint(cache, slice(2, 4)) == ops.ATTN_LONG_KEYS
    assert hint(cache, slice(3, 5)) == ops.ATTN_VERY_LONG_KEYS
    assert hint(cache, slice(0, 6)) == ops.ATTN_VERY_LONG_KEYS
    assert (ops.ATTN_LONG_KEYS, ops.ATTN_VERY_LONG_KEYS) == (6144, 12288)
    hdr = (ROOT / "include" / "exo_mi355x.h").read_text()
    assert "#define EXO_ATTN_MID_KEYS 3072" in hdr and "#define EXO_ATTN_LONG_KEYS 6144" in hdr and "#define EXO_ATTN_VERY_LONG_KEYS 12288" in hdr


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(native.NativeError):
        native.load()


# ------------------------------------------------------------------ config / loader


def test_named_configs_weight_bytes_match_the_stated_figures():
    def qbytes(n, k, bits):
        return n * k * bits // 8 + n * (k // 64) * 4

    c = named_config("llama-3.1-8b")
    H, D, I = c.hidden_size, c.head_dim, c.intermediate_size
    layer = (qbytes(c.num_attention_heads * D, H, 4) + 2 * qbytes(c.num_key_value_heads * D, H, 4)
             + qbytes(H, c.num_attention_heads * D, 4) + 2 * qbytes(I, H, 4) + qbytes(H, I, 4))
    assert layer == 122_683_392 and 32 * layer + qbytes(c.vocab_size, H, 4) == 4_221_370_368
    c1 = named_config("llama-3.2-1b")
    l1 = (qbytes(2048, 2048, 4) * 2 + 2 * qbytes(512, 2048, 4) + 3 * qbytes(8192, 2048, 4))
    assert 16 * l1 + qbytes(c1.vocab_size, 2048, 4) == 695_107_584


def test_config_round_trip_and_rejects():
    c = tiny_config("qwen3_moe", 8)
    d = c.to_dict()
    assert d["quantization"] == {"group_size": 64, "bits": 8}
    assert ModelConfig.from_dict(json.loads(json.dumps(d))) == c
    with pytest.raises(ValueError):
        ModelConfig.from_dict(dict(d, model_type="gpt2"))
    with pytest.raises(ValueError):
        ModelConfig.from_dict(dict(d, quantization={"group_size": 32, "bits": 4}))


def test_per_module_bit_width_comes_from_the_tensor_shapes(tmp_path):
    """A checkpoint that keeps single modules at another width (per-path entries of
    config.json's quantization map): the map round-trips, the synthesised router tensor
    has the 8-bit shape, and a tensor's width is read off its own shapes."""
    from exo_amd.ops import QuantizedWeight
    c = tiny_config("qwen3_moe_router8")
    d = json.loads(json.dumps(c.to_dict()))
    assert d["quantization"]["bits"] == 4
    assert d["quantization"]["model.layers.1.mlp.gate"] == {"group_size": 64, "bits": 8}
    assert ModelConfig.from_dict(d) == c and c.bits_for("model.layers.0.mlp.gate") == 8
    assert c.bits_for("model.layers.0.self_attn.o_proj") == 4
    w = synth_weights(c, seed=2)
    H, E = c.hidden_size, c.num_experts
    assert w["model.layers.0.mlp.gate.weight"].shape == (E, H * 8 // 32)
    assert w["model.layers.0.self_attn.o_proj.weight"].shape[-1] == c.num_attention_heads * c.head_dim * 4 // 32
    gate = QuantizedWeight.from_tensors(*(w[f"model.layers.0.mlp.gate.{k}"] for k in ("weight", "scales", "biases")))
    o = QuantizedWeight.from_tensors(*(w[f"model.layers.0.self_attn.o_proj.{k}"] for k in ("weight", "scales", "biases")))
    ex = QuantizedWeight.from_tensors(*(w[f"model.layers.0.mlp.switch_mlp.up_proj.{k}"] for k in ("weight", "scales", "biases")))
    assert (gate.bits, gate.K, o.bits, ex.bits, ex.K) == (8, H, 4, 4, H)
    with pytest.raises(ValueError):  # 3 words per group of 64: no 4- or 8-bit layout
        QuantizedWeight.from_tensors(torch.zeros(4, 6, dtype=torch.int32),
                                     torch.zeros(4, 2, dtype=torch.bfloat16),
                                     torch.zeros(4, 2, dtype=torch.bfloat16), name="bad")


def test_shard_tensor_selection_rule():
    c = tiny_config("llama")
    assert layer_index_of("model.layers.12.self_attn.q_proj.weight") == 12
    assert layer_index_of("model.norm.weight") is None
    assert wanted("model.layers.1.mlp.up_proj.scales", c, 1, 2)
    assert not wanted("model.layers.0.mlp.up_proj.scales", c, 1, 2)
    assert wanted("model.embed_tokens.weight", c, 0, 1) and not wanted("model.embed_tokens.weight", c, 1, 3)
    assert wanted("lm_head.weight", c, 1, 3) and not wanted("lm_head.weight", c, 0, 2)
    tied = tiny_config("llama_tied_d128")
    assert wanted("model.embed_tokens.weight", tied, 1, 2)  # tied head lives in the embedding


@pytest.mark.parametrize("kind", ["llama", "qwen3_moe"])
def test_checkpoint_round_trip_and_progress(tmp_path, kind):
    cfg = tiny_config(kind)
    path = write_checkpoint(tmp_path / "m", cfg, seed=1)
    ref = synth_weights(cfg, seed=1)
    it = load_shard_weights(path, cfg, 0, cfg.num_hidden_layers, "cpu")
    prog = []
    try:
        while True:
            prog.append(next(it))
    except StopIteration as stop:
        got = stop.value
    assert prog == [(i + 1, cfg.num_hidden_layers) for i in range(cfg.num_hidden_layers)]
    assert set(got) == set(ref)
    for k in ref:
        assert got[k].dtype == ref[k].dtype and torch.equal(got[k], ref[k]), k
    # a middle shard gets only its own layer
    it = load_shard_weights(path, cfg, 1, 2, "cpu")
    try:
        while True:
            next(it)
    except StopIteration as stop:
        mid = stop.value
    is_last = cfg.num_hidden_layers == 2  # then the shard also owns final norm + head
    assert all(layer_index_of(k) == 1 or (is_last and layer_index_of(k) is None) for k in mid)
    assert len(mid) > 5 and not any(k.startswith("model.embed_tokens") for k in mid)
    # shapes follow the MLX layout
    w = got["model.layers.0.self_attn.q_proj.weight"]
    assert w.shape == (cfg.num_attention_heads * cfg.head_dim, cfg.hidden_size * cfg.bits // 32)
    if cfg.is_moe:
        assert got["model.layers.0.mlp.switch_mlp.down_proj.scales"].shape == (
            cfg.num_experts, cfg.hidden_size, cfg.moe_intermediate_size // 64)


def test_build_model_path_search_order(tmp_path, monkeypatch):
    ro, rw, default = tmp_path / "ro", tmp_path / "rw", tmp_path / "def"
    for d in (ro, rw, default):
        (d / "org--name").mkdir(parents=True)
    monkeypatch.setenv("EXO_MODELS_READ_ONLY_DIRS", str(ro))
    monkeypatch.setenv("EXO_MODELS_DIRS", str(rw))
    monkeypatch.setenv("EXO_DEFAULT_MODELS_DIR", str(default))
    assert build_model_path("org/name") == default / "org--name"  # nothing complete yet
    (rw / "org--name" / "config.json").write_text("{}")
    assert build_model_path("org/name") == rw / "org--name"
    (ro / "org--name" / "config.json").write_text("{}")
    assert build_model_path("org/name") == ro / "org--name"


def test_tokenizers():
    t = load_tokenizer("/nonexistent", 100)
    assert isinstance(t, IdTokenizer) and t.encode("5 17 205") == [5, 17, 5] and t.decode([3, 4]) == "3 4 "


# ------------------------------------------------------------------ sampling


def test_samplers():
    lp = torch.log_softmax(torch.tensor([[0.0, 3.0, 1.0, 2.5]]), -1)
    assert make_sampler(0.0)(lp).tolist() == [1]
    g = torch.Generator().manual_seed(0)
    draws = torch.stack([make_sampler(1.0, top_k=2, generator=g)(lp) for _ in range(200)])
    assert set(draws.flatten().tolist()) == {1, 3}
    draws = torch.stack([make_sampler(1.0, min_p=0.9, generator=g)(lp) for _ in range(50)])
    assert set(draws.flatten().tolist()) == {1}
    draws = torch.stack([make_sampler(1.0, top_p=0.5, generator=g)(lp) for _ in range(50)])
    assert set(draws.flatten().tolist()) == {1}
    banned = ban_token_ids([1])(torch.tensor([0]), torch.tensor([[0.0, 3.0, 1.0, 2.5]]))
    assert banned[0, 1] == -1e9 and torch.argmax(banned) == 3
    lpv, top = extract_top_logprobs(lp[0], None, 3, 2)
    assert [t.token for t in top] == ["1", "3", "2"] and abs(lpv - float(lp[0, 2])) < 1e-6


# ------------------------------------------------------------------ Engine event ordering


class FakeGen:
    """Port of the reference's FakeExoBatchGenerator
    (src/exo/worker/tests/unittests/test_runner/test_event_ordering.py:161-198)."""

    def __init__(self, fail_on_step=False):
        self.active, self.cancelled, self.next_uid = {}, [], 0
        self.fail_on_step = fail_on_step

    @property
    def has_work(self):
        return bool(self.active)

    def submit(self, task_params, prompt, on_prefill_progress=None,
               distributed_prompt_progress_callback=None, on_generation_token=None):
        if distributed_prompt_progress_callback:
            distributed_prompt_progress_callback()
        if on_prefill_progress:
            on_prefill_progress(len(prompt), len(prompt))
        uid = self.next_uid
        self.next_uid += 1
        self.active[uid] = [0, task_params.max_output_tokens or 3, on_generation_token]
        return uid

    def step(self):
        if self.fail_on_step:
            raise RuntimeError("device fault")
        out = []
        for uid, st in list(self.active.items()):
            st[0] += 1
            done = st[0] >= st[1]
            if st[2]:
                st[2]()
            out.append((uid, GenerationResponse(text="x", token=st[0], finish_reason="length" if done else None)))
            if done:
                del self.active[uid]
        return out

    def cancel(self, uids):
        self.cancelled += uids
        for u in uids:
            self.active.pop(u, None)

    def close(self):
        self.active.clear()


class _Sender:
    def __init__(self):
        self.sent = []

    def send(self, e):
        self.sent.append(e)


class _Receiver:
    def __init__(self):
        self.pending = []

    def collect(self):
        p, self.pending = self.pending, []
        return p


def _engine(**kw):
    s, r = _Sender(), _Receiver()
    gen = FakeGen(**kw)
    e = BatchGenerator(model=None, tokenizer=IdTokenizer(100), model_id="m", cancel_receiver=r,
                       event_sender=s, gen_factory=lambda: gen)
    return e, gen, s, r


def _task(tid, n=2, prompt=(1, 2, 3)):
    return GenerationTask(tid, "cmd-" + tid, TextGenerationTaskParams(model="m", input=list(prompt), max_output_tokens=n))


def test_engine_event_sequence():
    e, gen, s, _ = _engine()
    assert list(e.step()) == []
    e.submit(_task("a", 2))
    e.submit(_task("b", 3))
    ev = []
    for _ in range(4):
        ev += [(t, type(x).__name__, getattr(x, "finish_reason", None)) for t, x in e.step()]
    assert ev == [("a", "TokenChunk", None), ("b", "TokenChunk", None),
                  ("a", "TokenChunk", "length"), ("a", "FinishedResponse", None), ("b", "TokenChunk", None),
                  ("b", "TokenChunk", "length"), ("b", "FinishedResponse", None)]
    # prefill progress chunks were sent on the event channel, tagged with the command id
    assert [(c, type(x).__name__) for c, x in s.sent] == [("cmd-a", "PrefillProgressChunk"), ("cmd-b", "PrefillProgressChunk")]


def test_engine_concurrency_cap_and_cancellation():
    e, gen, _, r = _engine()
    for i in range(10):
        e.submit(_task(f"t{i}", 50))
    e.step()
    assert len(gen.active) == 8 and len(e._queue) == 2  # EXO_MAX_CONCURRENT_REQUESTS
    r.pending += ["t3", "unknown-task"]
    e.check_for_cancel_every = 1
    out = []
    for _ in range(3):
        out += [(t, type(x).__name__) for t, x in e.step()]
    assert ("t3", "CancelledResponse") in out and 3 in gen.cancelled
    r.pending.append("CANCEL_ALL_TASKS")
    out = []
    for _ in range(3):
        out += [(t, type(x).__name__) for t, x in e.step()]
    assert {t for t, k in out if k == "CancelledResponse"} >= {"t0", "t1", "t2"}
    assert not gen.has_work or len(gen.active) <= 2


def test_engine_prefill_cancel_and_errors():
    e, gen, s, r = _engine()
    r.pending.append("z")
    e._all_tasks["z"] = None
    e.submit(_task("z"))
    assert list(e.step()) == [] or True
    assert not gen.active  # PrefillCancelled swallowed, task dropped
    e2, gen2, s2, _ = _engine(fail_on_step=True)
    e2.submit(_task("q"))
    with pytest.raises(RuntimeError):
        e2.step()
    assert type(s2.sent[-1][1]).__name__ == "ErrorChunk" and s2.sent[-1][0] == "cmd-q"
    from exo_amd.disaggregated import PrefillRequest
    with pytest.raises(ValueError, match="exceeds the cache"):
        e2.serve_prefill(PrefillRequest("r", "m", list(range(e2.max_seq + 1)), 0), None)
    with pytest.raises(PrefillCancelled):
        raise PrefillCancelled()


# ---------------------------------------------------------------- KV prefix cache


@pytest.mark.parametrize("a,b,want", [
    ([1, 2, 3, 4, 5], [1, 2, 3, 4, 5], 5), ([1, 2, 3], [4, 5, 6], 0),
    ([1, 2, 3, 4, 5], [1, 2, 3, 7, 8], 3), ([1, 2, 3, 4, 5], [1, 2, 3], 3),
    ([1, 2, 3], [1, 2, 3, 4, 5], 3), ([1, 2, 3], [1, 5, 6], 1),
    ([], [1, 2, 3], 0), ([1, 2, 3], [], 0), ([], [], 0)])
def test_get_prefix_length(a, b, want):
    """The nine cases of the reference's TestGetPrefixLength
    (src/exo/worker/tests/unittests/test_mlx/test_kv_prefix_cache.py:33-77)."""
    from exo_amd.prefix_cache import get_prefix_length
    assert get_prefix_length(a, b) == want


def _filled_cache(n_tokens, seed, layers=2, batch=2, max_seq=32):
    from exo_amd.cache import ShardKVCache
    c = ShardKVCache(layers, batch, 2, 8, max_seq, "cpu")
    g = torch.Generator().manual_seed(seed)
    for t in c.k + c.v:
        t.copy_(torch.randn(t.shape, generator=g).bfloat16())
    c.offsets[0] = n_tokens
    c.sync_pos()
    return c


def test_prefix_cache_store_fetch_and_isolation():
    """Exact hit leaves the last token(s) to feed, a partial hit the unmatched suffix,
    and the stored entry is a detached copy (test_kv_prefix_cache.py:161-201,253-298)."""
    from exo_amd.prefix_cache import KVPrefixCache, cache_length
    pc = KVPrefixCache(None)
    assert len(pc.prompts) == 0 and len(pc.caches) == 0
    prompt = list(range(100, 112))                      # 12 tokens, 10 of them cached
    src = _filled_cache(10, seed=1)
    pc.add_kv_cache(prompt, src, row=0, prefill_tps=123.0)
    assert len(pc.prompts) == 1 and cache_length(pc.caches[0]) == 10
    want_k = src.k[1][0, :, :10].clone()
    src.k[1].zero_()                                    # the live cache moves on
    dst = _filled_cache(0, seed=2)
    _, remaining, idx, exact = pc.get_kv_cache(dst, prompt, row=1)
    assert idx == 0 and exact and remaining == prompt[-2:] and dst.offsets[1] == 10
    assert torch.equal(dst.k[1][1, :, :10], want_k)
    assert dst.pos.tolist() == [0, 10]
    # a stored entry longer than the query is cut back to len-1
    _, remaining, idx, exact = pc.get_kv_cache(dst, prompt[:6], row=1)
    assert exact and remaining == prompt[5:6] and dst.offsets[1] == 5
    # partial hit: 7 common tokens
    other = prompt[:7] + [1, 2, 3, 4]
    _, remaining, idx, exact = pc.get_kv_cache(dst, other, row=0)
    assert idx == 0 and not exact and remaining == [1, 2, 3, 4] and dst.offsets[0] == 7
    dst.k[0][0].zero_()                                 # generation mutates the row, not the entry
    assert cache_length(pc.caches[0]) == 10 and torch.equal(pc.caches[0].layers[1][0], want_k)
    # no common prefix: the row is reset
    _, remaining, idx, exact = pc.get_kv_cache(dst, [9, 9, 9], row=0)
    assert idx is None and not exact and remaining == [9, 9, 9] and dst.offsets[0] == 0
    pc.clear()
    assert len(pc.prompts) == 0 and len(pc.caches) == 0


def test_prefix_cache_update_in_place_rule(monkeypatch):
    """generator/batch_generate.py:493-535: a hit of >= min length and >= half the prompt
    replaces the matched entry, anything else adds one."""
    import exo_amd.prefix_cache as P
    from exo_amd.prefix_cache import KVPrefixCache, cache_length, save_prefix_cache
    monkeypatch.setattr(P, "get_memory_used_percentage", lambda device=None: 0.1)
    monkeypatch.setenv("EXO_MEMORY_THRESHOLD", "0.9")
    pc = KVPrefixCache(None)
    c = _filled_cache(10, seed=3)
    save_prefix_cache(pc, list(range(12)), c, 0, 0, None, min_prefix_hit_length=4)
    c.offsets[0] = 18
    save_prefix_cache(pc, list(range(20)), c, 0, 10, 0, min_prefix_hit_length=4)
    assert len(pc.prompts) == 1 and cache_length(pc.caches[0]) == 18 and len(pc.prompts[0]) == 20
    save_prefix_cache(pc, list(range(3)) + [77] * 9, c, 0, 3, 0, min_prefix_hit_length=4)
    assert len(pc.prompts) == 2
    save_prefix_cache(pc, list(range(5)) + [78] * 9, c, 0, 5, 0, min_prefix_hit_length=4)
    assert len(pc.prompts) == 3                          # long enough, but under half the prompt


def test_prefix_cache_evicts_lru_under_memory_pressure(monkeypatch):
    """test_kv_prefix_cache.py:534-602: with usage pinned above the threshold every old
    entry goes, least recently used first, and only the new one survives."""
    import exo_amd.prefix_cache as P
    monkeypatch.setenv("EXO_MEMORY_THRESHOLD", "0.9")
    usage = {"v": 0.5}
    monkeypatch.setattr(P, "get_memory_used_percentage", lambda device=None: usage["v"])
    pc = P.KVPrefixCache(None)
    for i in range(3):
        pc.add_kv_cache([i, i, i], _filled_cache(3, seed=i))
        pc._last_used[i] = float(i)
    pc._last_used[2] = 100.0
    assert len(pc.prompts) == 3
    order = []
    usage["v"] = 0.95
    # record which prompts leave, in order
    class Spy(list):
        def pop(self, i):
            order.append(int(self[i][0]))
            return super().pop(i)
    pc.prompts = Spy(pc.prompts)
    pc.add_kv_cache([7, 7, 7, 7], _filled_cache(4, seed=9))
    assert order == [0, 1, 2]
    assert len(pc.prompts) == 1 and P.get_prefix_length(pc.prompts[0], [7, 7, 7, 7]) == 4


def test_logits_processors():
    """Penalties as the reference requests them (generator/generate.py:599-612), checked
    on values worked by hand."""
    from exo_amd.generate import make_logits_processors, processors_for
    logits = torch.tensor([[2.0, -2.0, 1.0, 0.5, -1.0]])
    assert make_logits_processors() == []
    assert make_logits_processors(repetition_penalty=0.0, presence_penalty=0.0, frequency_penalty=None) == []
    (rep,) = make_logits_processors(repetition_penalty=2.0, repetition_context_size=3)
    # context = last three tokens {1, 0, 1}; token 4 is older than the window
    out = rep(torch.tensor([4, 1, 0, 1]), logits)
    assert out.tolist() == [[1.0, -4.0, 1.0, 0.5, -1.0]] and logits[0, 0] == 2.0  # input untouched
    (pres,) = make_logits_processors(presence_penalty=0.5)
    assert pres(torch.tensor([2, 2, 3]), logits).tolist() == [[2.0, -2.0, 0.5, 0.0, -1.0]]
    (freq,) = make_logits_processors(frequency_penalty=0.25)
    assert freq(torch.tensor([2, 2, 3]), logits).tolist() == [[2.0, -2.0, 0.5, 0.25, -1.0]]
    assert rep(torch.tensor([], dtype=torch.int64), logits) is logits
    with pytest.raises(ValueError):
        make_logits_processors(repetition_penalty=-1.0)
    p = TextGenerationTaskParams(model="m", bench=True, repetition_penalty=1.1, frequency_penalty=0.1)
    procs = processors_for(p, [3])
    assert len(procs) == 3 and procs[0](None, logits)[0, 3] == -1e9
    assert processors_for(TextGenerationTaskParams(model="m", bench=True), []) == []


# ------------------------------------------------------------------ detokeniser, token stream


def _byte_level_tokenizer():
    """A byte-level BPE without merges: one id per UTF-8 byte, decoded by the ByteLevel
    decoder - the smallest tokenizer in which a character is split over several ids."""
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers
    from exo_amd.tokenizer import HFTokenizer
    vocab = {ch: i for i, ch in enumerate(sorted(pre_tokenizers.ByteLevel.alphabet()))}
    tok = Tokenizer(models.BPE(vocab=vocab, merges=[]))
    tok.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tok.decoder = decoders.ByteLevel()
    return HFTokenizer(tok, [])


def test_streaming_detokenizer_holds_back_incomplete_characters():
    from exo_amd.tokenizer import StreamingDetokenizer
    t = _byte_level_tokenizer()
    text = "h\u00e9llo \u4e16\u754c \U0001f600!"
    ids = t.encode(text)
    assert len(ids) > len(text)                       # multi-byte characters span ids
    assert "\ufffd" in "".join(t.decode([i]) for i in ids)  # one by one they would be garbled
    d = StreamingDetokenizer(t)
    segs = []
    for i in ids:
        d.add_token(i)
        segs.append(d.last_segment)
    d.finalize()
    segs.append(d.last_segment)
    assert "".join(segs) == text and not any("\ufffd" in s for s in segs)
    assert segs[1] == "" and segs[2] == "\u00e9"     # the first byte of the e-acute is held back
    # a sequence cut inside a character: finalize releases what there is
    d = StreamingDetokenizer(t)
    for i in ids[:2]:
        d.add_token(i)
    assert d.last_segment == "h"
    d.finalize()
    assert d.last_segment == "\ufffd"


def test_token_stream_finish_reasons_and_stop_sequences():
    from exo_amd.generate import TokenStream
    t = _byte_level_tokenizer()
    ids = t.encode("ab\u00e9cd STOP tail")
    task = TextGenerationTaskParams(model="m", stop=["STOP"])
    ts = TokenStream(t, task, [], 100, 5, 10.0, "none", "cpu")
    out = []
    with pytest.MonkeyPatch.context() as mp:
        mp.setattr(torch.cuda, "max_memory_allocated", lambda d=None: 0)
        for k, i in enumerate(ids):
            r = ts.push(i, float(k))
            out.append(r)
            if r.finish_reason:
                break
    # as in the reference (batch_generate.py:371-385) only the chunk that completes the stop
    # sequence is trimmed: the characters of it that earlier chunks carried are already out
    assert "".join(r.text for r in out) == "ab\u00e9cd STO" and out[-1].finish_reason == "stop"
    assert out[-1].text == "" and out[-1].token == ids[len(out) - 1]
    assert out[-1].usage.completion_tokens == len(out) and out[-1].stats.generation_tokens == len(out)
    assert out[-1].stats.generation_tps == pytest.approx((len(out) - 1) / (len(out) - 1.0))
    # EOS: the token is not detokenised; length: the last token is
    eos = t.encode("z")[0]
    with pytest.MonkeyPatch.context() as mp:
        mp.setattr(torch.cuda, "max_memory_allocated", lambda d=None: 0)
        ts = TokenStream(t, TextGenerationTaskParams(model="m"), [eos], 100, 5, 10.0, "none", "cpu")
        assert ts.push(t.encode("q")[0], 0.0).text == "q"
        r = ts.push(eos, 1.0)
        assert r.finish_reason == "stop" and r.text == ""
        ts = TokenStream(t, TextGenerationTaskParams(model="m", bench=True), [eos], 2, 5, 10.0, "none", "cpu")
        assert ts.push(eos, 0.0).finish_reason is None   # bench mode: EOS does not stop
        r = ts.push(t.encode("q")[0], 1.0)
        assert r.finish_reason == "length" and r.text == "q"
        items = ts.top_items([t.encode("a")[0], -1, t.encode("b")[0]], [-0.5, float("nan"), -1.5], 5)
        assert [(i.token, i.logprob) for i in items] == [("a", -0.5), ("b", -1.5)]
