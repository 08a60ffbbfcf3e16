#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a Llama-3.1-8B-architecture model on MLX
4-bit g64 weights, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one decoded token: the full shard forward (32 layers + head) as a HIP
graph replay at a context of about 2048 tokens, weights and KV cache resident in HBM,
greedy sampling on the device.  Prints ONE JSON line: decode tok/s (`value`), the
roofline of the dominant kernel (the fused dequant-GEMV, measured live with HIP events)
and the CPU oracle timed on this box's host cores (`cpu_baseline`, reported only).

Weights are synthetic (N(0,0.02) -> bf16 -> mx.quantize-style affine 4-bit g64), the
prompt is 2048 uniform random token ids; see `data` in the output.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--config", default="llama-3.1-8b")
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="debug: truncate the model")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-engine", action="store_true", help="skip the run through the Engine")
    ap.add_argument("--batch", type=int, default=1, help="sequences decoded together (1..16)")
    ap.add_argument("--shard-layers", type=int, default=None,
                    help="run layers [0, n) as a first pipeline shard (output: hidden state)")
    ap.add_argument("--pmc-copy", action="store_true",
                    help="also launch one plain 256 MiB copy kernel: the known-size dispatch that "
                         "calibrates FETCH_SIZE / WRITE_SIZE in a rocprofv3 --pmc pass")
    ap.add_argument("--workload", default="decode", choices=["decode", "qmatmul_sweep"],
                    help="decode (default, the headline) or the quantised-matmul shape sweep")
    return ap.parse_args()


def qbytes(n: int, k: int, bits: int) -> int:
    return n * k * bits // 8 + n * (k // 64) * 4


def measure_kernels(model, torch, reps: int = 20):
    """Per-kernel HBM roofline of the GEMV launches of one decode step.  Each group of
    same-shaped launches (one per layer, distinct weights, 4.2 GB in total so nothing
    is served from cache) is captured into a HIP graph and timed with events on the
    launch stream; average launch duration = elapsed / launches."""
    from exo_amd import ops
    from exo_amd.model import capture_graph

    c = model.cfg
    dev = model.device
    H, D = c.hidden_size, c.head_dim
    Hq, Hkv, I = c.num_attention_heads, c.num_key_value_heads, c.intermediate_size
    bf = dict(dtype=torch.bfloat16, device=dev)
    xh = torch.randn(1, H, device=dev).to(torch.bfloat16)
    xa = torch.randn(1, Hq * D, device=dev).to(torch.bfloat16)
    xi = torch.randn(1, I, device=dev).to(torch.bfloat16)
    y_qkv = torch.empty(1, (Hq + 2 * Hkv) * D, **bf)
    y_h = torch.empty(1, H, **bf)
    y_i = torch.empty(1, I, **bf)
    y_v = torch.empty(1, c.vocab_size, **bf)
    def kernel_name(nmat, K):  # template arguments <bits, rows of x, matrices, 1 KiB units per row, self-routing>
        return "qmv_rows_kernel<%d,1,%d,%d,false>" % (c.bits, nmat, K * c.bits // 8 // 1024)

    nw, eps = torch.ones(H, **bf), c.rms_norm_eps

    def timed_rounds(graph, launches, rounds=5):
        """Average launch duration in us: `rounds` timed regions of `reps` replays each,
        the median region (the first one after a capture runs 2-3 % slow)."""
        avg = []
        for _ in range(rounds):
            st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            st.record()
            for _ in range(reps):
                graph.replay()
            en.record()
            torch.cuda.synchronize()
            avg.append(st.elapsed_time(en) * 1e3 / (reps * launches))
        return sorted(avg)[len(avg) // 2]

    groups = {
        "norm_gate_up_swiglu": (lambda L: ops.qmv_swiglu(xh, L.gate, L.up, out=y_i, norm_weight=nw, eps=eps),
                                2 * qbytes(I, H, c.bits) + 2 * (2 * H + I), kernel_name(2, H)),
        "down_residual": (lambda L: ops.quantized_matmul(xi, L.down, residual=y_h, out=y_h),
                          qbytes(H, I, c.bits) + 2 * (I + 2 * H), kernel_name(1, I)),
        "norm_qkv": (lambda L: ops.quantized_matmul(xh, L.qkv, out=y_qkv, norm_weight=nw, eps=eps),
                     qbytes((Hq + 2 * Hkv) * D, H, c.bits) + 2 * (2 * H + (Hq + 2 * Hkv) * D),
                     kernel_name(1, H)),
        "o_residual": (lambda L: ops.quantized_matmul(xa, L.o, residual=y_h, out=y_h),
                       qbytes(H, Hq * D, c.bits) + 2 * (Hq * D + 2 * H), kernel_name(1, Hq * D)),
    }
    out = []
    for name, (fn, nbytes, kname) in groups.items():
        for L in model.layers:  # warm-up (also sets kernel attributes outside capture)
            fn(L)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with capture_graph(g):
            for L in model.layers:
                fn(L)
        g.replay()
        torch.cuda.synchronize()
        us = timed_rounds(g, len(model.layers))
        out.append(dict(name=name, kernel=kname, launches_per_token=len(model.layers),
                        bytes_per_launch=nbytes, avg_us=us, GBps=nbytes / us * 1e-3))
    # lm_head: once per token, with 4 GB of layer weights streamed since its last use, so
    # the 256 MB last-level cache holds none of it when it runs.  Re-reading ONE matrix back to
    # back would find most of it there (5.0 against 4.7 TB/s measured), so the launches of the
    # timed graph rotate over four copies of the matrix (1.2 GB).
    from exo_amd.ops import QuantizedWeight
    hd = model.lm_head
    heads = [hd] + [QuantizedWeight(hd.weight.clone(), hd.scales.clone(), hd.biases.clone(), hd.bits)
                    for _ in range(3)]
    for q in heads:
        ops.quantized_matmul(xh, q, out=y_v, norm_weight=nw, eps=eps)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with capture_graph(g):
        for q in heads:
            ops.quantized_matmul(xh, q, out=y_v, norm_weight=nw, eps=eps)
    g.replay()
    torch.cuda.synchronize()
    us = timed_rounds(g, len(heads))
    del heads
    nbytes = qbytes(c.vocab_size, H, c.bits) + 2 * (2 * H + c.vocab_size)
    out.append(dict(name="norm_lm_head", kernel=kernel_name(1, H), launches_per_token=1,
                    bytes_per_launch=nbytes, avg_us=us, GBps=nbytes / us * 1e-3))
    return out


def cpu_baseline(model, torch, seconds: float, context: int):
    """The CPU oracle (C restatement of the quantised matmul + numpy ops) timed on this
    host: one decode token of the same architecture at the same context length.
    Bounded sample: 2 layers + head are run and the layer time is scaled to the full
    depth."""
    from oracle import cref
    from oracle import models as OM

    c = model.cfg
    n_sample = min(2, len(model.layers))

    def to_np(t):
        t = t.detach().cpu().contiguous()
        if t.dtype == torch.int32:
            return t.numpy().view(np.uint32)
        return t.view(torch.int16).numpy().view(np.uint16)

    w = {}

    def put(prefix, q):
        w[prefix + ".weight"], w[prefix + ".scales"], w[prefix + ".biases"] = (
            to_np(q.weight), to_np(q.scales), to_np(q.biases))

    Hq, Hkv, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
    for i in range(n_sample):
        L = model.layers[i]
        p = f"model.layers.{i}."
        nq, nk = Hq * D, Hkv * D
        put(p + "self_attn.q_proj", L.qkv[0:nq])
        put(p + "self_attn.k_proj", L.qkv[nq : nq + nk])
        put(p + "self_attn.v_proj", L.qkv[nq + nk : nq + 2 * nk])
        put(p + "self_attn.o_proj", L.o)
        put(p + "mlp.gate_proj", L.gate)
        put(p + "mlp.up_proj", L.up)
        put(p + "mlp.down_proj", L.down)
        w[p + "input_layernorm.weight"] = to_np(L.in_norm)
        w[p + "post_attention_layernorm.weight"] = to_np(L.post_norm)
    put("model.embed_tokens", model.embed_tokens)
    put("lm_head", model.lm_head)
    w["model.norm.weight"] = to_np(model.norm)
    ocfg = OM.Config(model_type=c.model_type, hidden_size=c.hidden_size, num_hidden_layers=n_sample,
                     num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D,
                     intermediate_size=c.intermediate_size, vocab_size=c.vocab_size,
                     rms_norm_eps=c.rms_norm_eps, rope_theta=c.rope_theta, rope_scaling=c.rope_scaling,
                     tie_word_embeddings=False, group_size=64, bits=c.bits)
    om = OM.ShardModel(ocfg, w, use_c=True)
    rng = np.random.default_rng(0)
    cache = OM.make_kv_cache(n_sample)
    from oracle.affine import bf16_round

    for kv in cache:  # a context of `context` cached tokens (synthetic K/V)
        kv.k = bf16_round(rng.standard_normal((1, Hkv, context, D)).astype(np.float32))
        kv.v = bf16_round(rng.standard_normal((1, Hkv, context, D)).astype(np.float32))
        kv.offset = context
    tok = np.array([[1]])
    om(tok, cache)  # warm-up
    for kv in cache:
        kv.trim(1)
    t_full, n_full, t0 = 0.0, 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds * 0.7 or n_full < 2:
        a = time.perf_counter()
        om(tok, cache)
        t_full += time.perf_counter() - a
        n_full += 1
        for kv in cache:
            kv.trim(1)
    x = bf16_round(rng.standard_normal((1, c.hidden_size)).astype(np.float32))
    t_head, n_head, t0 = 0.0, 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds * 0.3 or n_head < 2:
        a = time.perf_counter()
        om.linear(x, "lm_head")
        t_head += time.perf_counter() - a
        n_head += 1
    t_full /= n_full
    t_head /= n_head
    t_layer = max(t_full - t_head, 1e-9) / n_sample
    t_token = t_layer * c.num_hidden_layers + t_head
    import importlib.util
    have = {m: importlib.util.find_spec(m) is not None for m in ("mlx", "mlx_lm")}
    mlx_note = ("mlx_lm: unavailable on this box (importlib finds neither mlx nor mlx_lm), so the baseline "
                "is this repository's own CPU restatement; " if not all(have.values()) else
                "mlx / mlx_lm are importable here but are not driven by this build; ")
    return dict(value=1.0 / t_token, unit="tok/s", cores=cref.num_threads(), kind="port",
                mlx_importable=have,
                sample=(mlx_note +
                        f"{n_full} decode steps of {n_sample} layers + lm_head at context {context} "
                        f"(layer {t_layer * 1e3:.1f} ms, head {t_head * 1e3:.1f} ms), layer time "
                        f"scaled to {c.num_hidden_layers} layers; oracle/qmm_ref.c with OpenMP + numpy"),
                host_cpus=os.cpu_count(), affinity=len(os.sched_getaffinity(0)))


PMC_SUMMARY = "profiles/decode_llama8b_4bit_bs1_pmc_traffic.md"


def pmc_traffic(launch: str):
    """HBM bytes per launch of one GEMV group as measured by the committed
    `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` passes of this command (a text summary
    under profiles/; counters cannot be read from inside the process).  Returns (bytes,
    where the figure comes from) or (None, None): it is a recorded measurement of that
    earlier run, not of this one."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), PMC_SUMMARY)
    val, commit = None, "unknown"
    try:
        with open(path) as fh:
            for line in fh:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == launch:
                    val = int(parts[2])
                if len(parts) >= 2 and parts[0] == "measured_at_commit":
                    commit = parts[1]
    except OSError:
        pass
    if val is None:
        return None, None
    return val, f"{PMC_SUMMARY} (rocprofv3 --pmc passes recorded at commit {commit}; not re-measured by this run)"


def engine_rates(model, cfg, args, torch):
    """The same workload through the Engine the runner drives (BatchGenerator.step(): queue,
    prefill, double-buffered graph replays with device sampling, detokeniser, chunks):
    `generation_tps` as the reference defines it, (n-1)/(t_last - t_first) per request
    (src/exo/worker/engines/mlx/generator/batch_generate.py:418-426), summed over the
    requests of the batch; once greedy, once with the reference's default sampler
    (temperature 0.7, min-p 0.05)."""
    from exo_amd.engine import BatchGenerator
    from exo_amd.types import GenerationTask, TextGenerationTaskParams

    B, K = args.batch, args.steps + args.warmup
    eng = BatchGenerator(model=model, tokenizer=None, model_id=args.config,
                         max_seq=args.prompt + K + 72)
    g = torch.Generator().manual_seed(1234)
    prompts = [torch.randint(0, cfg.vocab_size, (args.prompt,), generator=g).tolist() for _ in range(B)]
    res = {}
    for label, temp in (("engine_tok_s", 0.0), ("engine_tok_s_sampled", 0.7)):
        for i, p in enumerate(prompts):
            eng.submit(GenerationTask(f"{label}-{i}", f"cmd-{i}", TextGenerationTaskParams(
                model=args.config, input=p, max_output_tokens=K, temperature=temp, bench=True)))
        tps, n_done = 0.0, 0
        while n_done < B:
            for _tid, ev in eng.step():
                st = getattr(ev, "stats", None)
                if st is not None:
                    tps += st.generation_tps
                    n_done += 1
        res[label] = tps
    res["engine_note"] = (f"{B} request(s) of {K} tokens through BatchGenerator.step(); generation_tps per "
                          "request as the reference defines it, summed")
    eng.close()
    return res


def active_token_bytes(model, cfg, ctx: int, batch: int) -> int:
    """Algorithmic HBM bytes of one decode step: every weight the step multiplies by (for
    MoE layers the router plus top-k experts per sequence, at most all experts) once,
    plus the K/V read of every sequence."""
    n = 0
    for L in model.layers:
        n += L.qkv.nbytes + L.o.nbytes
        if cfg.is_moe:
            per_expert = (L.gate.nbytes + L.up.nbytes + L.down.nbytes) // cfg.num_experts
            n += L.router.nbytes + per_expert * min(cfg.num_experts, cfg.num_experts_per_tok * batch)
        else:
            n += L.gate.nbytes + L.up.nbytes + L.down.nbytes
    if model.lm_head is not None:
        n += model.lm_head.nbytes
    kv = 2 * len(model.layers) * cfg.num_key_value_heads * cfg.head_dim * ctx * 2 * batch
    return n + kv


def qmatmul_sweep(args):
    """configs[1] of the baseline: y = x @ dq(W)^T over the listed (N, K), bits and M.
    Weight copies rotate so that nothing is served from cache; one HIP-graph replay holds
    one launch per copy; events on the launch stream give the average launch duration."""
    import torch

    from exo_amd import native, ops
    from exo_amd.model import capture_graph
    from exo_amd.ops import QuantizedWeight

    native.load()
    dev = torch.device("cuda:0")
    shapes = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]
    rows = []
    g = torch.Generator(device=dev).manual_seed(4321)
    for bits in (4, 8):
        for (N, K) in shapes:
            wbytes = qbytes(N, K, bits)
            copies = max(4, min(32, int(1.5e9 // wbytes) + 1))
            ws = []
            for _ in range(copies):
                w = torch.randint(-2**31, 2**31 - 1, (N, K * bits // 32), dtype=torch.int32, device=dev, generator=g)
                sc = (torch.rand(N, K // 64, device=dev, generator=g) * 0.01).bfloat16()
                bi = (torch.rand(N, K // 64, device=dev, generator=g) * -0.08).bfloat16()
                ws.append(QuantizedWeight(w, sc, bi, bits))
            for M in (1, 4, 16, 32, 64, 128, 2048):
                if M >= 128 and N * M * 2 > (1 << 30):
                    continue  # 128256 x 2048 outputs: not a shape the models produce
                x = torch.randn(M, K, device=dev, generator=g).bfloat16()
                y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                fns = [(lambda q=q: ops.quantized_matmul(x, q, out=y)) for q in ws]
                for f in fns:
                    f()
                torch.cuda.synchronize()
                gr = torch.cuda.CUDAGraph()
                with capture_graph(gr):
                    for f in fns:
                        f()
                gr.replay()
                torch.cuda.synchronize()
                reps = 10 if M <= 128 else 3
                st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                st.record()
                for _ in range(reps):
                    gr.replay()
                en.record()
                torch.cuda.synchronize()
                us = st.elapsed_time(en) * 1e3 / (reps * copies)
                nbytes = wbytes + 2 * M * (K + N)
                flops = 2.0 * M * N * K
                rows.append(dict(bits=bits, N=N, K=K, M=M, us=round(us, 2), GBps=round(nbytes / us * 1e-3, 1),
                                 frac_hbm=round(nbytes / us * 1e-3 / 8000.0, 3),
                                 TFLOPs=round(flops / us * 1e-6, 1), frac_mfma=round(flops / us * 1e-6 / 2500.0, 3)))
                print(f"[sweep] b{bits} N={N} K={K} M={M}: {us:.1f} us", file=sys.stderr, flush=True)
            del ws
    best = max((r for r in rows if r["M"] == 1), key=lambda r: r["GBps"])
    dom = next(r for r in rows if (r["bits"], r["N"], r["K"], r["M"]) == (4, 14336, 4096, 1))
    print(json.dumps({
        "metric": "qmatmul HBM GB/s (% of 8 TB/s) over the shape sweep", "value": dom["GBps"], "unit": "GB/s",
        "n_gpus": 1, "steps": len(rows), "warmup": 1, "ms_per_step": dom["us"] * 1e-3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: quantised matmul sweep, bits {4,8} x 5 shapes x M {1,4,16,32,64,128,2048}; "
                               "value = 4-bit 14336x4096 at M=1"},
        "roofline": {"bound": "hbm", "achieved": dom["GBps"], "peak": 8000.0, "unit": "GB/s",
                     "frac": dom["GBps"] / 8000.0, "traffic": None},
        "best_M1": best, "rows": rows, "cpu_baseline": None}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (per-shard forward); --gpus {args.gpus} is not "
              "supported: every figure here is one GPU's throughput.",
              file=sys.stderr)
        sys.exit(2)
    if args.workload == "qmatmul_sweep":
        return qmatmul_sweep(args)
    import torch

    from exo_amd import native
    from exo_amd.config import named_config
    from exo_amd.generate import prefill
    from exo_amd.model import ShardModel
    from exo_amd.synth import synth_weights

    native.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cfg = named_config(args.config)
    if args.layers:
        cfg.num_hidden_layers = args.layers
    B = args.batch
    if not 1 <= B <= 16:
        sys.exit("bench.py: --batch must be 1..16")
    end = args.shard_layers or cfg.num_hidden_layers
    t0 = time.perf_counter()
    weights = synth_weights(cfg, 0, end, seed=0, device=dev)
    model = ShardModel(cfg, weights, 0, end, device=dev)
    del weights
    torch.cuda.synchronize()
    t_build = time.perf_counter() - t0
    print(f"[bench] weights ready in {t_build:.1f} s", file=sys.stderr, flush=True)

    g = torch.Generator().manual_seed(1234)
    K, W = args.steps, args.warmup
    cache = model.make_cache(B, args.prompt + K + W + 64)

    # prefill with the reference's protocol (one sequence at a time, as its batch engine
    # does), then the last-but-one prompt token of every sequence as a GEMV step
    tps_prefill, n_prefill, last = 0.0, 0, []
    for row in range(B):
        prompt = torch.randint(0, cfg.vocab_size, (args.prompt,), generator=g).tolist()
        # untimed warm-up of the same call (buffers, code objects, the captured single-token
        # step of this cache row, as in an engine whose cache outlives its requests), then rewind
        prefill(model, prompt[:-1], cache, row=row, faithful_extra_steps=model.is_last, graph_steps=True)
        cache.reset(rows=range(row, row + 1))
        tps, n = prefill(model, prompt[:-1], cache, row=row,
                         faithful_extra_steps=model.is_last, graph_steps=True)
        tps_prefill, n_prefill = tps, n
        model(torch.tensor([[prompt[-2]]], dtype=torch.int32), cache, logits="none",
              rows=slice(row, row + 1))
        last.append(prompt[-1])
        print(f"[bench] row {row}: prefill {n} tokens at {tps:.0f} tok/s", file=sys.stderr, flush=True)
    bufs = model._buffers(B, 1)
    bufs.tokens.copy_(torch.tensor(last, dtype=torch.int32))

    def step():
        return model.decode_step(cache, B, use_graph=not args.no_graph, feedback=model.is_last)

    for _ in range(W):
        step()
    torch.cuda.synchronize()
    ctx0 = cache[0].offset
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    last_token = int(bufs.next_token[0]) if model.is_last else None
    tok_s = B * K / dt
    token_bytes = active_token_bytes(model, cfg, ctx0, B)

    if args.pmc_copy:
        # plain 16-byte-per-lane copy of 256 MiB (the KV re-layout kernel with one head is
        # exactly that): reads 256 MiB, writes 256 MiB
        from exo_amd import ops
        a = torch.zeros(1, 1 << 20, 128, dtype=torch.bfloat16, device=dev)
        ops.kv_export_nhd(a, 0, 1 << 20)
        torch.cuda.synchronize()
        del a

    headline = (args.config == "llama-3.1-8b" and B == 1 and model.is_last and not cfg.is_moe)
    if not cfg.is_moe and model.is_last and B == 1:
        # (a counter pass serialises every dispatch: one replay per region is plenty there)
        kernels = measure_kernels(model, torch, reps=1 if args.pmc_copy else 20)
        for k in kernels:
            k["frac_of_8TBps"] = k["GBps"] / 8000.0
            k["us_per_token"] = k["avg_us"] * k["launches_per_token"]
        dom = max(kernels, key=lambda k: k["us_per_token"])
        traffic, traffic_src = pmc_traffic(dom["name"]) if headline else (None, None)
        gemv_us = sum(k["us_per_token"] for k in kernels)
        gemv_bytes = sum(k["bytes_per_launch"] * k["launches_per_token"] for k in kernels)
        roofline = dict(bound="hbm", achieved=dom["GBps"], peak=8000.0, unit="GB/s",
                        frac=dom["GBps"] / 8000.0,
                        traffic=traffic, traffic_source=traffic_src, kernel=dom["kernel"],
                        launch=dom["name"], avg_us=dom["avg_us"], bytes_per_launch=dom["bytes_per_launch"],
                        all_gemv_GBps=gemv_bytes / gemv_us * 1e-3, all_gemv_us_per_token=gemv_us)
    else:
        # no single dominant launch is isolated here: the whole step against its bytes
        kernels = None
        gbps = token_bytes / (dt / K) * 1e-9
        roofline = dict(bound="hbm", achieved=gbps, peak=8000.0, unit="GB/s", frac=gbps / 8000.0,
                        traffic=None, kernel="all launches of one decode step",
                        bytes_per_launch=token_bytes, avg_us=dt / K * 1e6)

    engine = None
    if model.is_last and not args.no_engine:
        engine = engine_rates(model, cfg, args, torch)

    what = {"llama-3.2-1b": "configs[0]", "llama-3.1-8b": "configs[2]", "qwen3-30b-a3b": "configs[3]",
            "qwen3-235b-a22b": "configs[4]"}.get(args.config, "custom")
    shard = "" if model.is_last else f", pipeline shard of layers [0,{end}) (output: hidden state)"
    out = {
        "metric": ("decode tok/s + qmatmul HBM GB/s (% peak), Llama-3.1-8B 4-bit g64 bs1" if headline
                   else f"decode tok/s, {args.config} {cfg.bits}-bit g64 batch {B}"),
        "value": tok_s, "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": dt / K * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{what}: {args.config} architecture, MLX affine {cfg.bits}-bit g64, "
                               f"random prompt of {args.prompt} tokens, greedy decode, batch {B}{shard}",
                   "layers": len(model.layers), "context_at_start": ctx0, "hip_graph": not args.no_graph},
        "roofline": roofline,
        "prefill_tok_s": tps_prefill, "prefill_tokens": n_prefill,
        "token_bytes": token_bytes, "effective_GBps": token_bytes * (K / dt) * 1e-9,
        "kernels": kernels, "build_s": t_build, "last_token": last_token,
    }
    if engine is not None:
        out.update(engine)
    if not args.no_cpu_baseline and kernels is not None:
        out["cpu_baseline"] = cpu_baseline(model, torch, args.cpu_seconds, ctx0)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
