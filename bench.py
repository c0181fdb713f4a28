#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen3-8B layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  `value` is decoded tokens per second at batch 8 and the context
length the configuration names (the last timed step ends at that length); a "step" is one
decode step through the engine's own step function (mixed-batch path, paged cache,
kernels) followed by greedy sampling on the GPU, launched as the engine launches its steps:
the sampled ids reach the next step on the device and travel to the host beside it, so the
host prepares a step while the GPU runs the one before (the timed steps lie between two
synchronizations, and all of their tokens have reached the host at the second).  Beside it: the prefill of one
2,048-token prompt, the decode step's bandwidth roofline, decode at batch 1 and 64 (`points`,
and each one's own roofline in `points_roofline`), and decode at batch 8 with four times the
context (`further`).

`--product M,N,K[,slices[,shape]]` times one bfloat16 product alone, in the hand-written many-row
tiled kernel and in the vendor library.

`--peaks` adds what this card itself reaches (a read-only stream, one large square product) and
the fractions of those, beside the fractions of the published peaks that the line always has.

Data is synthetic: weights are seeded random values of the architecture's shapes made
on the GPU, token ids are seeded uniform, and the cache contents the decode steps read
are random values (decode timing does not depend on what the cache holds).

`--workload serve14b` and `--workload long32b` instead run the two serving workloads of the
larger configurations through the whole engine (scheduler, chunked prefill, continuous
batching, greedy sampling) and print their own JSON line: total generated tokens per second.
`--workload many06b` is the one run the reference publishes a figure for (Qwen3-0.6B, 256
concurrent requests, 1,024 new tokens each); its line carries the ratio to that figure, which
was measured on other hardware.  `--workload many8b` is 192 concurrent requests (prompts of 64
to 512 tokens, 256 new tokens each) at Qwen3-8B sizes: decode steps of 129 to 256 rows.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], hidden_size=4096, intermediate_size=12288,
    num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False,
    max_position_embeddings=40960, hidden_act="silu")
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40,
                 num_attention_heads=40, num_key_value_heads=8)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64,
                 num_attention_heads=64, num_key_value_heads=8)
QWEN3_0_6B = dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
                  num_attention_heads=16, num_key_value_heads=8, tie_word_embeddings=True)
# the serving workloads of the two larger configurations, and the one the reference publishes a
# figure for: Qwen3-0.6B, 256 concurrent requests of 16 prompt tokens, 1,024 new tokens each
# (/root/reference/python/ReadMe.md:2-13: 10,944.62 generated tokens/s on a CUDA GPU)
WORKLOADS = {
    "many06b": dict(model=QWEN3_0_6B, name="Qwen3-0.6B layer sizes", requests=256, prompt=(16, 16), new_tokens=1024,
                    chunk=2048, max_model_len=1088, reference_tok_s=10944.62),
    "serve14b": dict(model=QWEN3_14B, name="Qwen3-14B layer sizes", requests=64, prompt=(128, 2048), new_tokens=256,
                     chunk=2048, max_model_len=2304),
    "many8b": dict(model=QWEN3_8B, name="Qwen3-8B layer sizes", requests=192, prompt=(64, 512), new_tokens=256,
                   chunk=2048, max_model_len=768),
    "long32b": dict(model=QWEN3_32B, name="Qwen3-32B layer sizes", requests=16, prompt=(8192, 8192), new_tokens=512,
                    chunk=2048, max_model_len=8704),
}
MODELS = {"0.6b": QWEN3_0_6B, "8b": QWEN3_8B, "14b": QWEN3_14B, "32b": QWEN3_32B}
CONTEXT = 4096
PREFILL_TOKENS = 2048


def weight_bytes(cfg, esize=2):
    h, i, nq, nkv, d, v, L = (cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                              cfg.num_key_value_heads, cfg.head_dim, cfg.vocab_size, cfg.num_hidden_layers)
    per_layer = (nq + 2 * nkv) * d * h + h * nq * d + 2 * i * h + h * i
    return (L * per_layer + v * h) * esize          # every linear weight once, and the head


def kv_bytes_per_token(cfg, esize=2):
    return 2 * cfg.num_key_value_heads * cfg.head_dim * esize * cfg.num_hidden_layers


def prefill_flops(cfg, T):
    h, i, nq, nkv, d, v, L = (cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads,
                              cfg.num_key_value_heads, cfg.head_dim, cfg.vocab_size, cfg.num_hidden_layers)
    per_layer = (nq + 2 * nkv) * d * h + h * nq * d + 2 * i * h + h * i
    linear = 2.0 * T * L * per_layer + 2.0 * v * h          # the head runs on one row
    attn = L * 4.0 * nq * d * (T * (T + 1) / 2.0)           # causal QK^T and PV
    return linear + attn


def serve(workload: str, layers, run_ahead: bool = True) -> int:
    """One of the serving workloads through the whole engine."""
    import torch
    from xinfer_amd import EngineConfig, SamplingParams
    from xinfer_amd.engine import build_model
    from xinfer_amd.engine.llm_engine import LLMEngine
    from xinfer_amd.models import config_from_dict
    from xinfer_amd.weights.random_init import random_store_for

    w = WORKLOADS[workload]
    full = w["model"]["num_hidden_layers"]
    raw = dict(w["model"], num_hidden_layers=layers or full)
    _, cfg = config_from_dict(raw)
    t0 = time.time()
    model = build_model(cfg, random_store_for(cfg, seed=0), "bf16", "cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] {w['name']}, {cfg.num_hidden_layers} layers, built in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    page = 64
    n = w["requests"]
    pages = n * (-(-w["max_model_len"] // page)) + 8
    eng = LLMEngine(EngineConfig(max_num_seqs=n, max_model_len=w["max_model_len"], num_pages=pages, page_size=page,
                                 prefill_chunk_size=w["chunk"], seed=1, run_ahead=run_ahead),     # a step's token budget is the chunk
                    model=model)
    g = torch.Generator().manual_seed(4)
    lo, hi = w["prompt"]
    lens = [lo] * n if lo == hi else torch.randint(lo, hi + 1, (n,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (m,), generator=g).tolist() for m in lens]
    sp = SamplingParams(temperature=0.0, max_tokens=w["new_tokens"], ignore_eos=True)
    eng.generate(prompts[:2], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))   # warm-up
    steps0 = eng.steps
    eng.step_log = []
    torch.cuda.synchronize()
    t = time.perf_counter()
    outs = eng.generate(prompts, sp)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t
    new = sum(o.decoded_length for o in outs)
    # The least time the steps that ran could take: a step reads every weight once and the cache of its
    # requests, and computes its tokens' products and its attention's pairs; it is bound by the slower
    # of the two at the published peaks.
    h, i_, nq, nkv, d, L = (cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                            cfg.head_dim, cfg.num_hidden_layers)
    per_layer = (nq + 2 * nkv) * d * h + h * nq * d + 3 * i_ * h
    wb, kvb = weight_bytes(cfg), kv_bytes_per_token(cfg)
    least = mem_s = 0.0
    for tokens, keys, pairs in eng.step_log:
        mem = (wb + keys * kvb) / (HBM_GBPS * 1e9)
        flop = (2.0 * tokens * L * per_layer + L * 4.0 * nq * d * pairs) / (PEAK_TFLOPS["bf16"] * 1e12)
        least += max(mem, flop)
        mem_s += mem
    print(json.dumps({
        "metric": f"generated tok/s, {workload} workload, bf16", "value": round(new / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "seconds": round(dt, 3), "engine_steps": eng.steps - steps0, "higher_is_better": True,
        "vs_reference_published": round(new / dt / w["reference_tok_s"], 2) if "reference_tok_s" in w else None,
        "roofline": {"bound": "hbm or mfma, step by step", "least_seconds": round(least, 3),
                     "least_seconds_memory_alone": round(mem_s, 3), "frac": round(least / dt, 4)},
        "dtype": "bf16", "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {"model": w["name"], "layers": cfg.num_hidden_layers, "layers_of_model": full, "requests": n,
                   "prompt_tokens": sum(lens), "new_tokens": new, "prefill_chunk": w["chunk"],
                   "preemptions": eng.num_preemptions, "total_tok_per_s": round((sum(lens) + new) / dt, 1)}}), flush=True)
    return 0


def product(spec: str, dev="cuda:0") -> int:
    """One bfloat16 product x [M, K] @ w [N, K]^T alone: the many-row tiled kernel (with `slices` of K as
    float32 partial sums, in tile `shape`; left out: what `kernels.tile_split_plan` chooses, or one slice
    in the shape of fewest tiles) beside the vendor library's plain product, each the best of 5 runs of 20
    launches in a HIP graph."""
    import torch
    from xinfer_amd import kernels
    parts = [int(v) for v in spec.split(",")]
    M, N, K = parts[:3]
    slices, shape = (parts[3], parts[4] if len(parts) > 4 else None) if len(parts) > 3 else kernels.tile_split_plan(M, N, K)
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    x = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device=dev, dtype=torch.float32) * 0.05).to(torch.bfloat16)

    def timed(f, n=20):
        f()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(n):
                f()
        best = None
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b) / n
            best = ms if best is None else min(best, ms)
        return best * 1e3

    tile_us = timed(lambda: kernels.linear_tile(x, w, slices, partial=slices > 1, shape=shape))
    lib_us = timed(lambda: torch.nn.functional.linear(x, w))
    y = kernels.linear_tile(x, w, slices, partial=slices > 1, shape=shape)
    y = y.sum(0) if y.dim() == 3 else y.float()
    ref = x.float() @ w.float().t()
    flops = 2.0 * M * N * K
    print(json.dumps({"product": [M, N, K], "slices": slices, "tile_shape": shape, "linear_tile_us": round(tile_us, 1),
                      "library_us": round(lib_us, 1), "linear_tile_tflops": round(flops / tile_us / 1e6, 1),
                      "library_tflops": round(flops / lib_us / 1e6, 1),
                      "max_error_of_largest": float((y - ref).abs().max() / ref.abs().max())}), flush=True)
    return 0


def measured_peaks(dev="cuda:0"):
    """(GB/s of a read-only stream over 4 GiB, TFLOP/s of one square bfloat16 product of 8192 in the
    vendor library): what this card reaches, beside the published peaks.  Best of five runs each."""
    import torch
    from xinfer_amd import kernels
    buf = torch.empty(1 << 30, dtype=torch.int32, device=dev)         # 4 GiB: sixteen times the memory-side cache
    buf.zero_()
    best = None
    for workgroups, chunk in ((256, 1 << 18), (256, 1 << 16), (1024, 1 << 14)):     # the shapes that read fastest
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            kernels.stream_read(buf, workgroups, chunk)
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b)
            best = ms if best is None else min(best, ms)
    gbps = buf.numel() * 4 / (best * 1e-3) / 1e9
    del buf
    n = 8192
    x = torch.randn(n, n, device=dev, dtype=torch.float32).to(torch.bfloat16)
    w = torch.randn(n, n, device=dev, dtype=torch.float32).to(torch.bfloat16)
    best = None
    for _ in range(6):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        torch.nn.functional.linear(x, w)
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b)
        best = ms if best is None else min(best, ms)
    tflops = 2.0 * n * n * n / (best * 1e-3) / 1e12
    return gbps, tflops


def main() -> int:
    global CONTEXT, PREFILL_TOKENS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the configuration has (reported in config)")
    ap.add_argument("--workload", choices=["decode"] + sorted(WORKLOADS), default="decode",
                    help="decode: the contract's run (default); the others: a serving workload end to end")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=CONTEXT,
                    help="context length at the end of the decode run (default: the contract's)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="length of the prefilled prompt (default: the contract's)")
    ap.add_argument("--model", choices=sorted(MODELS), default="8b",
                    help="layer sizes of the decode and prefill runs (default: the contract's Qwen3-8B)")
    ap.add_argument("--skip-points", action="store_true", help="only the default decode run")
    ap.add_argument("--only", choices=["all", "decode", "prefill"], default="all",
                    help="run one phase only (for profiling); the JSON line then lacks the other")
    ap.add_argument("--no-run-ahead", action="store_true",
                    help="serving workloads: read every step's tokens on the host before the next step is planned")
    ap.add_argument("--product", default=None, metavar="M,N,K[,slices[,shape]]",
                    help="time one bfloat16 product alone in the many-row tiled kernel and in the vendor library")
    ap.add_argument("--peaks", action="store_true",
                    help="also measure what this card reaches on a read-only stream of 4 GiB and on one square "
                         "bfloat16 product of 8192, and report the fractions of those beside the fractions of the "
                         "published peaks")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.product:
        return product(args.product)
    if args.workload != "decode":
        return serve(args.workload, args.layers, not args.no_run_ahead)
    full_layers = MODELS[args.model]["num_hidden_layers"]
    model_name = {"0.6b": "Qwen3-0.6B", "8b": "Qwen3-8B", "14b": "Qwen3-14B", "32b": "Qwen3-32B"}[args.model]
    if args.layers is None:
        args.layers = full_layers
    CONTEXT, PREFILL_TOKENS = args.context, args.prefill_tokens     # the sizes of this run

    import torch
    from xinfer_amd.engine import ModelRunner, StepEntry, build_model
    from xinfer_amd.models import config_from_dict
    from xinfer_amd.sampling import Sampler
    from xinfer_amd.weights.random_init import random_store_for

    dev = "cuda:0"
    raw = dict(MODELS[args.model], num_hidden_layers=args.layers)
    _, cfg = config_from_dict(raw)
    store = random_store_for(cfg, seed=0, linear_std=0.02, norm_std=0.1)
    t0 = time.time()
    model = build_model(cfg, store, "bf16", dev)
    torch.cuda.synchronize()
    print(f"[bench] model of {args.layers} layers built in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)

    page = 64
    max_batch = 8 if (args.skip_points or args.only != "all") else 64
    max_batch = max(max_batch, args.batch)
    num_pages = max_batch * (-(-CONTEXT // page)) + -(-PREFILL_TOKENS // page) + 8
    runner = ModelRunner(model, page_size=page, num_pages=num_pages, max_requests=max_batch + 1)
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    for lc in runner.layer_caches.values():          # random cache contents for the decode runs
        lc.k.copy_(torch.randn(lc.k.shape, generator=g, device=dev, dtype=torch.float32).to(lc.k.dtype))
        lc.v.copy_(torch.randn(lc.v.shape, generator=g, device=dev, dtype=torch.float32).to(lc.v.dtype))
    sampler = Sampler(dev)
    cpu_gen = torch.Generator().manual_seed(2)

    def sync():
        torch.cuda.synchronize()

    def decode_run(batch, steps, warmup, context=None):
        """`batch` requests whose caches already hold context - steps - warmup tokens decode
        steps + warmup tokens, so that the last timed step ends at `context` (CONTEXT unless given)."""
        prep = runner.graph_after          # steps before the warm-up in which the decode graph is recorded
        start = (context or CONTEXT) - steps - warmup - prep
        rids = list(range(100, 100 + batch))
        for rid in rids:
            runner.add_request(rid)
            runner.cache.reserve(rid, start)
            runner.cache.commit(rid, start)
        toks = torch.randint(0, cfg.vocab_size, (batch,), generator=cpu_gen).tolist()
        places = list(range(batch))
        pins = [torch.empty((batch,), dtype=torch.int32, pin_memory=True) for _ in range(2)]
        state = {"turn": 0}

        def one(prev):
            """One decode step as the engine launches it (`LLMEngine.step` with its default
            `run_ahead`): the tokens that the step before sampled are handed over on the device,
            greedy sampling follows on the GPU, and the sampled ids start their way to the host
            without anything waiting for them; the host prepares the next step meanwhile."""
            if prev is None:
                logits = runner.step([StepEntry(r, [t], [0]) for r, t in zip(rids, toks)])
            else:
                logits = runner.step([StepEntry(r, [0], [0]) for r in rids], device_tokens=(prev, places, places))
            tok = sampler.argmax(logits)
            pins[state["turn"]].copy_(tok, non_blocking=True)
            state["turn"] ^= 1
            return tok

        prev = None
        for _ in range(prep + warmup):
            prev = one(prev)
        sync()
        t = time.perf_counter()
        for _ in range(steps):
            prev = one(prev)
        sync()
        dt = time.perf_counter() - t
        assert 0 <= int(prev.min()) and int(prev.max()) < cfg.vocab_size
        for rid in rids:
            runner.release(rid)
        return dt / steps

    def prefill_run(reps=3):
        ids = torch.randint(0, cfg.vocab_size, (PREFILL_TOKENS,), generator=cpu_gen).tolist()
        best = None
        for _ in range(reps + 1):                  # the first run warms up
            runner.add_request(7)
            sync()
            t = time.perf_counter()
            logits = runner.step([StepEntry(7, ids, [PREFILL_TOKENS - 1])])
            sampler.argmax(logits).tolist()
            sync()
            dt = time.perf_counter() - t
            runner.release(7)
            best = dt if best is None else min(best, dt)
        return best

    if args.only == "prefill":
        psec = prefill_run()
        print(json.dumps({"prefill_ms": round(psec * 1e3, 3), "layers": args.layers}), flush=True)
        return 0
    sec = decode_run(args.batch, args.steps, args.warmup)
    wb, kvb = weight_bytes(cfg), kv_bytes_per_token(cfg)

    def stream_rate(batch, steps, seconds, context):
        """GB/s of a decode step: every weight once and the cache of its requests, over its time.  The
        cache length is the mean over the timed steps (it grows by one a step and ends at `context`)."""
        return (wb + batch * (context - (steps - 1) / 2.0) * kvb) / seconds / 1e9

    achieved = stream_rate(args.batch, args.steps, sec, CONTEXT)
    out = {
        "metric": f"decode tok/s at batch {args.batch}, {model_name} bf16", "value": round(args.batch / sec, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: seeded random weights, uniform random token ids, random cache contents",
        "config": {
            "model": f"{model_name} layer sizes", "global_batch": args.batch, "seq_len": CONTEXT,
            "parallelism": "single GPU", "layers": args.layers, "layers_of_model": full_layers,
            "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "vocab_size": cfg.vocab_size, "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps, "tie_word_embeddings": cfg.tie_word_embeddings,
            "page_size": page, "prefill_tokens": PREFILL_TOKENS, "kv_dtype": "bf16"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    print(f"[bench] decode b{args.batch}: {sec * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    peaks = None
    if args.peaks:
        peaks = measured_peaks(dev)
        out["peaks_measured"] = {"hbm_read_GBps": round(peaks[0], 1), "bf16_product_TFLOPs": round(peaks[1], 1)}
        out["roofline"]["frac_of_measured"] = round(achieved / peaks[0], 4)
        print(f"[bench] measured peaks: {peaks[0]:.0f} GB/s read-only stream, {peaks[1]:.0f} TFLOP/s square bf16 product",
              file=sys.stderr, flush=True)
    if args.only == "decode":
        print(json.dumps(out), flush=True)
        return 0
    psec = prefill_run()
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    out["prefill"] = {"value": round(PREFILL_TOKENS / psec, 1), "tokens": PREFILL_TOKENS,
                      "ms": round(psec * 1e3, 3),
                      "frac": round(flops / psec / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    if peaks is not None:
        out["prefill"]["frac_of_measured"] = round(flops / psec / (peaks[1] * 1e12), 4)
    print(f"[bench] prefill {PREFILL_TOKENS}: {psec * 1e3:.2f} ms", file=sys.stderr, flush=True)
    if not args.skip_points:
        points, roofs = {}, {}
        k, w = max(8, args.steps // 2), max(2, args.warmup // 2)
        for b in (1, 64):
            s = decode_run(b, k, w)
            points[f"decode_b{b}"] = round(b / s, 2)
            rate = stream_rate(b, k, s, CONTEXT)
            roofs[f"decode_b{b}"] = {"ms_per_step": round(s * 1e3, 4), "achieved": round(rate, 1),
                                     "frac": round(rate / HBM_GBPS, 4)}
            print(f"[bench] decode b{b}: {s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
        out["points"] = points
        out["points_roofline"] = roofs          # GB/s of each point's step and its fraction of the 8 TB/s peak
        # one point at a longer context: batch 8 with 16,384 tokens in every request's cache
        far = 4 * CONTEXT
        if max_batch * (-(-CONTEXT // page)) >= 8 * (-(-far // page)) and far <= cfg.max_position_embeddings:
            s = decode_run(8, k, w, context=far)
            rate = stream_rate(8, k, s, far)
            out["further"] = {"decode_b8_ctx": far, "value": round(8 / s, 2), "ms_per_step": round(s * 1e3, 4),
                              "achieved": round(rate, 1), "frac": round(rate / HBM_GBPS, 4)}
            print(f"[bench] decode b8 at context {far}: {s * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
