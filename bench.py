"""Decode and prefill throughput of the engine on one MI355X, Llama-3.1-8B layer sizes, random
bfloat16 weights, synthetic token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]
                    [--shape 8b|1b|70b] [--workload decode|serve|small-kernels]

A step is one decode step of the whole batch: ``Engine.step`` on one token per request followed by
the sampling kernel and the copy of the chosen tokens to the host, as generation does it.  The
requests' earlier context is not computed: their pages are filled with random keys and values,
which costs a decode step the same reads.  One JSON line is printed: ``value`` is decoded tokens a
second at the default batch; ``prefill`` times one 2,048-token prompt; ``roofline`` sets the decode
step's unavoidable reads (every weight once, the live requests' cache) against HBM's 8 TB/s;
``points`` holds decode at batch 1 and 64.

``--shape`` takes the layer sizes of Llama-3.2-1B or Llama-3.1-70B instead (the default is the
headline's 8B).  ``--workload serve`` runs the scheduler instead of fixed batches: 64 requests at
once, prompts of 128 to 4,096 random tokens, 512 tokens generated for each at temperature 0.7; its
line reports generated tokens a second over the whole run, prefill included.  ``--workload
small-kernels`` times what a norm kernel adds to a replayed graph of large products, without a
profiler (under rocprofv3 no dispatch is shorter than about 4.6 us, an empty kernel included, so a
kernel trace overstates the small kernels of a step).
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_GBS = 8000.0  # MI355X HBM3E, published
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}  # dense MFMA, published

# the model of the headline benchmark: Llama-3.1-8B layer sizes, random weights
LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256, rms_norm_eps=1e-5,
    rope_theta=500000.0, max_position_embeddings=131072, tie_word_embeddings=False,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)


SHAPES = {
    "8b": LLAMA_8B,
    "1b": dict(LLAMA_8B, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               intermediate_size=8192, tie_word_embeddings=True,
               rope_scaling=dict(LLAMA_8B["rope_scaling"], factor=32.0)),
    "70b": dict(LLAMA_8B, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=28672),
}
SHAPE_NAMES = {"8b": "Llama-3.1-8B shape", "1b": "Llama-3.2-1B shape", "70b": "Llama-3.1-70B shape"}


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=32)
    p.add_argument("--warmup", type=int, default=4)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=8192)
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (both numbers are reported)")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes (default: the headline's)")
    p.add_argument("--workload", default="decode", choices=["decode", "serve", "small-kernels"])
    p.add_argument("--requests", type=int, default=64, help="serve: requests running at once")
    p.add_argument("--new-tokens", type=int, default=512, help="serve: tokens generated for every request")
    p.add_argument("--no-look-ahead", action="store_true", help="plan every decode step when it runs, not during the step before")
    return p.parse_args(argv)


def weight_bytes(engine) -> int:
    """Bytes of every tensor a decode step reads once: all layers, final norm, output matrix; of the
    embedding table only the rows of the batch (counted by the caller)."""
    total = 0
    seen = set()
    m = engine.model

    def add(t):
        if t is not None and t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            nonlocal total
            total += t.numel() * t.element_size()

    for part in m.all_parts():
        if part is m.embedding:
            continue  # a step reads as many rows of it as it has tokens
        for v in vars(part).values():
            if hasattr(v, "data_ptr"):
                add(v)
    return total


def fill_context(engine, rids, n_tokens, seed=0):
    """Give every request ``n_tokens`` cached tokens without computing them: pages are claimed and
    filled with random keys and values."""
    import torch

    for rid in rids:
        engine.admit(rid)
        engine.cache.extend(rid, n_tokens)
        engine.cache.advance(rid, n_tokens)
    g = torch.Generator(device=engine.device).manual_seed(seed)
    for pages in list(engine.cache.k_pages) + list(engine.cache.v_pages):
        flat = pages.view(-1)
        chunk = 1 << 28
        for lo in range(0, flat.numel(), chunk):
            flat[lo : lo + chunk].normal_(0.0, 1.0, generator=g)


def decode_run(engine, sampler, batch, context, steps, warmup, vocab, look_ahead=True):
    """Time ``steps`` decode steps of ``batch`` requests whose context ends at ``context`` tokens.
    A step is what the generation loop does for one: run the batch, sample, read the tokens; with
    ``look_ahead`` the next step's plan is made while the GPU runs this one, as the loop does."""
    import torch

    from torchllms_amd.engine import StepEntry
    from torchllms_amd.sampling import SamplingParams

    rids = [f"d{i}" for i in range(batch)]
    # a decode shape is recorded as a HIP graph once it has come back a few times: these steps are
    # part of setting the engine up, before the warm-up steps that the caller asked for
    prime = 3
    start = context - (steps + warmup + prime) - 1
    fill_context(engine, rids, start)
    params = [SamplingParams(temperature=0.0, seed=i) for i in range(batch)]
    tokens = [(7 * i + 3) % vocab for i in range(batch)]

    prepared = None

    def one_step(k):
        nonlocal tokens, prepared
        entries = [StepEntry(r, [t], [0]) for r, t in zip(rids, tokens)]
        logits = engine.step_prepared(prepared, entries) if prepared is not None else None
        if logits is None:
            logits = engine.step(entries)
        pending = sampler.launch(logits, params, [k] * batch)
        prepared = engine.prepare_decode() if look_ahead else None
        tokens = pending.tolist()

    for k in range(prime + warmup):
        one_step(k)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        one_step(prime + warmup + k)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    mean_ctx = start + prime + warmup + (steps + 1) / 2
    for r in rids:
        engine.free(r)
    return dt / steps, mean_ctx


def prefill_run(engine, n_tokens, vocab, repeats=3):
    import torch

    from torchllms_amd.engine import StepEntry

    toks = torch.randint(0, vocab, (n_tokens,), generator=torch.Generator().manual_seed(1)).tolist()
    times = []
    for i in range(repeats + 1):
        engine.admit("p")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry("p", toks, [n_tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.free("p")
    times = sorted(times[1:])  # the first run warms up
    return times[len(times) // 2]


def prefill_flops(cfg, n_layers, T):
    """Multiply-adds x 2 of one prompt of T tokens: projections, causal attention (half the square),
    feed-forward, and the output matrix for the one wanted row."""
    D, Hq, Hkv, dh, F, V = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size, cfg.vocab_size
    per_token = 2 * D * (Hq + 2 * Hkv) * dh + 2 * Hq * dh * D + 3 * 2 * D * F
    attn = 2 * 2 * Hq * dh * (T * (T + 1) / 2)
    return n_layers * (T * per_token + attn) + 2 * D * V


def serve_run(args, shape) -> int:
    """The continuous-batching workload: every request is admitted at once, prompts are cut into
    portions under the token budget beside the running requests' decode tokens."""
    import random

    import torch

    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.engine import Engine
    from torchllms_amd.inference.llm import GenerationLoop
    from torchllms_amd.sampling import Sampler, SamplingParams

    n_layers = args.layers or shape["num_hidden_layers"]
    cfg = LlamaConfig.from_dict(dict(shape, num_hidden_layers=n_layers))
    longest, budget = 4096, 4096
    engine = Engine.from_random(cfg, seed=0, dtype=args.dtype, draw_on_device=True, page_size=args.page_size,
                                max_seqs=args.requests, max_model_len=longest + args.new_tokens)
    rng = random.Random(0)
    prompts = [[rng.randrange(cfg.vocab_size) for _ in range(rng.randint(128, longest))] for _ in range(args.requests)]
    params = [SamplingParams(temperature=0.7, max_new_tokens=args.new_tokens, seed=i) for i in range(args.requests)]
    loop = GenerationLoop(engine, Sampler(), max_num_seqs=args.requests, max_num_batched_tokens=budget,
                          max_model_len=longest + args.new_tokens, look_ahead=not args.no_look_ahead)
    steps = [0]

    def count(plan):
        steps[0] += 1

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    requests = loop.run(prompts, params, count)
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    generated = sum(len(r.output) for r in requests)
    prompt_tokens = sum(len(p) for p in prompts)
    engine.cache.check_invariants()
    print(json.dumps({
        "metric": f"generated tok/s, {args.requests} requests at once, prompts of 128..{longest} tokens, {args.new_tokens} new tokens each, {SHAPE_NAMES[args.shape]}",
        "value": round(generated / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps[0], "warmup": 0,
        "ms_per_step": round(sec / steps[0] * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random-init weights, random token ids",
        "config": {"model": SHAPE_NAMES[args.shape], "global_batch": args.requests, "seq_len": longest + args.new_tokens,
                   "parallelism": "single GPU", "n_layers": n_layers, "n_layers_full": shape["num_hidden_layers"],
                   "hidden_size": cfg.hidden_size, "n_heads": cfg.num_attention_heads, "n_kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "page_size": args.page_size, "token_budget": budget, "temperature": 0.7},
        "seconds": round(sec, 3), "prompt_tokens": prompt_tokens, "generated_tokens": generated,
        "total_tokens_per_s": round((prompt_tokens + generated) / sec, 1),
        "preemptions": loop.scheduler.stats["preemptions"], "prepared_steps": loop.stats["prepared_steps"],
    }))
    return 0


def small_kernels_run(args, shape) -> int:
    """What a small kernel costs between two large ones of a replayed graph: the time of a graph of
    32 gate/up products of a decode step (each on a matrix of its own turn, caches flushed before
    every replay), and of the same graph with 1, 2 and 4 norm kernels behind each product."""
    import torch

    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    hidden, inter, rows, n = shape["hidden_size"], shape["intermediate_size"], args.batch, 32
    weights = [torch.randn(2 * inter, hidden, device=dev, dtype=torch.float32).mul_(0.02).to(torch.bfloat16) for _ in range(4)]
    x = torch.randn(rows, hidden, device=dev, dtype=torch.float32).to(torch.bfloat16)
    h, delta = torch.randn_like(x), torch.randn_like(x)
    gain = torch.ones(hidden, device=dev, dtype=torch.bfloat16)
    flush = torch.zeros(512 << 18, device=dev)

    def graph_us(norms_behind_each: int) -> float:
        def run():
            for i in range(n):
                ops.gemm_stream_glu(x, weights[i % 4], 4, 8)
                for _ in range(norms_behind_each):
                    ops.rmsnorm(h, gain, 1e-5, delta=delta, return_sum=True)

        with torch.inference_mode():
            run()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run()
            best = float("inf")
            for _ in range(7):
                flush.sum()
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                graph.replay()
                stop.record()
                stop.synchronize()
                best = min(best, start.elapsed_time(stop) * 1e3)
        return best

    base = graph_us(0)
    added = {k: (graph_us(k) - base) / n / k for k in (1, 2, 4)}
    print(json.dumps({
        "metric": "microseconds a norm kernel adds behind a large kernel of a replayed graph", "unit": "us",
        "rows": rows, "hidden_size": hidden, "product_us": round(base / n, 2),
        "norm_us": {f"{k}_behind_each": round(v, 2) for k, v in added.items()},
    }))
    return 0


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    shape = SHAPES[args.shape]
    if args.workload == "serve":
        return serve_run(args, shape)
    if args.workload == "small-kernels":
        return small_kernels_run(args, shape)
    import torch

    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.engine import Engine
    from torchllms_amd.sampling import Sampler

    full_layers = shape["num_hidden_layers"]
    n_layers = args.layers or full_layers
    cfg = LlamaConfig.from_dict(dict(shape, num_hidden_layers=n_layers))
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b]
    max_batch = max(batches)
    pages_per_req = -(-args.context // args.page_size) + 1
    engine = Engine.from_random(
        cfg, seed=0, dtype=args.dtype, draw_on_device=True, page_size=args.page_size,
        num_pages=max_batch * pages_per_req, max_seqs=max_batch, max_model_len=args.context,
    )
    sampler = Sampler()
    elt = 2 if args.dtype == "bfloat16" else 4
    wbytes = weight_bytes(engine)
    kv_per_token = 2 * n_layers * cfg.num_key_value_heads * cfg.head_dim * elt

    results = {}
    for b in batches:
        steps = args.steps if b == args.batch else max(args.steps // 2, 4)
        sec, mean_ctx = decode_run(engine, sampler, b, args.context, steps, args.warmup, cfg.vocab_size, not args.no_look_ahead)
        step_bytes = wbytes + b * cfg.hidden_size * elt + b * mean_ctx * kv_per_token
        results[b] = dict(sec=sec, tps=b / sec, bytes=step_bytes)

    pre_sec = prefill_run(engine, args.prefill_tokens, cfg.vocab_size)
    flops = prefill_flops(cfg, n_layers, args.prefill_tokens)

    main_r = results[args.batch]
    achieved = main_r["bytes"] / main_r["sec"] / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {SHAPE_NAMES[args.shape]} (plus batch {'/'.join(str(b) for b in batches[1:]) or 'none'}"
                  f" and prefill tok/s at {args.prefill_tokens} tokens)",
        "value": round(main_r["tps"], 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_r["sec"] * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random-init weights, random token ids, cache of earlier context filled with random values",
        "config": {
            "model": SHAPE_NAMES[args.shape],
            "global_batch": args.batch,
            "seq_len": args.context,
            "parallelism": "single GPU",
            "n_layers": n_layers,
            "n_layers_full": full_layers,
            "hidden_size": cfg.hidden_size,
            "n_heads": cfg.num_attention_heads,
            "n_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size,
            "vocab_size": cfg.vocab_size,
            "page_size": args.page_size,
            "prefill_tokens": args.prefill_tokens,
            "rope": f"llama3 factor {shape['rope_scaling']['factor']:g} theta 5e5",
        },
        "prefill": {
            "value": round(args.prefill_tokens / pre_sec, 1),
            "tokens": args.prefill_tokens,
            "ms": round(pre_sec * 1e3, 3),
            "frac": round(flops / pre_sec / (PEAK_TFLOPS[args.dtype] * 1e12), 4),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBS, 4),
        },
        "points": {f"decode_b{b}": round(r["tps"], 2) for b, r in results.items() if b != args.batch},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
