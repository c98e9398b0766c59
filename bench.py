"""Decode and prefill throughput of the engine on one MI355X, Llama-3.1-8B layer sizes, random
bfloat16 weights, synthetic token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 8192] [--layers L]
                    [--shape 8b|1b|70b] [--workload decode|serve|peaks|small-kernels|attention|products]

Everything runs through the generation loop: the scheduler admits the requests, cuts their prompts
into portions under its token budget, and plans every decode step; the step function runs it; the
sampling kernel picks the tokens (greedy), and they travel to the host, as in serving.  Nothing of
the context is faked: prompts of random token ids are prefilled for real.

One JSON line is printed.  ``value``: decoded tokens a second of ``--batch`` requests whose context
ends at ``--context``: the prompts are ``context`` less the generated tokens long, and K decode
steps are timed after W warm-up steps (a step is one decode step of the whole batch).  ``points``:
the same at batch 1 and 64.  ``prefill``: one prompt of 2,048 tokens in one step.  ``roofline``: the
bytes a decode step has to read (every weight once, the live requests' cache) over its time, against
HBM's published 8 TB/s and against what a plain read kernel reaches on this GPU.  ``workload``: the
reference's own decode benchmark (reference: torchllms/inference/throughput_bench.py:498-563):
prompts of 2,048 tokens, 256 generated, batch 1, 8 and 64, tokens a second = B * (new - 1) /
seconds from the end of the prefill to the last token, with the bytes per step at the mean context
of 2,176 and their share of 8 TB/s.

``--shape`` takes the layer sizes of Llama-3.2-1B or Llama-3.1-70B instead (the default is the
headline's 8B).  ``--workload serve`` runs 64 requests at once with prompts of 128 to 4,096 random
tokens and 512 tokens generated for each at temperature 0.7; its line reports generated tokens a
second over the whole run, prefill included.  ``--workload peaks`` measures what this GPU reaches:
a read of 4 GiB with 16-byte loads, a device copy, a loop of MFMA instructions on registers, and the
library's large matrix product.  ``--workload small-kernels`` times what a norm kernel adds to a
replayed graph of large products, without a profiler (under rocprofv3 no dispatch is shorter than
about 4.6 us, an empty kernel included, so a kernel trace overstates the small kernels of a step).
``--workload attention``: the decode attention and the merge of its splits alone, by batch size, context and
split size.  ``--workload products``: a decode layer's four products alone at 1 to 128 rows, the library against
this package's kernels.  Both as a step runs them: in a replayed graph, caches flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

from ctypes import c_int, c_size_t, c_void_p

HBM_GBS = 8000.0  # MI355X HBM3E, published
PEAK_SIGNATURES = {"tl_peak_stream_read": [c_void_p, c_size_t, c_int, c_void_p, c_void_p],
                   "tl_peak_mfma_bf16": [c_int, c_int, c_void_p, c_void_p],
                   "tl_peak_fma_f32": [c_int, c_int, c_void_p, c_void_p]}
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
    p.add_argument("--workload", default="decode", choices=["decode", "serve", "peaks", "small-kernels", "attention", "products"])
    p.add_argument("--token-budget", type=int, default=8192, help="tokens a step may hold (the scheduler cuts prompts to it)")
    p.add_argument("--no-reference-workload", action="store_true",
                   help="leave out the reference's benchmark (2,048-token prompts, 256 new tokens at batch 1, 8, 64)")
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


def generation_run(engine, sampler, batch, prompt_len, new_tokens, vocab, budget, look_ahead=True, timed_steps=None, warmup=0,
                   seed=0):
    """``batch`` random prompts of ``prompt_len`` tokens through the generation loop, ``new_tokens``
    greedy tokens each.  The scheduler decodes first: a request whose prompt is in the cache decodes
    while the others' prompts are still being prefilled, so the decode phase of the whole batch
    begins when the last prompt is in, and lasts until the first request ends.  Returns the seconds
    from the end of the prefill to the end of the run (``decode_s``; with a token budget that holds
    all prompts in one step every request decodes in lock step all the way, as in the reference's
    benchmark) and, with ``timed_steps`` = K, the seconds of exactly K decode steps of the whole
    batch after ``warmup`` + 3 further ones (the steps in which the decode shape is met for the first
    times and recorded as a HIP graph), bracketed by synchronisations."""
    import random

    import torch

    from torchllms_amd.inference.llm import GenerationLoop
    from torchllms_amd.sampling import SamplingParams

    rng = random.Random(seed)
    prompts = [[rng.randrange(vocab) for _ in range(prompt_len)] for _ in range(batch)]
    params = [SamplingParams(temperature=0.0, max_new_tokens=new_tokens, stop_token_ids=(), seed=i) for i in range(batch)]
    loop = GenerationLoop(engine, sampler, max_num_seqs=batch, max_num_batched_tokens=budget,
                          max_model_len=prompt_len + new_tokens, look_ahead=look_ahead)
    skip = 3 + warmup
    state = {"decode_steps": 0, "kv_tokens": 0, "t0": None, "t1": None, "t_start": None, "prefill_done": None}

    def on_step(plan):
        # (called when the step's tokens are booked) a decode step of the whole batch fed every request a
        # token that it had generated; while prompts are still being prefilled, or once a request has
        # ended, a step is not one
        if len(plan.entries) != batch or not all(len(e.tokens) == 1 and len(e.request.output) >= 2 for e in plan.entries):
            return
        state["decode_steps"] += 1
        if timed_steps is not None:
            if skip < state["decode_steps"] <= skip + timed_steps:
                state["kv_tokens"] += sum(e.request.num_computed for e in plan.entries)  # keys each row read
            if state["decode_steps"] == skip:
                torch.cuda.synchronize()
                state["t0"] = time.perf_counter()
            elif state["decode_steps"] == skip + timed_steps:
                torch.cuda.synchronize()
                state["t1"] = time.perf_counter()

    # the end of the prefill: the scheduler's own books say when every prompt is in the cache
    sched = loop.scheduler
    update = sched.update

    def update_and_watch(plan, sampled):
        done = update(plan, sampled)
        if state["prefill_done"] is None and not sched.waiting and all(r.output for r in sched.running):
            torch.cuda.synchronize()
            state["prefill_done"] = time.perf_counter()
        return done

    sched.update = update_and_watch
    torch.cuda.synchronize()
    state["t_start"] = time.perf_counter()
    requests = loop.run(prompts, params, on_step)
    torch.cuda.synchronize()
    t_end = time.perf_counter()
    assert all(len(r.output) == new_tokens for r in requests)
    engine.cache.check_invariants()
    out = {
        "prefill_s": state["prefill_done"] - state["t_start"],
        "decode_s": t_end - state["prefill_done"],
        "decode_steps": state["decode_steps"],
        "prepared_steps": loop.stats["prepared_steps"],
    }
    if timed_steps is not None:
        if state["t1"] is None:
            raise RuntimeError(f"only {state['decode_steps']} decode steps ran, {skip + timed_steps} were needed")
        out["timed_s"] = state["t1"] - state["t0"]
        out["mean_kv_tokens"] = state["kv_tokens"] / timed_steps  # keys all rows of a timed step read, on average
    return out


def measured_read_gbs(device, gib: int = 4) -> float:
    """What a plain read kernel (16-byte loads, four in flight per thread, 2,048 blocks) reaches on
    this GPU, in GB/s: the best of five passes over ``gib`` GiB."""
    import torch

    from torchllms_amd.kernels import lib

    peaks = lib.variant("peaks", 1, PEAK_SIGNATURES)
    buf = torch.empty(gib << 30, dtype=torch.uint8, device=device)
    buf.view(torch.int32).fill_(1)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(6):
        start.record()
        lib.check(peaks.tl_peak_stream_read(buf.data_ptr(), buf.numel(), 2048, None, stream), peaks, "tl_variant_last_error")
        stop.record()
        stop.synchronize()
        best = min(best, start.elapsed_time(stop))
    return buf.numel() / (best * 1e-3) / 1e9


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


def peaks_run(args) -> int:
    """What this GPU reaches at its clocks of today, beside the published figures: a read of 4 GiB by a
    kernel of 16-byte loads, a device-to-device copy (its bytes counted once read, once written), MFMA
    bfloat16 16x16x32 instructions issued from registers alone, the library's product of two
    8,192 x 8,192 bfloat16 matrices, and plain 32-bit multiply-adds from registers alone (the
    arithmetic of the 32-bit path's products)."""
    import torch

    from torchllms_amd.kernels import lib

    dev = "cuda:0"
    peaks = lib.variant("peaks", 1, PEAK_SIGNATURES)
    stream = torch.cuda.current_stream().cuda_stream
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(fn, repeats=6):
        best = float("inf")
        for _ in range(repeats):
            start.record()
            fn()
            stop.record()
            stop.synchronize()
            best = min(best, start.elapsed_time(stop))
        return best

    read_gbs = measured_read_gbs(dev)
    src = torch.empty(2 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    src.view(torch.int32).fill_(3)
    copy_ms = best_ms(lambda: dst.copy_(src))
    iters, blocks = 20000, 256 * 8
    mfma_ms = best_ms(lambda: lib.check(peaks.tl_peak_mfma_bf16(iters, blocks, None, stream), peaks, "tl_variant_last_error"))
    mfma_tflops = blocks * 4 * iters * 8 * (2 * 16 * 16 * 32) / (mfma_ms * 1e-3) / 1e12
    fma_iters = 4000
    fma_ms = best_ms(lambda: lib.check(peaks.tl_peak_fma_f32(fma_iters, blocks, None, stream), peaks, "tl_variant_last_error"))
    fma_tflops = blocks * 256 * fma_iters * 16 * 2 / (fma_ms * 1e-3) / 1e12
    a = torch.randn(8192, 8192, device=dev).to(torch.bfloat16)
    b = torch.randn(8192, 8192, device=dev).to(torch.bfloat16)
    mm_ms = best_ms(lambda: torch.matmul(a, b))
    print(json.dumps({
        "metric": "measured peaks of this GPU", "unit": "GB/s and TFLOP/s",
        "hbm_read_gbs": round(read_gbs, 1), "hbm_read_frac_of_published": round(read_gbs / HBM_GBS, 4),
        "hbm_copy_gbs_read_plus_write": round(2 * src.numel() / (copy_ms * 1e-3) / 1e9, 1),
        "mfma_bf16_tflops": round(mfma_tflops, 1), "mfma_bf16_frac_of_published": round(mfma_tflops / PEAK_TFLOPS["bfloat16"], 4),
        "library_matmul_bf16_tflops": round(2 * 8192 ** 3 / (mm_ms * 1e-3) / 1e12, 1),
        "fma_f32_tflops": round(fma_tflops, 1), "fma_f32_frac_of_published": round(fma_tflops / PEAK_TFLOPS["float32"], 4),
        "published": {"hbm_gbs": HBM_GBS, "mfma_bf16_tflops": PEAK_TFLOPS["bfloat16"], "fp32_tflops": PEAK_TFLOPS["float32"]},
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


def _cold_graph_us(fn, repeats: int, flush) -> float:
    """Microseconds per call of ``fn(i)``, i = 0 .. repeats - 1, recorded into one HIP graph and replayed with the
    caches flushed before each of five replays (the least counts): as a kernel runs inside a decode step."""
    import gc

    import torch

    with torch.inference_mode():
        for i in range(repeats):
            fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                for i in range(repeats):
                    fn(i)
        finally:
            if collecting:
                gc.enable()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(5):
            flush.sum()
            start.record()
            graph.replay()
            stop.record()
            stop.synchronize()
            best = min(best, start.elapsed_time(stop) * 1e3)
    return best / repeats


def attention_run(args, shape) -> int:
    """The decode attention kernel and the merge of its splits alone: every request at context C, behind a
    gate/up product that evicts the caches, in a replayed graph; per batch size and context the time with the
    planned splits and with splits of 128 to 2,048 keys."""
    import torch

    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    hq, hkv, dh, page = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"], args.page_size
    x = torch.randn(8, shape["hidden_size"], device=dev).to(torch.bfloat16)
    big = [torch.randn(2 * shape["intermediate_size"], shape["hidden_size"], device=dev).mul_(0.02).to(torch.bfloat16) for _ in range(4)]
    flush = torch.zeros(512 << 18, device=dev)
    layers = 8
    between = lambda i: ops.gemm_stream_glu(x, big[i % 4], 0, 16)
    base = _cold_graph_us(between, layers, flush)
    table = {}
    for batch in (1, 2, 4, 8, 16, 64):
        for ctx in (2176, 8192, 32768):
            if batch * ctx > 600000:
                continue
            n_pages = batch * ctx // page
            caches = [(torch.randn(n_pages, hkv, page, dh, device=dev).to(torch.bfloat16), torch.randn(n_pages, hkv, page, dh, device=dev).to(torch.bfloat16))
                      for _ in range(3)]
            tables = torch.arange(n_pages, dtype=torch.int32, device=dev).view(batch, -1).contiguous()
            q = torch.randn(batch, (hq + 2 * hkv) * dh, device=dev).to(torch.bfloat16)
            seq = torch.arange(batch, dtype=torch.int32, device=dev)
            pos = torch.full((batch,), ctx - 1, dtype=torch.int32, device=dev)
            row = {}
            for split in (None, 128, 256, 512, 1024, 2048):
                if split is not None and ctx // split > 512:
                    continue

                def step(i, split=split):
                    between(i)
                    k, v = caches[i % 3]
                    ops.attention_decode(q, hq, hkv, dh, k, v, seq, pos, tables, 0, dh ** -0.5, ctx, split_size=split)

                row["planned" if split is None else str(split)] = round(_cold_graph_us(step, layers, flush) - base, 1)
            plan = ops.plan_decode_splits(batch, hkv, ctx, dh)
            mb = batch * ctx * hkv * dh * 4 / 1e6
            table[f"b{batch}_ctx{ctx}"] = {"plan": list(plan), "mb": round(mb, 1), "us": row}
            del caches
    print(json.dumps({"metric": "decode attention and merge alone, cold, behind a large product", "unit": "us",
                      "model": SHAPE_NAMES[args.shape], "by_split_size": table}))
    return 0


def products_run(args, shape) -> int:
    """The four matrix products of a decode layer alone at 1 to 128 rows, cold weights in a replayed graph: the
    library, and the kernels of this package in the launch that the measurement at engine start would pick."""
    import torch

    from torchllms_amd.kernels import ops, products

    dev = "cuda:0"
    d, f = shape["hidden_size"], shape["intermediate_size"]
    qkv = (shape["num_attention_heads"] + 2 * shape["num_key_value_heads"]) * shape["head_dim"]
    shapes = {"qkv": (qkv, d, "qkv"), "o": (d, shape["num_attention_heads"] * shape["head_dim"], "sum"), "gate_up": (2 * f, d, "glu"), "down": (d, f, "sum")}
    flush = torch.zeros(512 << 18, device=dev)
    out = {}
    for name, (n, k, use) in shapes.items():
        weights = [torch.randn(n, k, device=dev).mul_(0.02).to(torch.bfloat16) for _ in range(4)]
        timed = {}
        ops.tune_linear(weights, torch.bfloat16, use, report=lambda bucket, choice, us: timed.setdefault(bucket, []).append((choice, us)))
        rows = {}
        for bucket, cands in sorted(timed.items()):
            chosen = products.LINEAR_CHOICE[(n, k, bucket, use)]
            lib = next(us for c, us in cands if c is None)
            best = min(us for _, us in cands)
            rows[str(bucket)] = {"library_us": round(lib, 1), "chosen": None if chosen is None else list(chosen),
                                 "chosen_us": round(next(us for c, us in cands if c == chosen), 1), "least_us": round(best, 1)}
        out[name] = {"n": n, "k": k, "use": use, "mb": round(n * k * 2 / 1e6, 1), "by_rows": rows}
        del weights
    print(json.dumps({"metric": "decode products alone, cold weights in a replayed graph (times as the engine's measurement charges them)",
                      "unit": "us", "model": SHAPE_NAMES[args.shape], "products": out}))
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
    if args.workload == "attention":
        return attention_run(args, shape)
    if args.workload == "products":
        return products_run(args, shape)
    if args.workload == "peaks":
        return peaks_run(args)
    import torch

    from torchllms_amd.config import LlamaConfig
    from torchllms_amd.engine import Engine
    from torchllms_amd.sampling import Sampler

    full_layers = shape["num_hidden_layers"]
    n_layers = args.layers or full_layers
    cfg = LlamaConfig.from_dict(dict(shape, num_hidden_layers=n_layers))
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b]
    max_batch = max(batches)
    def tokens_to_generate(b, steps):
        """Enough for ``steps`` timed decode steps of the whole batch: the first token comes from the
        prefill, the first request decodes alone while the other prompts are prefilled (at most so many
        steps), 3 + W steps record and warm up, and the last token is never fed back."""
        prefill_steps = -(-b * args.context // max(args.token_budget - b, 1)) + 1
        return 1 + prefill_steps + 3 + args.warmup + steps + 1

    new_tokens = tokens_to_generate(args.batch, args.steps)
    prompt_len = args.context - new_tokens
    if prompt_len < 1:
        print(f"--context {args.context} is too short for {new_tokens} generated tokens")
        return 2
    pages_per_req = -(-args.context // args.page_size) + 1
    engine = Engine.from_random(
        cfg, seed=0, dtype=args.dtype, draw_on_device=True, page_size=args.page_size,
        num_pages=max_batch * pages_per_req, max_seqs=max_batch, max_model_len=args.context,
    )
    sampler = Sampler()
    elt = 2 if args.dtype == "bfloat16" else 4
    wbytes = weight_bytes(engine)
    kv_per_token = 2 * n_layers * cfg.num_key_value_heads * cfg.head_dim * elt
    look_ahead = not args.no_look_ahead

    def step_bytes(b, mean_ctx):
        return wbytes + b * cfg.hidden_size * elt + b * mean_ctx * kv_per_token

    results = {}
    for b in batches:
        steps = args.steps if b == args.batch else max(args.steps // 2, 4)
        new_b = tokens_to_generate(b, steps)
        run = generation_run(engine, sampler, b, args.context - new_b, new_b, cfg.vocab_size, args.token_budget, look_ahead,
                             timed_steps=steps, warmup=args.warmup)
        sec = run["timed_s"] / steps
        nbytes = wbytes + b * cfg.hidden_size * elt + run["mean_kv_tokens"] * kv_per_token
        results[b] = dict(sec=sec, tps=b / sec, bytes=nbytes, steps=steps, mean_ctx=run["mean_kv_tokens"] / b)

    pre_sec = prefill_run(engine, args.prefill_tokens, cfg.vocab_size)
    flops = prefill_flops(cfg, n_layers, args.prefill_tokens)

    # the reference's own decode benchmark: 2,048-token prompts, 256 new tokens
    workload = {}
    if not args.no_reference_workload:
        ref_prompt, ref_new = 2048, 256
        if ref_prompt + ref_new <= args.context:
            for b in sorted(set([1, 8, 64]) & set(range(1, max_batch + 1))):
                # the whole batch's prompts in one step, as the reference's benchmark prefills them in one forward pass:
                # every request then decodes in lock step from the first token to the last
                one_step = b * ref_prompt
                generation_run(engine, sampler, b, ref_prompt, 8, cfg.vocab_size, one_step, look_ahead, seed=1)  # records the shape
                run = generation_run(engine, sampler, b, ref_prompt, ref_new, cfg.vocab_size, one_step, look_ahead, seed=2)
                assert run["decode_steps"] == ref_new - 1, run
                sec = run["decode_s"] / (ref_new - 1)
                nbytes = step_bytes(b, ref_prompt + ref_new / 2)
                workload[f"b{b}"] = {
                    "decode_tps": round(b * (ref_new - 1) / run["decode_s"], 1), "ms_per_step": round(sec * 1e3, 4),
                    "gb_per_step": round(nbytes / 1e9, 3), "frac": round(nbytes / sec / 1e9 / HBM_GBS, 4),
                    "prefill_tps": round(b * ref_prompt / run["prefill_s"], 1),
                }

    read_gbs = measured_read_gbs(engine.device)
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
        "data": "synthetic: random-init weights, prompts of random token ids prefilled through the scheduler, greedy decoding",
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
            "prompt_tokens": prompt_len,
            "new_tokens": new_tokens,
            "prefill_tokens": args.prefill_tokens,
            "token_budget": args.token_budget,
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
            "measured_read_peak": round(read_gbs, 1),
            "frac_of_measured": round(achieved / read_gbs, 4),
        },
        "points": {f"decode_b{b}": round(r["tps"], 2) for b, r in results.items() if b != args.batch},
        "points_frac": {f"decode_b{b}": round(r["bytes"] / r["sec"] / 1e9 / HBM_GBS, 4) for b, r in results.items() if b != args.batch},
        "mean_context": {f"b{b}": round(r["mean_ctx"], 1) for b, r in results.items()},
        "workload": dict(workload, prompt_tokens=2048, new_tokens=256, mean_context=2176) if workload else None,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
