#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Gemma 2 2B layer sizes, random weights.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step: every live request advances by one token, through the scheduler, the step
function and the sampler, exactly as generation does.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# the benchmark configuration: Gemma 2 2B layer sizes
GEMMA2_2B = dict(
    architectures=["Gemma2ForCausalLM"], hidden_size=2304, num_hidden_layers=26, num_attention_heads=8,
    num_key_value_heads=4, head_dim=256, intermediate_size=9216, vocab_size=256000, rms_norm_eps=1e-6,
    rope_theta=10000.0, sliding_window=4096, query_pre_attn_scalar=256, attn_logit_softcapping=50.0,
    final_logit_softcapping=30.0, tie_word_embeddings=True, max_position_embeddings=8192,
    hidden_activation="gelu_pytorch_tanh", initializer_range=0.02)


def weight_bytes(cfg, esize=2):
    D, H, K, hd, F, V, L = (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                            cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers)
    per_layer = D * (H + 2 * K) * hd + H * hd * D + 3 * D * F + 4 * D
    return (L * per_layer + V * D + D) * esize


def kv_bytes_per_request(cfg, kv_len, esize=2):
    """Bytes of keys and values that one decode step reads for a request with kv_len tokens."""
    total = 0
    for kind in cfg.layer_types:
        seen = min(kv_len, cfg.sliding_window) if kind == "sliding_attention" else kv_len
        total += 2 * cfg.num_key_value_heads * cfg.head_dim * esize * seen
    return total


def prefill_flops(cfg, T):
    D, H, K, hd, F, V, L = (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                            cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers)
    gemm = 2 * T * (D * (H + 2 * K) * hd + H * hd * D + 3 * D * F) * L
    attn = 0
    for kind in cfg.layer_types:
        w = cfg.sliding_window if kind == "sliding_attention" else None
        keys = sum(min(t + 1, w) if w else t + 1 for t in range(T))
        attn += 4 * H * hd * keys
    return gemm + attn + 2 * D * V


# the larger Gemma 2 layer sizes, for --shape
SHAPES = {
    "2b": {},
    "9b": dict(hidden_size=3584, num_hidden_layers=42, num_attention_heads=16, num_key_value_heads=8, head_dim=256,
               intermediate_size=14336, query_pre_attn_scalar=256),
    "27b": dict(hidden_size=4608, num_hidden_layers=46, num_attention_heads=32, num_key_value_heads=16, head_dim=128,
                intermediate_size=36864, query_pre_attn_scalar=144),
}


def sync():
    import torch
    torch.cuda.synchronize()


def fill_cache_random(lm, std: float = 0.5, seed: int = 0, repeat_block: bool = False) -> None:
    """Fills every page of keys and values with N(0, std), so that decode steps over a long context can be timed
    without running the prompts that would have written them.  repeat_block: one block of 64 M random values copied
    over and over (for pools of a hundred gigabytes, whose every value need not be drawn)."""
    import torch
    gen = torch.Generator(device=lm.executor.device)
    gen.manual_seed(seed)
    block = None
    for v in lm.executor.cache.views:
        if v.pages and v.write:
            for t in v.pages.values():
                flat = t.view(-1)     # in slices, so that no float32 copy of a whole pool is made
                step = 1 << 26
                for i in range(0, flat.numel(), step):
                    n = min(step, flat.numel() - i)
                    if block is None or block.dtype != t.dtype or not repeat_block:
                        block = (torch.randn(step, generator=gen, device=t.device, dtype=torch.float32) * std).to(t.dtype)
                    flat[i:i + n] = block[:n]


def self_check(lm) -> dict:
    """Outside the timed steps: the next decode step is run twice, once eagerly (no recorded graph; the kernels plan
    for the real context) and once as the engine runs it (a replay of the recorded step), over the same cache.  The
    token that the engine's step draws must be the best of the eager step's logits, or within rounding of it
    (the two steps may cut the keys differently, so their logits differ in the last bits)."""
    import dataclasses
    import torch
    from simply_amd.engine.executor import StepEntry

    ex, reqs = lm.executor, sorted(lm.scheduler.running, key=lambda r: r.arrival)
    entries = [StepEntry(r.request_id, [r.all_token_ids[-1]], [0], r.num_computed) for r in reqs]
    config = ex.config
    ex.config = dataclasses.replace(config, use_graphs=False)
    try:
        eager = ex.step(entries).float().clone()
    finally:
        ex.config = config
    before = [len(r.output_token_ids) for r in reqs]
    lm.step(max_decode_steps=1)
    drawn = [r.output_token_ids[-1] for r in reqs]
    assert all(len(r.output_token_ids) == n + 1 for r, n in zip(reqs, before))
    assert torch.isfinite(eager).all(), "the eager step's logits are not finite"
    best = eager.max(dim=1).values
    of_drawn = eager[torch.arange(len(reqs)), torch.tensor(drawn, device=eager.device)]
    gap = float((best - of_drawn).max())
    same = int((eager.argmax(dim=1).cpu() == torch.tensor(drawn)).sum())
    scale = float(eager.abs().max())
    assert gap <= 1e-2 * scale, f"the engine's step drew tokens that the eager step's logits do not support: gap {gap}"
    return {"same_token": same, "of": len(reqs), "distinct_tokens": len(set(drawn)), "largest_gap": round(gap, 5),
            "largest_logit": round(scale, 3)}


def percentile(values, p):
    v = sorted(values)
    return v[min(len(v) - 1, int(round(p / 100.0 * (len(v) - 1))))]


def run_decode(model, cfg, batch, context, steps, warmup, page_size, dtype, latency_steps=0, memory_fraction=None):
    """Returns (seconds per step, mean kv length over the timed steps, latencies, self-check): `steps` decode steps as
    the engine runs them when nobody waits (several in a row on the device), then one step whose tokens are checked
    (`self_check`), then `latency_steps` more one at a time, the host reading each step's tokens before the next:
    their seconds are the latencies."""
    import torch
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    max_len = context + steps + warmup + latency_steps + 10
    lm = LMInterface(config=cfg, random_weights=0, activation_dtype=dtype, batch_size=batch, max_seq_len=max_len,
                     page_size=page_size, max_num_issue_tokens=2048, memory_fraction=memory_fraction, _model=model)
    fill_cache_random(lm, repeat_block=memory_fraction is not None)
    g = torch.Generator().manual_seed(1)
    params = SamplingParams(temperature=0.0, max_decode_steps=steps + warmup + latency_steps + 6, ignore_eos=True)
    for i in range(batch):
        prompt = torch.randint(0, cfg.vocab_size, (context,), generator=g).tolist()
        lm.adopt_request(f"b{i}", prompt, context - 1, params)
    def decode(k):
        """Exactly k decode steps (the engine runs several in a row on the device where it can)."""
        target = lm.stats["steps"] + k
        while lm.stats["steps"] < target:
            lm.step(max_decode_steps=target - lm.stats["steps"])

    decode(warmup)
    sync()
    t0 = time.perf_counter()
    decode(steps)
    sync()
    dt = (time.perf_counter() - t0) / steps
    first = context + warmup          # kv length seen by the first timed step
    mean_kv = first + (steps - 1) / 2
    assert all(len(r.output_token_ids) == warmup + steps for r in lm.scheduler.running)
    check = self_check(lm)
    latencies = []
    if latency_steps:
        lm.step(max_decode_steps=1)   # the single-step graph is recorded outside the timed steps
        lm.step_log = []
        for _ in range(latency_steps - 1):
            lm.step(max_decode_steps=1)
        latencies = [sec for _, _, sec in lm.step_log]
    del lm
    torch.cuda.empty_cache()
    return dt, mean_kv, latencies, check


def run_prefill(model, cfg, tokens, reps, page_size, dtype, portion=None):
    """Seconds for a prompt of `tokens` tokens and its first sampled token: in one step, or in portions of `portion`
    tokens (the scheduler cuts it under that token budget)."""
    import torch
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    lm = LMInterface(config=cfg, random_weights=0, activation_dtype=dtype, batch_size=1, max_seq_len=tokens + 8,
                     page_size=page_size, max_num_issue_tokens=portion or tokens, _model=model)
    g = torch.Generator().manual_seed(2)
    params = SamplingParams(temperature=0.0, max_decode_steps=1, ignore_eos=True)
    times = []
    for i in range(reps + 1):
        prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist()
        sync()
        t0 = time.perf_counter()
        steps_before = lm.stats["steps"]
        lm.generate(prompt, sampling_params=params)   # the whole prompt, then one sampled token
        sync()
        times.append(time.perf_counter() - t0)
        assert lm.stats["steps"] - steps_before == -(-tokens // (portion or tokens))
    del lm
    torch.cuda.empty_cache()
    return min(times[1:])


def run_requests(model, cfg, requests, prompt_min, prompt_max, new_tokens, page_size, dtype):
    """A whole workload through the scheduler: `requests` prompts of uniform-random lengths, all submitted at once,
    each generating `new_tokens` greedily (portions of prompts beside decoded tokens, continuous batching)."""
    import torch
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    g = torch.Generator().manual_seed(3)
    lengths = torch.randint(prompt_min, prompt_max + 1, (requests,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]
    lm = LMInterface(config=cfg, random_weights=0, activation_dtype=dtype, batch_size=requests,
                     max_seq_len=prompt_max + new_tokens + 8, page_size=page_size, max_num_issue_tokens=2048, _model=model)
    params = SamplingParams(temperature=0.0, max_decode_steps=new_tokens, ignore_eos=True)
    lm.generate(prompts[:2], sampling_params=SamplingParams(temperature=0.0, max_decode_steps=4, ignore_eos=True))
    sync()
    before = dict(lm.stats)
    lm.step_log = []
    t0 = time.perf_counter()
    outs = lm.generate(prompts, sampling_params=params)
    sync()
    dt = time.perf_counter() - t0
    assert all(len(o.output_token_ids) == new_tokens for o in outs)
    stats = {k: lm.stats[k] - before.get(k, 0) for k in lm.stats if isinstance(lm.stats[k], (int, float))}
    # steps that ran a portion of some prompt (beside decoded tokens of others) against steps that only decoded
    log = lm.step_log
    stats["prompt_step_seconds"] = sum(sec for n, _, sec in log if n == 0)
    stats["decode_step_seconds"] = sum(sec for n, _, sec in log if n > 0)
    stats["prompt_steps"] = sum(1 for n, _, _ in log if n == 0)
    stats["decode_steps"] = sum(n for n, _, _ in log if n > 0)
    stats["prompt_step_tokens"] = sum(t for n, t, _ in log if n == 0)
    per_decode_step = [sec / n for n, _, sec in log if n > 0]
    stats["decode_step_ms_p50"] = 1e3 * percentile(per_decode_step, 50) if per_decode_step else None
    stats["decode_step_ms_p99"] = 1e3 * percentile(per_decode_step, 99) if per_decode_step else None
    prompt_steps = [sec for n, _, sec in log if n == 0]
    stats["prompt_step_ms_p50"] = 1e3 * percentile(prompt_steps, 50) if prompt_steps else None
    stats["prompt_step_ms_p99"] = 1e3 * percentile(prompt_steps, 99) if prompt_steps else None
    del lm
    torch.cuda.empty_cache()
    return dt, sum(lengths), requests * new_tokens, stats


def run_products(which: str):
    """Times of the three bfloat16 product kernels (few-rows, tiled, wide) and of the library's own choice, for 1 to 64
    rows against weights of many sizes streamed from HBM (several copies of a weight in turn, so that no cache holds
    them), beside the times that the library expects: one JSON line per size and number of rows.  This is the sweep
    that the kernels' time models (`sa_gemm_plan`) are fitted to and judged by."""
    import torch
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles

    def graph_time(fs, reps=8):
        for f in fs:
            f()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for f in fs:
                f()
        g.replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(reps):
            g.replay()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / reps / len(fs) * 1e3

    # q/k/v, output and down projections of the 2B, 9B and 27B sizes, sizes of no model, the head; gated: the three
    # feed-forwards and two sizes of no model
    plain = [(4096, 2304), (2304, 2048), (2304, 9216), (8192, 3584), (3584, 4096), (3584, 14336), (8192, 4608),
             (4608, 4096), (4608, 36864), (3072, 3072), (5120, 8192), (1024, 1024), (11008, 4096), (2048, 16384),
             (256000, 2304)]
    gated = [(9216, 2304), (14336, 3584), (36864, 4608), (8192, 3072), (4096, 1024)]
    names = {ops.ALGO_SKINNY: "skinny", ops.ALGO_TILED: "tiled", ops.ALGO_WIDE: "wide"}
    for (N, K) in (gated if which == "gated" else plain):
        nbytes = N * K * 2 * (2 if which == "gated" else 1)
        copies = max(1, min(12, -(-(700 << 20) // nbytes)))
        ws = []
        for _ in range(copies):
            w = (torch.randn(N, K, device="cuda") * 0.03).to(torch.bfloat16)
            ws.append(pack_gate_up(w, (torch.randn(N, K, device="cuda") * 0.03).to(torch.bfloat16))
                      if which == "gated" else pack_tiles(w))
            del w
        for M in (1, 2, 4, 8, 9, 12, 16, 17, 24, 32, 48, 64):
            a = torch.randn(M, K, device="cuda").to(torch.bfloat16)
            out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            res = {}
            for name, algo in (("skinny", ops.ALGO_SKINNY), ("tiled", ops.ALGO_TILED), ("wide", ops.ALGO_WIDE),
                               ("chosen", ops.ALGO_AUTO)):
                try:
                    fs = [(lambda w=w: ops.gemm(a, w, out=out, algo=algo)) for w in ws]
                    res[name] = round(graph_time(fs * (2 if copies < 4 else 1)), 2)
                except ops.KernelError:
                    res[name] = None
            kernel, expected = ops.gemm_plan(M, N, K, gated=which == "gated")
            print(json.dumps({"product": which, "M": M, "N": N, "K": K, "us": res, "choice": names.get(kernel),
                              "expected_us": {k: round(v, 1) for k, v in expected.items()}}), flush=True)
        del ws
        torch.cuda.empty_cache()


def measure_ceilings():
    """What this GPU reaches by itself, with the library's two probe kernels: reading HBM with all CUs (2 GiB,
    contiguously and in shuffled 8 KiB pieces, as a cache's pages lie) and retiring bfloat16 MFMA instructions
    (operands of zeros, and of random values: the clock held under that load depends on the bits that toggle).
    The decode step's kernels cannot read faster than the first, the prompt's products cannot multiply faster than
    the last; the published peaks are higher than both."""
    import torch
    from simply_amd.kernels import ops

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            fn()
            end.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(end) * 1e-3)
        return best

    nbytes = 2 << 30
    buffer = torch.zeros(nbytes // 4, dtype=torch.float32, device="cuda:0")
    order = torch.randperm(nbytes // 8192, device="cuda:0").to(torch.int32)
    out = {"hbm_read_gbps": round(nbytes / timed(lambda: ops.probe_hbm_read(buffer), 5) / 1e9, 1),
           "hbm_read_8k_pieces_gbps": round(nbytes / timed(lambda: ops.probe_hbm_read(buffer, order), 5) / 1e9, 1)}
    del buffer, order
    iters = 40000  # about 5 ms a launch: long enough for the clock to settle
    for name, operands in (("zeros", torch.zeros(8192, dtype=torch.bfloat16, device="cuda:0")),
                           ("random", (torch.rand(8192, device="cuda:0") - 0.5).to(torch.bfloat16))):
        flops = [0.0]

        def run():
            flops[0] = ops.probe_mfma(operands, iters)
        seconds = timed(run, 8)
        out[f"mfma_bf16_{name}_tflops"] = round(flops[0] / seconds / 1e12, 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--batches", default="1,8,32,64", help="--only decode-grid: the batch sizes")
    ap.add_argument("--contexts", default="1024,4096,8192", help="--only decode-grid: the context lengths")
    ap.add_argument("--only", default="all", choices=["all", "decode", "decode-grid", "prefill", "prefill-chunked", "products",
                                                      "gated-products", "ceilings"],
                    help="measure one part alone (for profiles); the line then holds that part only.  products / "
                         "gated-products: the sweep of the product kernels over rows and weight sizes; ceilings: "
                         "what the GPU itself reaches in reading HBM and in bfloat16 MFMA instructions")
    ap.add_argument("--latency-steps", type=int, default=100,
                    help="decode steps run one at a time after the timed ones, for the p50 and p99 of a step's latency")
    ap.add_argument("--shape", default="2b", choices=sorted(SHAPES), help="layer sizes: Gemma 2 2B (the default), 9B, 27B")
    ap.add_argument("--requests", type=int, default=0,
                    help="instead of timed decode steps: a workload of this many requests through the scheduler")
    ap.add_argument("--prompt-min", type=int, default=128)
    ap.add_argument("--prompt-max", type=int, default=4096)
    ap.add_argument("--new-tokens", type=int, default=256)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        sys.exit(2)

    import torch
    from simply_amd.config import config_from_dict
    from simply_amd.engine.loading import random_model
    from simply_amd.kernels import lib

    lib.load()
    if args.only == "ceilings":
        print(json.dumps({"metric": "measured ceilings of this GPU", **measure_ceilings(),
                          "published": {"hbm_gbps": HBM_GBPS, "mfma_bf16_tflops": PEAK_TFLOPS["bf16"]}}), flush=True)
        return
    if args.only in ("products", "gated-products"):
        run_products("gated" if args.only == "gated-products" else "plain")
        return
    d = dict(GEMMA2_2B, **SHAPES[args.shape])
    full_layers = d["num_hidden_layers"]
    if args.layers:
        d["num_hidden_layers"] = args.layers
    cfg = config_from_dict(d)
    tdtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    esize = 2 if args.dtype == "bfloat16" else 4
    model = random_model(cfg, 0, tdtype, torch.device("cuda:0"))

    if args.requests:
        dt, prompt_tokens, new_tokens, stats = run_requests(model, cfg, args.requests, args.prompt_min, args.prompt_max,
                                                            args.new_tokens, args.page_size, args.dtype)
        print(json.dumps({
            "metric": "tokens/s of a workload (prompt and generated tokens, continuous batching)",
            "value": round((prompt_tokens + new_tokens) / dt, 1), "unit": "tokens/s", "n_gpus": 1,
            "generated_per_s": round(new_tokens / dt, 1), "seconds": round(dt, 3), "prompt_tokens": prompt_tokens,
            "generated_tokens": new_tokens, "engine_steps": stats.get("steps"), "higher_is_better": True,
            "phases": {"prompt_steps": stats["prompt_steps"], "prompt_step_seconds": round(stats["prompt_step_seconds"], 3),
                       "prompt_step_tokens": stats["prompt_step_tokens"], "decode_steps": stats["decode_steps"],
                       "decode_step_seconds": round(stats["decode_step_seconds"], 3)},
            "latency_ms": {f"{k}_{q}": (round(stats[f"{k}_ms_{q}"], 3) if stats[f"{k}_ms_{q}"] else None)
                           for k in ("decode_step", "prompt_step") for q in ("p50", "p99")},
            "preemptions": stats.get("preemptions"),
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": {"model": f"gemma2-{args.shape}-shape", "layers": cfg.num_hidden_layers,
                       "layers_of_full_model": full_layers, "requests": args.requests, "prompt_min": args.prompt_min,
                       "prompt_max": args.prompt_max, "new_tokens": args.new_tokens, "page_size": args.page_size}}),
              flush=True)
        return

    if args.only == "decode-grid":
        # decode steps at every batch size and context of the lists, one line each; the cache pools are sized from
        # the device memory that the weights leave free (`memory_fraction`), never more than the requests need
        for context in [int(c) for c in args.contexts.split(",")]:
            for batch in [int(b) for b in args.batches.split(",")]:
                dt, mean_kv, _, check = run_decode(model, cfg, batch, context, args.steps, args.warmup, args.page_size,
                                                   args.dtype, memory_fraction=0.9)
                step_bytes = weight_bytes(cfg, esize) + batch * kv_bytes_per_request(cfg, mean_kv, esize)
                print(json.dumps({"metric": "decode tokens/s", "model": f"gemma2-{args.shape}-shape",
                                  "layers": cfg.num_hidden_layers, "batch": batch, "context": context,
                                  "value": round(batch / dt, 1), "ms_per_step": round(dt * 1e3, 3),
                                  "step_gb": round(step_bytes / 1e9, 2),
                                  "roofline_frac": round(step_bytes / dt / 1e9 / HBM_GBPS, 4),
                                  "self_check": f"{check['same_token']} of {check['of']}"}), flush=True)
        return

    if args.only in ("prefill", "prefill-chunked"):
        T = args.prefill_tokens
        portion = -(-T // 4) if args.only == "prefill-chunked" else None
        pt = run_prefill(model, cfg, T, max(3, args.steps), args.page_size, args.dtype, portion=portion)
        peak = PEAK_TFLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
        print(json.dumps({"metric": f"prefill tokens/s ({T} tokens" + (", 4 portions)" if portion else ")"),
                          "value": round(T / pt, 1), "unit": "tokens/s", "ms": round(pt * 1e3, 3),
                          "frac": round(prefill_flops(cfg, T) / pt / 1e12 / peak, 4), "n_gpus": 1,
                          "config": {"model": f"gemma2-{args.shape}-shape", "layers": cfg.num_hidden_layers}}), flush=True)
        return

    dt, mean_kv, latencies, check = run_decode(model, cfg, args.batch, args.context, args.steps, args.warmup,
                                               args.page_size, args.dtype, latency_steps=args.latency_steps)
    step_bytes = weight_bytes(cfg, esize) + args.batch * kv_bytes_per_request(cfg, mean_kv, esize)
    achieved = step_bytes / dt / 1e9

    if args.only == "decode":
        print(json.dumps({"metric": "decode tokens/s (batch %d, context %d)" % (args.batch, args.context),
                          "value": round(args.batch / dt, 1), "unit": "tokens/s", "ms_per_step": round(dt * 1e3, 4),
                          "roofline_frac": round(achieved / HBM_GBPS, 4), "n_gpus": 1, "steps": args.steps,
                          "config": {"model": f"gemma2-{args.shape}-shape", "layers": cfg.num_hidden_layers}}), flush=True)
        return

    T = args.prefill_tokens
    pt = run_prefill(model, cfg, T, 3, args.page_size, args.dtype)
    peak = PEAK_TFLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    prefill = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
               "frac": round(prefill_flops(cfg, T) / pt / 1e12 / peak, 4)}
    # the same prompt in four portions, as it runs beside other requests under a token budget of a quarter of it
    pc = run_prefill(model, cfg, T, 3, args.page_size, args.dtype, portion=-(-T // 4))
    prefill_chunked = {"value": round(T / pc, 1), "tokens": T, "portions": 4, "ms": round(pc * 1e3, 3),
                       "frac": round(prefill_flops(cfg, T) / pc / 1e12 / peak, 4)}

    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps_b = max(10, min(args.steps, 30))
            dtb, _, _, _ = run_decode(model, cfg, b, args.context, steps_b, 8, args.page_size, args.dtype)
            points[f"decode_b{b}"] = round(b / dtb, 1)

    out = {
        "metric": "decode tokens/s (Gemma 2 %s shape, batch %d, context %d)" % (args.shape.upper(), args.batch, args.context),
        "value": round(args.batch / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {"model": f"gemma2-{args.shape}-shape", "layers": cfg.num_hidden_layers, "layers_of_full_model": full_layers,
                   "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
                   "sliding_window": cfg.sliding_window, "global_batch": args.batch, "seq_len": args.context,
                   "page_size": args.page_size, "prefill_tokens": T, "weights": "random N(0,0.02)",
                   "parallelism": "single-gpu"},
        "prefill": prefill,
        "prefill_chunked": prefill_chunked,
        "step_latency_ms": {"p50": round(1e3 * percentile(latencies, 50), 4), "p99": round(1e3 * percentile(latencies, 99), 4),
                            "steps": len(latencies), "what": "one decode step at a time, tokens read by the host"}
        if latencies else None,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points,
        "self_check": check,
    }
    try:  # (an extra: whatever goes wrong with it must not cost the line)
        out["measured_ceilings"] = measure_ceilings()
    except Exception as exc:  # noqa: BLE001
        out["measured_ceilings"] = {"error": repr(exc)[:200]}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
