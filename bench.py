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


def run_decode(model, cfg, batch, context, steps, warmup, page_size, dtype):
    """Returns (seconds per step, mean kv length over the timed steps)."""
    import torch
    from simply_amd.engine.llm import LMInterface, fill_cache_random, preload
    from simply_amd.sampling import SamplingParams

    max_len = context + steps + warmup + 8
    lm = LMInterface(config=cfg, random_weights=0, activation_dtype=dtype, batch_size=batch, max_seq_len=max_len,
                     page_size=page_size, max_num_issue_tokens=max(batch, 16), _model=model)
    fill_cache_random(lm)
    g = torch.Generator().manual_seed(1)
    params = SamplingParams(temperature=0.0, max_decode_steps=steps + warmup + 4, ignore_eos=True)
    for i in range(batch):
        prompt = torch.randint(0, cfg.vocab_size, (context,), generator=g).tolist()
        preload(lm, f"b{i}", prompt, params)
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
    del lm
    torch.cuda.empty_cache()
    return dt, mean_kv


def run_prefill(model, cfg, tokens, reps, page_size, dtype):
    import torch
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    lm = LMInterface(config=cfg, random_weights=0, activation_dtype=dtype, batch_size=1, max_seq_len=tokens + 8,
                     page_size=page_size, max_num_issue_tokens=tokens, _model=model)
    g = torch.Generator().manual_seed(2)
    params = SamplingParams(temperature=0.0, max_decode_steps=1, ignore_eos=True)
    times = []
    for i in range(reps + 1):
        prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist()
        sync()
        t0 = time.perf_counter()
        lm.generate(prompt, sampling_params=params)   # one step: the whole prompt, then one sampled token
        sync()
        times.append(time.perf_counter() - t0)
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
    t0 = time.perf_counter()
    outs = lm.generate(prompts, sampling_params=params)
    sync()
    dt = time.perf_counter() - t0
    assert all(len(o.output_token_ids) == new_tokens for o in outs)
    stats = {k: lm.stats[k] - before.get(k, 0) for k in lm.stats if isinstance(lm.stats[k], (int, float))}
    del lm
    torch.cuda.empty_cache()
    return dt, sum(lengths), requests * new_tokens, stats


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
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": {"model": f"gemma2-{args.shape}-shape", "layers": cfg.num_hidden_layers,
                       "layers_of_full_model": full_layers, "requests": args.requests, "prompt_min": args.prompt_min,
                       "prompt_max": args.prompt_max, "new_tokens": args.new_tokens, "page_size": args.page_size}}),
              flush=True)
        return

    dt, mean_kv = run_decode(model, cfg, args.batch, args.context, args.steps, args.warmup, args.page_size, args.dtype)
    step_bytes = weight_bytes(cfg, esize) + args.batch * kv_bytes_per_request(cfg, mean_kv, esize)
    achieved = step_bytes / dt / 1e9

    T = args.prefill_tokens
    pt = run_prefill(model, cfg, T, 3, args.page_size, args.dtype)
    peak = PEAK_TFLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    prefill = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
               "frac": round(prefill_flops(cfg, T) / pt / 1e12 / peak, 4)}

    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps_b = max(10, min(args.steps, 30))
            dtb, _ = run_decode(model, cfg, b, args.context, steps_b, 8, args.page_size, args.dtype)
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
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
