"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives `Executor.step`,
the step function that generation uses.  Steps arrive as JSON lines:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the wanted places,
in the order of the entries and of `want`, as little-endian float32 [wanted, vocab].
"""
from __future__ import annotations

import json
import os
import sys
from typing import IO

import numpy as np
import torch

from ..config import EngineConfig
from .executor import Executor, StepEntry
from .loading import load_model

#: requests that may be live at a time
MAX_LIVE_REQUESTS = 4
#: each request's token count is rounded up to a multiple of this when the pool is sized
ROUND_TOKENS_TO = 64


class ReplayError(RuntimeError):
    """A step that could not be run: the line, and what the engine said."""


def build_executor(model_dir: str, dtype: str, max_tokens: int, *, device: str = "cuda:0",
                   page_size: int = 16, poison: bool = False) -> Executor:
    if ROUND_TOKENS_TO % page_size:
        raise ValueError(f"page size {page_size} does not divide {ROUND_TOKENS_TO}")
    cfg0 = EngineConfig(activation_dtype=dtype)
    model, config = load_model(model_dir, cfg0.dtype, torch.device(device))
    max_tokens = max(int(max_tokens), ROUND_TOKENS_TO)
    engine_config = EngineConfig(
        activation_dtype=dtype, page_size=page_size, batch_size=MAX_LIVE_REQUESTS,
        max_seq_len=max_tokens, max_num_issue_tokens=max_tokens,
        total_num_pages=-(-max_tokens // page_size), poison_freed_pages=poison, use_graphs=False, device=device)
    return Executor(model, engine_config)


def run_step(executor: Executor, record: dict, out_dir: str) -> None:
    entries = []
    for e in record.get("entries", []):
        rid = e["id"]
        if not executor.has_request(rid):
            executor.add_request(rid)
        entries.append(StepEntry(rid, e.get("tokens", []), e.get("want", [])))
    logits = executor.step(entries)
    if logits is not None:
        arr = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
        path = os.path.join(out_dir, f"{record['step']}.f32")
        tmp = path + ".tmp"
        with open(tmp, "wb") as f:
            f.write(arr.tobytes())
        os.replace(tmp, path)
    elif executor.device.type == "cuda":
        torch.cuda.synchronize(executor.device)
    for rid in record.get("end", []):
        if executor.has_request(rid):
            executor.finish_request(rid)


def replay(executor: Executor, lines: IO[str], out_dir: str, done: IO[str] = sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        try:
            record = json.loads(line)
            if not isinstance(record, dict) or "step" not in record:
                raise ValueError('a step is a JSON object with "step", "entries" and "end"')
            run_step(executor, record, out_dir)
        except Exception as e:  # which step, then the error as it is
            raise ReplayError(f"line {n + 1} ({line[:60]}{'...' if len(line) > 60 else ''}): "
                              f"{type(e).__name__}: {e}") from e
        print(f"done {record['step']}", file=done, flush=True)
        n += 1
    return n


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens that live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--poison", action="store_true", help="fill freed pages with NaN")
    args = ap.parse_args(argv)
    import torch

    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; this engine has no CPU path", file=sys.stderr, flush=True)
        return 3
    print("[trace_run] loading kernels and model ...", file=sys.stderr, flush=True)
    from ..kernels import lib

    lib.load()
    executor = build_executor(args.model, args.dtype, args.max_tokens, page_size=args.page_size, poison=args.poison)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    try:
        replay(executor, sys.stdin, args.out)
    except ReplayError as e:
        print(f"trace_run: {e}", file=sys.stderr, flush=True)
        return 1
    return 0
