"""Command line: `python -m simply_amd <command> ...`

generate   token ids in, generated token ids out (JSON lines)
replay     the trace replay of bin/trace_run
random     write a model folder with random weights from a config.json and a seed

Options of `generate` carry the names of simply/serving/common_flags.py:19-132 where the reference
has the option (--batch_size, --activation_dtype, --max_seq_len, --max_decode_steps, --page_size,
--temperature, --top_k, --top_p, --max_num_issue_tokens, --intermediate_steps, --ckpt_dir) and of
simply/eval/page_decode_eval.py (--seed); dashes are accepted for underscores.
"""
from __future__ import annotations

import argparse
import json
import sys


def _flag(ap, name, **kw):
    ap.add_argument("--" + name, "--" + name.replace("_", "-"), dest=name, **kw)


def _read_prompts(args) -> list[list[int]]:
    prompts = []
    for p in args.prompt_ids or []:
        prompts.append([int(t) for t in p.replace(",", " ").split()])
    if args.prompt_file:
        with (sys.stdin if args.prompt_file == "-" else open(args.prompt_file)) as f:
            for line in f:
                line = line.strip()
                if line:
                    rec = json.loads(line)
                    prompts.append([int(t) for t in (rec["tokens"] if isinstance(rec, dict) else rec)])
    if not prompts:
        raise SystemExit("generate: no prompts (use --prompt_ids or --prompt_file)")
    return prompts


def cmd_generate(argv) -> int:
    ap = argparse.ArgumentParser(prog="python -m simply_amd generate")
    _flag(ap, "ckpt_dir", help="model folder: config.json and model.safetensors")
    ap.add_argument("--model", dest="ckpt_dir", help="same as --ckpt_dir")
    _flag(ap, "config", help="a config.json, with --random_weights")
    _flag(ap, "random_weights", type=int, help="seed of random weights for --config")
    _flag(ap, "prompt_ids", action="append", help='token ids of one prompt, "1,2,3"; may be repeated')
    _flag(ap, "prompt_file", help="JSON lines: a list of token ids, or {\"tokens\": [...]}; - is standard input")
    _flag(ap, "batch_size", type=int, default=8)
    _flag(ap, "activation_dtype", choices=["float32", "bfloat16"], default="bfloat16")
    ap.add_argument("--dtype", dest="activation_dtype", choices=["float32", "bfloat16"])
    _flag(ap, "max_seq_len", type=int, default=None)
    _flag(ap, "max_decode_steps", type=int, default=256)
    ap.add_argument("--max-tokens", dest="max_decode_steps", type=int)
    _flag(ap, "page_size", type=int, default=16)
    _flag(ap, "total_num_pages", type=int, default=None, help="pages of a cache group that keeps every token")
    _flag(ap, "windowed_num_pages", type=int, default=None, help="pages of a cache group that keeps a window only")
    _flag(ap, "memory_fraction", type=float, default=None,
          help="size the cache pools to this fraction of the free device memory (when --total_num_pages is not given)")
    _flag(ap, "temperature", type=float, default=1.0)
    _flag(ap, "top_k", type=int, default=-1)
    _flag(ap, "top_p", type=float, default=1.0)
    _flag(ap, "max_num_issue_tokens", type=int, default=2048)
    _flag(ap, "intermediate_steps", type=int, default=64,
          help="decode steps that may run in a row without a new scheduling decision (a run ends when a request ends)")
    _flag(ap, "seed", type=int, default=0)
    _flag(ap, "ignore_eos", action="store_true")
    args = ap.parse_args(argv)
    from .engine.llm import LMInterface
    from .sampling import SamplingParams

    kw = dict(activation_dtype=args.activation_dtype, batch_size=args.batch_size, max_seq_len=args.max_seq_len,
              page_size=args.page_size, max_num_issue_tokens=args.max_num_issue_tokens,
              total_num_pages=args.total_num_pages, windowed_num_pages=args.windowed_num_pages,
              memory_fraction=args.memory_fraction, seed=args.seed, intermediate_steps=args.intermediate_steps)
    if args.ckpt_dir:
        lm = LMInterface(args.ckpt_dir, **kw)
    elif args.config and args.random_weights is not None:
        from .config import config_from_dict

        with open(args.config) as f:
            lm = LMInterface(config=config_from_dict(json.load(f)), random_weights=args.random_weights, **kw)
    else:
        raise SystemExit("generate: give --ckpt_dir, or --config with --random_weights")
    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            max_decode_steps=args.max_decode_steps, ignore_eos=args.ignore_eos)
    outs = lm.generate(_read_prompts(args), sampling_params=params)
    for i, o in enumerate(outs):
        print(json.dumps({"index": i, "input_len": len(o.input_token_ids), "tokens": o.output_token_ids,
                          "logprobs": o.output_token_logprobs, "truncated": o.is_truncated,
                          "finish_reason": o.finish_reason}), flush=True)
    s = lm.stats
    print(f"[simply_amd] {s['tokens']} tokens in {s['steps']} steps, {s['seconds']:.3f} s, "
          f"{s['preemptions']} preemptions", file=sys.stderr)
    return 0


def cmd_random(argv) -> int:
    ap = argparse.ArgumentParser(prog="python -m simply_amd random")
    ap.add_argument("--config", required=True, help="config.json of the model to write")
    ap.add_argument("--out", required=True, help="folder to write config.json and model.safetensors into")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", choices=["float32", "bfloat16"], default="bfloat16")
    _flag(ap, "norm_std", type=float, default=0.1)
    _flag(ap, "std", type=float, default=None, help="default: initializer_range of the config")
    args = ap.parse_args(argv)
    from .config import config_from_dict, parse_dtype
    from .weights import write_random_model

    with open(args.config) as f:
        cfg = config_from_dict(json.load(f))
    print(write_random_model(cfg, args.out, args.seed, parse_dtype(args.dtype), std=args.std, norm_std=args.norm_std))
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    commands = {"generate": cmd_generate, "random": cmd_random}
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0
    if argv[0] == "replay":
        from .engine.replay import main as replay_main

        return replay_main(argv[1:])
    if argv[0] not in commands:
        raise SystemExit(f"unknown command {argv[0]!r}; known: generate, replay, random")
    return commands[argv[0]](argv[1:])


if __name__ == "__main__":
    sys.exit(main())
