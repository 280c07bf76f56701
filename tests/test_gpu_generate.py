"""Greedy and sampled generation through the entry point and the command line, on the GPU."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_gemma2 as plain
import tiny
from simply_amd.engine.llm import LMInterface
from simply_amd.sampling import SamplingParams

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def lm(d, **kw):
    args = dict(activation_dtype="float32", batch_size=3, max_seq_len=64, page_size=4, max_num_issue_tokens=16)
    args.update(kw)
    return LMInterface(d, **args)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_matches_plain(tmp_path, gpu_lib, dtype):
    d = tiny.write_model("A", str(tmp_path / "A"), dtype=torch.bfloat16, std=0.5)
    w, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 50 + n) for n in (5, 11, 17)]
    want = [plain.greedy(w, cfg, p, 8, torch.float64) for p in prompts]
    params = SamplingParams(temperature=0.0, max_decode_steps=8)
    outs = lm(d, activation_dtype=dtype).generate(prompts, sampling_params=params)
    assert [o.output_token_ids for o in outs] == want
    small = lm(d, activation_dtype=dtype, total_num_pages=11, poison_freed_pages=True)
    outs = small.generate(prompts, sampling_params=params)
    assert [o.output_token_ids for o in outs] == want
    assert small.stats["preemptions"] > 0
    small.executor.cache.check()


def test_sampling_is_per_request(tmp_path, gpu_lib):
    """BASELINE workload of the second tiny configuration: prompts of 1, 9, 23 and 40 tokens, pages of 4,
    mixed portions and decoding, temperature 0.7."""
    d = tiny.write_model("B", str(tmp_path / "B"), dtype=torch.float32, std=0.1)
    _, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 70 + n) for n in (1, 9, 23, 40)]
    plist = [SamplingParams(temperature=0.7, max_decode_steps=6, seed=1 + i) for i in range(4)]
    together = lm(d, batch_size=4).generate(prompts, sampling_params=plist)
    alone = [lm(d, batch_size=1).generate([p], sampling_params=[sp])[0] for p, sp in zip(prompts, plist)]
    assert [o.output_token_ids for o in together] == [o.output_token_ids for o in alone]
    w, cfg = plain.load(d)
    for o in together:   # the reported log-probability is log_softmax(logits / T) of the plain implementation
        seq = o.input_token_ids + o.output_token_ids
        logits = plain.forward(w, cfg, seq[:-1], torch.float64)
        for j, (tok, lp) in enumerate(zip(o.output_token_ids, o.output_token_logprobs)):
            assert abs(plain.log_prob(logits[len(o.input_token_ids) - 1 + j], tok, 0.7) - lp) < 1e-3


def test_command_line(tmp_path, gpu_lib):
    d = tiny.write_model("A", str(tmp_path / "A"), dtype=torch.bfloat16, std=0.5)
    w, cfg = plain.load(d)
    prompt = tiny.random_tokens(7, cfg["vocab_size"], 4)
    r = subprocess.run([sys.executable, "-m", "simply_amd", "generate", "--ckpt_dir", d, "--prompt_ids",
                        ",".join(map(str, prompt)), "--temperature", "0", "--max_decode_steps", "5",
                        "--activation_dtype", "float32", "--batch_size", "2", "--max_seq_len", "64"],
                       cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    assert rec["tokens"] == plain.greedy(w, cfg, prompt, 5, torch.float64) and rec["finish_reason"] == "length"
