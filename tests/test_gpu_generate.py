"""Greedy and sampled generation through the entry point and the command line, on the GPU."""
import dataclasses
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_gemma2 as plain
import tiny
from simply_amd.engine.llm import LMInterface
from simply_amd.sampling import SamplingParams, ScoringParams

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
    """The workload of the second tiny configuration: prompts of 1, 9, 23 and 40 tokens, pages of 4,
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_in_a_row_on_the_device(tmp_path, gpu_lib, dtype):
    """Decoding several steps without the host in between (drawn tokens fed on the device, positions, slots and
    draw counters advanced by a kernel) gives what step-by-step decoding gives: greedy and sampled, across page
    edges and a window, with requests that end at different times, an end-of-sequence token among them."""
    d = tiny.write_model("D", str(tmp_path / "D"), dtype=torch.bfloat16, std=0.3)
    _, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 90 + n) for n in (3, 14, 31, 18)]
    plist = [SamplingParams(temperature=0.0, max_decode_steps=37), SamplingParams(temperature=0.8, max_decode_steps=21, seed=5),
             SamplingParams(temperature=1.1, top_k=20, max_decode_steps=40, seed=6),
             SamplingParams(temperature=0.0, max_decode_steps=9)]
    kw = dict(activation_dtype=dtype, batch_size=4, max_seq_len=96, page_size=16, max_num_issue_tokens=64)
    one = LMInterface(d, intermediate_steps=1, **kw).generate(prompts, sampling_params=plist)
    for steps in (2, 8, 64):
        lm_many = LMInterface(d, intermediate_steps=steps, **kw)
        many = lm_many.generate(prompts, sampling_params=plist)
        assert [o.output_token_ids for o in many] == [o.output_token_ids for o in one], steps
        for a, b in zip(many, one):
            torch.testing.assert_close(torch.tensor(a.output_token_logprobs), torch.tensor(b.output_token_logprobs),
                                       rtol=1e-5, atol=1e-5)
        lm_many.executor.cache.check()
        # a second call goes through the recorded graph from its first step
        again = lm_many.generate(prompts, sampling_params=plist)
        assert [o.output_token_ids for o in again] == [o.output_token_ids for o in one], steps
    # an end-of-sequence token in the middle of a run of steps ends that request there
    eos = one[0].output_token_ids[5]
    lm_eos = LMInterface(d, intermediate_steps=8, **kw)
    lm_eos.model.spec = dataclasses.replace(lm_eos.model.spec, eos_token_ids=(eos,))
    out = lm_eos.generate([prompts[0]], sampling_params=[SamplingParams(temperature=0.0, max_decode_steps=37)])[0]
    assert out.output_token_ids == one[0].output_token_ids[:one[0].output_token_ids.index(eos) + 1]
    assert out.finish_reason == "eos"
    # ... and the others go on as if nothing had happened, although the host learns of the end a few steps late, when
    # further steps are already launched: a token that two of the four requests draw, at different times, as the end
    # of sequence for all of them; freed pages are overwritten at once
    common = [t for t in one[1].output_token_ids[3:] if t in one[2].output_token_ids[3:]]
    eos = common[0] if common else one[2].output_token_ids[7]

    def with_eos(steps):
        m = LMInterface(d, intermediate_steps=steps, poison_freed_pages=True, **kw)
        m.model.spec = dataclasses.replace(m.model.spec, eos_token_ids=(eos,))
        outs = m.generate(prompts, sampling_params=plist)
        m.executor.cache.check()
        return [(o.output_token_ids, o.finish_reason) for o in outs]

    want = with_eos(1)
    assert sum(reason == "eos" for _, reason in want) >= 1
    assert with_eos(64) == want and with_eos(3) == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_score_tokens(tmp_path, gpu_lib, dtype):
    """`score_tokens` against the log-softmax of the plain implementation's logits, in portions, beside live
    requests' pages; what `generate` reports for the tokens it drew is what scoring them gives."""
    d = tiny.write_model("D", str(tmp_path / "D"), dtype=torch.bfloat16, std=0.15)
    w, cfg = plain.load(d)
    toks = tiny.random_tokens(150, cfg["vocab_size"], 91)
    logits = plain.forward(w, cfg, toks[:-1], torch.float64)
    tol = 1e-4 if dtype == "float32" else 0.15
    m = lm(d, activation_dtype=dtype, max_seq_len=256, page_size=16, max_num_issue_tokens=48)
    for temp in (1.0, 0.6):
        got = m.score_tokens(toks, ScoringParams(temperature=temp))
        want = [plain.log_prob(logits[i], toks[i + 1], temp) for i in range(len(toks) - 1)]
        assert len(got) == len(want) and max(abs(a - b) for a, b in zip(got, want)) < tol
    sp = SamplingParams(temperature=0.8, top_k=20, max_decode_steps=12, seed=5, ignore_eos=True)
    out = m.generate([toks[:30]], sampling_params=sp)[0]
    seq = out.input_token_ids + out.output_token_ids
    scores = m.score_tokens(seq, ScoringParams.from_sampling_params(sp))
    tail = scores[len(out.input_token_ids) - 1:]
    assert max(abs(a - b) for a, b in zip(tail, out.output_token_logprobs)) < (1e-4 if dtype == "float32" else 0.1)
    m.executor.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.executor.cache.groups)
