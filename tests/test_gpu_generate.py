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


def run_cli(args, stdin=None):
    r = subprocess.run([sys.executable, "-m", "simply_amd", *args], cwd=ROOT, capture_output=True, text=True, timeout=110,
                       input=stdin)
    assert r.returncode == 0, r.stderr
    return r.stdout


def test_command_line_with_a_config_random_weights_and_prompts_from_standard_input(tmp_path, gpu_lib):
    """`random --config C --seed S` writes a folder (weights drawn on the host); `generate --model` on that folder and
    `generate --config C --random_weights S` (weights drawn on the device from the same seed, in the same order of
    tensors, by the device's own generator) each generate what the plain implementation generates from the same
    tensors, for prompts that arrive on standard input as JSON lines in both accepted forms."""
    from simply_amd.config import config_from_dict
    from simply_amd.models import DecoderModel
    from simply_amd.weights import random_tensors

    d = dict(tiny.TINY_U, initializer_range=0.3)
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(d))
    folder = run_cli(["random", "--config", str(cfg_path), "--out", str(tmp_path / "m"), "--seed", "7", "--dtype", "float32",
                      "--norm_std", "0.1"]).strip().splitlines()[-1]
    w_folder, cfg = plain.load(folder)
    model = DecoderModel(config_from_dict(d).model_spec())
    w_device = {n: t.cpu() for n, t in random_tensors(model, 7, torch.float32, norm_std=0.1, device="cuda:0")}
    assert set(w_device) == set(w_folder)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 40 + n) for n in (6, 13)]
    lines = json.dumps(prompts[0]) + "\n\n" + json.dumps({"tokens": prompts[1]}) + "\n"
    common = ["--prompt_file", "-", "--temperature", "0", "--max-tokens", "5", "--dtype", "float32", "--batch-size", "2",
              "--max_seq_len", "64", "--page_size", "4", "--intermediate-steps", "3"]
    for source, w in ((["--config", str(cfg_path), "--random_weights", "7"], w_device), (["--model", folder], w_folder)):
        want = [plain.greedy(w, cfg, p, 5, torch.float64) for p in prompts]
        assert all(len(set(t)) > 1 for t in want)
        recs = [json.loads(l) for l in run_cli(["generate", *source, *common], stdin=lines).strip().splitlines()]
        assert [r["index"] for r in recs] == [0, 1] and [r["input_len"] for r in recs] == [6, 13]
        assert [r["tokens"] for r in recs] == want, source


def test_command_line_replay(tmp_path, gpu_lib):
    """`python -m simply_amd replay` is the replay of bin/trace_run: the same options, the same files."""
    import numpy as np
    d = tiny.write_model("A", str(tmp_path / "A"), dtype=torch.bfloat16, std=0.5)
    w, cfg = plain.load(d)
    toks = tiny.random_tokens(12, cfg["vocab_size"], 8)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:7], "want": [6]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[7:9], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[9:], "want": [0, 2]}], "end": ["a"]}]
    out = run_cli(["replay", "--model", d, "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                  stdin="".join(json.dumps(s) + "\n" for s in steps))
    assert out.split() == ["done", "0", "done", "1", "done", "2"]
    want = plain.forward(w, cfg, toks, torch.float64)
    assert sorted(os.listdir(tmp_path / "o")) == ["0.f32", "2.f32"]
    got0 = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(1, -1).copy()).double()
    got2 = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(2, -1).copy()).double()
    scale = want.abs().max().item()
    assert (got0 - want[6:7]).abs().max().item() <= 2e-5 * scale
    assert (got2 - want[[9, 11]]).abs().max().item() <= 2e-5 * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_top_p_and_top_k_in_steps_in_a_row(tmp_path, gpu_lib, dtype):
    """Requests with top-p, top-k, both and neither decode together, eight steps in a row on the device (the recorded
    graph holds the sampler's kernels for those modes): the tokens and log-probabilities are those of one step at a
    time, and every drawn token lies in the nucleus that the plain implementation's masks leave."""
    d = tiny.write_model("D", str(tmp_path / "D"), dtype=torch.bfloat16, std=0.3)
    w, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 120 + n) for n in (4, 19, 33, 11)]
    plist = [SamplingParams(temperature=0.9, top_p=0.6, max_decode_steps=24, seed=11, ignore_eos=True),
             SamplingParams(temperature=1.2, top_p=0.8, top_k=12, max_decode_steps=17, seed=12, ignore_eos=True),
             SamplingParams(temperature=0.7, top_k=5, max_decode_steps=24, seed=13, ignore_eos=True),
             SamplingParams(temperature=1.0, max_decode_steps=20, seed=14, ignore_eos=True)]
    kw = dict(activation_dtype=dtype, batch_size=4, max_seq_len=96, page_size=16, max_num_issue_tokens=64)
    one = LMInterface(d, intermediate_steps=1, **kw).generate(prompts, sampling_params=plist)
    m = LMInterface(d, intermediate_steps=8, **kw)
    many = m.generate(prompts, sampling_params=plist)
    assert any(k[0] == "many" for k in m.executor._graphs)
    assert [o.output_token_ids for o in many] == [o.output_token_ids for o in one]
    for a, b in zip(many, one):
        torch.testing.assert_close(torch.tensor(a.output_token_logprobs), torch.tensor(b.output_token_logprobs),
                                   rtol=1e-5, atol=1e-5)
    if dtype == "float32":
        for o, sp in zip(many, plist):
            seq = o.input_token_ids + o.output_token_ids
            logits = plain.forward(w, cfg, seq[:-1], torch.float64)[len(o.input_token_ids) - 1:]
            for row, tok, lp in zip(logits, o.output_token_ids, o.output_token_logprobs):
                # the k largest stay, then among those the nucleus of mass top_p (simply/utils/sampling_lib.py:427-469)
                x = row / sp.temperature
                if sp.top_k > 0:
                    x = torch.where(plain.top_k_mask(x, sp.top_k), x, torch.full_like(x, -float("inf")))
                if sp.top_p < 1.0:
                    x = torch.where(plain.top_p_mask(x, sp.top_p), x, torch.full_like(x, -float("inf")))
                assert torch.isfinite(x[tok]), (sp, tok)
                assert abs(float(torch.log_softmax(x, -1)[tok]) - lp) < 1e-3


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
    # log_softmax moves by at most twice the largest change of a logit; the logits' own bound is derived from the
    # plain implementation with bfloat16 rounding (tests/bounds.py)
    import bounds
    ref = bounds.reference(w, cfg, toks[:-1], dtype)
    m = lm(d, activation_dtype=dtype, max_seq_len=256, page_size=16, max_num_issue_tokens=48)
    for temp in (1.0, 0.6):
        tol = 1e-4 if dtype == "float32" else 2 * ref.max_bound() * ref.scale / temp
        got = m.score_tokens(toks, ScoringParams(temperature=temp))
        want = [plain.log_prob(logits[i], toks[i + 1], temp) for i in range(len(toks) - 1)]
        assert len(got) == len(want) and max(abs(a - b) for a, b in zip(got, want)) < tol, tol
    sp = SamplingParams(temperature=0.8, top_k=20, max_decode_steps=12, seed=5, ignore_eos=True)
    out = m.generate([toks[:30]], sampling_params=sp)[0]
    seq = out.input_token_ids + out.output_token_ids
    scores = m.score_tokens(seq, ScoringParams.from_sampling_params(sp))
    tail = scores[len(out.input_token_ids) - 1:]
    # scoring runs the tokens in portions, generation one by one: in bfloat16 other kernels, the same bound twice
    seq_ref = bounds.reference(w, cfg, seq[:-1], dtype)
    tol = 1e-4 if dtype == "float32" else 4 * seq_ref.max_bound() * seq_ref.scale / sp.temperature
    assert max(abs(a - b) for a, b in zip(tail, out.output_token_logprobs)) < tol, tol
    m.executor.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.executor.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_score_tokens_while_requests_are_live(tmp_path, gpu_lib, dtype):
    """Scoring runs as a request of its own beside whatever else is live: two requests are in the middle of their
    generation (one still in its prompt) when a sequence is scored; the scores are those of scoring alone, and the two
    requests go on to the tokens that they generate undisturbed.  So few pages that the scored sequence takes pages
    that others gave back."""
    d = tiny.write_model("D", str(tmp_path / "D"), dtype=torch.bfloat16, std=0.15)
    w, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 300 + n) for n in (21, 70)]
    params = SamplingParams(temperature=0.0, max_decode_steps=12, ignore_eos=True)
    toks = tiny.random_tokens(60, cfg["vocab_size"], 92)
    kw = dict(activation_dtype=dtype, max_seq_len=128, page_size=16, max_num_issue_tokens=32, intermediate_steps=2,
              poison_freed_pages=True)
    alone = lm(d, **kw)
    undisturbed = [o.output_token_ids for o in alone.generate(prompts, sampling_params=params)]
    want = alone.score_tokens(toks, ScoringParams(temperature=0.8))
    m = lm(d, total_num_pages=12, **kw)
    reqs = [m.add_request(i, p, params) for i, p in enumerate(prompts)]
    m.step()
    m.step()                    # the first decodes, the second is in its prompt's third portion
    assert len(reqs[0].output_token_ids) >= 1 and reqs[1].num_computed < 70 and len(m.scheduler.running) == 2
    got = m.score_tokens(toks, ScoringParams(temperature=0.8))
    m.executor.cache.check()
    while m.scheduler.has_work():
        m.step()
    assert [r.output_token_ids for r in reqs] == undisturbed
    import bounds
    ref = bounds.reference(w, cfg, toks[:-1], dtype)
    # (beside other requests the portions go through other kernels than alone: twice the bound on either)
    assert max(abs(a - b) for a, b in zip(got, want)) < (1e-5 if dtype == "float32" else 4 * ref.max_bound() * ref.scale / 0.8)
    logits = plain.forward(w, cfg, toks[:-1], torch.float64)
    exact = [plain.log_prob(logits[i], toks[i + 1], 0.8) for i in range(len(toks) - 1)]
    assert max(abs(a - b) for a, b in zip(got, exact)) < (1e-4 if dtype == "float32" else 2 * ref.max_bound() * ref.scale / 0.8)
    assert all(g.pool.num_free == g.pool.num_pages for g in m.executor.cache.groups)
