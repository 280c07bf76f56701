"""The entry point's loop (scheduler, step function, sampler) with the kernels replaced by their plain
references: greedy generation equals the plain implementation's, also when pages run out."""
import torch

import plain_gemma2 as plain
import tiny
from simply_amd.engine.llm import LMInterface
from simply_amd.sampling import SamplingParams, ScoringParams


def lm(d, **kw):
    args = dict(activation_dtype="float32", batch_size=3, max_seq_len=64, page_size=4, max_num_issue_tokens=16,
                device="cpu", use_graphs=False)
    args.update(kw)
    return LMInterface(d, **args)


def test_greedy_generation_matches_plain(tmp_path, cpu_ops):
    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)
    w, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 50 + n) for n in (5, 11, 17)]
    want = [plain.greedy(w, cfg, p, 8) for p in prompts]
    params = SamplingParams(temperature=0.0, max_decode_steps=8)
    outs = lm(d).generate(prompts, sampling_params=params)
    assert [o.output_token_ids for o in outs] == want
    assert all(o.finish_reason == "length" and o.is_truncated for o in outs)
    assert all(lp == 0.0 for o in outs for lp in o.output_token_logprobs)
    # so few pages that requests give way and are recomputed: the tokens stay the same
    small = lm(d, total_num_pages=11)
    outs2 = small.generate(prompts, sampling_params=params)
    assert [o.output_token_ids for o in outs2] == want
    assert small.stats["preemptions"] > 0
    small.executor.cache.check()
    assert all(g.pool.num_free == 11 for g in small.executor.cache.groups)


def test_windowed_layers_have_a_smaller_pool(tmp_path, cpu_ops):
    """Prompts much longer than the window, in portions of 16: the windowed layers' pool holds a window and a portion
    per request (simply/utils/ragged_paged_attention.py:95-110), a third of what the other layers' pool holds, and
    generation equals the plain implementation's."""
    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)      # window 8
    w, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 90 + n) for n in (90, 61, 75)]
    want = [plain.greedy(w, cfg, p, 6) for p in prompts]
    m = lm(d, max_seq_len=128, intermediate_steps=1)
    windowed, rest = sorted(m.executor.cache.groups, key=lambda g: g.need.window is None)
    assert windowed.need.window == 8 and rest.need.window is None
    assert rest.pool.num_pages == 3 * 32 and windowed.pool.num_pages == 3 * (2 + 2) + 4
    most = 0
    for i, p in enumerate(prompts):
        m.add_request(i, p, SamplingParams(temperature=0.0, max_decode_steps=6))
    done = []
    while m.scheduler.has_work():
        done += m.step()
        most = max(most, windowed.pool.num_pages - windowed.pool.num_free)
        m.executor.cache.check()
    assert [r.output_token_ids for r in sorted(done, key=lambda r: r.request_id)] == want
    assert m.stats["preemptions"] == 0 and 6 <= most <= windowed.pool.num_pages
    assert windowed.pool.num_free == windowed.pool.num_pages


def test_a_full_batch_past_the_window_still_runs_all_its_steps_in_a_row(tmp_path, cpu_ops):
    """The windowed pool leaves room for `intermediate_steps` tokens ahead of every request: a full batch whose
    requests are all past the window gets runs of that many decode steps, not runs halved for want of pages."""
    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)      # window 8, pages of 4
    _, cfg = plain.load(d)
    m = lm(d, max_seq_len=160, intermediate_steps=16)
    windowed = next(g for g in m.executor.cache.groups if g.need.window is not None)
    assert windowed.pool.num_pages == 3 * (2 + 2) + 3 * 16 // 4
    for i, n in enumerate((40, 33, 47)):     # staggered: the requests cross page edges at different steps
        m.add_request(i, tiny.random_tokens(n, cfg["vocab_size"], 20 + n), SamplingParams(temperature=0.0, max_decode_steps=64,
                                                                                         ignore_eos=True))
    m.step_log = []
    full_runs = 0
    while m.scheduler.has_work():
        left = min((64 - len(r.output_token_ids) for r in m.scheduler.running), default=0)
        decoding = bool(m.scheduler.running) and not m.scheduler.waiting and all(
            r.num_computed == r.num_tokens - 1 for r in m.scheduler.running)
        m.step()
        m.executor.cache.check()
        if decoding:      # a run is as long as the requests' own limits allow: pages never cut it short
            assert m.step_log[-1][0] == min(16, left), (m.step_log[-1], left)
            full_runs += m.step_log[-1][0] == 16
    assert full_runs == 3
    assert m.stats["preemptions"] == 0 and windowed.pool.num_free == windowed.pool.num_pages


def test_an_adopted_request_goes_on_where_one_that_ran_its_prompt_stands(tmp_path, cpu_ops):
    """`adopt_request` (what the benchmark uses to start decoding at a long context): the pages are reserved and given
    back as the prompt's portions would have done, so with the keys and values that the real run left in them the
    adopted request generates the same tokens, windowed layers included; and nothing is left behind afterwards."""
    import pytest
    from simply_amd.cache import OutOfPages

    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)      # window 8, pages of 4, budget 16
    _, cfg = plain.load(d)
    prompt = tiny.random_tokens(45, cfg["vocab_size"], 5)
    params = SamplingParams(temperature=0.0, max_decode_steps=9, ignore_eos=True)
    a = lm(d, max_seq_len=128, intermediate_steps=4)
    want = a.generate([prompt], sampling_params=params)[0].output_token_ids
    b = lm(d, max_seq_len=128, intermediate_steps=4)
    r = b.adopt_request("r", prompt, len(prompt) - 1, params)
    windowed = next(g for g in b.executor.cache.groups if g.need.window is not None)
    assert len(windowed.pages_of("r")) == 5 and r.num_computed == 44       # blocks 6 to 10: the window and the last portion
    for va, vb in zip(a.executor.cache.views, b.executor.cache.views):
        for name, t in va.pages.items():
            vb.pages[name].copy_(t)                                       # the same pages in the same order: see above
    while b.scheduler.has_work():
        b.step()
        b.executor.cache.check()
    assert r.output_token_ids == want
    assert all(g.pool.num_free == g.pool.num_pages for g in b.executor.cache.groups)
    # what does not fit is refused and leaves nothing behind
    c = lm(d, max_seq_len=128, total_num_pages=13)
    c.adopt_request("p", prompt[:20], 19, params)                         # 5 of the 13 pages
    keeps_all = next(g for g in c.executor.cache.groups if g.need.window is None)
    assert keeps_all.pool.num_free == 8
    with pytest.raises(OutOfPages):
        c.adopt_request("r", prompt, len(prompt) - 1, params)             # 11 more do not fit
    assert [r.request_id for r in c.scheduler.running] == ["p"] and list(c.executor.cache.requests) == ["p"]
    assert keeps_all.pool.num_free == 8 and len(keeps_all.pages_of("p")) == 5
    c.executor.cache.check()
    with pytest.raises(ValueError, match="computed tokens"):
        c.adopt_request("q", prompt, len(prompt), params)


def test_sampled_tokens_do_not_depend_on_the_batch(tmp_path, cpu_ops):
    d = tiny.write_model("B", str(tmp_path / "B"), std=0.1)
    _, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 70 + n) for n in (1, 9, 23, 40)]
    plist = [SamplingParams(temperature=0.7, max_decode_steps=6, seed=1000 + i) for i in range(4)]
    together = lm(d, batch_size=4).generate(prompts, sampling_params=plist)
    alone = [lm(d, batch_size=1).generate([p], sampling_params=[sp])[0] for p, sp in zip(prompts, plist)]
    assert [o.output_token_ids for o in together] == [o.output_token_ids for o in alone]
    for a, b in zip(together, alone):
        torch.testing.assert_close(torch.tensor(a.output_token_logprobs), torch.tensor(b.output_token_logprobs),
                                   rtol=1e-4, atol=1e-4)
    # another seed gives another continuation
    other = lm(d, batch_size=1).generate([prompts[3]], sampling_params=[SamplingParams(temperature=0.7, max_decode_steps=6, seed=5)])
    assert other[0].output_token_ids != together[3].output_token_ids


def test_eos_stops(tmp_path, cpu_ops):
    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)
    w, cfg = plain.load(d)
    prompt = tiny.random_tokens(6, cfg["vocab_size"], 3)
    free_run = plain.greedy(w, cfg, prompt, 6)
    import json, os
    cfg["eos_token_id"] = free_run[2]
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    out = lm(d).generate(prompt, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=6))[0]
    stop = free_run.index(free_run[2]) + 1
    assert out.output_token_ids == free_run[:stop] and out.finish_reason == "eos" and not out.is_truncated


def test_steps_in_a_row_change_nothing(tmp_path, cpu_ops):
    """The entry point's bookkeeping for several decode steps per scheduling decision (here through the host,
    step by step): the same tokens as one step at a time, also when requests end inside a run of steps and when
    the pages are so few that runs shrink."""
    d = tiny.write_model("B", str(tmp_path / "B"), std=0.1)
    _, cfg = plain.load(d)
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 80 + n) for n in (2, 9, 13)]
    plist = [SamplingParams(temperature=0.7, max_decode_steps=n, seed=50 + n) for n in (5, 12, 9)]
    one = lm(d, intermediate_steps=1).generate(prompts, sampling_params=plist)
    for steps, pages in ((4, None), (16, None), (16, 9)):
        many = lm(d, intermediate_steps=steps, total_num_pages=pages)
        outs = many.generate(prompts, sampling_params=plist)
        assert [o.output_token_ids for o in outs] == [o.output_token_ids for o in one], (steps, pages)
        assert [o.finish_reason for o in outs] == [o.finish_reason for o in one]
        many.executor.cache.check()
        assert many.stats["steps"] >= max(len(o.output_token_ids) for o in one)


def test_score_tokens(tmp_path, cpu_ops):
    """Scores are the log-softmax of the plain implementation's logits at the next token, in portions beside a
    pool that is used again; greedy scoring says 0 where the token is the argmax."""
    d = tiny.write_model("A", str(tmp_path / "A"), std=0.5)
    w, cfg = plain.load(d)
    toks = tiny.random_tokens(41, cfg["vocab_size"], 90)
    logits = plain.forward(w, cfg, toks[:-1], torch.float64)
    m = lm(d, max_num_issue_tokens=7)
    for _ in range(2):
        got = m.score_tokens(toks)
        want = [plain.log_prob(logits[i], toks[i + 1], 1.0) for i in range(40)]
        assert len(got) == 40 and max(abs(a - b) for a, b in zip(got, want)) < 1e-4
    got = m.score_tokens(toks, ScoringParams(temperature=0.7))
    want = [plain.log_prob(logits[i], toks[i + 1], 0.7) for i in range(40)]
    assert max(abs(a - b) for a, b in zip(got, want)) < 1e-4
    best = [int(torch.argmax(logits[i])) for i in range(40)]
    got = m.score_tokens(toks, ScoringParams(temperature=0.0))
    assert all((g == 0.0) == (toks[i + 1] == best[i]) for i, g in enumerate(got)) and min(got) < -1e37
    assert m.score_tokens([5]) == [] and m.score_tokens([]) == []
    m.executor.cache.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.executor.cache.groups)
