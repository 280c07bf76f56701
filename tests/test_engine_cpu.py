"""The engine's host logic (step function, cache bookkeeping) with the kernels replaced by their
plain torch references: every way of cutting the work gives the plain implementation's logits."""
import numpy as np
import pytest
import torch

import plain_gemma2 as plain
import tiny
from simply_amd.config import EngineConfig
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.loading import load_model


def make_executor(model_dir, page_size=4, num_pages=64, batch=4, max_len=256):
    model, _ = load_model(model_dir, torch.float32, "cpu")
    cfg = EngineConfig(activation_dtype="float32", page_size=page_size, batch_size=batch, max_seq_len=max_len,
                       max_num_issue_tokens=max_len, total_num_pages=num_pages, device="cpu", use_graphs=False)
    return Executor(model, cfg)


def run_cut(ex, rid, tokens, cuts):
    """Feeds `tokens` in portions of the given sizes, wanting every position; returns [T, V]."""
    out, i = [], 0
    ex.add_request(rid)
    for c in cuts:
        part = tokens[i:i + c]
        out.append(ex.step([StepEntry(rid, part, list(range(len(part))))]))
        i += len(part)
    assert i == len(tokens)
    ex.finish_request(rid)
    ex.cache.check()
    return torch.cat(out)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuts_match_plain(tmp_path, cpu_ops, name):
    d = tiny.write_model(name, str(tmp_path / name), std=0.3)
    w, cfg = plain.load(d)
    tokens = tiny.random_tokens(45, cfg["vocab_size"], 7)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d)
    scale = want.abs().max().item()
    for cuts in ([45], [13] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 13], [1] * 45):
        got = run_cut(ex, "r", tokens, cuts)
        assert (got - want).abs().max().item() <= 2e-5 * scale, cuts


@pytest.mark.parametrize("head_dim", [2, 6, 24, 40])
def test_head_sizes_that_are_even_but_no_multiple_of_16(tmp_path, cpu_ops, head_dim):
    """Every even head size that the configuration allows builds and runs (rotary pairs are all that the
    architecture asks of it: simply/utils/position_encoding.py:83-84)."""
    d = tiny.write_config_model(tiny.odd_head_size_config(head_dim), str(tmp_path / "m"), seed=head_dim, std=0.3)
    w, cfg = plain.load(d)
    tokens = tiny.random_tokens(30, cfg["vocab_size"], 3)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d)
    for cuts in ([30], [12] + [1] * 18, [7, 5, 3, 2, 11, 2]):
        got = run_cut(ex, "r", tokens, cuts)
        assert (got - want).abs().max().item() <= 2e-5 * want.abs().max().item(), cuts


def test_mixed_with_page_reuse(tmp_path, cpu_ops):
    d = tiny.write_model("B", str(tmp_path / "B"), std=0.3)
    w, cfg = plain.load(d)
    V = cfg["vocab_size"]
    reqs = {f"r{i}": tiny.random_tokens(n, V, 100 + i) for i, n in enumerate([40, 23, 9, 31, 17, 1, 26])}
    want = {r: plain.forward(w, cfg, t) for r, t in reqs.items()}
    # 28 pages of 4 tokens: far fewer than the 147 tokens of all requests need, so pages are used again
    ex = make_executor(d, page_size=4, num_pages=28, batch=4, max_len=64)
    pending = list(reqs)
    live, done_at, got = {}, {}, {r: [] for r in reqs}
    rng = np.random.default_rng(0)
    step = 0
    while pending or live:
        while pending and len(live) < 4:
            nxt = pending[0]
            need = -(-len(reqs[nxt]) // 4)
            held = sum(-(-len(reqs[r]) // 4) for r in live)
            if held + need > 28:
                break
            pending.pop(0)
            live[nxt] = 0
            ex.add_request(nxt)
        entries = []
        for r in list(live):
            left = len(reqs[r]) - live[r]
            if rng.random() < 0.2 and len(live) > 1:
                continue  # left out of this step
            n = 1 if rng.random() < 0.4 else int(rng.integers(1, min(left, 9) + 1))
            entries.append(StepEntry(r, reqs[r][live[r]:live[r] + n], list(range(n))))
        if not entries:
            continue
        logits = ex.step(entries)
        i = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request_id].append(logits[i:i + n])
            i += n
            live[e.request_id] += n
            if live[e.request_id] == len(reqs[e.request_id]):
                ex.finish_request(e.request_id)
                del live[e.request_id]
        ex.cache.check()
        step += 1
    for r in reqs:
        g = torch.cat(got[r])
        assert (g - want[r]).abs().max().item() <= 2e-5 * want[r].abs().max().item(), r
    assert all(g.pool.num_free == 28 for g in ex.cache.groups)
