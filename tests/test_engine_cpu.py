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


def test_a_mixer_with_pages_of_its_own_layout(cpu_ops):
    """A toy mixer (tests/toy_parts.py) that keeps one latent vector per token in pages [page, rank, page_size] of
    float32: its need is a class of the test's own, the cache manager forms groups for it (one windowed, one that
    keeps everything), counts their pages and poisons what is given back, and knows nothing of the layout.  Whole,
    cut, and mixed with page reuse give the same logits; the mixer alone equals its whole-sequence formula."""
    import toy_parts
    from simply_amd import registry
    from simply_amd.models import DecoderModel
    from simply_amd.weights import init_random

    registry.MIXERS.register("toy_latent_mean", toy_parts.LatentMeanMixer)
    try:
        model = DecoderModel(toy_parts.latent_model_spec())
        init_random(model, 0, torch.float32, torch.device("cpu"), std=0.2)
        cfg = EngineConfig(activation_dtype="float32", page_size=4, batch_size=3, max_seq_len=64, max_num_issue_tokens=32,
                           total_num_pages=24, device="cpu", use_graphs=False, poison_freed_pages=True, intermediate_steps=1)
        ex = Executor(model, cfg)
        assert len(ex.cache.groups) == 3
        assert [type(g.need).__name__ for g in ex.cache.groups] == ["PagedKVNeed", "LatentNeed", "LatentNeed"]
        assert [g.window for g in ex.cache.groups] == [7, 6, None]
        lat = ex.cache.views[1]
        assert list(lat.pages) == ["latent"] and lat.pages["latent"].shape == (ex.cache.groups[1].pool.num_pages, 12, 4)
        assert lat.k_pages is None and ex.cache.bytes_per_token() == 2 * 2 * 16 * 4 + 48 + 48
        assert ex.cache.groups[1].pool.num_pages == 20 and ex.cache.groups[2].pool.num_pages == 24   # a window's worth only
        reqs = {f"r{i}": tiny.random_tokens(n, 128, 40 + i) for i, n in enumerate((30, 17, 26, 9, 22))}
        whole = {}
        for r, t in reqs.items():
            whole[r] = run_cut(ex, r, t, [len(t)])
            assert torch.isfinite(whole[r]).all() and whole[r].abs().max() > 0
        torch.testing.assert_close(run_cut(ex, "x", reqs["r0"], [7, 2, 9, 1, 11]), whole["r0"], rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(run_cut(ex, "y", reqs["r2"], [1] * 26), whole["r2"], rtol=1e-4, atol=1e-4)
        # mixed, three live at a time in 24 pages of 4 (29 pages' worth in all): pages are used again, poisoned in between
        pending, live, got = list(reqs), {}, {r: [] for r in reqs}
        rng = np.random.default_rng(1)
        while pending or live:
            while pending and len(live) < 3 and sum(-(-len(reqs[r]) // 4) for r in live) + -(-len(reqs[pending[0]]) // 4) <= 24:
                live[pending[0]] = 0
                ex.add_request(pending.pop(0))
            entries = []
            for r in list(live):
                n = min(len(reqs[r]) - live[r], int(rng.integers(1, 8)))
                entries.append(StepEntry(r, reqs[r][live[r]:live[r] + n], list(range(n))))
            logits, i = ex.step(entries), 0
            for e in entries:
                n = len(e.tokens)
                got[e.request_id].append(logits[i:i + n])
                i += n
                live[e.request_id] += n
                if live[e.request_id] == len(reqs[e.request_id]):
                    ex.finish_request(e.request_id)
                    del live[e.request_id]
            ex.cache.check()
        for r in reqs:
            torch.testing.assert_close(torch.cat(got[r]), whole[r], rtol=1e-4, atol=1e-4)
        assert all(g.pool.num_free == g.pool.num_pages for g in ex.cache.groups)
        # the mixer alone against its formula over the whole sequence
        mixer = model.layers[1].mixer
        x = torch.randn(19, 64, generator=torch.Generator().manual_seed(3))
        ex.add_request("m")
        ex.cache.reserve("m", 0, 19)
        from simply_amd.engine.context import GroupStep, StepContext
        tables = ex.cache.sync_tables()
        slot = ex.cache.slot_of("m")
        groups = {g.group_id: GroupStep(tables[g.group_id], torch.from_numpy(ex.cache.slot_mapping(g.group_id, "m", 0, 19)))
                  for g in ex.cache.groups}
        ctx = StepContext(dtype=torch.float32, num_tokens=19, positions=torch.arange(19, dtype=torch.int32),
                          token_seq=torch.full((19,), slot, dtype=torch.int32),
                          seq_meta=torch.tensor([[slot, 0, 19, 0]], dtype=torch.int32), groups=groups, request_ids=["m"],
                          seq_slots=[slot], seq_starts=[0], q_lens=[19], cu_q_lens=[0, 19])
        want = toy_parts.latent_mean_reference(x, mixer.w_in, mixer.w_out, 6)
        torch.testing.assert_close(mixer.forward(x, ctx, ex.cache.views[1]).double(), want, rtol=1e-5, atol=1e-6)
    finally:
        registry.MIXERS.unregister("toy_latent_mean")


def test_an_unknown_kind_of_need_is_refused_with_what_it_lacks():
    from simply_amd.cache import CacheError, CacheManager

    class Odd:
        pass

    with pytest.raises(CacheError, match="neither page_tensors.*nor slot_tensor"):
        CacheManager([(Odd(), None)], page_size=4, num_pages=4, num_slots=1, max_seq_len=16)


def test_partial_sums_are_refused_once_the_workspace_has_been_handed_on():
    """The cuts of a product lie in the one workspace that every kernel with scratch memory shares: reading them
    after another kernel has been given the workspace is an error, not a wrong sum."""
    from simply_amd.kernels import ops

    cpu = torch.device("cpu")
    out = torch.empty(2, 4, dtype=torch.bfloat16)
    ps = ops.PartialSums(torch.zeros(3, 2, 4), out)
    ps.check_fresh()
    ops._workspace(cpu)                   # (as the next kernel with scratch memory would)
    with pytest.raises(ops.KernelError, match="after another kernel had been given the workspace"):
        ps.materialize()
    with pytest.raises(ops.KernelError, match="workspace"):
        ops.add_rmsnorm(ps, torch.zeros(2, 4))
    done = ops.PartialSums(torch.zeros(3, 2, 4), out)
    done.planes = None                    # added up already: nothing to go stale
    ops._workspace(cpu)
    assert done.materialize() is out
