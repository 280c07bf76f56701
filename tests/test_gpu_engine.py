"""The engine on the GPU against the plain implementation, in float32 and in bfloat16, under every
way of cutting the work."""
import numpy as np
import pytest
import torch

import bounds
import plain_gemma2 as plain
import tiny
from simply_amd.config import EngineConfig
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.loading import load_model

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


def make_executor(model_dir, dtype, page_size=4, num_pages=64, batch=4, max_len=256, poison=True):
    cfg = EngineConfig(activation_dtype=dtype, page_size=page_size, batch_size=batch, max_seq_len=max_len,
                       max_num_issue_tokens=max_len, total_num_pages=num_pages, device="cuda:0", use_graphs=False,
                       poison_freed_pages=poison)
    model, _ = load_model(model_dir, cfg.dtype, "cuda:0")
    return Executor(model, cfg)


def run_cut(ex, rid, tokens, cuts):
    out, i = [], 0
    ex.add_request(rid)
    for c in cuts:
        part = tokens[i:i + c]
        out.append(ex.step([StepEntry(rid, part, list(range(len(part))))]).cpu())
        i += len(part)
    assert i == len(tokens)
    ex.finish_request(rid)
    ex.cache.check()
    return torch.cat(out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "U"])
def test_cuts_match_plain(tmp_path, name, dtype):
    d = tiny.write_model(name, str(tmp_path / name), std=0.3)
    vocab = plain.load(d)[1]["vocab_size"]
    tokens = tiny.random_tokens(77, vocab, 7)
    ref = bounds.reference_of(d, tokens, dtype)
    ex = make_executor(d, dtype)
    for cuts in ([77], [45] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 13, 17, 2, 13], [1] * 77):
        ref.check(run_cut(ex, "r", tokens, cuts), what=cuts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_match_plain_at_kernel_sizes(tmp_path, dtype):
    """Head size 64 and pages of 16: the sizes at which the bfloat16 path runs its MFMA kernels."""
    d = tiny.write_model("D", str(tmp_path / "D"), std=0.15)
    vocab = plain.load(d)[1]["vocab_size"]
    tokens = tiny.random_tokens(150, vocab, 8)
    ref = bounds.reference_of(d, tokens, dtype)
    ex = make_executor(d, dtype, page_size=16, num_pages=24, max_len=320)
    for cuts in ([150], [118] + [1] * 32, [40, 7, 5, 3, 2, 30, 2, 2, 13, 17, 2, 27], [1] * 150, [3, 4, 2] * 16 + [6]):
        ref.check(run_cut(ex, "r", tokens, cuts), what=cuts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_match_eager(tmp_path, dtype):
    """Decode-only steps run through captured HIP graphs: every replay (with the host's own work and
    synchronisation between them) gives what the eager step gives, for changing numbers of requests."""
    d = tiny.write_model("D", str(tmp_path / "D"), std=0.15)
    vocab = plain.load(d)[1]["vocab_size"]
    reqs = {f"r{i}": tiny.random_tokens(40 + 7 * i, vocab, 20 + i) for i in range(3)}
    outs = {}
    for graphs in (False, True):
        cfg = EngineConfig(activation_dtype=dtype, page_size=16, batch_size=4, max_seq_len=128, max_num_issue_tokens=128,
                           total_num_pages=32, device="cuda:0", use_graphs=graphs)
        model, _ = load_model(d, cfg.dtype, "cuda:0")
        ex = Executor(model, cfg)
        got = {r: [] for r in reqs}
        for r, t in reqs.items():
            ex.add_request(r)
            got[r].append(ex.step([StepEntry(r, t[:20], [19])]).cpu())
        pos = {r: 20 for r in reqs}
        live = list(reqs)
        while live:
            logits = ex.step([StepEntry(r, [reqs[r][pos[r]]], [0]) for r in live]).cpu()
            for i, r in enumerate(live):
                got[r].append(logits[i:i + 1])
                pos[r] += 1
            for r in [r for r in live if pos[r] == len(reqs[r])]:
                ex.finish_request(r)
                live.remove(r)
        if graphs:
            assert sorted({k[0] for k in ex._graphs}) == [1, 2, 3]   # recorded per number of requests (and context scale)
        outs[graphs] = {r: torch.cat(v) for r, v in got.items()}
    for r in reqs:
        assert torch.equal(outs[False][r], outs[True][r]), r
    for r, t in reqs.items():
        bounds.reference_of(d, t, dtype).check(outs[True][r], rows=slice(19, None), what=r)


def mixed_requests_in_a_tight_pool(model_dir, page, lens, seed, rms_per_request=True):
    """Up to four live requests cut at random into portions and single tokens, in a pool that is smaller than what
    all requests hold: in 32-bit against the plain implementation; in bfloat16 against the plain implementation
    (within the bound derived for the model, `bounds`) and against the same requests run whole and alone, where only
    the rounding of other kernels may differ.  rms_per_request=False: the RMS criterion over all requests together
    only (for models whose rounding noise has too few independent sources for one request's sample to mean much)."""
    w0, pcfg = plain.load(model_dir)
    rng = np.random.default_rng(seed)
    reqs = {f"r{i}": tiny.random_tokens(n, pcfg["vocab_size"], seed * 100 + i) for i, n in enumerate(lens)}
    pages_of = lambda n: -(-n // page) + 1
    num_pages = max(pages_of(max(lens)) + 2, int(sum(pages_of(n) for n in lens) * 0.6))
    for dtype in ("float32", "bfloat16"):
        refs = {r: bounds.reference(w0, pcfg, t, dtype) for r, t in reqs.items()}
        ex = make_executor(model_dir, dtype, page_size=page, num_pages=num_pages)
        pending, live, got = list(reqs), {}, {r: {} for r in reqs}
        while pending or live:
            while pending and len(live) < 4:
                if sum(pages_of(len(reqs[r])) for r in live) + pages_of(len(reqs[pending[0]])) > num_pages:
                    break
                live[pending[0]] = 0
                ex.add_request(pending.pop(0))
            entries = []
            for r in list(live):
                left = len(reqs[r]) - live[r]
                if rng.random() < 0.25 and len(live) > 1:
                    continue
                n = 1 if (left < 2 or rng.random() < 0.4) else int(rng.integers(2, min(left, 40) + 1))
                entries.append(StepEntry(r, reqs[r][live[r]:live[r] + n], list(range(n)) if rng.random() < 0.8 else []))
            if not entries:
                continue
            logits = ex.step(entries)
            i = 0
            for e in entries:
                r = e.request_id
                for at in e.want:
                    got[r][live[r] + at] = logits[i].cpu()
                    i += 1
                live[r] += len(e.tokens)
                if live[r] == len(reqs[r]):
                    ex.finish_request(r)
                    del live[r]
            ex.cache.check()
        pooled = bounds.Pooled()      # short requests have too few rows for the RMS criterion alone: all of them together
        for r, t in reqs.items():
            at = sorted(got[r])
            if not at:
                continue
            g = torch.stack([got[r][p] for p in at]).double()
            refs[r].check(g, rows=at, what=(dtype, r), rms=rms_per_request)
            pooled.add(refs[r], g, rows=at)
            if dtype == "bfloat16":
                # cut and mixed against whole and alone: the same arithmetic but for the kernels that few rows and
                # many rows go through; bounded by the same rounded run
                ex.add_request(r)
                whole = ex.step([StepEntry(r, t, list(range(len(t))))]).cpu().double()
                ex.finish_request(r)
                refs[r].check(whole, what=(dtype, r, "whole"), rms=rms_per_request)
                assert (g - whole[at]).abs().max().item() / refs[r].scale <= refs[r].max_bound(), (dtype, r)
        pooled.check((dtype, "all requests"))


@pytest.mark.parametrize("seed", range(100, 112))
def test_random_configurations_mixed(tmp_path, seed):
    """Configurations drawn at random (tiny.random_config): head counts and sizes, widths that are no multiple of 8,
    layer kinds in any order."""
    d = tiny.write_random_config_model(seed, str(tmp_path / "m"))
    rng = np.random.default_rng(seed)
    page = int(rng.choice([4, 8, 16, 16, 32]))
    lens = [int(rng.integers(2, 130)) for _ in range(int(rng.integers(3, 6)))]
    mixed_requests_in_a_tight_pool(d, page, lens, seed)


@pytest.mark.parametrize("head_dim", [2, 6, 24, 40, 72])
def test_head_sizes_that_are_even_but_no_multiple_of_16(tmp_path, head_dim):
    """Every even head size that the configuration allows runs (on the kernels that take every size), in both
    element types, mixed in a tight pool (simply/utils/position_encoding.py:83-84 asks only for halves)."""
    d = tiny.write_config_model(tiny.odd_head_size_config(head_dim), str(tmp_path / "m"), seed=head_dim, std=0.2)
    # With heads of one rotary pair the ratio of the engine's RMS error to the rounded plain run's scatters from 0.6
    # to 1.4 from request to request, whole or cut alike (0.85 to 1.16 from six dimensions on), and from 0.85 to 1.18
    # over four requests together: there the RMS criterion is applied to the requests together.
    mixed_requests_in_a_tight_pool(d, 8 if head_dim != 24 else 16, [33, 70, 9, 51], 300 + head_dim,
                                   rms_per_request=head_dim > 2)


@pytest.mark.parametrize("case", [4, 11, 21, 36, 94, 135, "smallest"])
def test_configurations_with_the_largest_bfloat16_error(tmp_path, case):
    """The configurations on which bfloat16 logits lie furthest from the float64 ones (tiny.drawn_case): 4 to 9 % of
    the largest logit, where the usual configuration gives 0.3 to 1 %.  The plain implementation with rounding at the
    same places is as far off (tests/test_plain.py shows on the CPU where the error enters), so the bound that is
    derived from it holds here as everywhere."""
    d, page, lens = tiny.write_drawn_case(case, str(tmp_path / "m"))
    mixed_requests_in_a_tight_pool(d, page, lens, 7 if case == "smallest" else case)
