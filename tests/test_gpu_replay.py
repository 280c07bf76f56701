"""bin/trace_run as a user runs it (a child process fed through standard input), in float32 and in
bfloat16: whole requests, the last 32 tokens one by one, portions of changing size down to two tokens,
and up to four live requests mixed with so few pages that they are used again; long decoding and the
first tokens of a sequence.  All compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import bounds
import plain_gemma2 as plain
import tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class TraceRun:
    def __init__(self, model_dir, dtype, out_dir, max_tokens, extra=()):
        self.out_dir = out_dir
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out",
             out_dir, "--max-tokens", str(max_tokens), *extra],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.step = 0

    def run(self, entries, end=()):
        """entries: [(id, tokens, want)].  Returns the logits [wanted, vocab] or None."""
        rec = {"step": self.step, "entries": [{"id": i, "tokens": list(t), "want": list(w)} for i, t, w in entries],
               "end": list(end)}
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {self.step}", (line, self.proc.poll())
        path = os.path.join(self.out_dir, f"{self.step}.f32")
        self.step += 1
        n = sum(len(w) for _, _, w in entries)
        if n == 0:
            assert not os.path.exists(path)
            return None
        return torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n, -1).copy())

    def close(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=60) == 0


def feed(tr, rid, tokens, cuts, end=True):
    out, i = [], 0
    for j, c in enumerate(cuts):
        part = tokens[i:i + c]
        last = j == len(cuts) - 1
        out.append(tr.run([(rid, part, range(len(part)))], end=[rid] if (end and last) else []))
        i += len(part)
    assert i == len(tokens)
    return torch.cat(out)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_all_cuts(tmp_path, name, dtype):
    d = tiny.write_model(name, str(tmp_path / "m"), dtype=torch.bfloat16, std=0.3)
    w, cfg = plain.load(d)
    V = cfg["vocab_size"]
    reqs = {f"r{i}": tiny.random_tokens(n, V, 10 + i) for i, n in enumerate([70, 45, 100, 33, 64, 2, 90])}
    refs = {r: bounds.reference(w, cfg, t, dtype) for r, t in reqs.items()}
    # 320 tokens = 20 pages of 16: less than the 404 tokens that all requests hold together
    tr = TraceRun(d, dtype, str(tmp_path / "out"), 320, extra=["--poison"])
    try:
        toks = reqs["r0"]
        refs["r0"].check(feed(tr, "whole", toks, [len(toks)]), what="whole")
        refs["r0"].check(feed(tr, "tail", toks, [len(toks) - 32] + [1] * 32), what="tail")
        refs["r0"].check(feed(tr, "cuts", toks, [9, 7, 5, 3, 2, 16, 2, 2, 11, 13]), what="cuts")
        refs["r0"].check(feed(tr, "first", toks, [1, 1, 1, 2, 3, 62]), what="first")
        # mixed: up to four live requests, portions of some beside single tokens of others, requests left out of
        # steps, nothing wanted in some portions
        rng = np.random.default_rng(1)
        pending, live, got = list(reqs), {}, {r: {} for r in reqs}
        while pending or live:
            while pending and len(live) < 4:
                held = sum(-(-len(reqs[r]) // 64) * 64 for r in live)
                if held + -(-len(reqs[pending[0]]) // 64) * 64 > 320:
                    break
                live[pending.pop(0)] = 0
            entries, ends = [], []
            for r in list(live):
                left = len(reqs[r]) - live[r]
                if rng.random() < 0.25 and len(live) > 1:
                    continue
                n = 1 if rng.random() < 0.4 else int(rng.integers(2, min(left, 23) + 1)) if left >= 2 else 1
                wanted = list(range(n)) if rng.random() < 0.8 else []
                entries.append((r, reqs[r][live[r]:live[r] + n], wanted))
            if not entries:
                continue
            for r, t, _ in entries:
                if live[r] + len(t) == len(reqs[r]):
                    ends.append(r)
            logits = tr.run(entries, end=ends)
            i = 0
            for r, t, wanted in entries:
                for wpos in wanted:
                    got[r][live[r] + wpos] = logits[i]
                    i += 1
                live[r] += len(t)
                if r in ends:
                    del live[r]
        for r in reqs:
            pos = sorted(got[r])
            assert len(pos) > 0
            refs[r].check(torch.stack([got[r][p] for p in pos]), rows=pos, what=r)
    finally:
        tr.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_long_decoding(tmp_path, dtype):
    """300 tokens one by one after a short prompt: windows slide over many pages, pages are given back on the way."""
    d = tiny.write_model("A", str(tmp_path / "m"), dtype=torch.bfloat16, std=0.3)
    w, cfg = plain.load(d)
    toks = tiny.random_tokens(320, cfg["vocab_size"], 99)
    ref = bounds.reference(w, cfg, toks, dtype)
    tr = TraceRun(d, dtype, str(tmp_path / "out"), 320, extra=["--poison"])
    try:
        ref.check(feed(tr, "long", toks, [20] + [1] * 300), what="long")
    finally:
        tr.close()


def test_replay_says_which_line_is_wrong(tmp_path):
    """A step that cannot be run ends the program with status 1 and one line that names it: broken JSON, a wanted
    place outside the tokens, a token outside the vocabulary, more tokens than the pool holds."""
    d = tiny.write_model("A", str(tmp_path / "m"), dtype=torch.bfloat16, std=0.3)
    good = '{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [2]}], "end": []}'
    bad = {
        "JSONDecodeError": '{"step": 1, "entries": [',
        "wanted place": '{"step": 1, "entries": [{"id": "a", "tokens": [5, 6], "want": [2]}], "end": []}',
        "token id": '{"step": 1, "entries": [{"id": "a", "tokens": [5, 100000], "want": []}], "end": []}',
        "OutOfPages": json.dumps({"step": 1, "entries": [{"id": "b", "tokens": [1] * 64, "want": []}], "end": []}),
    }
    for what, line in bad.items():
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                            "--out", str(tmp_path / "out"), "--max-tokens", "64"], input=good + "\n" + line + "\n",
                           capture_output=True, text=True, timeout=120)
        assert p.returncode == 1, (what, p.returncode, p.stderr[-300:])
        assert p.stdout.strip() == "done 0"
        last = p.stderr.strip().splitlines()[-1]
        assert last.startswith("trace_run: line 2") and what in last, (what, last)
