"""The step function at the batch sizes and the context at which the engine is measured: 17 to 64 decoding requests
in one step (the kernels for many rows: products with K cut over workgroups and their sum kernel, the wide gated
product, the separate residual/norm and rotary kernels, decode attention over many requests, graphs of more than 16
rows), a portion of a prompt beside them, several steps in a row on the device, and a context of more than 8192
tokens over a window of 4096.  Every logit is compared with the plain implementation
(batch-composition invariance as simply/model_lib_test.py:664-692 tests it for the reference)."""
import numpy as np
import pytest
import torch

import bounds
import plain_gemma2 as plain
import tiny
from simply_amd.config import EngineConfig, config_from_dict
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.llm import LMInterface
from simply_amd.engine.loading import load_model
from simply_amd.sampling import SamplingParams
from simply_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

GEMMA2_2B_LAYER = dict(hidden_size=2304, num_attention_heads=8, num_key_value_heads=4, head_dim=256,
                       intermediate_size=9216, query_pre_attn_scalar=256)


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


def write_2b_shape(out_dir, window, vocab=2000, seed=5, layers=2):
    d = dict(architectures=["Gemma2ForCausalLM"], num_hidden_layers=layers, vocab_size=vocab, rms_norm_eps=1e-6,
             rope_theta=10000.0, sliding_window=window, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
             max_position_embeddings=16384, initializer_range=0.02, **GEMMA2_2B_LAYER)
    return write_random_model(config_from_dict(d), out_dir, seed, torch.bfloat16, norm_std=0.1)


def decode_together(ex, reqs, first, refs, what, extra_portion=None):
    """Admits every request, runs its first `first[r]` tokens as a portion (several requests to a step), then decodes
    all of them together, one token each per step, until each has run out of tokens (so the number of rows shrinks
    on the way).  `extra_portion` = (request id, tokens): a further request whose prompt runs in portions of 40 beside
    the decoding ones.  Checks every logit that comes back."""
    pos = {}
    batch = []
    portions, decoded = bounds.Pooled(), bounds.Pooled()     # single rows of many requests, pooled for the RMS criterion
    for r, t in reqs.items():
        ex.add_request(r)
        batch.append(StepEntry(r, t[:first[r]], [first[r] - 1]))
        pos[r] = first[r]
        if len(batch) == 8 or r == list(reqs)[-1]:
            logits = ex.step(batch).cpu()
            for i, e in enumerate(batch):
                refs[e.request_id].check(logits[i:i + 1], rows=[first[e.request_id] - 1], what=(what, "portion", e.request_id))
                portions.add(refs[e.request_id], logits[i:i + 1], rows=[first[e.request_id] - 1])
            batch = []
    portions.check((what, "portions"))
    live = list(reqs)
    got = {r: [] for r in reqs}
    extra_at = 0
    if extra_portion is not None:
        ex.add_request(extra_portion[0])
    steps = 0
    while live:
        entries = [StepEntry(r, [reqs[r][pos[r]]], [0]) for r in live]
        if extra_portion is not None and extra_at < len(extra_portion[1]):
            part = extra_portion[1][extra_at:extra_at + 40]
            entries.insert(len(entries) // 2, StepEntry(extra_portion[0], part, list(range(len(part)))))
        logits = ex.step(entries).cpu()
        i = 0
        for e in entries:
            if e.request_id in reqs:
                got[e.request_id].append(logits[i:i + 1])
                i += 1
            else:
                refs[e.request_id].check(logits[i:i + len(e.want)], rows=list(range(extra_at, extra_at + len(e.want))),
                                         what=(what, "portion beside decoding", extra_at))
                i += len(e.want)
                extra_at += len(e.tokens)
        for r in live:
            pos[r] += 1
        for r in [r for r in live if pos[r] == len(reqs[r])]:
            ex.finish_request(r)
            live.remove(r)
        steps += 1
        ex.cache.check()
    for r, t in reqs.items():
        refs[r].check(torch.cat(got[r]), rows=list(range(first[r], len(t))), what=(what, "decode", r))
        decoded.add(refs[r], torch.cat(got[r]), rows=list(range(first[r], len(t))))
    decoded.check((what, "decode steps"))
    if extra_portion is not None:
        ex.finish_request(extra_portion[0])
    return steps


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("num", [17, 33, 64])
def test_many_decoding_requests_tiny(tmp_path, num, dtype, graphs):
    """Head size 64, pages of 16 (the bfloat16 MFMA kernels), 17, 33 and 64 requests of different lengths decoding
    together, finishing at different times."""
    d = tiny.write_model("D", str(tmp_path / "D"), std=0.15)
    w, cfg = plain.load(d)
    rng = np.random.default_rng(num)
    reqs = {f"r{i}": tiny.random_tokens(int(rng.integers(12, 70)), cfg["vocab_size"], 1000 + i) for i in range(num)}
    first = {r: int(rng.integers(1, len(t) - 8)) for r, t in reqs.items()}
    refs = {r: bounds.reference(w, cfg, t, dtype) for r, t in reqs.items()}
    ecfg = EngineConfig(activation_dtype=dtype, page_size=16, batch_size=num, max_seq_len=96, max_num_issue_tokens=512,
                        device="cuda:0", use_graphs=graphs, poison_freed_pages=True)
    model, _ = load_model(d, ecfg.dtype, "cuda:0")
    ex = Executor(model, ecfg)
    steps = decode_together(ex, reqs, first, refs, (num, dtype, graphs))
    assert steps >= 20
    if graphs:
        assert max(k[0] for k in ex._graphs) == num and len(ex._graphs) >= 5   # recorded on the way down, too


LAYER_SIZES = {
    "2b": GEMMA2_2B_LAYER,
    "9b": dict(hidden_size=3584, num_attention_heads=16, num_key_value_heads=8, head_dim=256, intermediate_size=14336,
               query_pre_attn_scalar=256),
    "27b": dict(hidden_size=4608, num_attention_heads=32, num_key_value_heads=16, head_dim=128, intermediate_size=36864,
                query_pre_attn_scalar=144),
}
_drawn = {}


def real_size_model(shape, dtype, window=24, vocab=2000, layers=2):
    """Two layers of the Gemma 2 2B, 9B or 27B sizes with random weights drawn on the GPU (no files: the 27B sizes
    have a billion parameters in two layers).  Returns (model for the engine, the same tensors for the plain
    implementation, the configuration as config.json holds it, the typed configuration)."""
    from simply_amd.models import DecoderModel
    from simply_amd.weights import random_tensors

    d = dict(architectures=["Gemma2ForCausalLM"], num_hidden_layers=layers, vocab_size=vocab, rms_norm_eps=1e-6,
             rope_theta=10000.0, sliding_window=window, attn_logit_softcapping=50.0, final_logit_softcapping=30.0,
             max_position_embeddings=16384, initializer_range=0.02, tie_word_embeddings=True, **LAYER_SIZES[shape])
    cfg = config_from_dict(d)
    key = (shape, window, vocab, layers)
    if key not in _drawn:
        _drawn.clear()          # one set of weights at a time on the GPU
        torch.cuda.empty_cache()
        _drawn[key] = dict(random_tensors(DecoderModel(cfg.model_spec()), 5, torch.bfloat16, norm_std=0.1, device="cuda:0"))
    w = _drawn[key]
    model = DecoderModel(cfg.model_spec())
    model.load_tensors({n: (t.float() if dtype == "float32" else t) for n, t in w.items()})
    return model, w, d, cfg


@pytest.fixture(scope="module", autouse=True)
def _forget_drawn_weights():
    yield
    _drawn.clear()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,num", [("2b", 40), ("9b", 40), ("9b", 64), ("27b", 40), ("27b", 64)])
def test_many_decoding_requests_at_real_layer_sizes(shape, num, dtype):
    """The layer sizes that the engine is measured at (two layers of Gemma 2 2B, 9B and 27B): 40 and 64 requests
    decoding together and finishing at different times (every number of rows from there down to one: the products'
    routes for 17 to 64 rows, for 9 to 16 and for fewer, the norms in front of the products at widths 2304, 3584 and
    4608, decode attention with 2, 2 and 2 query heads per key head at head sizes 256 and 128), a prompt of 200
    tokens running in portions beside them, recorded graphs where the step is decode-only."""
    model, w, cfg, _ = real_size_model(shape, dtype)
    rng = np.random.default_rng(3)
    reqs = {f"r{i}": tiny.random_tokens(int(rng.integers(14, 34)), 2000, 2000 + i) for i in range(num)}
    first = {r: int(rng.integers(1, len(t) - 8)) for r, t in reqs.items()}
    extra = ("long", tiny.random_tokens(200, 2000, 77))
    everything = dict(reqs, long=extra[1])
    refs = {r: bounds.reference(w, cfg, t, dtype, device="cuda:0") for r, t in everything.items()}
    ecfg = EngineConfig(activation_dtype=dtype, page_size=16, batch_size=num + 1, max_seq_len=256, max_num_issue_tokens=512,
                        device="cuda:0", use_graphs=True, poison_freed_pages=True)
    ex = Executor(model, ecfg)
    decode_together(ex, reqs, first, refs, (shape, num, dtype), extra_portion=extra)
    assert ex._graphs, "the steps after the long prompt's last portion are decode-only and recorded"


@pytest.mark.parametrize("shape", ["9b", "27b"])
def test_generation_at_real_layer_sizes(shape):
    """Through the entry point at the 9B and 27B layer sizes: 20 requests generating greedily, eight decode steps in
    a row on the device (the recorded graph of model, sampler and hand-over at more than 16 rows).  In 32-bit the
    tokens are the plain implementation's.  In bfloat16 every token is the best of the exact logits given the tokens
    before it, or within the bound on the logits' error of the best; and the same tokens come out one step at a time."""
    num, new = 20, 10
    rng = np.random.default_rng(11)
    prompts = [tiny.random_tokens(int(rng.integers(3, 40)), 2000, 500 + i) for i in range(num)]
    params = SamplingParams(temperature=0.0, max_decode_steps=new, ignore_eos=True)
    kw = dict(batch_size=num, max_seq_len=64, page_size=16, max_num_issue_tokens=256, device="cuda:0")
    model, w, cfg, typed = real_size_model(shape, "float32")
    on_gpu = {k: v.to("cuda:0") for k, v in w.items()}
    lm = LMInterface(config=typed, activation_dtype="float32", intermediate_steps=8, _model=model, **kw)
    got = [o.output_token_ids for o in lm.generate(prompts, sampling_params=params)]
    assert any(k[0] == "many" and k[1] > 16 for k in lm.executor._graphs)
    for p, g in zip(prompts, got):
        logits = plain.forward(on_gpu, cfg, list(p) + g[:-1], torch.float64, device="cuda:0")[len(p) - 1:]
        assert logits.argmax(dim=-1).tolist() == g, p
    del lm, model
    model, w, cfg, typed = real_size_model(shape, "bfloat16")
    runs = {}
    for steps in (8, 1):
        lm = LMInterface(config=typed, activation_dtype="bfloat16", intermediate_steps=steps, _model=model, **kw)
        runs[steps] = [o.output_token_ids for o in lm.generate(prompts, sampling_params=params)]
        lm.executor.cache.check()
    assert runs[8] == runs[1]
    for p, g in zip(prompts, runs[8]):
        ref = bounds.reference(on_gpu, cfg, list(p) + g[:-1], "bfloat16", device="cuda:0", rows=slice(len(p) - 1, None))
        slack = 2 * ref.max_bound() * ref.scale
        for i, tok in enumerate(g):
            assert ref.want[i][tok] >= ref.want[i].max() - slack, (p, i, float(ref.want[i].max() - ref.want[i][tok]), slack)


@pytest.mark.parametrize("num", [17, 33, 64])
def test_generation_with_many_requests(tmp_path, num):
    """Through the entry point: greedy generation of 17, 33 and 64 requests at once, several decode steps in a row on
    the device (recorded graphs that hold model, sampler and the hand-over of the drawn tokens).  In 32-bit the tokens
    are the plain implementation's; in bfloat16 they are the same whether the steps run in a row on the device, one
    at a time through graphs, or without graphs (the same kernels, the same numbers), and every token is the best of
    the exact logits given the tokens before it, or within the bound on the logits' error of the best."""
    d = tiny.write_model("D", str(tmp_path / "D"), std=0.15)
    w, cfg = plain.load(d)
    rng = np.random.default_rng(100 + num)
    prompts = [tiny.random_tokens(int(rng.integers(1, 40)), cfg["vocab_size"], 3000 + i) for i in range(num)]
    steps = [int(rng.integers(9, 20)) for _ in range(num)]    # the first eight decode steps run in a row, all rows
    plist = [SamplingParams(temperature=0.0, max_decode_steps=s, ignore_eos=True) for s in steps]
    want = [plain.greedy(w, cfg, p, s, torch.float64) for p, s in zip(prompts, steps)]

    def run(dtype, **kw):
        lm = LMInterface(d, activation_dtype=dtype, batch_size=num, max_seq_len=64, page_size=16, max_num_issue_tokens=256,
                         device="cuda:0", **kw)
        outs = lm.generate(prompts, sampling_params=plist)
        lm.executor.cache.check()
        return [o.output_token_ids for o in outs], lm

    got, lm = run("float32", intermediate_steps=8)
    assert got == want
    assert any(k[0] == "many" and k[1] > 16 for k in lm.executor._graphs)   # steps in a row on the device, > 16 rows
    in_a_row, _ = run("bfloat16", intermediate_steps=8)
    one_by_one, _ = run("bfloat16", intermediate_steps=1)
    eager, _ = run("bfloat16", intermediate_steps=1, use_graphs=False)
    assert in_a_row == one_by_one == eager
    for p, g in zip(prompts, in_a_row):
        ref = bounds.reference(w, cfg, list(p) + g[:-1], "bfloat16", rows=slice(len(p) - 1, None))
        slack = 2 * ref.max_bound() * ref.scale      # both the best and the chosen logit may be off by the bound
        for i, tok in enumerate(g):
            assert ref.want[i][tok] >= ref.want[i].max() - slack, (p, i, float(ref.want[i].max() - ref.want[i][tok]), slack)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_context_of_8192_over_a_window_of_4096(tmp_path, dtype):
    """The measured context: two layers of Gemma 2 2B (one windowed, 4096 keys; one that sees everything), pages of
    16, a prompt of 8200 tokens in portions of 2048, then 64 decode steps through recorded graphs.  The last portion's
    logits and every decode step's are compared with the plain implementation (computed in float64 by torch on the
    GPU: 4 Tflop); on the way the windowed layer never holds more than its window and the step's portion
    (simply/utils/ragged_paged_attention.py:437-472 releases what the window has passed before every step)."""
    d = write_2b_shape(str(tmp_path / "m"), window=4096, vocab=512, seed=9)
    w, cfg = plain.load(d)
    prompt, steps, portion, P = 8200, 64, 2048, 16
    tokens = tiny.random_tokens(prompt + steps, 512, 55)
    last = (prompt - 1) // portion * portion          # where the prompt's last portion begins
    ref = bounds.reference(w, cfg, tokens, dtype, device="cuda:0", rows=slice(last, None))
    torch.cuda.empty_cache()
    ecfg = EngineConfig(activation_dtype=dtype, page_size=P, batch_size=2, max_seq_len=prompt + steps + 8,
                        max_num_issue_tokens=portion, device="cuda:0", use_graphs=True, poison_freed_pages=True)
    model, _ = load_model(d, ecfg.dtype, "cuda:0")
    ex = Executor(model, ecfg)
    windowed = next(g for g in ex.cache.groups if g.need.window == 4096)
    assert windowed.pool.num_pages == 2 * (256 + 2) + portion // P          # a window per request and a step's tokens
    ex.add_request("r")
    got, most = [], 0
    for at in range(0, prompt, portion):
        part = tokens[at:min(at + portion, prompt)]
        logits = ex.step([StepEntry("r", part, list(range(len(part))) if at == last else [])])
        most = max(most, len(windowed.pages_of("r")))
        assert len(windowed.pages_of("r")) <= 4096 // P + 1 + portion // P
        if logits is not None:
            got.append(logits.cpu())
    for i in range(steps):
        got.append(ex.step([StepEntry("r", [tokens[prompt + i]], [0])]).cpu())
        assert len(windowed.pages_of("r")) <= 4096 // P + 1
    assert most > 4096 // P and len(ex._graphs) == 1
    ex.cache.check()
    ref.check(torch.cat(got), what=dtype)
    ex.finish_request("r")
    assert windowed.pool.num_free == windowed.pool.num_pages
