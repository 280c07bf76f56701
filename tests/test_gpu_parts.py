"""Each part alone against the plain implementation's function for it, and the framework's generality:
a toy mixer with state of its own, a toy feed-forward with routing and another position encoding are
defined here, registered, built into a model and stepped, without a change to the framework's files."""
import dataclasses
import math

import pytest
import torch

import plain_gemma2 as plain
import tiny
from simply_amd import registry
from simply_amd.cache import CacheManager
from simply_amd.config import EngineConfig, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, config_from_dict
from simply_amd.engine import Executor, StepEntry
from simply_amd.engine.context import GroupStep, StepContext
from simply_amd.kernels import ops
from simply_amd.models import DecoderModel
from simply_amd.parts.base import FeedForward, Mixer, PagedKVNeed, ParamSpec, PositionEncoding, StateNeed
from simply_amd.weights import init_random

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


def rand(shape, seed, scale=1.0, dtype=torch.float32):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype).to(DEV)


def whole_sequence_ctx(T, dtype, page_size, needs, num_pages=64):
    """One request of T tokens from position 0, with a cache for `needs`."""
    cache = CacheManager([(n, None) for n in needs], page_size=page_size, num_pages=num_pages, num_slots=2,
                         max_seq_len=num_pages * page_size, dtype=dtype, device=torch.device(DEV))
    cache.admit("r")
    cache.reserve("r", 0, T)
    tables = cache.sync_tables()
    slot = cache.slot_of("r")
    groups = {g.group_id: GroupStep(tables[g.group_id],
                                    torch.from_numpy(cache.slot_mapping(g.group_id, "r", 0, T)).to(DEV))
              for g in cache.groups}
    ctx = StepContext(dtype=dtype, num_tokens=T, positions=torch.arange(T, dtype=torch.int32, device=DEV),
                      token_seq=torch.full((T,), slot, dtype=torch.int32, device=DEV),
                      seq_meta=torch.tensor([[slot, 0, T, 0]], dtype=torch.int32, device=DEV), groups=groups,
                      request_ids=["r"], seq_slots=[slot], seq_starts=[0], q_lens=[T], cu_q_lens=[0, T])
    return ctx, cache


# ------------------------------------------------------------------ the built-in parts, one by one
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    part = registry.NORMS.build("rmsnorm", dim=100, eps=1e-5, scale_plus_one=True)
    w = rand((100,), 1, 0.2)
    part.load({"scale": w.to(dtype)})
    x = rand((7, 100), 2, 3.0)
    want = plain.rms_norm(x.double().cpu(), w.to(dtype).double().cpu(), 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    torch.testing.assert_close(part.forward(x, dtype).double().cpu(), want, rtol=tol, atol=tol)
    # residual += norm(y), fused with the next norm
    nxt = registry.NORMS.build("rmsnorm", dim=100, eps=1e-6, scale_plus_one=True)
    w2 = rand((100,), 3, 0.2)
    nxt.load({"scale": w2.to(dtype)})
    h, y = rand((7, 100), 4), rand((7, 100), 5).to(dtype)
    h_want = h.double().cpu() + plain.rms_norm(y.double().cpu(), w.to(dtype).double().cpu(), 1e-5)
    out = part.add_into(h, y, nxt, dtype)
    torch.testing.assert_close(h.double().cpu(), h_want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(out.double().cpu(), plain.rms_norm(h_want, w2.to(dtype).double().cpu(), 1e-6),
                               rtol=tol, atol=tol)


def test_rope_part():
    part = registry.POSITION_ENCODINGS.build("rope", head_dim=32, base=1000000.0)
    part.to_device(torch.device(DEV))
    x = rand((9, 3 * 32), 6)
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 7, 511, 5], dtype=torch.int32, device=DEV)
    want = plain.rope(x.double().cpu().reshape(9, 3, 32), pos.cpu(), 1000000.0).reshape(9, 96) / 4.0
    part.apply(x, pos, 3, 32, 4.0)
    torch.testing.assert_close(x.double().cpu(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    D, F = 96, 200
    part = registry.FEED_FORWARDS.build("gated_dense", hidden_size=D, intermediate_size=F)
    w = {n: rand(s, 10 + i, 0.1).to(dtype) for i, (n, s) in enumerate((("gate_proj", (F, D)), ("up_proj", (F, D)),
                                                                       ("down_proj", (D, F))))}
    part.load(w)
    x = rand((11, D), 13).to(dtype)
    pw = {"p." + n + ".weight": t.double().cpu() for n, t in w.items()}
    want = plain.feed_forward(x.double().cpu(), pw, "p.")
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    torch.testing.assert_close(part.forward(x).double().cpu(), want, rtol=tol, atol=tol * want.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("activation", ["silu", "squared_relu"])
def test_feed_forward_part_with_another_activation(dtype, activation):
    """The gated feed-forward takes its activation by name from the registry; the ones beside Gemma 2's own."""
    D, F = 96, 200
    part = registry.FEED_FORWARDS.build("gated_dense", hidden_size=D, intermediate_size=F, activation=activation)
    w = {n: rand(s, 10 + i, 0.1).to(dtype) for i, (n, s) in enumerate((("gate_proj", (F, D)), ("up_proj", (F, D)),
                                                                       ("down_proj", (D, F))))}
    part.load(w)
    x = rand((11, D), 13).to(dtype)
    g, u, d = (w[n].double().cpu() for n in ("gate_proj", "up_proj", "down_proj"))
    xd = x.double().cpu()
    act = {"silu": torch.nn.functional.silu, "squared_relu": lambda v: torch.relu(v) ** 2}[activation]
    want = (act(xd @ g.T) * (xd @ u.T)) @ d.T
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    torch.testing.assert_close(part.forward(x).double().cpu(), want, rtol=tol, atol=tol * want.abs().max().item())
    with pytest.raises(ValueError, match="unknown activation"):
        registry.FEED_FORWARDS.build("gated_dense", hidden_size=D, intermediate_size=F, activation="swish7")


@pytest.mark.parametrize("dtype,hd,page", [(torch.float32, 16, 4), (torch.bfloat16, 16, 4), (torch.bfloat16, 64, 16)])
@pytest.mark.parametrize("window", [None, 8])
def test_attention_part(dtype, hd, page, window):
    D, H, K, T = 64, 4, 2, 40
    cfg = dict(num_attention_heads=H, num_key_value_heads=K, head_dim=hd, rope_theta=10000.0, query_pre_attn_scalar=24,
               attn_logit_softcapping=50.0)
    part = registry.MIXERS.build(
        "paged_attention", hidden_size=D, num_heads=H, num_kv_heads=K, head_dim=hd, query_scale=math.sqrt(24),
        soft_cap=50.0, window=window, position_encoding=PartSpec("rope", {"head_dim": hd, "base": 10000.0}))
    w = {n: rand(s, 20 + i, 0.2).to(dtype) for i, (n, s) in enumerate((("q_proj", (H * hd, D)), ("k_proj", (K * hd, D)),
                                                                       ("v_proj", (K * hd, D)), ("o_proj", (D, H * hd))))}
    part.load(w)
    x = rand((T, D), 25).to(dtype)
    ctx, cache = whole_sequence_ctx(T, dtype, page, [part.cache_need()])
    got = part.forward(x, ctx, cache.views[0])
    pw = {"a." + n + ".weight": t.double().cpu() for n, t in w.items()}
    want = plain.attention_layer(x.double().cpu(), torch.arange(T), pw, "a.", cfg, window)
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    torch.testing.assert_close(got.double().cpu(), want, rtol=tol, atol=tol * want.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(dtype):
    from simply_amd.parts.embedding import LinearHead, ScaledEmbedding
    V, D = 333, 72
    table = rand((V, D), 30, 0.3).to(dtype)
    emb, head = ScaledEmbedding(V, D, math.sqrt(D)), LinearHead(V, D, 15.0)
    emb.load({"table": table})
    head.load({"weight": table})
    tokens = torch.tensor([0, 5, 332, 5], dtype=torch.int32, device=DEV)
    scale = float(torch.tensor(math.sqrt(D), dtype=dtype))
    torch.testing.assert_close(emb.forward(tokens).double().cpu(), table.double().cpu()[tokens.long().cpu()] * scale,
                               rtol=1e-6, atol=1e-6)
    x = rand((4, D), 31).to(dtype)
    want = 15 * torch.tanh(x.double().cpu() @ table.double().cpu().T / 15)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got = head.forward(x)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double().cpu(), want, rtol=tol, atol=tol)


# ------------------------------------------------------------------ toy parts, defined and registered here
class RunningMeanMixer(Mixer):
    """A toy mixer with a state of fixed size per request: y_t = W (decay * s_{t-1} + x_t), s_t = decay * s_{t-1} + x_t.
    It keeps no keys: its state lives in the request's state slot, from which a portion continues and into which
    the portion's last state is written back.  Steps in which every request brings one token take the slots from
    the device (`ctx.token_seq`), so that such a step can be recorded once and replayed for other requests."""

    def __init__(self, hidden_size: int, decay: float):
        self.hidden_size, self.decay = hidden_size, decay
        self.proj = None

    def param_specs(self):
        return {"proj": ParamSpec((self.hidden_size, self.hidden_size))}

    def cache_need(self):
        return StateNeed((self.hidden_size,), torch.float32)

    def forward(self, x, ctx, cache):
        if ctx.max_q_len == 1:
            slots = ctx.token_seq.long()
            s = self.decay * cache.state.index_select(0, slots) + x.float()
            cache.state.index_copy_(0, slots, s)
            return ops.gemm(s, self.proj.float()).to(x.dtype)
        out = torch.empty_like(x)
        for slot, a, b in zip(ctx.seq_slots, ctx.cu_q_lens[:-1], ctx.cu_q_lens[1:]):
            s = cache.state[slot]
            for t in range(a, b):
                s = self.decay * s + x[t].float()
                out[t] = (self.proj.float() @ s).to(x.dtype)
            cache.state[slot] = s
        return out


class TopOneRouted(FeedForward):
    """A toy feed-forward with routing: each token goes through the one of E small linear maps that its router
    logit picks."""

    def __init__(self, hidden_size: int, experts: int):
        self.hidden_size, self.experts = hidden_size, experts
        self.router = self.maps = None

    def param_specs(self):
        return {"router": ParamSpec((self.experts, self.hidden_size)),
                "maps": ParamSpec((self.experts, self.hidden_size, self.hidden_size))}

    def forward(self, x, ctx=None):
        choice = (x.float() @ self.router.float().T).argmax(-1)
        return torch.einsum("tij,tj->ti", self.maps.float()[choice], x.float()).to(x.dtype)


class AlibiLikeShift(PositionEncoding):
    """A toy position encoding: adds position / 1000 to the first element of every head."""

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        v = x[:, :num_heads * head_dim].view(x.shape[0], num_heads, head_dim)
        v[:, :, 0] += (positions.float() / 1000.0).to(x.dtype)[:, None]
        v /= div


@pytest.fixture
def toy_registry():
    registry.MIXERS.register("toy_running_mean", RunningMeanMixer)
    registry.FEED_FORWARDS.register("toy_top_one", TopOneRouted)
    registry.POSITION_ENCODINGS.register("toy_shift", AlibiLikeShift)
    yield
    registry.MIXERS.unregister("toy_running_mean")
    registry.FEED_FORWARDS.unregister("toy_top_one")
    registry.POSITION_ENCODINGS.unregister("toy_shift")


def toy_spec():
    D, V = 64, 128
    norm = lambda name: PartSpec("rmsnorm", {"dim": D, "eps": 1e-6}, {"scale": name})
    norms = lambda p: {"pre_mixer": norm(p + "n0"), "post_mixer": norm(p + "n1"), "pre_ffn": norm(p + "n2"),
                       "post_ffn": norm(p + "n3")}
    attn = PartSpec("paged_attention", {"hidden_size": D, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                        "query_scale": 4.0, "soft_cap": None, "window": 6,
                                        "position_encoding": PartSpec("toy_shift")},
                    {n: "l0." + n for n in ("q_proj", "k_proj", "v_proj", "o_proj")})
    dense = PartSpec("gated_dense", {"hidden_size": D, "intermediate_size": 96},
                     {n: "l0." + n for n in ("gate_proj", "up_proj", "down_proj")})
    layers = (
        LayerSpec(PartSpec("sandwich"), attn, dense, norms("l0.")),
        LayerSpec(PartSpec("sandwich"), PartSpec("toy_running_mean", {"hidden_size": D, "decay": 0.5}, {"proj": "l1.proj"}),
                  PartSpec("toy_top_one", {"hidden_size": D, "experts": 3}, {"router": "l1.router", "maps": "l1.maps"}),
                  norms("l1.")),
    )
    # the attention layer runs twice (its second run reads the first run's cache), the toy layer between them
    schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_from=0), ScheduleEntry(1))
    return ModelSpec("ToyModel", D, V, PartSpec("scaled_embedding", {"vocab_size": V, "dim": D, "scale": 8.0}, {"table": "emb"}),
                     layers, schedule, norm("final"), PartSpec("linear_head", {"vocab_size": V, "dim": D, "soft_cap": None},
                                                               {"weight": "emb"}), max_position=256)


def test_toy_parts_are_registered_built_and_stepped(toy_registry):
    model = DecoderModel(toy_spec())
    needs = model.cache_needs()
    assert [type(n).__name__ for n, _ in needs] == ["PagedKVNeed", "StateNeed", "PagedKVNeed", "StateNeed"]
    assert needs[2][1] == 0
    init_random(model, 0, torch.float32, torch.device(DEV), std=0.2)
    cfg = EngineConfig(activation_dtype="float32", page_size=4, batch_size=3, max_seq_len=64, max_num_issue_tokens=64,
                       total_num_pages=24, device=DEV, use_graphs=False)
    ex = Executor(model, cfg)
    # the two runs of the toy layer keep separate states; the second attention run shares the first one's pages
    assert ex.cache.views[1].state is not ex.cache.views[3].state
    assert ex.cache.views[2].k_pages is ex.cache.views[0].k_pages and not ex.cache.views[2].write
    tokens = tiny.random_tokens(30, 128, 3)

    def run(rid, cuts):
        ex.add_request(rid)
        out, i = [], 0
        for c in cuts:
            out.append(ex.step([StepEntry(rid, tokens[i:i + c], list(range(c)))]).cpu())
            i += c
        ex.finish_request(rid)
        return torch.cat(out)

    whole = run("a", [30])
    assert torch.isfinite(whole).all() and whole.abs().max() > 0
    for cuts in ([1] * 30, [7, 2, 9, 1, 11], [28, 2]):
        torch.testing.assert_close(run("b", cuts), whole, rtol=1e-4, atol=1e-4)
    # two requests mixed: the state slots keep them apart
    ex.add_request("x")
    ex.add_request("y")
    other = tiny.random_tokens(30, 128, 4)
    got = []
    for i in range(0, 30, 5):
        logits = ex.step([StepEntry("x", tokens[i:i + 5], list(range(5))), StepEntry("y", other[i:i + 5], [])]).cpu()
        got.append(logits)
    torch.testing.assert_close(torch.cat(got), whole, rtol=1e-4, atol=1e-4)
    # a new request in a slot that was used before starts from a zero state
    ex.finish_request("x")
    torch.testing.assert_close(run("z", [30]), whole, rtol=1e-4, atol=1e-4)


def test_toy_state_advances_once_per_step_under_graphs(toy_registry):
    """Decode-only steps are recorded in HIP graphs and replayed.  A mixer with a state of its own shows whether a
    step runs exactly once (the step that is recorded included) and whether a replay serves other requests in
    other slots than those it was recorded with: three requests decode together, finish at different times (so
    the number of rows changes and new graphs are recorded on the way), a fourth takes over a freed slot; every
    logit equals the request run whole."""
    model = DecoderModel(toy_spec())
    init_random(model, 0, torch.float32, torch.device(DEV), std=0.2)
    reqs = {r: tiny.random_tokens(n, 128, 30 + i) for i, (r, n) in enumerate((("a", 24), ("b", 17), ("c", 30), ("d", 21)))}

    def run(graphs):
        cfg = EngineConfig(activation_dtype="float32", page_size=4, batch_size=3, max_seq_len=64,
                           max_num_issue_tokens=64, total_num_pages=36, device=DEV, use_graphs=graphs)
        ex = Executor(model, cfg)
        got = {r: [] for r in reqs}
        live, pending, pos = [], list(reqs), {}
        while live or pending:
            while pending and len(live) < 3:
                r = pending.pop(0)
                ex.add_request(r)
                got[r].append(ex.step([StepEntry(r, reqs[r][:5], [0, 1, 2, 3, 4])]).cpu())   # its first portion, alone
                pos[r] = 5
                live.append(r)
            logits = ex.step([StepEntry(r, [reqs[r][pos[r]]], [0]) for r in live]).cpu()
            torch.cuda.synchronize()
            for i, r in enumerate(live):
                got[r].append(logits[i:i + 1])
                pos[r] += 1
            for r in [r for r in live if pos[r] == len(reqs[r])]:
                ex.finish_request(r)
                live.remove(r)
        return {r: torch.cat(v) for r, v in got.items()}, ex

    eager, _ = run(False)
    replayed, ex = run(True)
    assert {k[0] for k in ex._graphs} == {1, 2, 3}
    whole_ex = Executor(model, EngineConfig(activation_dtype="float32", page_size=4, batch_size=3, max_seq_len=64,
                                            max_num_issue_tokens=64, total_num_pages=36, device=DEV, use_graphs=False))
    for r, t in reqs.items():
        whole_ex.add_request(r)
        whole = whole_ex.step([StepEntry(r, t, list(range(len(t))))]).cpu()
        whole_ex.finish_request(r)
        torch.testing.assert_close(eager[r], whole, rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(replayed[r], whole, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_pages_of_its_own_layout(dtype):
    """A toy mixer (tests/toy_parts.py) that keeps one latent vector per token in float32 pages [page, rank,
    page_size], through a need class of the test's own: two more cache groups beside the attention layer's, one of
    them windowed.  Whole, cut and mixed in a pool so small that pages are used again (poisoned in between) give the
    same logits, in both element types; the framework's files know nothing of the layout."""
    import numpy as np
    import toy_parts

    registry.MIXERS.register("toy_latent_mean", toy_parts.LatentMeanMixer)
    try:
        model = DecoderModel(toy_parts.latent_model_spec())
        tdtype = torch.float32 if dtype == "float32" else torch.bfloat16
        init_random(model, 0, tdtype, torch.device(DEV), std=0.2)
        cfg = EngineConfig(activation_dtype=dtype, page_size=4, batch_size=3, max_seq_len=64, max_num_issue_tokens=32,
                           total_num_pages=24, device=DEV, use_graphs=False, poison_freed_pages=True, intermediate_steps=1)
        ex = Executor(model, cfg)
        assert [type(g.need).__name__ for g in ex.cache.groups] == ["PagedKVNeed", "LatentNeed", "LatentNeed"]
        assert ex.cache.views[1].pages["latent"].dtype == torch.float32 and ex.cache.views[0].k_pages.dtype == tdtype
        reqs = {f"r{i}": tiny.random_tokens(n, 128, 40 + i) for i, n in enumerate((30, 17, 26, 9, 22))}
        tol = dict(rtol=1e-4, atol=1e-4) if dtype == "float32" else dict(rtol=5e-2, atol=5e-2)

        def run(rid, t, cuts):
            ex.add_request(rid)
            out, i = [], 0
            for c in cuts:
                out.append(ex.step([StepEntry(rid, t[i:i + c], list(range(c)))]).cpu())
                i += c
            ex.finish_request(rid)
            return torch.cat(out)

        whole = {r: run(r, t, [len(t)]) for r, t in reqs.items()}
        assert all(torch.isfinite(v).all() and v.abs().max() > 0 for v in whole.values())
        torch.testing.assert_close(run("x", reqs["r0"], [7, 2, 9, 1, 11]), whole["r0"], **tol)
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
            logits, i = ex.step(entries).cpu(), 0
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
            torch.testing.assert_close(torch.cat(got[r]), whole[r], **tol)
        assert all(g.pool.num_free == g.pool.num_pages for g in ex.cache.groups)
    finally:
        registry.MIXERS.unregister("toy_latent_mean")


def test_unknown_part_names_are_refused():
    spec = toy_spec()   # the toy kinds are not registered here
    with pytest.raises(ValueError, match="unknown (mixer|feed-forward|position encoding)"):
        DecoderModel(spec)
