"""Each HIP kernel alone against its plain torch reference, at sizes other than the engine's."""
import math

import pytest
import torch

import torch_ops as ref

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]


def bf16_step(x: torch.Tensor) -> torch.Tensor:
    """The spacing of bfloat16 numbers at the magnitude of x (8 bits of significand): 2^(floor(log2 |x|) - 7)."""
    return torch.exp2(torch.floor(torch.log2(x.abs().clamp_min(1e-30))) - 7)


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(bf16_steps=1.0)


def gated(t):
    """The tolerance of a gated product: both of its products are rounded to bfloat16 before the activation and
    the multiplication (act(g) * u with |act'| <= 1.13), and the result once more: three rounding steps."""
    return dict(t, bf16_steps=3.0 * t["bf16_steps"]) if "bf16_steps" in t else t


def check(got, want, *, rtol=None, atol=None, bf16_steps=None, msg=None):
    """A kernel's result against its plain reference.  With rtol / atol: torch's criterion (32-bit results).  With
    bf16_steps: both sides were computed in 32-bit from the same bfloat16 inputs and rounded to bfloat16 once, so they
    differ by a rounding step where the 32-bit values behind them differ in their last bits; every element must lie
    within that many bfloat16 steps at the largest magnitude of its row (one step there is 0.39 to 0.78 % of that
    magnitude; the reference's bars for its own attention kernel are 5e-3 and 1e-2 of such outputs:
    simply/utils/ragged_paged_attention_test.py:471, simply/utils/rpa_shard_window_repro_test.py:234)."""
    if bf16_steps is None:
        torch.testing.assert_close(got, want, rtol=rtol, atol=atol, msg=msg)
        return
    got, want = got.float(), want.float()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all()
    rows = want.reshape(-1, want.shape[-1])
    bound = bf16_steps * bf16_step(rows.abs().amax(dim=-1, keepdim=True))
    excess = (got.reshape(rows.shape) - rows).abs() - bound
    worst = int(excess.argmax())
    assert excess.max().item() <= 0, (
        msg, f"element {worst} of {tuple(want.shape)}: got {got.reshape(-1)[worst].item()}, want "
             f"{want.reshape(-1)[worst].item()}, allowed {bound[worst // rows.shape[1]].item()}")


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("V,D,T", [(50, 24, 7), (333, 1000, 33)])
def test_embed(dtype, V, D, T):
    from simply_amd.kernels import ops
    table = rand((V, D), dtype, 0)
    tokens = torch.randint(0, V, (T,), dtype=torch.int32).cuda()
    got = ops.embed(table, tokens, 3.25)
    check(got, ref.embed(table, tokens, 3.25), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,D", [(1, 16), (5, 100), (3, 2304), (2, 5000)])
def test_rmsnorm(dtype, T, D):
    from simply_amd.kernels import ops
    x = rand((T, D), torch.float32, 1, 3.0)
    w = rand((D,), dtype, 2, 0.3)
    for plus_one in (True, False):
        got = ops.rmsnorm(x, w, 1e-5, plus_one, dtype)
        check(got.float(), ref.rmsnorm(x, w, 1e-5, plus_one, dtype).float(), **tol(dtype))
    xa = x.to(dtype)
    got = ops.rmsnorm(xa, w, 1e-6, True, dtype)
    check(got.float(), ref.rmsnorm(xa, w, 1e-6, True, dtype).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,D", [(1, 48), (6, 100), (3, 2304), (600, 2304), (513, 100), (515, 5000), (512, 6000), (517, 50),
                                 (64, 2304), (100, 3584), (2049, 2304), (2050, 4608), (2051, 1028), (2048, 5120)])
def test_add_rmsnorm(dtype, T, D):
    from simply_amd.kernels import ops
    y = rand((T, D), dtype, 3, 2.0)
    h0 = rand((T, D), torch.float32, 4, 5.0)
    w1, w2 = rand((D,), dtype, 5, 0.3), rand((D,), torch.float32, 6, 0.3)
    for with_post in (True, False):
        for with_next in (True, False):
            h_got, h_ref = h0.clone(), h0.clone()
            kw = dict(post_weight=w1 if with_post else None, post_eps=1e-6, next_weight=w2 if with_next else None,
                      next_eps=1e-5, out_dtype=dtype)
            o_got = ops.add_rmsnorm(y, h_got, **kw)
            o_ref = ref.add_rmsnorm(y, h_ref, **kw)
            check(h_got, h_ref, rtol=1e-5, atol=1e-5)
            assert (o_got is None) == (o_ref is None)
            if o_got is not None:
                check(o_got.float(), o_ref.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("H,K,hd,P", [(4, 2, 16, 4), (6, 1, 32, 3), (8, 4, 256, 16), (3, 3, 48, 5)])
@pytest.mark.parametrize("T,order", [(11, "random"), (300, "random"), (300, "run"), (300, "run from 5"), (333, "runs")])
def test_rope_cache_write(dtype, H, K, hd, P, T, order):
    """Few tokens: a block per (token, head); many: a block per token, or (bfloat16, head sizes in steps of 16)
    blocks of 8 and 16 tokens with 16-byte accesses, which write the values of 16 tokens in one piece where their
    slots are a run inside a page."""
    from simply_amd.kernels import ops
    pages = 2 * -(-T // P) + 6
    qkv = rand((T, (H + 2 * K) * hd), dtype, 7)
    positions = torch.tensor(([0, 1, 2, 3, 100, 101, 7, 8000, 5, 6, 7] * 32)[:T], dtype=torch.int32).cuda()
    ts = (10000.0 ** (2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().cuda()
    if order == "random":
        slots = torch.randperm(pages * P)[:T]
    elif order == "run":
        slots = torch.arange(T) + P          # one run from a page's edge
    elif order == "run from 5":
        slots = torch.arange(T) + 5          # one run that starts inside a page
    else:                                    # runs of 40 slots at scattered places: some blocks of 16 are a run, some not
        starts = torch.randperm(pages * P // 48)[: -(-T // 40)] * 48
        slots = torch.cat([st + torch.arange(40) for st in starts])[:T]
    slots = slots.to(torch.int64).cuda()
    kp, vp = torch.zeros((pages, K, P, hd), dtype=dtype).cuda(), torch.zeros((pages, K, hd, P), dtype=dtype).cuda()
    kp2, vp2, qkv2 = kp.clone(), vp.clone(), qkv.clone()
    ops.rope_cache_write(qkv, positions, ts, 1.0, 12.0, H, K, hd, slots, kp, vp)
    ref.rope_cache_write(qkv2, positions, ts, 1.0, 12.0, H, K, hd, slots, kp2, vp2)
    t = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else tol(dtype)  # sin/cos of angles up to 8000 rad
    check(qkv[:, :H * hd].float(), qkv2[:, :H * hd].float(), **t)
    check(kp.float(), kp2.float(), **t)
    check(vp, vp2, rtol=0, atol=0)
    # without rotation and without a cache: only the query scale
    q3 = rand((T, (H + 2 * K) * hd), dtype, 8)
    q4 = q3.clone()
    ops.rope_cache_write(q3, positions, None, 1.0, 3.0, H, K, hd)
    check(q3[:, :H * hd].float(), (q4[:, :H * hd].float() / 3.0).to(dtype).float(), **tol(dtype))
    check(q3[:, H * hd:], q4[:, H * hd:], rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 64, 64), (65, 130, 100), (17, 333, 72), (128, 96, 2304)])
def test_gemm_generic(dtype, M, N, K):
    from simply_amd.kernels import ops
    a, w, w2 = rand((M, K), dtype, 9), rand((N, K), dtype, 10, 0.1), rand((N, K), dtype, 11, 0.1)
    t = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else tol(dtype)
    for algo in (ops.ALGO_AUTO, ops.ALGO_GENERIC):
        check(ops.gemm(a, w, algo=algo).float(), ref.gemm(a, w).float(), **t)
        check(ops.gemm(a, w, w2=w2, algo=algo).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
        got = ops.gemm(a, w, soft_cap=2.0, out_dtype=torch.float32, algo=algo)
        assert got.dtype == torch.float32
        check(got, ref.gemm(a, w, soft_cap=2.0, out_dtype=torch.float32), **t)
    # rows of a wider buffer as input (a view), as the attention output is
    wide = rand((M, K + 24), dtype, 12)
    check(ops.gemm(wide[:, 8:8 + K], w).float(), ref.gemm(wide[:, 8:8 + K], w).float(), **t)


def test_gemm_rows_do_not_depend_on_the_batch():
    """float32: a row's product is bit-identical whatever other rows are in the batch."""
    from simply_amd.kernels import ops
    a, w = rand((70, 200), torch.float32, 13), rand((150, 200), torch.float32, 14)
    full = ops.gemm(a, w)
    for rows in ([0], [69], [3, 4, 5], list(range(64, 70))):
        part = ops.gemm(a[rows].contiguous(), w)
        assert torch.equal(part, full[rows])


def paged_setup(dtype, S, H, Kh, hd, P, lens, seed):
    """Random cache contents for S requests of the given lengths, pages handed out in a shuffled order."""
    max_blocks = max(-(-l // P) for l in lens) + 1
    num_pages = S * max_blocks + 3
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    table = torch.full((S, max_blocks), -1, dtype=torch.int32)
    kp = torch.full((num_pages, Kh, P, hd), float("nan"), dtype=dtype)
    vp = torch.full((num_pages, Kh, hd, P), float("nan"), dtype=dtype)
    for s, l in enumerate(lens):
        for b in range(-(-l // P)):
            page = perm.pop()
            table[s, b] = page
            n = min(P, l - b * P)
            kp[page, :, :n] = torch.randn((Kh, n, hd), generator=g).to(dtype)
            vp[page, :, :, :n] = torch.randn((Kh, hd, n), generator=g).to(dtype)
    return ref.rows_as_stored_keys(kp).cuda(), vp.cuda(), table.cuda()


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("H,Kh,hd,P,window,cap", [
    (4, 2, 16, 4, None, 50.0), (4, 2, 16, 4, 8, 50.0), (6, 1, 32, 3, 16, None), (8, 4, 256, 16, None, 50.0),
    (6, 3, 48, 5, 5, 20.0), (16, 1, 64, 16, 70, None), (2, 2, 128, 64, 100, 30.0)])
def test_paged_attention_generic(dtype, H, Kh, hd, P, window, cap):
    from simply_amd.kernels import ops
    lens = [1, 37, 150, 64]
    kp, vp, table = paged_setup(dtype, len(lens), H, Kh, hd, P, lens, 21)
    # queries: the last tokens of each request, several per request (a portion), unfilled page tails are NaN
    token_seq, positions = [], []
    for s, l in enumerate(lens):
        for p in range(max(0, l - 5), l):
            token_seq.append(s)
            positions.append(p)
    T = len(positions)
    q = rand((T, H * hd + 32), dtype, 22, 0.5)[:, :H * hd]
    ts = torch.tensor(token_seq, dtype=torch.int32).cuda()
    ps = torch.tensor(positions, dtype=torch.int32).cuda()
    got = ops.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=cap, algo=ops.ALGO_GENERIC)
    want = ref.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=cap)
    assert torch.isfinite(got.float()).all()
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else tol(dtype)
    check(got.float(), want.float(), **t)


@pytest.mark.parametrize("P,hd", [(16, 32), (32, 256), (48, 64), (16, 48), (4, 32), (24, 64)])
def test_key_page_layout(P, hd):
    """The layout of a stored page of keys, three ways: the index arithmetic of the tests' reference (written from
    the interface's description), the product's re-layout functions, and the kernel that writes keys into pages."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import keys_to_rows, rows_to_keys
    rows = torch.arange(3 * 2 * P * hd, dtype=torch.float32).reshape(3, 2, P, hd).cuda()
    assert torch.equal(rows_to_keys(rows), ref.rows_as_stored_keys(rows))
    assert torch.equal(keys_to_rows(rows_to_keys(rows)), rows) and torch.equal(ref.stored_keys_as_rows(rows_to_keys(rows)), rows)
    # the kernel: token t's key (no rotation) lands where the arithmetic says
    T, K = 3 * P, 2
    qkv = rand((T, (1 + 2 * K) * hd), torch.float32, 5)
    slots = torch.randperm(3 * P).to(torch.int64).cuda()
    kp, vp = torch.zeros((3, K, P, hd)).cuda(), torch.zeros((3, K, hd, P)).cuda()
    ops.rope_cache_write(qkv, torch.zeros(T, dtype=torch.int32).cuda(), None, 1.0, 1.0, 1, K, hd, slots, kp, vp)
    got = ref.stored_keys_as_rows(kp)
    want = qkv[:, hd:(1 + K) * hd].reshape(T, K, hd)
    assert torch.equal(got[slots // P, :, slots % P], want)


def test_paged_attention_far_key_and_window_edge():
    """One key far back gets a score that stands out: a global layer must find it, a windowed layer
    must see it exactly while it is inside the window."""
    from simply_amd.kernels import ops
    H = Kh = 1
    hd, P, L = 32, 16, 300
    kp, vp, table = paged_setup(torch.float32, 1, H, Kh, hd, P, [L], 31)
    kp = ref.stored_keys_as_rows(kp) * 0.01
    far = 37
    page, off = int(table[0, far // P]), far % P
    kp[page, 0, off] = 0.0
    kp[page, 0, off, 3] = 50.0
    kp = ref.rows_as_stored_keys(kp)
    vp[page, 0, :, off] = 7.0
    q = torch.zeros((1, hd)).cuda()
    q[0, 3] = 1.0
    ts = torch.zeros(1, dtype=torch.int32).cuda()
    for window, pos, sees in [(None, L - 1, True), (100, far + 99, True), (100, far + 100, False), (1, far, True)]:
        ps = torch.tensor([pos], dtype=torch.int32).cuda()
        out = ops.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=None)
        assert (abs(out.mean().item() - 7.0) < 1e-3) == sees, (window, pos, out.mean().item())
        check(out, ref.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=None),
                                   rtol=1e-4, atol=1e-5)


def test_sampling_kernel():
    from simply_amd.kernels import ops
    V, R = 1000, 6
    logits = rand((R, V), torch.float32, 41, 3.0)
    temperature = torch.tensor([0.0, 1.0, 0.7, 1.0, 1.3, 1.0]).cuda()
    top_k = torch.tensor([-1, -1, -1, 1, 20, 50], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 1.0, 1.0, 1.0, 1.0, 0.6]).cuda()
    seed = torch.tensor([1, 2, 3, 4, 5, 2**40 + 17], dtype=torch.int64).cuda()
    counter = torch.tensor([0, 5, 9, 0, 3, 77], dtype=torch.int32).cuda()
    tok, lp = ops.sample(logits, temperature, top_k, top_p, seed, counter)
    rtok, rlp = ref.sample(logits, temperature, top_k, top_p, seed, counter)
    assert tok.tolist() == rtok.tolist()
    check(lp, rlp, rtol=1e-4, atol=1e-4)
    assert tok[0].item() == int(logits[0].argmax()) and tok[3].item() == int(logits[3].argmax())
    # same seed and counter: same token; another counter: (almost surely) another stream
    tok2, _ = ops.sample(logits, temperature, top_k, top_p, seed, counter)
    assert tok.tolist() == tok2.tolist()
    # host copy of the generator agrees with the reference implementation
    assert ops.philox4x32_10((1, 2, 3, 4), (5, 6)) == ref.philox4x32_10((1, 2, 3, 4), (5, 6))


def test_sampling_frequencies():
    """10^4 draws from a 4-way distribution lie within 4 sigma of softmax(logits / T)
    (after simply/utils/sampling_lib_test.py:138-152)."""
    from simply_amd.kernels import ops
    n, T = 10000, 0.7
    base = torch.tensor([1.0, 0.0, -1.0, 2.0])
    logits = base.repeat(n, 1).cuda()
    tok, _ = ops.sample(logits, torch.full((n,), T).cuda(), torch.full((n,), -1, dtype=torch.int32).cuda(),
                        torch.ones(n).cuda(), torch.full((n,), 1234, dtype=torch.int64).cuda(),
                        torch.arange(n, dtype=torch.int32).cuda())
    freq = torch.bincount(tok.long().cpu(), minlength=4).double() / n
    p = torch.softmax(base.double() / T, -1)
    sigma = torch.sqrt(p * (1 - p) / n)
    assert ((freq - p).abs() < 4 * sigma).all(), (freq, p)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 72), (2304, 2048), (333, 1000), (4096, 2304)])
def test_gemm_skinny(M, N, K):
    """The few-rows bfloat16 kernel, with its own choice of rows per workgroup and waves and with forced ones."""
    from simply_amd.kernels import ops
    a, w, w2 = rand((M, K), torch.bfloat16, 50), rand((N, K), torch.bfloat16, 51, 0.05), rand((N, K), torch.bfloat16, 52, 0.05)
    blocks = 1 if M <= 16 else 2 if M <= 32 else 4
    for shape in (0, 1604, 808, 407, 1601):
        if (shape % 100) * 2 * blocks * 16 * 17 * 4 > 65536:
            continue   # the waves' tiles of the gated product would not fit in LDS: the library refuses that
        kw = dict(algo=ops.ALGO_SKINNY, shape=shape)
        check(ops.gemm(a, w, **kw).float(), ref.gemm(a, w).float(), bf16_steps=1.0)
        check(ops.gemm(a, w, w2=w2, **kw).float(), ref.gemm(a, w, w2=w2).float(), bf16_steps=3.0)
        got = ops.gemm(a, w, soft_cap=3.0, out_dtype=torch.float32, **kw)
        check(got, ref.gemm(a, w, soft_cap=3.0, out_dtype=torch.float32), rtol=2e-3, atol=2e-3)
    # the same call twice gives the same bits (the order of the partial sums is fixed)
    assert torch.equal(ops.gemm(a, w, algo=ops.ALGO_SKINNY, shape=804), ops.gemm(a, w, algo=ops.ALGO_SKINNY, shape=804))
    # a view with a row stride, as the attention output is
    wide = rand((M, K + 16), torch.bfloat16, 53)
    check(ops.gemm(wide[:, 8:8 + K], w, algo=ops.ALGO_SKINNY).float(), ref.gemm(wide[:, 8:8 + K], w).float(),
                               bf16_steps=1.0)


@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 7, 8, 9])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 96), (2304, 2048), (333, 1120), (1000, 2304), (200, 9216)])
def test_gemm_skinny_with_tiled_weights_and_few_rows(M, N, K):
    """Up to 8 rows against tiled weights: one load of activations brings two or four chunks of K, each chunk's product
    has an accumulator of its own (right in its own columns only) and they are added up after the loop.  Numbers of
    chunks per wave that are and are not multiples of the four chunks of a register set, rows that do not fill their
    share of the columns (3 of 4, 5 and 7 of 8), plain, gated and soft-capped; a hot row and a hot column of K show
    a chunk that lands in the wrong accumulator or a wrong column."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles
    a, w, w2 = rand((M, K), torch.bfloat16, 58), rand((N, K), torch.bfloat16, 59, 0.05), rand((N, K), torch.bfloat16, 60, 0.05)
    a[M - 1, K // 3] = 40.0      # one activation that stands out: its chunk must meet its own weights
    a[0, K - 1] = -30.0
    t = dict(bf16_steps=1.0)
    for waves in (0, 1, 3, 8):
        kw = dict(algo=ops.ALGO_SKINNY, shape=1600 + waves if waves else 0)
        if waves and waves > K // 64:
            continue
        check(ops.gemm(a, pack_tiles(w), **kw).float(), ref.gemm(a, w).float(), **t)
        check(ops.gemm(a, pack_gate_up(w, w2), **kw).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
        check(ops.gemm(a, pack_tiles(w), soft_cap=3.0, out_dtype=torch.float32, **kw),
                                   ref.gemm(a, w, soft_cap=3.0, out_dtype=torch.float32), rtol=2e-3, atol=2e-3)
    # rows of wider rows, as the attention output is
    big = rand((M, K + 32), torch.bfloat16, 61)
    check(ops.gemm(big[:, 16:16 + K], pack_tiles(w), algo=ops.ALGO_SKINNY).float(),
                               ref.gemm(big[:, 16:16 + K], w).float(), **t)
    # the same rows to the bit whoever else is in the batch, within the kernel's variants of up to 4, up to 8 and more rows
    if M in (2, 3, 4):
        assert torch.equal(ops.gemm(a, pack_tiles(w), algo=ops.ALGO_SKINNY)[:1], ops.gemm(a[:1], pack_tiles(w), algo=ops.ALGO_SKINNY))


def test_gemm_skinny_refuses_what_it_does_not_take():
    from simply_amd.kernels import ops
    from simply_amd.kernels.lib import KernelError
    a, w = rand((4, 100), torch.bfloat16, 54), rand((8, 100), torch.bfloat16, 55)   # K is no multiple of 8
    with pytest.raises(KernelError, match="few-rows"):
        ops.gemm(a, w, algo=ops.ALGO_SKINNY)
    check(ops.gemm(a, w).float(), ref.gemm(a, w).float(), bf16_steps=1.0)   # auto falls back
    with pytest.raises(KernelError):
        ops.gemm(rand((65, 64), torch.bfloat16, 56), rand((8, 64), torch.bfloat16, 57), algo=ops.ALGO_SKINNY)


def seq_meta_for(lens, q_lens):
    """Requests whose last q tokens are this step's; returns (meta [S, 4], token_seq, positions)."""
    meta, token_seq, positions, t0 = [], [], [], 0
    for s, (l, q) in enumerate(zip(lens, q_lens)):
        meta.append((s, t0, q, l - q))
        token_seq += [s] * q
        positions += list(range(l - q, l))
        t0 += q
    return (torch.tensor(meta, dtype=torch.int32).cuda(), torch.tensor(token_seq, dtype=torch.int32).cuda(),
            torch.tensor(positions, dtype=torch.int32).cuda())


@pytest.mark.parametrize("H,Kh,hd,P,window,cap", [
    (8, 4, 256, 16, None, 50.0), (8, 4, 256, 16, 100, 50.0), (4, 2, 64, 16, 33, None), (16, 1, 128, 32, None, 30.0),
    (2, 2, 128, 64, 200, None), (6, 3, 64, 16, 1, 20.0), (32, 16, 128, 16, 500, 50.0)])
@pytest.mark.parametrize("splits", [0, 1, 5])
def test_paged_attention_decode(H, Kh, hd, P, window, cap, splits):
    """The few-tokens bfloat16 kernel against the plain reference: lengths around page and tile edges, one
    to several tokens per request, unwritten page tails holding NaN, keys cut over workgroups."""
    from simply_amd.kernels import ops
    G = H // Kh
    lens = [1, 16, 17, 33, 250, 700, 64, 1000]
    max_q = max(1, 16 // G)
    q_lens = [min(l, 1 + (i * 3) % max_q) for i, l in enumerate(lens)]
    order = sorted(range(len(lens)), key=lambda i: q_lens[i])
    lens, q_lens = [lens[i] for i in order], [q_lens[i] for i in order]
    kp, vp, table = paged_setup(torch.bfloat16, len(lens), H, Kh, hd, P, lens, 61)
    meta, ts, ps = seq_meta_for(lens, q_lens)
    T = ts.numel()
    q = rand((T, (H + 2 * Kh) * hd), torch.bfloat16, 62, 0.3)
    out = torch.zeros((T, H * hd), dtype=torch.bfloat16).cuda()
    assert ops.decode_attention_takes(q, kp, H, max(q_lens))
    ops.paged_attention_decode(q, kp, vp, table, meta, 0, len(lens), H, window=window, soft_cap=cap,
                               max_kv_len=max(lens), max_q_len=max(q_lens), out=out, num_splits=splits)
    want = ref.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=cap)
    assert torch.isfinite(out.float()).all()
    check(out.float(), want.float(), bf16_steps=2.0)
    # a sub-range of the requests: the others' rows stay untouched
    out2 = torch.full_like(out, 7.0)
    ops.paged_attention_decode(q, kp, vp, table, meta, 2, 3, H, window=window, soft_cap=cap, max_kv_len=max(lens),
                               max_q_len=max(q_lens), out=out2, num_splits=splits)
    a, b = int(meta[2, 1]), int(meta[4, 1] + meta[4, 2])
    # (with its own choice of key ranges the library cuts differently for 3 requests than for 8: equal up to rounding)
    if splits:
        assert torch.equal(out2[a:b], out[a:b])
    check(out2[a:b].float(), out[a:b].float(), bf16_steps=2.0)
    assert (out2[:a] == 7).all() and (out2[b:] == 7).all()


@pytest.mark.parametrize("stated", [40000, 700])
def test_paged_attention_decode_with_a_range_longer_than_one_look_up(stated):
    """One range of 40,000 keys (more than the 32,768 whose pages a workgroup looks up at a time), and a caller that
    understates the longest context: the kernel works through the range in passes and reads every key."""
    from simply_amd.kernels import ops
    H, Kh, hd, P, L = 2, 1, 64, 16, 40000
    kp, vp, table = paged_setup(torch.bfloat16, 1, H, Kh, hd, P, [L], 77)
    q = rand((1, H * hd), torch.bfloat16, 78, 0.5)
    meta = torch.tensor([[0, 0, 1, L - 1]], dtype=torch.int32).cuda()
    out = torch.zeros((1, H * hd), dtype=torch.bfloat16).cuda()
    ops.paged_attention_decode(q, kp, vp, table, meta, 0, 1, H, window=None, soft_cap=30.0, max_kv_len=stated, max_q_len=1,
                               out=out, num_splits=1)
    want = ref.paged_attention(q, kp, vp, table, torch.zeros(1, dtype=torch.int32).cuda(),
                               torch.tensor([L - 1], dtype=torch.int32).cuda(), H, window=None, soft_cap=30.0)
    check(out.float(), want.float(), bf16_steps=2.0)
    # a key in the second pass that stands out is found
    rows = ref.stored_keys_as_rows(kp) * 0.01
    far = 36000
    page, off = int(table[0, far // P]), far % P
    rows[page, 0, off] = 0.0
    rows[page, 0, off, 5] = 60.0
    vp[page, 0, :, off] = 9.0
    q2 = torch.zeros((1, H * hd), dtype=torch.bfloat16).cuda()
    q2[0, 5] = q2[0, hd + 5] = 1.0
    ops.paged_attention_decode(q2, ref.rows_as_stored_keys(rows), vp, table, meta, 0, 1, H, window=None, soft_cap=None,
                               max_kv_len=stated, max_q_len=1, out=out, num_splits=1)
    assert abs(out.float().mean().item() - 9.0) < 0.1, out.float().mean().item()


def test_paged_attention_decode_far_key():
    """A key 3000 positions back with a score that stands out, among keys cut over many workgroups."""
    from simply_amd.kernels import ops
    H, Kh, hd, P, L = 2, 1, 128, 16, 3100
    kp, vp, table = paged_setup(torch.bfloat16, 1, H, Kh, hd, P, [L], 63)
    kp = ref.stored_keys_as_rows(kp) * 0.01
    far = 71
    page, off = int(table[0, far // P]), far % P
    kp[page, 0, off] = 0.0
    kp[page, 0, off, 5] = 60.0
    kp = ref.rows_as_stored_keys(kp)
    vp[page, 0, :, off] = 3.0
    meta, ts, ps = seq_meta_for([L], [1])
    q = torch.zeros((1, 4 * hd), dtype=torch.bfloat16).cuda()
    q[0, 5] = 1.0
    q[0, hd + 5] = 1.0
    for window, sees in ((None, True), (L - far, True), (L - far - 1, False)):
        out = torch.zeros((1, H * hd), dtype=torch.bfloat16).cuda()
        ops.paged_attention_decode(q, kp, vp, table, meta, 0, 1, H, window=window, soft_cap=None, max_kv_len=L,
                                   max_q_len=1, out=out)
        assert (abs(out.float().mean().item() - 3.0) < 0.05) == sees, (window, out.float().mean().item())


@pytest.mark.parametrize("M", [1, 8, 33, 64, 100])
@pytest.mark.parametrize("N,K", [(48, 64), (100, 72), (333, 1000), (2304, 2048), (1000, 2304)])
def test_gemm_tiled_weights(M, N, K):
    """Weights in the tiled layout: the few-rows kernel (M <= 64) and the other kernels read the same numbers."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles, unpack_gate_up, unpack_tiles
    a, w, w2 = rand((M, K), torch.bfloat16, 70), rand((N, K), torch.bfloat16, 71, 0.05), rand((N, K), torch.bfloat16, 72, 0.05)
    tw, tw2 = pack_tiles(w), pack_gate_up(w, w2)
    assert torch.equal(unpack_tiles(tw), w)
    assert all(torch.equal(x, y) for x, y in zip(unpack_gate_up(tw2), (w, w2)))
    t = dict(bf16_steps=1.0)
    check(ops.gemm(a, tw).float(), ref.gemm(a, w).float(), **t)
    check(ops.gemm(a, tw2).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
    check(ops.gemm(a, tw2, algo=ops.ALGO_GENERIC).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
    check(ops.gemm(a, tw, soft_cap=3.0, out_dtype=torch.float32),
                               ref.gemm(a, w, soft_cap=3.0, out_dtype=torch.float32), rtol=2e-3, atol=2e-3)
    check(ops.gemm(a, tw, algo=ops.ALGO_GENERIC).float(), ref.gemm(a, w).float(), **t)
    tokens = torch.randint(0, N, (9,), dtype=torch.int32).cuda()
    check(ops.embed(tw, tokens, 1.5), ref.embed(w, tokens, 1.5), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("M,N,K", [(65, 48, 64), (100, 100, 72), (128, 333, 1000), (300, 2304, 2048), (1, 130, 96),
                                   (513, 4096, 2304), (2048, 256, 136), (17, 100, 200), (64, 2304, 9216), (33, 600, 328)])
def test_gemm_tiled(M, N, K):
    """The tiled MFMA kernel for many rows, all epilogues, edges in M, N and K."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles
    a, w, w2 = rand((M, K), torch.bfloat16, 80), rand((N, K), torch.bfloat16, 81, 0.05), rand((N, K), torch.bfloat16, 82, 0.05)
    tw, tw2 = pack_tiles(w), pack_gate_up(w, w2)
    t = dict(bf16_steps=1.0)
    kw = dict(algo=ops.ALGO_TILED)
    for cuts in (0, 1, 3):   # K whole, or cut over workgroups with the partial tiles added by a second kernel
        kw = dict(algo=ops.ALGO_TILED, shape=cuts)
        check(ops.gemm(a, tw, **kw).float(), ref.gemm(a, w).float(), **t)
        check(ops.gemm(a, tw2, **kw).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
        check(ops.gemm(a, tw, soft_cap=3.0, out_dtype=torch.float32, **kw),
                                   ref.gemm(a, w, soft_cap=3.0, out_dtype=torch.float32), rtol=2e-3, atol=2e-3)
    kw = dict(algo=ops.ALGO_TILED)
    wide = rand((M, K + 16), torch.bfloat16, 83)
    check(ops.gemm(wide[:, 8:8 + K], tw, **kw).float(), ref.gemm(wide[:, 8:8 + K], w).float(), **t)
    from simply_amd.kernels.lib import KernelError
    with pytest.raises(KernelError, match="tiled"):
        ops.gemm(a, w, **kw)     # row-major weights are refused


@pytest.mark.parametrize("M,N,K", [(257, 1000, 192), (300, 200, 128), (1, 16, 64), (700, 100, 64), (2048, 2304, 2048),
                                   (513, 4096, 2304), (1000, 388, 1088), (64, 2304, 2048), (200, 4096, 2304)])
def test_gemm_wide(M, N, K):
    """The wide-tile MFMA kernel for very many rows: its three tile shapes and its own choice, plain and gated,
    edges in M and N, odd numbers of slabs, strided rows in and out; and what it refuses."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.lib import KernelError
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles
    a, w, w2 = rand((M, K), torch.bfloat16, 90), rand((N, K), torch.bfloat16, 91, 0.05), rand((N, K), torch.bfloat16, 92, 0.05)
    tw, tw2 = pack_tiles(w), pack_gate_up(w, w2)
    t = dict(bf16_steps=1.0)
    want, want_gated = ref.gemm(a, w).float(), ref.gemm(a, w, w2=w2).float()
    # large tiles, and the small ones with deeper pipelines that products of a few hundred rows get
    for shape in (0, 2256192, 3256128, 3128256, 3192128, 2128192, 3128128, 3128064, 3064128, 3064064, 6064064, 5128064,
                  4128128, 6064128):
        kw = dict(algo=ops.ALGO_WIDE, shape=shape)
        check(ops.gemm(a, tw, **kw).float(), want, **t)
        check(ops.gemm(a, tw2, **kw).float(), want_gated, **gated(t))
    # K cut over two, three and seven workgroups per tile (their partial tiles summed by a second kernel); a cut
    # that K is too short for shrinks to what it allows
    for shape in (20000000 + 3128128, 30000000 + 6064064, 70000000 + 3256128, 20000000 + 5128064, 30000000 + 3192128):
        check(ops.gemm(a, tw, algo=ops.ALGO_WIDE, shape=shape).float(), want, **t)
    if K >= 128:
        with pytest.raises(KernelError, match="cuts K only without"):
            ops.gemm(a, tw2, algo=ops.ALGO_WIDE, shape=20000000 + 3128128)
    # the same rows whatever the tile and whoever else is in the batch, to the bit, while K is not cut: every sum
    # runs along K in order
    one = ops.gemm(a, tw, algo=ops.ALGO_WIDE, shape=2256192)
    assert torch.equal(one, ops.gemm(a, tw, algo=ops.ALGO_WIDE, shape=3128256))
    assert torch.equal(one[: M // 2 + 1], ops.gemm(a[: M // 2 + 1], tw, algo=ops.ALGO_WIDE, shape=3192128))
    assert torch.equal(one, ops.gemm(a, tw, algo=ops.ALGO_TILED, shape=1))   # (K in one piece: the same order)
    # rows inside wider rows, in and out
    kw = dict(algo=ops.ALGO_WIDE)
    big = rand((M, K + 16), torch.bfloat16, 93)
    out = torch.full((M, N + 12), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.gemm(big[:, 8:8 + K], tw, out=out[:, 4:4 + N], **kw)
    check(out[:, 4:4 + N].float(), ref.gemm(big[:, 8:8 + K], w).float(), **t)
    assert (out[:, :4] == 7.0).all() and (out[:, 4 + N:] == 7.0).all()
    with pytest.raises(KernelError, match="wide"):
        ops.gemm(a, w, **kw)                                     # row-major weights
    with pytest.raises(KernelError, match="wide"):
        ops.gemm(a, tw, soft_cap=3.0, out_dtype=torch.float32, **kw)   # the soft-cap epilogue
    with pytest.raises(KernelError, match="wide"):
        ops.gemm(a[:, :K - 32], pack_tiles(w[:, :K - 32].contiguous()), **kw)   # K that is no multiple of 64
    with pytest.raises(KernelError, match="wide"):
        ops.gemm(a, pack_tiles(w[:N - 2].contiguous()), **kw)  # N that is no multiple of 4
    # it is what the library chooses by itself for products that are not bound by streaming the weights; for what it
    # refuses, the tiled kernel
    check(ops.gemm(a, pack_tiles(w[:N - 2].contiguous())).float(), want[:, :N - 2], **t)


@pytest.mark.parametrize("D", [5000, 5200])
def test_add_rmsnorm_wide_rows(D):
    """Rows up to 5120 wide are held in registers by 1024 threads; wider ones take the kernel's second code path."""
    from simply_amd.kernels import ops
    T = 3
    y, h = rand((T, D), torch.bfloat16, 90, 2.0), rand((T, D), torch.float32, 91, 5.0)
    w1, w2 = rand((D,), torch.bfloat16, 92, 0.3), rand((D,), torch.bfloat16, 93, 0.3)
    h_ref = h.clone()
    o = ops.add_rmsnorm(y, h, post_weight=w1, post_eps=1e-6, next_weight=w2, next_eps=1e-6, out_dtype=torch.bfloat16)
    o_ref = ref.add_rmsnorm(y, h_ref, post_weight=w1, post_eps=1e-6, next_weight=w2, next_eps=1e-6, out_dtype=torch.bfloat16)
    check(h, h_ref, rtol=1e-5, atol=1e-5)
    check(o.float(), o_ref.float(), bf16_steps=1.0)


def test_sampling_rows_at_odd_addresses():
    """Rows whose stride is no multiple of four entries: the kernel's four-at-a-time reads start at an aligned
    entry and the rest is read singly."""
    from simply_amd.kernels import ops
    V, R = 1001, 5
    wide = rand((R, V + 2), torch.float32, 94, 3.0)
    logits = wide[:, 1:1 + V]
    temperature = torch.tensor([0.0, 0.8, 0.0, 1.2, 0.0]).cuda()
    top_k = torch.tensor([-1, -1, -1, 30, -1], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 1.0, 1.0, 0.9, 1.0]).cuda()
    seed = torch.tensor([9, 8, 7, 6, 5], dtype=torch.int64).cuda()
    counter = torch.tensor([0, 1, 2, 3, 4], dtype=torch.int32).cuda()
    tok, lp = ops.sample(logits, temperature, top_k, top_p, seed, counter)
    rtok, rlp = ref.sample(logits, temperature, top_k, top_p, seed, counter)
    assert tok.tolist() == rtok.tolist()
    check(lp, rlp, rtol=1e-4, atol=1e-4)
    for r in (0, 2, 4):
        assert tok[r].item() == int(logits[r].argmax())


@pytest.mark.parametrize("V,offset", [(16384, 0), (50001, 1), (256000, 0), (33333, 3)])
def test_sampling_greedy_rows_of_a_large_vocabulary(V, offset):
    """From 16384 entries on the greedy rows are searched in parts by many workgroups: the first of equal maxima
    wins wherever it lies (a part's edge, the last entry, an unaligned row), and the other rows are sampled as
    before."""
    from simply_amd.kernels import ops
    R = 6
    wide = rand((R, V + 8), torch.float32, 95, 2.0)
    logits = wide[:, offset:offset + V]
    part = ((V + 31) // 32 + 3) // 4 * 4
    top = 50.0
    logits[0, V - 1] = top                                   # the last entry
    logits[1, part - 1] = top; logits[1, part] = top         # equal maxima on both sides of a part's edge
    logits[2, 7 * part + 5] = top; logits[2, 20 * part] = top; logits[2, 3] = top   # the first of three
    logits[4, 0] = top
    temperature = torch.tensor([0.0, 0.0, 0.0, 0.9, 1.0, 0.0]).cuda()
    top_k = torch.tensor([-1, -1, -1, -1, 1, -1], dtype=torch.int32).cuda()   # row 4: greedy through top_k 1
    top_p = torch.ones(R).cuda()
    seed = torch.arange(R, dtype=torch.int64).cuda() + 3
    counter = torch.zeros(R, dtype=torch.int32).cuda()
    tok, lp = ops.sample(logits, temperature, top_k, top_p, seed, counter)
    rtok, rlp = ref.sample(logits, temperature, top_k, top_p, seed, counter)
    assert tok.tolist() == rtok.tolist()
    assert tok.tolist()[:3] == [V - 1, part - 1, 3] and tok[4].item() == 0
    assert tok[5].item() == int(logits[5].argmax())
    check(lp, rlp, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("V", [20000, 256000])
def test_sampling_top_k_and_top_p_of_a_large_vocabulary(V):
    """From 16384 entries on the boundaries of top-k and top-p are selected by 32 workgroups per row over several
    kernels (histograms added up with atomics): the same tokens and log-probabilities as the reference, for every
    mix of rows, with equal entries at a boundary, and whatever the caller says of what the rows may ask for (rows
    that ask for more than it says are served by the one-workgroup path)."""
    from simply_amd.kernels import ops
    R = 9
    logits = rand((R, V), torch.float32, 96, 2.5)
    logits[6, 100:105] = 20.0         # five equal largest entries against top_k 3: all of them stay
    logits[7, 7] = 30.0               # one entry holds nearly all the mass
    temperature = torch.tensor([0.8, 1.3, 0.7, 1.0, 0.0, 0.9, 0.5, 2.0, 1.1]).cuda()
    top_k = torch.tensor([40, -1, 50, V + 5, -1, -1, 3, -1, 2], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 0.9, 0.8, 1.0, 1.0, 1.0, 1.0, 0.05, 0.999]).cuda()
    seed = torch.arange(R, dtype=torch.int64).cuda() * 7 + 11
    rtok = rlp = None
    for counter0 in (0, 5):
        counter = torch.full((R,), counter0, dtype=torch.int32).cuda()
        rtok, rlp = ref.sample(logits, temperature, top_k, top_p, seed, counter)
        for modes in (7, 1, 3, 5, 0):
            tok, lp = ops.sample(logits, temperature, top_k, top_p, seed, counter, modes=modes)
            assert tok.tolist() == rtok.tolist(), (modes, tok.tolist(), rtok.tolist())
            check(lp, rlp, rtol=1e-4, atol=1e-4)
    assert rtok[6].item() in range(100, 105) and rtok[7].item() == 7
    # rows that ask for one thing only, with the kernels for exactly that
    for modes, rows in ((ops.SAMPLE_DRAWN | ops.SAMPLE_TOP_K, [0, 3, 6]), (ops.SAMPLE_DRAWN | ops.SAMPLE_TOP_P, [1, 7]),
                        (ops.SAMPLE_DRAWN, [5]), (0, [4])):
        idx = torch.tensor(rows).cuda()
        counter = torch.full((len(rows),), 5, dtype=torch.int32).cuda()
        tok, lp = ops.sample(logits[idx].contiguous(), temperature[idx], top_k[idx], top_p[idx], seed[idx], counter,
                             modes=modes)
        assert tok.tolist() == rtok[idx].tolist()
        check(lp, rlp[idx], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("V", [333, 1001, 20000])
def test_score(V):
    """The log-probability of a given token under temperature, top-k and top-p against the reference: the token
    that the sampler draws scores what the sampler reports for it; tokens inside and outside the masks; greedy rows;
    equal entries at a top-k boundary; rows at odd addresses."""
    from simply_amd.kernels import ops
    R = 9
    wide = rand((R, V + 3), torch.float32, 97, 2.5)
    logits = wide[:, 1:1 + V]
    logits[6, 100:105] = 20.0
    temperature = torch.tensor([0.8, 1.3, 0.7, 1.0, 0.0, 0.9, 0.5, 2.0, 1.0]).cuda()
    top_k = torch.tensor([40, -1, 50, V + 5, -1, -1, 3, -1, 1], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 0.9, 0.8, 1.0, 1.0, 1.0, 1.0, 0.3, 1.0]).cuda()
    seed = torch.arange(R, dtype=torch.int64).cuda() * 5 + 3
    counter = torch.full((R,), 2, dtype=torch.int32).cuda()
    tok, lp = ops.sample(logits, temperature, top_k, top_p, seed, counter)
    check(ops.score(logits, temperature, top_k, top_p, tok), lp, rtol=1e-5, atol=1e-5)
    best, worst = logits.argmax(-1).int(), logits.argmin(-1).int()
    fifth = logits.topk(5).indices[:, 4].int().contiguous()
    for given in (tok, best, worst, fifth, torch.full((R,), 104, dtype=torch.int32).cuda()):
        got = ops.score(logits, temperature, top_k, top_p, given)
        want = ref.score(logits, temperature, top_k, top_p, given)
        masked = want < -1e37
        assert torch.equal(got < -1e37, masked), (given.tolist(), got.tolist(), want.tolist())
        check(got[~masked], want[~masked], rtol=1e-4, atol=1e-4)
        assert (got[masked] == ops.SCORE_MASKED).all()
    got = ops.score(logits, temperature, top_k, top_p, worst)
    assert got[4] == ops.SCORE_MASKED and got[8] == ops.SCORE_MASKED and got[5] > -1e3   # greedy rows; a plain draw


@pytest.mark.parametrize("M", [17, 33, 48, 64, 100, 256, 400, 512, 768, 1100, 1536, 1537])
@pytest.mark.parametrize("N,K", [(4096, 2304), (2304, 2048), (2304, 4608), (1000, 9216), (2304, 9216)])
def test_gemm_dispatch_at_a_few_hundred_rows(M, N, K):
    """What the dispatcher chooses by itself for portions of a few hundred tokens and for many decoding requests
    (the wide kernel with a tile and a cut of K that it fits to the sizes; large tiles beyond) against the reference,
    plain and gated."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles
    a = rand((M, K), torch.bfloat16, 140)
    w, w2 = rand((N, K), torch.bfloat16, 141, 0.03), rand((N, K), torch.bfloat16, 142, 0.03)
    t = dict(bf16_steps=1.0)
    check(ops.gemm(a, pack_tiles(w)).float(), ref.gemm(a, w).float(), **t)
    if N <= 2304:
        check(ops.gemm(a, pack_gate_up(w, w2)).float(), ref.gemm(a, w, w2=w2).float(), **gated(t))
    # rows of wider rows in and out, as the attention output and the fused projection are
    big, out = rand((M, K + 64), torch.bfloat16, 143), torch.zeros((M, N + 8), dtype=torch.bfloat16, device="cuda")
    ops.gemm(big[:, 32:32 + K], pack_tiles(w), out=out[:, :N])
    check(out[:, :N].float(), ref.gemm(big[:, 32:32 + K], w).float(), **t)
    assert not out[:, N:].any()


@pytest.mark.parametrize("M,N,K", [(1, 1024, 24576), (8, 1024, 24576), (16, 520, 24640), (9, 2304, 9216), (12, 2304, 8192),
                                   (16, 2304, 9216), (13, 1000, 8256), (9, 2304, 8200), (24, 8192, 3584), (12, 4608, 4096),
                                   (32, 5000, 3584)])
def test_gemm_dispatch_of_few_rows_against_a_long_k(M, N, K):
    """Few rows against a very long K, 9 to 16 rows against a long one and 9 to 32 rows against a large weight are
    cut over workgroups by the dispatcher (the wide kernel; where K is no multiple of 64, what takes it): against the reference, also with
    rows of wider rows in and out."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_tiles
    a = rand((M, K), torch.bfloat16, 150)
    w = rand((N, K), torch.bfloat16, 151, 0.03)
    t = dict(bf16_steps=1.0)
    check(ops.gemm(a, pack_tiles(w)).float(), ref.gemm(a, w).float(), **t)
    big, out = rand((M, K + 64), torch.bfloat16, 152), torch.zeros((M, N + 8), dtype=torch.bfloat16, device="cuda")
    ops.gemm(big[:, 32:32 + K], pack_tiles(w), out=out[:, :N])
    check(out[:, :N].float(), ref.gemm(big[:, 32:32 + K], w).float(), **t)
    assert not out[:, N:].any()


@pytest.mark.parametrize("activation", [0, 1, 2])
@pytest.mark.parametrize("M", [5, 16, 40, 300])
def test_gated_activations_in_every_product_kernel(M, activation):
    """act(a.Wg^T) * (a.Wu^T) for the three activations that the reference registers (tanh-gelu, silu, squared relu:
    simply/model_lib.py:93-104), in each kernel that has the gated epilogue: the 32-bit one, the few-rows one, the
    one with the norms in front, the tiled one with and without its sum kernel, the wide one."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up
    N, K = 200, 256
    a = rand((M, K), torch.bfloat16, 130, 1.5)
    w, w2 = rand((N, K), torch.bfloat16, 131, 0.08), rand((N, K), torch.bfloat16, 132, 0.08)
    tg = pack_gate_up(w, w2)
    want = ref.gemm(a, w, w2=w2, activation=activation).float()
    assert want.abs().max() > 0.5
    if activation:
        assert not torch.allclose(want, ref.gemm(a, w, w2=w2).float(), rtol=2e-2, atol=2e-2)   # the activations differ
    # (the squared relu doubles the relative error of its argument: one step more than gelu and silu)
    t = dict(bf16_steps=4.0 if activation == 2 else 3.0)
    a32, w32, w232 = a.float(), w.float(), w2.float()
    check(ops.gemm(a32, w32, w2=w232, activation=activation),
                               ref.gemm(a32, w32, w2=w232, activation=activation), rtol=1e-4, atol=1e-4)
    check(ops.gemm(a, w, w2=w2, activation=activation, algo=ops.ALGO_GENERIC).float(), want, **t)
    check(ops.gemm(a, tg, activation=activation).float(), want, **t)      # the dispatcher's choice
    if M <= 16:
        check(ops.gemm(a, tg, activation=activation, algo=ops.ALGO_SKINNY).float(), want, **t)
        h = a.float() * 3.0
        wn = rand((K,), torch.bfloat16, 133, 0.3)
        normed = ref.rmsnorm(h, wn, 1e-6, True, torch.bfloat16)
        got = ops.gemm_normed(None, h, None, tg, post_weight=None, post_eps=0.0, post_plus_one=True, next_weight=wn,
                              next_eps=1e-6, next_plus_one=True, activation=activation)
        check(got.float(), ref.gemm(normed, w, w2=w2, activation=activation).float(), **t)
    for cuts in (1, 2):
        got = ops.gemm(a, tg, activation=activation, algo=ops.ALGO_TILED, shape=cuts)
        check(got.float(), want, **t)
    check(ops.gemm(a, tg, activation=activation, algo=ops.ALGO_WIDE).float(), want, **t)
    from simply_amd.kernels.lib import KernelError
    with pytest.raises(KernelError, match="activation"):
        ops.gemm(a, tg, activation=3)


@pytest.mark.parametrize("M", [1, 3, 8, 9, 13, 16])
@pytest.mark.parametrize("K,N", [(128, 96), (2304, 4096), (2560, 512), (2048, 200), (3584, 512), (4608, 64), (4640, 64),
                                 (96, 40), (72, 64), (3072, 200), (4096, 512), (2816, 96), (3328, 64)])
def test_gemm_normed(M, K, N):
    """Residual sum, two norms and the product in one kernel against the separate references."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_gate_up, pack_tiles
    y, h = rand((M, K), torch.bfloat16, 100, 2.0), rand((M, K), torch.float32, 101, 4.0)
    wp, wn = rand((K,), torch.bfloat16, 102, 0.3), rand((K,), torch.bfloat16, 103, 0.3)
    w, w2 = rand((N, K), torch.bfloat16, 104, 0.05), rand((N, K), torch.bfloat16, 105, 0.05)
    tw, tg = pack_tiles(w), pack_gate_up(w, w2)
    fits = (8 if M <= 8 else 16) * (K + 8) * 2 + 8 * 2 * 16 * 17 * 4 <= 160 * 1024   # activations and tiles in LDS
    assert ops.gemm_normed_takes(M, tw) == (fits and K % 32 == 0 and K <= 4608)
    # what it takes it computes; it says that it pays where it has a prologue for the width (the widths of the three
    # Gemma 2 sizes and other multiples of 256 such as 3072 and 4096) or the row is at most 2560 wide
    assert ops.gemm_normed_pays(M, tw) == (ops.gemm_normed_takes(M, tw)
                                           and (K <= 2560 or K in (3072, 3584, 4096, 4608)))
    assert not ops.gemm_normed_pays(M, pack_tiles(torch.zeros((16 * 8192 + 16, 64), dtype=torch.bfloat16).cuda()))
    if not ops.gemm_normed_takes(M, tw):
        return
    kw = dict(post_weight=wp, post_eps=1e-6, post_plus_one=True, next_weight=wn, next_eps=1e-5, next_plus_one=True)
    t = dict(bf16_steps=1.0)
    for with_y in (True, False):
        h_ref = h.clone()
        a_ref = ref.add_rmsnorm(y, h_ref, post_weight=wp, post_eps=1e-6, next_weight=wn, next_eps=1e-5,
                                out_dtype=torch.bfloat16) if with_y else ref.rmsnorm(h, wn, 1e-5, True, torch.bfloat16)
        h_out = torch.full_like(h, 7.0)
        got = ops.gemm_normed(y if with_y else None, h, h_out if with_y else None, tw, **kw)
        check(got.float(), ref.gemm(a_ref, w).float(), **t)
        if with_y:
            check(h_out, h_ref, rtol=1e-5, atol=1e-5)
        got = ops.gemm_normed(y if with_y else None, h, h_out if with_y else None, tg, **kw)
        check(got.float(), ref.gemm(a_ref, w, w2=w2).float(), **gated(t))
        got = ops.gemm_normed(y if with_y else None, h, h_out if with_y else None, tw, soft_cap=3.0,
                              out_dtype=torch.float32, **kw)
        check(got, ref.gemm(a_ref, w, soft_cap=3.0, out_dtype=torch.float32), rtol=5e-3, atol=5e-3)
    # without a post-norm the residual takes y as it is
    h_out = torch.empty_like(h)
    ops.gemm_normed(y, h, h_out, tw, **dict(kw, post_weight=None))
    check(h_out, h + y.float(), rtol=1e-6, atol=1e-6)
    assert not ops.gemm_normed_takes(17, tw) and not ops.gemm_normed_takes(M, w)


def prefill_units(lens, q_lens, per_unit):
    """Units of at most per_unit tokens of requests whose last q tokens are this step's, each request's units
    filled up to a multiple of the kernel's group: what the host hands to the prompt-portion kernel."""
    from simply_amd.kernels import ops
    units, t0 = [], 0
    for s, (l, q) in enumerate(zip(lens, q_lens)):
        for o in range(0, q, per_unit):
            units.append((s, t0 + o, min(per_unit, q - o), l - q + o))
        while len(units) % ops.prefill_units_per_group():
            units.append((s, t0 + q, 0, l))
        t0 += q
    return torch.tensor(units, dtype=torch.int32).cuda()


@pytest.mark.parametrize("H,Kh,hd,P,window,cap", [
    (8, 4, 256, 16, None, 50.0), (8, 4, 256, 16, 100, 50.0), (4, 2, 64, 16, 33, None), (16, 1, 128, 32, None, 30.0),
    (2, 2, 128, 64, 200, None), (6, 3, 64, 16, 1, 20.0), (6, 2, 128, 16, 40, 50.0), (5, 1, 64, 48, None, None)])
@pytest.mark.parametrize("splits", [0, 1, 3])
def test_paged_attention_prefill(H, Kh, hd, P, window, cap, splits):
    """The prompt-portion bfloat16 kernel against the plain reference: portions that start at 0 and after a
    history, with lengths around unit, tile and page edges, unwritten page tails holding NaN, keys also cut
    over workgroups."""
    from simply_amd.kernels import ops
    G = H // Kh
    per_unit = 16 // G
    lens = [300, 77, 1000, 64, 129, 5]
    q_lens = [300, 40, 130, 64, 2, 5]
    kp, vp, table = paged_setup(torch.bfloat16, len(lens), H, Kh, hd, P, lens, 71)
    _, ts, ps = seq_meta_for(lens, q_lens)
    units = prefill_units(lens, q_lens, per_unit)
    T = ts.numel()
    q = rand((T, (H + 2 * Kh) * hd), torch.bfloat16, 72, 0.3)
    out = torch.zeros((T, H * hd), dtype=torch.bfloat16).cuda()
    ops.paged_attention_prefill(q, kp, vp, table, units, 0, units.shape[0], H, window=window, soft_cap=cap,
                                max_kv_len=max(lens), max_q_len=per_unit, out=out, num_splits=splits)
    want = ref.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=cap)
    assert torch.isfinite(out.float()).all()
    check(out.float(), want.float(), bf16_steps=2.0)
    # the few-rows kernel on the same units gives the same up to rounding
    out2 = torch.zeros_like(out)
    ops.paged_attention_decode(q, kp, vp, table, units, 0, units.shape[0], H, window=window, soft_cap=cap,
                               max_kv_len=max(lens), max_q_len=per_unit, out=out2)
    check(out.float(), out2.float(), bf16_steps=2.0)
    # a sub-range of the units: the other rows stay untouched
    first = next(i for i in range(units.shape[0]) if int(units[i, 0]) == 2)
    count = sum(1 for i in range(units.shape[0]) if int(units[i, 0]) == 2)
    out3 = torch.full_like(out, 7.0)
    ops.paged_attention_prefill(q, kp, vp, table, units, first, count, H, window=window, soft_cap=cap,
                                max_kv_len=max(lens), max_q_len=per_unit, out=out3, num_splits=splits)
    a, b = sum(q_lens[:2]), sum(q_lens[:3])
    check(out3[a:b].float(), out[a:b].float(), bf16_steps=2.0)
    assert (out3[:a] == 7).all() and (out3[b:] == 7).all()
    with pytest.raises(Exception, match="groups of"):
        ops.paged_attention_prefill(q, kp, vp, table, units, 0, 3, H, window=window, soft_cap=cap,
                                    max_kv_len=max(lens), max_q_len=per_unit, out=out3)


def test_paged_attention_prefill_far_key_and_window_edge():
    """Every query row of a long portion must find one key far back whose score stands out, and a windowed
    layer must see it exactly while it is inside each row's own window."""
    from simply_amd.kernels import ops
    H, Kh, hd, P, L, Q = 2, 1, 128, 16, 2500, 600
    kp, vp, table = paged_setup(torch.bfloat16, 1, H, Kh, hd, P, [L], 73)
    kp = ref.stored_keys_as_rows(kp) * 0.01
    far = 1871
    page, off = int(table[0, far // P]), far % P
    kp[page, 0, off] = 0.0
    kp[page, 0, off, 5] = 60.0
    kp = ref.rows_as_stored_keys(kp)
    vp[page, 0, :, off] = 3.0
    units = prefill_units([L], [Q], 8)
    q = torch.zeros((Q, 4 * hd), dtype=torch.bfloat16).cuda()
    q[:, 5] = 1.0
    q[:, hd + 5] = 1.0
    positions = torch.arange(L - Q, L)
    for window in (None, 300):
        out = torch.zeros((Q, H * hd), dtype=torch.bfloat16).cuda()
        ops.paged_attention_prefill(q, kp, vp, table, units, 0, units.shape[0], H, window=window, soft_cap=None,
                                    max_kv_len=L, max_q_len=8, out=out)
        found = (out.float().mean(dim=1) - 3.0).abs().cpu() < 0.05
        sees = (positions >= far) & ((positions - far < window) if window else torch.ones_like(positions, dtype=torch.bool))
        assert torch.equal(found, sees), (window, (found != sees).nonzero().flatten().tolist()[:10])


@pytest.mark.parametrize("window", [None, 30000])
def test_paged_attention_far_keys_of_a_long_context(window):
    """70,000 keys (more than 16 bits count): every query must find the one key, planted 3 to 69,000 positions back,
    whose score stands out for it; in the prompt-portion kernel, the few-rows kernel (keys cut over workgroups) and
    the generic kernel, with and without a window."""
    from simply_amd.kernels import ops
    H, Kh, hd, P, L, Q = 2, 1, 128, 16, 70000, 64
    kp, vp, table = paged_setup(torch.bfloat16, 1, H, Kh, hd, P, [L], 75)
    kp = ref.stored_keys_as_rows(kp) * 0.01
    far = [3, 40001, 65535, 65536, 69000, L - 70]
    for f, at in enumerate(far):
        page, off = int(table[0, at // P]), at % P
        kp[page, 0, off] = 0.0
        kp[page, 0, off, 5 + f] = 60.0
        vp[page, 0, :, off] = float(f + 1)
    kp = ref.rows_as_stored_keys(kp)
    q = torch.zeros((Q, 4 * hd), dtype=torch.bfloat16).cuda()
    which = torch.arange(Q) % len(far)
    for i in range(Q):
        q[i, 5 + int(which[i])] = 1.0
        q[i, hd + 5 + int(which[i])] = 1.0
    positions = torch.arange(L - Q, L)
    at = torch.tensor(far)[which]
    sees = (at <= positions) & ((positions - at < window) if window else torch.ones(Q, dtype=torch.bool))
    want = torch.where(sees, (which + 1).float(), torch.zeros(Q))

    def found(out):
        m = out.float().mean(dim=1).cpu()
        return torch.where((m - m.round()).abs() < 0.05, m.round(), torch.full_like(m, -1.0)) * (m.abs() > 0.5)

    units = prefill_units([L], [Q], 8)
    out = torch.zeros((Q, H * hd), dtype=torch.bfloat16).cuda()
    ops.paged_attention_prefill(q, kp, vp, table, units, 0, units.shape[0], H, window=window, soft_cap=None,
                                max_kv_len=L, max_q_len=8, out=out)
    assert torch.equal(found(out), want), found(out).tolist()
    out = torch.zeros_like(out)
    ops.paged_attention_decode(q, kp, vp, table, units, 0, units.shape[0], H, window=window, soft_cap=None,
                               max_kv_len=L, max_q_len=8, out=out)
    assert torch.equal(found(out), want), found(out).tolist()
    out = torch.zeros_like(out)
    ts, ps = torch.zeros(Q, dtype=torch.int32).cuda(), positions.int().cuda()
    ops.paged_attention(q, kp, vp, table, ts, ps, H, window=window, soft_cap=None, out=out)
    assert torch.equal(found(out), want), found(out).tolist()


def test_bfloat16_rounding_of_the_kernels():
    """The device's conversion to bfloat16 rounds to nearest even, as torch does: all exponents, ties, subnormals."""
    from simply_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    bits = torch.randint(-2**31, 2**31 - 1, (64, 4096), generator=g, dtype=torch.int64).to(torch.int32)
    bits[0, :2048] = (torch.arange(2048, dtype=torch.int32) << 16) | 0x8000          # exact ties, even and odd
    bits[1, :2048] = (torch.arange(2048, dtype=torch.int32) << 16) | 0x7fff
    bits[2, :2048] = (torch.arange(2048, dtype=torch.int32) << 16) | 0x8001
    x = bits.view(torch.float32).cuda()
    idx = torch.arange(64, dtype=torch.int32).cuda()
    got = ops.gather_rows(x, idx, out_dtype=torch.bfloat16)
    want = x.to(torch.bfloat16)
    nan = torch.isnan(x)
    assert torch.equal(torch.isnan(got.float()), nan)
    assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan])


@pytest.mark.parametrize("M", [1, 8, 13])
@pytest.mark.parametrize("H,Kh,hd,P,K", [(8, 4, 256, 16, 2304), (4, 2, 64, 16, 128), (3, 1, 32, 48, 96), (2, 2, 128, 32, 2560), (4, 2, 256, 16, 3584),
                                         (4, 4, 128, 16, 4608), (6, 2, 128, 16, 3072), (4, 1, 64, 16, 4096), (2, 1, 32, 16, 2816)])
@pytest.mark.parametrize("rotate", [True, False])
def test_gemm_normed_rotary(M, H, Kh, hd, P, K, rotate):
    """Norms, q/k/v projection, rotation, query scale and cache write in one kernel against the same from the
    separate kernels (residual sum and norms in the projection, then the rotary kernel)."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_tiles
    N = (H + 2 * Kh) * hd
    y, h = rand((M, K), torch.bfloat16, 110, 2.0), rand((M, K), torch.float32, 111, 4.0)
    wp, wn = rand((K,), torch.bfloat16, 112, 0.3), rand((K,), torch.bfloat16, 113, 0.3)
    tw = pack_tiles(rand((N, K), torch.bfloat16, 114, 0.05))
    positions = torch.tensor([0, 1, 5, 100, 8000, 33, 7, 2, 4095, 4096, 9, 10, 11][:M], dtype=torch.int32).cuda()
    ts = (10000.0 ** (2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().cuda() if rotate else None
    pages = 5
    slots = torch.randperm(pages * P)[:M].to(torch.int64).cuda()
    norm = dict(post_weight=wp, post_eps=1e-6, post_plus_one=True, next_weight=wn, next_eps=1e-5, next_plus_one=True)
    if not ops.gemm_normed_takes(M, tw):   # 13 rows of 4,608 do not fit in LDS: refused, with the sizes in the message
        with pytest.raises(ops.KernelError, match=f"M={M} K={K}"):
            ops.gemm_normed_rotary(y, h, torch.empty_like(h), tw, **norm, positions=positions, timescale=ts, scale_factor=1.0,
                                   query_scale=12.0, num_heads=H, num_kv_heads=Kh, head_dim=hd)
        return
    for with_y in (True, False):
        kp, vp = torch.zeros((pages, Kh, P, hd), dtype=torch.bfloat16).cuda(), torch.zeros((pages, Kh, hd, P), dtype=torch.bfloat16).cuda()
        kp2, vp2 = kp.clone(), vp.clone()
        h_out, h_out2 = torch.full_like(h, 7.0), torch.full_like(h, 7.0)
        got = ops.gemm_normed_rotary(y if with_y else None, h, h_out if with_y else None, tw, **norm, positions=positions,
                                     timescale=ts, scale_factor=1.0, query_scale=12.0, num_heads=H, num_kv_heads=Kh,
                                     head_dim=hd, slot_mapping=slots, k_pages=kp, v_pages=vp)
        want = ops.gemm_normed(y if with_y else None, h, h_out2 if with_y else None, tw, **norm)
        ops.rope_cache_write(want, positions, ts, 1.0, 12.0, H, Kh, hd, slots, kp2, vp2)
        t = dict(rtol=1e-2, atol=1e-3)   # the same sums; the rotation's products may round one bfloat16 step apart
        check(got[:, :H * hd].float(), want[:, :H * hd].float(), **t)
        check(kp.float(), kp2.float(), **t)
        assert torch.equal(vp, vp2)
        assert torch.equal(h_out, h_out2)
    # without pages only the queries are produced
    got = ops.gemm_normed_rotary(None, h, None, tw, **norm, positions=positions, timescale=ts, scale_factor=1.0,
                                 query_scale=12.0, num_heads=H, num_kv_heads=Kh, head_dim=hd)
    check(got[:, :H * hd].float(), want[:, :H * hd].float(), rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("M,N,K", [(17, 2304, 2048), (64, 2304, 9216), (64, 2304, 2048), (100, 3584, 4096), (512, 2304, 9216),
                                   (40, 200, 512), (8, 2304, 2048), (2048, 2304, 2048)])
def test_deferred_sum_of_a_product_is_added_up_by_the_norm(M, N, K):
    """A product computed in cuts of K may leave their sum to the residual/norm kernel behind it: residual stream and
    normed activations are the same to the bit as with the product's own sum kernel in between, and `materialize()`
    is that product."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_tiles
    a = rand((M, K), torch.bfloat16, 95)
    w = pack_tiles(rand((N, K), torch.bfloat16, 96, 0.05))
    h0 = rand((M, N), torch.float32, 97, 3.0)
    w1, w2 = rand((N,), torch.bfloat16, 98, 0.3), rand((N,), torch.bfloat16, 99, 0.3)
    whole = ops.gemm(a, w)
    for with_next in (True, False):
        kw = dict(post_weight=w1, post_eps=1e-6, next_weight=w2 if with_next else None, next_eps=1e-6,
                  out_dtype=torch.bfloat16)
        h_want, h_got = h0.clone(), h0.clone()
        o_want = ops.add_rmsnorm(whole, h_want, **kw)
        y = ops.gemm(a, w, defer_sum=True)
        o_got = ops.add_rmsnorm(y, h_got, **kw)
        assert torch.equal(h_got, h_want)
        assert (o_got is None) == (o_want is None) and (o_got is None or torch.equal(o_got, o_want))
    y = ops.gemm(a, w, defer_sum=True)
    if isinstance(y, ops.PartialSums):
        assert y.planes.shape[0] > 1 and torch.equal(y.materialize(), whole)
    else:
        assert torch.equal(y, whole)
    if (M, N, K) in ((64, 2304, 9216), (512, 2304, 9216)):
        assert isinstance(ops.gemm(a, w, defer_sum=True), ops.PartialSums)   # these sizes do cut K


@pytest.mark.parametrize("T,H,K,hd,P", [(64, 8, 4, 256, 16), (17, 4, 2, 64, 16), (100, 16, 8, 128, 32), (33, 3, 1, 48, 4)])
def test_deferred_sum_of_the_projection_is_added_up_by_the_rotary_kernel(T, H, K, hd, P):
    """The fused q/k/v projection may leave the sum of its cuts of K to the rotate-and-write kernel: queries and
    pages are the same to the bit as with the product's own sum kernel in between."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.packing import pack_tiles
    D = 2304 if hd >= 128 else 512
    N = (H + 2 * K) * hd
    a = rand((T, D), torch.bfloat16, 101)
    w = pack_tiles(rand((N, D), torch.bfloat16, 102, 0.05))
    positions = (torch.arange(T, dtype=torch.int32) * 7 % 1000).cuda()
    ts = (10000.0 ** (2 * torch.arange(hd // 2, dtype=torch.float64) / hd)).float().cuda()
    pages = 2 * -(-T // P) + 3
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(5))[:T].to(torch.int64).cuda()
    results = []
    for defer in (False, True):
        kp = torch.zeros((pages, K, P, hd), dtype=torch.bfloat16, device="cuda")
        vp = torch.zeros((pages, K, hd, P), dtype=torch.bfloat16, device="cuda")
        y = ops.gemm(a, w, defer_sum=defer)
        qkv = ops.rope_cache_write(y, positions, ts, 1.0, 16.0, H, K, hd, slot_mapping=slots, k_pages=kp, v_pages=vp)
        results.append((qkv[:, :H * hd].clone(), kp, vp, isinstance(y, ops.PartialSums)))
    (q0, k0, v0, _), (q1, k1, v1, cut) = results
    assert torch.equal(q0, q1) and torch.equal(k0, k1) and torch.equal(v0, v1)
    if (T, hd) == (64, 256):
        assert cut   # this size does cut K


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("T,D,R", [(5, 100, 3), (16, 2304, 16), (9, 4608, 1), (40, 6000, 7), (3, 48, 3)])
def test_add_rmsnorm_rows(dtype, T, D, R):
    """The final norm of the rows whose logits are wanted, with the last residual sum, in one kernel: equals the sum
    over all rows, a gather and the norm; the residual stream is left as it was."""
    from simply_amd.kernels import ops
    y = rand((T, D), dtype, 150, 2.0)
    h = rand((T, D), torch.float32, 151, 5.0)
    w1, w2 = rand((D,), dtype, 152, 0.3), rand((D,), dtype, 153, 0.3)
    index = torch.randperm(T)[:R].to(torch.int32).cuda()
    for with_post in (True, False):
        h_ref = h.clone()
        ref.add_rmsnorm(y, h_ref, post_weight=w1 if with_post else None, post_eps=1e-6)
        want = ref.rmsnorm(h_ref[index.long()], w2, 1e-5, True, dtype)
        before = h.clone()
        got = ops.add_rmsnorm_rows(y, h, index, post_weight=w1 if with_post else None, post_eps=1e-6, next_weight=w2,
                                   next_eps=1e-5, out_dtype=dtype)
        assert torch.equal(h, before)
        check(got.float(), want.float(), **tol(dtype))


def test_decode_advance_with_slots():
    """Between two decode steps on the device: tokens handed on, positions and counters moved, and the slot of the
    next key in every cache group, in one launch: equals the separate kernels."""
    from simply_amd.kernels import ops
    B, P, steps = 5, 16, 4
    g = torch.Generator().manual_seed(9)
    positions = torch.tensor([15, 16, 0, 31, 100], dtype=torch.int32).cuda()
    token_seq = torch.tensor([3, 0, 4, 1, 2], dtype=torch.int32).cuda()
    tables = [torch.randint(0, 50, (6, 9), generator=g, dtype=torch.int32).cuda() for _ in range(3)]

    def state():
        return dict(counter=torch.zeros(1, dtype=torch.int32).cuda(), tokens_in=torch.zeros(B, dtype=torch.int32).cuda(),
                    positions=positions.clone(), meta=torch.arange(4 * B, dtype=torch.int32).reshape(B, 4).cuda().contiguous(),
                    draws=torch.arange(B, dtype=torch.int32).cuda(), out_tok=torch.zeros((steps, B), dtype=torch.int32).cuda(),
                    out_lp=torch.zeros((steps, B)).cuda(), slots=[torch.zeros(B, dtype=torch.int64).cuda() for _ in tables])

    a, b = state(), state()
    for k in range(3):
        toks = torch.randint(0, 1000, (B,), generator=g, dtype=torch.int32).cuda()
        lps = torch.randn(B, generator=g).cuda()
        ops.decode_advance(a["counter"], toks, lps, a["tokens_in"], a["positions"], a["meta"], a["draws"], a["out_tok"],
                           a["out_lp"])
        for t, s in zip(tables, a["slots"]):
            ops.decode_slots(a["positions"], token_seq, t, P, s)
        ops.decode_advance(b["counter"], toks, lps, b["tokens_in"], b["positions"], b["meta"], b["draws"], b["out_tok"],
                           b["out_lp"], token_seq=token_seq, page_size=P, groups=list(zip(tables, b["slots"])))
        for name in ("counter", "tokens_in", "positions", "meta", "draws", "out_tok", "out_lp"):
            assert torch.equal(a[name], b[name]), (k, name)
        for s1, s2, t in zip(a["slots"], b["slots"], tables):
            assert torch.equal(s1, s2)
            pos = b["positions"].long()
            assert torch.equal(s2, t[token_seq.long(), pos // P].long() * P + pos % P)
    assert int(b["counter"]) == 3 and torch.equal(b["positions"], positions + 3)


def test_machine_probes_run_and_refuse():
    """The two probe kernels (reading memory with all CUs, retiring MFMA instructions) run to their end, count the
    work they are said to do, and refuse buffers that do not fit."""
    from simply_amd.kernels import ops
    from simply_amd.kernels.lib import KernelError
    buffer = torch.ones(3 * 8192 // 4, dtype=torch.float32, device="cuda:0")  # three pieces: an odd count per wave
    ops.probe_hbm_read(buffer)
    ops.probe_hbm_read(buffer, torch.tensor([2, 0, 1], dtype=torch.int32, device="cuda:0"))
    operands = torch.randn(8192, device="cuda:0").to(torch.bfloat16)
    assert ops.probe_mfma(operands, 10, workgroups=4) == 2.0 * 16 * 16 * 32 * 16 * 10 * 8 * 4
    torch.cuda.synchronize()
    with pytest.raises(KernelError):
        ops.probe_hbm_read(torch.ones(1000, dtype=torch.float32, device="cuda:0"))
    with pytest.raises(KernelError):
        ops.probe_hbm_read(buffer, torch.tensor([0, 1], dtype=torch.int32, device="cuda:0"))
    with pytest.raises(KernelError):
        ops.probe_mfma(operands[:100], 10)
