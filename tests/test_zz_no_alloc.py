"""The decode attention entry point that allocates nothing (sa_paged_attention_decode_static: the partial results
of the key ranges go into an array inside the library) against the one that takes a workspace, called through
ctypes as a program without torch bindings would: two calls in a row on the same GPU, the second with a smaller
input, so that the first call's partial results are still in the array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

P_, I_, L_, F_ = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
COMMON = [P_, L_, P_, P_, P_, I_, P_, I_, I_, P_, L_, I_, I_, I_, I_, I_, F_, I_, I_, I_]


def load_library():
    from simply_amd.kernels import build

    path = build.find_library()
    assert path is not None, "the kernel library has not been built"
    lib = ctypes.CDLL(path)
    lib.sa_last_error.restype = ctypes.c_char_p
    lib.sa_paged_attention_decode.argtypes = COMMON + [P_, L_, P_]
    lib.sa_paged_attention_decode.restype = I_
    lib.sa_paged_attention_decode_static.argtypes = COMMON + [P_]
    lib.sa_paged_attention_decode_static.restype = I_
    lib.sa_paged_attention_decode_static_bytes.restype = I_
    return lib


def make_case(lens, H, Kh, hd, page, seed, device):
    """One decoding token per request at position len - 1 over random pages."""
    g = torch.Generator(device=device).manual_seed(seed)
    blocks = [-(-n // page) for n in lens]
    num_pages = sum(blocks) + 3
    k_pages = torch.randn(num_pages, Kh, page, hd, generator=g, device=device).to(torch.bfloat16)
    v_pages = torch.randn(num_pages, Kh, hd, page, generator=g, device=device).to(torch.bfloat16)
    order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.full((len(lens), max(blocks)), -1, dtype=torch.int32)
    meta = torch.zeros((len(lens), 4), dtype=torch.int32)
    for i, (n, b) in enumerate(zip(lens, blocks)):
        table[i, :b] = torch.tensor([order.pop() for _ in range(b)], dtype=torch.int32)
        meta[i] = torch.tensor([i, i, 1, n - 1], dtype=torch.int32)
    q = (torch.randn(len(lens), H * hd, generator=g, device=device) * 0.3).to(torch.bfloat16)
    return q, k_pages, v_pages, table.to(device), meta.to(device)


def run_both(lib, case, H, Kh, hd, page, window, max_len, num_splits, workspace):
    q, k_pages, v_pages, table, meta = case
    S = q.shape[0]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for static in (False, True):
        out = torch.full((S, H * hd), float("nan"), dtype=torch.bfloat16, device=q.device)
        args = [q.data_ptr(), q.stride(0), k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), table.stride(0),
                meta.data_ptr(), 0, S, out.data_ptr(), out.stride(0), H, Kh, hd, page, window, 50.0, max_len, 1,
                num_splits]
        if static:
            rc = lib.sa_paged_attention_decode_static(*args, stream)
        else:
            rc = lib.sa_paged_attention_decode(*args, workspace.data_ptr(), workspace.numel(), stream)
        assert rc == 0, lib.sa_last_error().decode()
        outs.append(out)
    torch.cuda.synchronize()
    return outs


@pytest.mark.parametrize("window", [0, 300])
def test_static_scratch_equals_workspace(window):
    lib = load_library()
    device = torch.device("cuda:0")
    H, Kh, hd, page = 8, 4, 256, 16
    assert lib.sa_paged_attention_decode_static_bytes() == 16 << 20
    workspace = torch.empty(64 << 20, dtype=torch.uint8, device=device)
    first = make_case([1500, 700, 333, 90, 2048, 17], H, Kh, hd, page, 1, device)
    second = make_case([400, 65], H, Kh, hd, page, 2, device)
    for num_splits in (0, 7):
        for case, max_len in ((first, 2048), (second, 400)):   # the second call is the smaller one
            want, got = run_both(lib, case, H, Kh, hd, page, window, max_len, num_splits, workspace)
            assert torch.isfinite(want.float()).all() and want.float().abs().max() > 0
            assert torch.equal(want, got), (num_splits, max_len, (want.float() - got.float()).abs().max().item())
            # ... and both against the plain torch attention over the same pages (a fault that the two entry points
            # shared would pass the comparison above): within two bfloat16 steps at each row's largest value
            import torch_ops
            q, k_pages, v_pages, table, meta = case
            plain = torch_ops.paged_attention(q, k_pages, v_pages, table, meta[:, 0].contiguous(), meta[:, 3].contiguous(), H,
                                              window=window or None, soft_cap=50.0).float()
            bound = 2 * torch.exp2(torch.floor(torch.log2(plain.abs().amax(dim=-1, keepdim=True))) - 7)
            assert ((got.float() - plain).abs() <= bound).all(), (num_splits, max_len)


def test_static_scratch_refuses_what_does_not_fit():
    lib = load_library()
    device = torch.device("cuda:0")
    H, Kh, hd, page = 8, 4, 256, 16
    case = make_case([300] * 64, H, Kh, hd, page, 3, device)
    q, k_pages, v_pages, table, meta = case
    out = torch.zeros((64, H * hd), dtype=torch.bfloat16, device=device)
    # 64 requests x 4 heads x 9 ranges x 16 rows x 260 floats = 38 MB of partial results
    rc = lib.sa_paged_attention_decode_static(
        q.data_ptr(), q.stride(0), k_pages.data_ptr(), v_pages.data_ptr(), table.data_ptr(), table.stride(0),
        meta.data_ptr(), 0, 64, out.data_ptr(), out.stride(0), H, Kh, hd, page, 0, 50.0, 300, 1, 9,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc != 0
    msg = lib.sa_last_error().decode()
    assert "scratch memory holds 16777216" in msg, msg
    assert not out.any()      # nothing ran
