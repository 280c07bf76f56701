"""Tensor-level calls of the gfx950 kernels.

Each function checks on the host that shapes, element types, strides and devices
are what the kernel assumes, then launches on torch's current stream.  Nothing
here computes on the CPU and nothing falls back to a library routine.
"""
from __future__ import annotations

import ctypes

import torch

from . import lib as _lib
from .lib import KernelError
from .packing import TiledWeight

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

ALGO_AUTO, ALGO_GENERIC, ALGO_SKINNY, ALGO_TILED, ALGO_WIDE = 0, 1, 2, 3, 4


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported by the kernels (float32, bfloat16)") from None


def _dev(*tensors) -> None:
    first = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("the kernels run on the GPU only: a tensor lies on " + str(t.device))
        if first is None:
            first = t.device
        elif t.device != first:
            raise KernelError(f"tensors lie on different devices: {first} and {t.device}")


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current torch stream's handle (through torch's own fast accessors where it has them: this is called once
    per kernel launch, and `torch.cuda.current_stream()` costs about as much as the launch)."""
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} "
                          f"strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, what: str, n: int | None = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what}: {t.numel()} entries, {n} needed")


# --------------------------------------------------------------------------- row-wise


def embed(table: "torch.Tensor | TiledWeight", tokens: torch.Tensor, scale: float,
          out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = float32(table[tokens[t]]) * scale.  The table may be row-major or tiled."""
    packed = isinstance(table, TiledWeight)
    data = table.data if packed else table
    _dev(data, tokens, out)
    V, D = table.shape
    T = tokens.numel()
    _i32(tokens, "embed: tokens")
    if not data.is_contiguous():
        raise KernelError("embed: the table must be contiguous")
    if out is None:
        out = torch.empty((T, D), dtype=torch.float32, device=data.device)
    if out.dtype != torch.float32 or not out.is_contiguous() or tuple(out.shape) != (T, D):
        raise KernelError("embed: the output must be a contiguous float32 [T, D] tensor")
    _lib.call("sa_embed", _ptr(data), _code(data), _ptr(tokens), _ptr(out), T, D, V, float(scale), int(packed),
              _stream())
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, plus_one: bool, out_dtype: torch.dtype,
            out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(x, weight, out)
    xs = _rows(x, "rmsnorm: x")
    T, D = x.shape
    if weight.numel() != D or not weight.is_contiguous():
        raise KernelError(f"rmsnorm: weight has {weight.numel()} entries for width {D}")
    if out is None:
        out = torch.empty((T, D), dtype=out_dtype, device=x.device)
    if tuple(out.shape) != (T, D):
        raise KernelError("rmsnorm: output shape differs from the input's")
    os_ = _rows(out, "rmsnorm: out")
    _lib.call("sa_rmsnorm", _ptr(x), _code(x), xs, _ptr(weight), _code(weight), _ptr(out), _code(out), os_, T, D,
              float(eps), int(plus_one), _stream())
    return out


class PartialSums:
    """A matrix product whose cuts of K have not been added up yet (`gemm(..., defer_sum=True)`): `planes`
    [cuts, M, N] float32 in the kernels' workspace, valid until the next kernel that is handed the workspace, and
    `out`, the tensor that the sum belongs in.  `add_rmsnorm` takes it in place of y and adds the planes up itself,
    which saves the sum kernel and its round trip; anyone else calls `materialize()`.  The planes remember how
    often the workspace had been handed out when they were written: whoever reads them after another kernel has
    been given the workspace is refused (`check_fresh`), instead of adding up someone else's partial results."""

    def __init__(self, planes: torch.Tensor, out: torch.Tensor):
        self.planes, self.out = planes, out
        self.shape, self.dtype, self.device = out.shape, out.dtype, out.device
        self._written_at = workspace_uses(out.device)

    def check_fresh(self) -> None:
        if self.planes is not None and workspace_uses(self.device) != self._written_at:
            raise KernelError(
                "partial sums of a matrix product were read after another kernel had been given the workspace that "
                "holds them: add them up (add_rmsnorm, rope_cache_write or materialize()) before anything else "
                "that uses the workspace runs (a product with K cut over workgroups, attention over key ranges, "
                "the sampler)")

    def materialize(self) -> torch.Tensor:
        """The product itself: the sum kernel, now."""
        if self.planes is not None:
            self.check_fresh()
            count, M, N = self.planes.shape
            _lib.call("sa_sum_planes", _ptr(self.planes), count, _ptr(self.out), _code(self.out), self.out.stride(0), M, N,
                      _stream())
            self.planes = None
        return self.out


def add_rmsnorm(y: "torch.Tensor | PartialSums", residual: torch.Tensor, *, post_weight: torch.Tensor | None = None,
                post_eps: float = 0.0, post_plus_one: bool = True, next_weight: torch.Tensor | None = None,
                next_eps: float = 0.0, next_plus_one: bool = True, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor | None:
    """residual += norm(y; post_weight) (or += y); returns norm(residual; next_weight) if asked."""
    T, D = residual.shape
    planes = None
    if isinstance(y, PartialSums):
        fits = (y.planes is not None and D % 4 == 0 and D <= 5120 and y.dtype == torch.bfloat16
                and tuple(y.shape) == (T, D) and all(w is None or w.data_ptr() % 16 == 0 for w in (post_weight, next_weight)))
        if fits:
            y.check_fresh()
            planes, y = y.planes, y.out   # (y stands for shape and type below; it is not read)
        else:
            y = y.materialize()
    _dev(y, residual, post_weight, next_weight, out)
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm: the residual stream must be contiguous float32")
    if tuple(y.shape) != (T, D) or not y.is_contiguous():
        raise KernelError(f"add_rmsnorm: y {tuple(y.shape)} does not match the residual {T, D}")
    for w in (post_weight, next_weight):
        if w is not None and (w.numel() != D or not w.is_contiguous()):
            raise KernelError("add_rmsnorm: a norm weight does not match the width")
    if next_weight is not None:
        if out is None:
            out = torch.empty((T, D), dtype=out_dtype or y.dtype, device=y.device)
        if tuple(out.shape) != (T, D) or not out.is_contiguous():
            raise KernelError("add_rmsnorm: bad output")
    else:
        out = None
    if planes is not None:
        _lib.call("sa_add_rmsnorm_planes", _ptr(planes), planes.shape[0], _ptr(post_weight),
                  _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
                  _ptr(residual), _ptr(next_weight), _code(next_weight) if next_weight is not None else 0,
                  float(next_eps), int(next_plus_one), _ptr(out), _code(out) if out is not None else 0, T, D, _stream())
        return out
    _lib.call("sa_add_rmsnorm", _ptr(y), _code(y), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(residual), _ptr(next_weight), _code(next_weight) if next_weight is not None else 0,
              float(next_eps), int(next_plus_one), _ptr(out), _code(out) if out is not None else 0, T, D, _stream())
    return out


def add_rmsnorm_rows(y: torch.Tensor, residual: torch.Tensor, index: torch.Tensor, *, post_weight: torch.Tensor | None,
                     post_eps: float = 0.0, post_plus_one: bool = True, next_weight: torch.Tensor, next_eps: float,
                     next_plus_one: bool = True, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """out[r] = norm(residual[index[r]] + norm(y[index[r]]; post_weight); next_weight), the residual left as it is:
    `add_rmsnorm` followed by a gather of the rows that are wanted, in one kernel that touches those rows only."""
    _dev(y, residual, index, post_weight, next_weight)
    T, D = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm_rows: the residual stream must be contiguous float32")
    if tuple(y.shape) != (T, D) or not y.is_contiguous():
        raise KernelError(f"add_rmsnorm_rows: y {tuple(y.shape)} does not match the residual {T, D}")
    for w in (post_weight, next_weight):
        if w is not None and (w.numel() != D or not w.is_contiguous()):
            raise KernelError("add_rmsnorm_rows: a norm weight does not match the width")
    _i32(index, "add_rmsnorm_rows: index")
    R = index.numel()
    out = torch.empty((R, D), dtype=out_dtype or y.dtype, device=y.device)
    _lib.call("sa_add_rmsnorm_rows", _ptr(y), _code(y), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one), _ptr(residual),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(out), _code(out),
              _ptr(index), R, D, _stream())
    return out


def _check_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, dtype: torch.dtype, what: str) -> int:
    """Key pages [pages, K, page_size, hd], value pages [pages, K, hd, page_size]; returns page_size."""
    if k_pages.dim() != 4 or v_pages.dim() != 4 or not k_pages.is_contiguous() or not v_pages.is_contiguous() \
            or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise KernelError(f"{what}: pages must be contiguous 4-D tensors of {dtype}")
    n, K, P, hd = k_pages.shape
    if tuple(v_pages.shape) != (n, K, hd, P):
        raise KernelError(f"{what}: key pages {tuple(k_pages.shape)} want value pages {(n, K, hd, P)}, "
                          f"got {tuple(v_pages.shape)}")
    return P


def rope_cache_write(qkv: "torch.Tensor | PartialSums", positions: torch.Tensor, timescale: torch.Tensor | None,
                     scale_factor: float, q_div: float, num_heads: int, num_kv_heads: int, head_dim: int,
                     slot_mapping: torch.Tensor | None = None, k_pages: torch.Tensor | None = None,
                     v_pages: torch.Tensor | None = None) -> torch.Tensor:
    """In place on the fused projection rows; writes keys and values into their pages.  A projection whose cuts of K
    are not added up yet is added up on the way (up to 256 tokens; its queries go to the tensor that it belongs in).
    Returns the projection's tensor, of which the queries are then the rotated and scaled ones."""
    planes = None
    if isinstance(qkv, PartialSums):
        if qkv.planes is not None and qkv.shape[0] <= 256 and qkv.dtype == torch.bfloat16:
            qkv.check_fresh()
            planes, qkv = qkv.planes, qkv.out
        else:
            qkv = qkv.materialize()
    _dev(qkv, positions, timescale, slot_mapping, k_pages, v_pages)
    stride = _rows(qkv, "rope_cache_write: qkv")
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"rope_cache_write: row width {qkv.shape[1]} is not (H + 2K) * hd = "
                          f"{(num_heads + 2 * num_kv_heads) * head_dim}")
    _i32(positions, "rope_cache_write: positions", T)
    if timescale is not None and (timescale.dtype != torch.float32 or timescale.numel() != head_dim // 2
                                  or not timescale.is_contiguous()):
        raise KernelError("rope_cache_write: timescale must be float32 [head_dim / 2]")
    page_size = 1
    if k_pages is not None:
        if v_pages is None or slot_mapping is None:
            raise KernelError("rope_cache_write: key pages, value pages and slots come together")
        page_size = _check_pages(k_pages, v_pages, qkv.dtype, "rope_cache_write")
        if k_pages.shape[1] != num_kv_heads or k_pages.shape[3] != head_dim:
            raise KernelError(f"rope_cache_write: pages {tuple(k_pages.shape)} do not match {num_kv_heads} heads of "
                              f"size {head_dim}")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < T or not slot_mapping.is_contiguous():
            raise KernelError("rope_cache_write: slot_mapping must be int64 [T]")
    if planes is not None:
        _lib.call("sa_rope_cache_write_planes", _ptr(planes), planes.shape[0], _ptr(qkv), stride, _ptr(positions),
                  _ptr(timescale), float(scale_factor), float(q_div), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages),
                  T, num_heads, num_kv_heads, head_dim, page_size, _stream())
        return qkv
    _lib.call("sa_rope_cache_write", _ptr(qkv), _code(qkv), stride, _ptr(positions), _ptr(timescale),
              float(scale_factor), float(q_div), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), T, num_heads,
              num_kv_heads, head_dim, page_size, _stream())
    return qkv


def rope(x: torch.Tensor, positions: torch.Tensor, timescale: torch.Tensor, scale_factor: float, div: float,
         num_heads: int, head_dim: int) -> None:
    """In place: x[t, h, :] rotated by positions[t], then divided by div.  x: [T, >= num_heads * head_dim]."""
    _dev(x, positions, timescale)
    stride = _rows(x, "rope: x")
    T = x.shape[0]
    if x.shape[1] < num_heads * head_dim:
        raise KernelError("rope: rows are shorter than heads * head size")
    _i32(positions, "rope: positions", T)
    if timescale.dtype != torch.float32 or timescale.numel() != head_dim // 2 or not timescale.is_contiguous():
        raise KernelError("rope: timescale must be float32 [head_dim / 2]")
    _lib.call("sa_rope", _ptr(x), _code(x), stride, _ptr(positions), _ptr(timescale), float(scale_factor), float(div),
              T, num_heads, head_dim, _stream())


def gather_rows(x: torch.Tensor, index: torch.Tensor, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(x, index, out)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("gather_rows: x must be contiguous 2-D")
    _i32(index, "gather_rows: index")
    R, D = index.numel(), x.shape[1]
    if out is None:
        out = torch.empty((R, D), dtype=out_dtype or x.dtype, device=x.device)
    if tuple(out.shape) != (R, D) or not out.is_contiguous():
        raise KernelError("gather_rows: bad output")
    _lib.call("sa_gather_rows", _ptr(x), _code(x), _ptr(index), _ptr(out), _code(out), R, D, _stream())
    return out


def fill_(t: torch.Tensor, value_bits: int = 0) -> None:
    """Sets every 32-bit word of `t` to `value_bits` with a kernel (safe inside a captured graph)."""
    _dev(t)
    nbytes = t.numel() * t.element_size()
    if not t.is_contiguous() or nbytes % 4:
        raise KernelError("fill_: needs a contiguous tensor of a multiple of 4 bytes")
    _lib.call("sa_fill_u32", _ptr(t), value_bits & 0xFFFFFFFF, nbytes // 4, _stream())


def decode_advance(step_counter: torch.Tensor, sampled_tokens: torch.Tensor, sampled_logprobs: torch.Tensor,
                   tokens_in: torch.Tensor, positions: torch.Tensor, seq_meta: torch.Tensor,
                   draw_counters: torch.Tensor, out_tokens: torch.Tensor, out_logprobs: torch.Tensor, *,
                   token_seq: torch.Tensor | None = None, page_size: int = 0,
                   groups: "list[tuple[torch.Tensor, torch.Tensor]] | None" = None) -> None:
    """Between two decode steps that the host does not see: what was drawn is recorded as row step_counter[0] of
    out_tokens / out_logprobs [max_steps, B] and becomes the next step's input; positions, the requests' first
    positions (seq_meta[:, 3]), their draw counters and the step counter go up by one.  groups: (block table, slot
    mapping) of up to four cache groups, whose slot mappings are set for the new positions in the same launch (what
    `decode_slots` does for one group): needs token_seq and page_size."""
    _dev(step_counter, sampled_tokens, sampled_logprobs, tokens_in, positions, seq_meta, draw_counters, out_tokens,
         out_logprobs)
    B = tokens_in.numel()
    for t, name in ((step_counter, "step_counter"), (sampled_tokens, "sampled_tokens"), (tokens_in, "tokens_in"),
                    (positions, "positions"), (seq_meta, "seq_meta"), (draw_counters, "draw_counters"),
                    (out_tokens, "out_tokens")):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise KernelError(f"decode_advance: {name} must be contiguous int32")
    for t, name in ((sampled_logprobs, "sampled_logprobs"), (out_logprobs, "out_logprobs")):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError(f"decode_advance: {name} must be contiguous float32")
    if out_tokens.dim() != 2 or out_tokens.shape[1] != B or tuple(out_logprobs.shape) != tuple(out_tokens.shape):
        raise KernelError("decode_advance: the records are [max_steps, B]")
    if min(sampled_tokens.numel(), sampled_logprobs.numel(), positions.numel(), draw_counters.numel()) < B \
            or seq_meta.numel() < 4 * B or step_counter.numel() < 1:
        raise KernelError("decode_advance: an array is shorter than the number of requests")
    if groups:
        if token_seq is None or page_size < 1 or len(groups) > 4:
            raise KernelError("decode_advance: slot mappings need token_seq, a page size and at most four groups")
        _i32(token_seq, "decode_advance: token_seq", B)
        n = len(groups)
        for table, slots in groups:
            _dev(table, slots)
            if table.dim() != 2 or table.dtype != torch.int32 or table.stride(1) != 1:
                raise KernelError("decode_advance: a block table must be int32 [sequences, blocks]")
            if slots.dtype != torch.int64 or slots.numel() < B or not slots.is_contiguous():
                raise KernelError("decode_advance: a slot mapping must be contiguous int64 with one entry per token")
        tables = (ctypes.c_void_p * n)(*[t.data_ptr() for t, _ in groups])
        strides = (ctypes.c_int * n)(*[t.stride(0) for t, _ in groups])
        mappings = (ctypes.c_void_p * n)(*[m.data_ptr() for _, m in groups])
        _lib.call("sa_decode_advance_slots", B, _ptr(step_counter), _ptr(sampled_tokens), _ptr(sampled_logprobs),
                  _ptr(tokens_in), _ptr(positions), _ptr(seq_meta), _ptr(draw_counters), _ptr(out_tokens),
                  _ptr(out_logprobs), out_tokens.shape[0], _ptr(token_seq), n, tables, strides, mappings, int(page_size),
                  _stream())
        return
    _lib.call("sa_decode_advance", B, _ptr(step_counter), _ptr(sampled_tokens), _ptr(sampled_logprobs), _ptr(tokens_in),
              _ptr(positions), _ptr(seq_meta), _ptr(draw_counters), _ptr(out_tokens), _ptr(out_logprobs),
              out_tokens.shape[0], _stream())


def decode_slots(positions: torch.Tensor, token_seq: torch.Tensor, block_table: torch.Tensor, page_size: int,
                 slot_mapping: torch.Tensor) -> None:
    """slot_mapping[b] = block_table[token_seq[b], positions[b] // page_size] * page_size + positions[b] % page_size."""
    _dev(positions, token_seq, block_table, slot_mapping)
    B = positions.numel()
    _i32(positions, "decode_slots: positions", B)
    _i32(token_seq, "decode_slots: token_seq", B)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("decode_slots: block_table must be int32 [sequences, blocks]")
    if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < B or not slot_mapping.is_contiguous():
        raise KernelError("decode_slots: slot_mapping must be contiguous int64 with one entry per token")
    _lib.call("sa_decode_slots", B, _ptr(positions), _ptr(token_seq), _ptr(block_table), block_table.stride(0),
              int(page_size), _ptr(slot_mapping), _stream())


# --------------------------------------------------------------------------- matrix products

EPILOGUE_NONE, EPILOGUE_GATED, EPILOGUE_SOFT_CAP = 0, 1, 2
#: activations of the gated epilogue (simply_amd/csrc/activations.h); the epilogue argument is 1 + 16 * activation
ACT_GELU_TANH, ACT_SILU, ACT_SQUARED_RELU = 0, 1, 2


def _gated(activation: int) -> int:
    if activation not in (ACT_GELU_TANH, ACT_SILU, ACT_SQUARED_RELU):
        raise KernelError(f"unknown activation code {activation!r}")
    return EPILOGUE_GATED + 16 * activation


#: scratch memory for partial results (attention over key ranges, products with K cut over workgroups), one per
#: device, allocated at first use; kernels on one stream use it one after the other
WORKSPACE_BYTES = 256 << 20
_scratch: dict = {}
_scratch_uses: dict = {}


def _workspace(device) -> torch.Tensor:
    """The device's workspace, for a kernel that is about to be launched with it: what an earlier kernel left there
    is lost from now on (`workspace_uses` counts these hand-outs)."""
    key = (device.type, device.index)
    if key not in _scratch:
        _scratch[key] = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    _scratch_uses[key] = _scratch_uses.get(key, 0) + 1
    return _scratch[key]


def workspace_uses(device) -> int:
    """How often the device's workspace has been handed to a kernel."""
    device = torch.device(device)
    return _scratch_uses.get((device.type, device.index), 0)


def gemm(a: torch.Tensor, w: "torch.Tensor | TiledWeight", *, w2: "torch.Tensor | TiledWeight | None" = None,
         soft_cap: float | None = None, out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
         algo: int = ALGO_AUTO, shape: int = 0, activation: int = ACT_GELU_TANH,
         defer_sum: bool = False) -> "torch.Tensor | PartialSums":
    """a[M, K] . w[N, K]^T.  With w2 (row-major weights) or a paired `TiledWeight`: act(a.wg^T) * (a.wu^T) with
    the activation of that code.  With soft_cap: cap * tanh(. / cap).  w is a row-major tensor or a `TiledWeight`.
    defer_sum: where the product is computed in cuts of K, leave their sum to the caller: the result is then a
    `PartialSums` (else the tensor as always)."""
    packed = isinstance(w, TiledWeight)
    wd = w.data if packed else w
    w2d = None
    paired = packed and w.paired
    if paired and (w2 is not None or soft_cap):
        raise KernelError("gemm: a paired tiled weight is the gated product by itself")
    if w2 is not None:
        if packed or isinstance(w2, TiledWeight):
            raise KernelError("gemm: tiled weights of a gated product come as one paired weight (pack_gate_up)")
        w2d = w2
    _dev(a, wd, w2d, out)
    lda = _rows(a, "gemm: a")
    M, K = a.shape
    if not wd.is_contiguous() or (not packed and w.dim() != 2) or w.shape[1] != K:
        raise KernelError(f"gemm: weight {tuple(w.shape)} does not match a {tuple(a.shape)} (expects [N, K] contiguous)")
    N = w.shape[0]
    if wd.dtype != a.dtype:
        raise KernelError(f"gemm: a is {a.dtype} but the weight is {wd.dtype}")
    epi, cap = EPILOGUE_NONE, 0.0
    if paired:
        epi = _gated(activation)
    elif w2 is not None:
        if soft_cap:
            raise KernelError("gemm: the gated and the soft-cap epilogue do not combine")
        if tuple(w2.shape) != tuple(w.shape) or w2d.dtype != wd.dtype or not w2d.is_contiguous():
            raise KernelError("gemm: the second weight must match the first")
        epi = _gated(activation)
    elif soft_cap:
        epi, cap = EPILOGUE_SOFT_CAP, float(soft_cap)
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    if tuple(out.shape) != (M, N):
        raise KernelError("gemm: bad output shape")
    ldc = _rows(out, "gemm: out")
    ws = _workspace(a.device)
    if defer_sum and epi == EPILOGUE_NONE and out.dtype == torch.bfloat16 and out.is_contiguous():
        count = ctypes.c_int(1)
        _lib.call("sa_gemm_planes", _ptr(a), _code(a), lda, _ptr(wd), _ptr(w2d), _code(wd), _ptr(out), _code(out), ldc, M, N,
                  K, epi, cap, algo, int(packed), int(shape), _ptr(ws), ws.numel(), ctypes.byref(count), _stream())
        if count.value > 1:
            words = count.value * M * N
            return PartialSums(ws.view(torch.float32)[:words].view(count.value, M, N), out)
        return out
    _lib.call("sa_gemm", _ptr(a), _code(a), lda, _ptr(wd), _ptr(w2d), _code(wd), _ptr(out), _code(out), ldc, M, N, K, epi,
              cap, algo, int(packed), int(shape), _ptr(ws), ws.numel(), _stream())
    return out


def gemm_plan(M: int, N: int, K: int, *, gated: bool = False, soft_cap: bool = False,
              out_dtype: torch.dtype = torch.bfloat16) -> tuple[int, dict[str, float]]:
    """Which kernel `gemm` would run for bfloat16 rows against a tiled [N, K] weight (ALGO_SKINNY, ALGO_TILED or
    ALGO_WIDE), and the microseconds that the library expects of each (negative: not eligible).  A host function:
    it needs no GPU."""
    us = (ctypes.c_double * 3)()
    epi = EPILOGUE_GATED if gated else (EPILOGUE_SOFT_CAP if soft_cap else EPILOGUE_NONE)
    kernel = _lib.load().sa_gemm_plan(int(M), int(N), int(K), epi, _CODES[out_dtype], WORKSPACE_BYTES, us)
    return kernel, {"skinny": us[0], "tiled": us[1], "wide": us[2]}


def gemm_normed_takes(M: int, w) -> bool:
    """Whether `gemm_normed` takes M rows against the weight `w`."""
    if not isinstance(w, TiledWeight) or not w.data.is_cuda:
        return False
    return bool(_lib.load().sa_gemm_normed_takes(int(M), int(w.rows), int(w.cols)))


def gemm_normed_pays(M: int, w) -> bool:
    """Whether `gemm_normed` takes M rows against the weight `w` and is expected to beat the separate norm and
    product kernels there (the library's own answer: it knows for which widths it has which prologue)."""
    if not isinstance(w, TiledWeight) or not w.data.is_cuda:
        return False
    return bool(_lib.load().sa_gemm_normed_pays(int(M), int(w.rows), int(w.cols)))


_few_rows: int | None = None


def few_rows_limit() -> int:
    """The most rows of a step for which the kernels that fuse the norms into the following product exist."""
    global _few_rows
    if _few_rows is None:
        _few_rows = int(_lib.load().sa_gemm_normed_max_rows())
    return _few_rows


def gemm_normed(y: torch.Tensor | None, h_in: torch.Tensor, h_out: torch.Tensor | None, w: TiledWeight, *,
                post_weight: torch.Tensor | None, post_eps: float, post_plus_one: bool, next_weight: torch.Tensor,
                next_eps: float, next_plus_one: bool, soft_cap: float | None = None,
                out_dtype: torch.dtype = torch.bfloat16, out: torch.Tensor | None = None,
                activation: int = ACT_GELU_TANH) -> torch.Tensor:
    """h_out = h_in + norm(y; post) (y None: the residual stays h_in); returns epilogue(norm(h_out; next) . w^T),
    in one kernel, for up to 16 rows.  The residual buffers are float32 [M, K] and must differ."""
    _dev(y, h_in, h_out, post_weight, next_weight, w.data)
    M, K = h_in.shape
    if h_in.dtype != torch.float32 or not h_in.is_contiguous() or w.cols != K:
        raise KernelError("gemm_normed: the residual must be contiguous float32 [M, K] with K the weight's width")
    if y is not None:
        if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, K) or not y.is_contiguous():
            raise KernelError("gemm_normed: y must be contiguous bfloat16 [M, K]")
        if h_out is None or h_out.dtype != torch.float32 or tuple(h_out.shape) != (M, K) or not h_out.is_contiguous() \
                or h_out.data_ptr() == h_in.data_ptr():
            raise KernelError("gemm_normed: the updated residual needs its own contiguous float32 [M, K] buffer")
    for t in (post_weight, next_weight):
        if t is not None and (t.numel() != K or not t.is_contiguous()):
            raise KernelError("gemm_normed: a norm weight does not match the width")
    epi, cap = EPILOGUE_NONE, 0.0
    if w.paired:
        epi = _gated(activation)
    elif soft_cap:
        epi, cap = EPILOGUE_SOFT_CAP, float(soft_cap)
    if out is None:
        out = torch.empty((M, w.rows), dtype=out_dtype, device=h_in.device)
    if tuple(out.shape) != (M, w.rows) or out.stride(1) != 1 or out.device != h_in.device:
        raise KernelError(f"gemm_normed: the output must be [{M}, {w.rows}] with contiguous rows on the inputs' device")
    _lib.call("sa_gemm_normed", _ptr(y), _ptr(h_in), _ptr(h_out), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(w.data), _ptr(out),
              _code(out), out.stride(0), M, w.rows, K, epi, cap, _stream())
    return out


def gemm_normed_rotary(y: torch.Tensor | None, h_in: torch.Tensor, h_out: torch.Tensor | None, w: TiledWeight, *,
                       post_weight: torch.Tensor | None, post_eps: float, post_plus_one: bool,
                       next_weight: torch.Tensor, next_eps: float, next_plus_one: bool, positions: torch.Tensor,
                       timescale: torch.Tensor | None, scale_factor: float, query_scale: float, num_heads: int,
                       num_kv_heads: int, head_dim: int, slot_mapping: torch.Tensor | None = None,
                       k_pages: torch.Tensor | None = None, v_pages: torch.Tensor | None = None) -> torch.Tensor:
    """`gemm_normed` for the fused q/k/v projection (w has (H + 2 K) * hd rows) followed by `rope_cache_write` in
    the same kernel.  Returns [M, (H + 2 K) * hd] of which only the query columns are written."""
    _dev(y, h_in, h_out, post_weight, next_weight, w.data, positions, timescale, slot_mapping, k_pages, v_pages)
    M, K = h_in.shape
    H, Kh, hd = num_heads, num_kv_heads, head_dim
    if w.paired or w.rows != (H + 2 * Kh) * hd or w.cols != K:
        raise KernelError("gemm_normed_rotary: the weight must have (H + 2 K) * hd rows of the residual's width")
    if h_in.dtype != torch.float32 or not h_in.is_contiguous():
        raise KernelError("gemm_normed_rotary: the residual must be contiguous float32 [M, K]")
    if y is not None:
        if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, K) or not y.is_contiguous():
            raise KernelError("gemm_normed_rotary: y must be contiguous bfloat16 [M, K]")
        if h_out is None or h_out.dtype != torch.float32 or tuple(h_out.shape) != (M, K) or not h_out.is_contiguous() \
                or h_out.data_ptr() == h_in.data_ptr():
            raise KernelError("gemm_normed_rotary: the updated residual needs its own contiguous float32 [M, K] buffer")
    for t in (post_weight, next_weight):
        if t is not None and (t.numel() != K or not t.is_contiguous()):
            raise KernelError("gemm_normed_rotary: a norm weight does not match the width")
    _i32(positions, "gemm_normed_rotary: positions", M)
    if timescale is not None and (timescale.dtype != torch.float32 or timescale.numel() != hd // 2):
        raise KernelError("gemm_normed_rotary: timescale must be float32 [hd / 2]")
    page_size = 1
    if slot_mapping is not None:
        if k_pages is None or v_pages is None:
            raise KernelError("gemm_normed_rotary: slots come with key and value pages")
        _check_pages(k_pages, v_pages, torch.bfloat16, "gemm_normed_rotary")
        if k_pages.shape[1] != Kh or k_pages.shape[3] != hd:
            raise KernelError("gemm_normed_rotary: the pages do not match the heads")
        page_size = k_pages.shape[2]
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < M or not slot_mapping.is_contiguous():
            raise KernelError("gemm_normed_rotary: slot_mapping must be contiguous int64 with one entry per row")
    out = torch.empty((M, w.rows), dtype=torch.bfloat16, device=h_in.device)
    _lib.call("sa_gemm_normed_rotary", _ptr(y), _ptr(h_in), _ptr(h_out), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(w.data), _ptr(out),
              _code(out), out.stride(0), M, K, _ptr(positions), _ptr(timescale), float(scale_factor),
              float(query_scale), _ptr(slot_mapping), _ptr(k_pages) if slot_mapping is not None else None,
              _ptr(v_pages) if slot_mapping is not None else None, H, Kh, hd, int(page_size), _stream())
    return out


# --------------------------------------------------------------------------- attention


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                    token_seq: torch.Tensor, positions: torch.Tensor, num_heads: int, *, window: int | None,
                    soft_cap: float | None, out: torch.Tensor | None = None, algo: int = ALGO_AUTO) -> torch.Tensor:
    """q: [T, >= H * hd] rows (a view into the fused projection is fine).  Returns [T, H * hd]."""
    _dev(q, k_pages, v_pages, block_table, token_seq, positions, out)
    q_stride = _rows(q, "paged_attention: q")
    T = q.shape[0]
    _check_pages(k_pages, v_pages, q.dtype, "paged_attention")
    num_pages, Kh, page_size, hd = k_pages.shape
    if q.shape[1] < num_heads * hd:
        raise KernelError("paged_attention: query rows are shorter than heads * head size")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("paged_attention: block_table must be int32 [sequences, blocks]")
    _i32(token_seq, "paged_attention: token_seq", T)
    _i32(positions, "paged_attention: positions", T)
    if out is None:
        out = torch.empty((T, num_heads * hd), dtype=q.dtype, device=q.device)
    if tuple(out.shape) != (T, num_heads * hd) or out.dtype != q.dtype:
        raise KernelError("paged_attention: bad output")
    out_stride = _rows(out, "paged_attention: out")
    _lib.call("sa_paged_attention", _ptr(q), _code(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(token_seq), _ptr(positions), _ptr(out), out_stride, T, num_heads, Kh, hd,
              page_size, int(window or 0), float(soft_cap or 0.0), algo, _stream())
    return out


def decode_attention_takes(q: torch.Tensor, k_pages: torch.Tensor, num_heads: int, max_q_len: int) -> bool:
    """Whether `paged_attention_decode` takes requests of up to max_q_len tokens at these sizes."""
    _, Kh, page_size, hd = k_pages.shape
    return q.dtype == torch.bfloat16 and q.is_cuda and bool(_lib.load().sa_paged_attention_decode_takes(
        int(num_heads), int(Kh), int(hd), int(page_size), int(max_q_len), q.stride(0), _ptr(q)))


def _attention_units(entry: str, q, k_pages, v_pages, block_table, seq_meta, begin, count, num_heads, window, soft_cap,
                     max_kv_len, max_q_len, out, num_splits):
    _dev(q, k_pages, v_pages, block_table, seq_meta, out)
    name = entry[3:]
    if q.dtype != torch.bfloat16:
        raise KernelError(f"{name}: bfloat16 only")
    q_stride = _rows(q, f"{name}: q")
    _check_pages(k_pages, v_pages, q.dtype, name)
    _, Kh, page_size, hd = k_pages.shape
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError(f"{name}: block_table must be int32 [sequences, blocks]")
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or begin < 0 or begin + count > seq_meta.shape[0]:
        raise KernelError(f"{name}: seq_meta must be int32 [S, 4] covering the requested range")
    if out.dtype != q.dtype or out.shape[0] != q.shape[0] or out.shape[1] != num_heads * hd:
        raise KernelError(f"{name}: bad output")
    out_stride = _rows(out, f"{name}: out")
    ws = _workspace(q.device)
    _lib.call(entry, _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(seq_meta), begin, count, _ptr(out), out_stride, num_heads, Kh, hd,
              page_size, int(window or 0), float(soft_cap or 0.0), int(max_kv_len), int(max_q_len), int(num_splits),
              _ptr(ws), ws.numel(), _stream())
    return out


def paged_attention_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                           seq_meta: torch.Tensor, seq_begin: int, seq_count: int, num_heads: int, *,
                           window: int | None, soft_cap: float | None, max_kv_len: int, max_q_len: int,
                           out: torch.Tensor, num_splits: int = 0) -> torch.Tensor:
    """Attention of requests seq_begin .. seq_begin + seq_count - 1 of seq_meta, each with few tokens
    ((heads per key head) * tokens <= 16).  q and out are the whole step's rows."""
    return _attention_units("sa_paged_attention_decode", q, k_pages, v_pages, block_table, seq_meta, seq_begin,
                            seq_count, num_heads, window, soft_cap, max_kv_len, max_q_len, out, num_splits)


def prefill_units_per_group() -> int:
    """How many units one workgroup of the portion kernel takes (they must belong to one request)."""
    return int(_lib.load().sa_paged_attention_prefill_group())


def paged_attention_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                            units: torch.Tensor, unit_begin: int, unit_count: int, num_heads: int, *,
                            window: int | None, soft_cap: float | None, max_kv_len: int, max_q_len: int,
                            out: torch.Tensor, num_splits: int = 0) -> torch.Tensor:
    """Attention of portions of prompts cut into units of few tokens ((heads per key head) * tokens <= 16), rows
    unit_begin .. unit_begin + unit_count - 1 of `units` in the layout of seq_meta.  One workgroup takes a group of
    consecutive units, which must belong to one request (units without tokens fill up the last group), and
    reads the keys once for all of them."""
    if unit_count % prefill_units_per_group():
        raise KernelError(f"paged_attention_prefill: units come in groups of {prefill_units_per_group()}")
    return _attention_units("sa_paged_attention_prefill", q, k_pages, v_pages, block_table, units, unit_begin,
                            unit_count, num_heads, window, soft_cap, max_kv_len, max_q_len, out, num_splits)


# --------------------------------------------------------------------------- measurements of the machine


def probe_hbm_read(buffer: torch.Tensor, order: torch.Tensor | None = None) -> None:
    """All CUs read `buffer` (whole 8 KiB pieces) once from memory, piece after piece or in the order given (int32
    piece numbers): the caller times it.  What the decode step's kernels, which are bound by reading weights and
    cache, can reach at most."""
    _dev(buffer, order)
    nbytes = buffer.numel() * buffer.element_size()
    if not buffer.is_contiguous() or nbytes % 8192:
        raise KernelError("probe_hbm_read: a contiguous buffer of whole 8 KiB pieces")
    if order is not None:
        _i32(order, "probe_hbm_read: order", nbytes // 8192)
    sink = _workspace(buffer.device)
    _lib.call("sa_probe_hbm_read", _ptr(buffer), nbytes, _ptr(order), _ptr(sink), _stream())


def probe_mfma(operands: torch.Tensor, iters: int, workgroups: int = 256) -> float:
    """`workgroups` workgroups of eight waves each retire 16 * iters bfloat16 MFMA instructions per wave on the
    16 KiB of `operands`; returns the floating-point operations that this is (the caller times it).  The rate
    depends on the operands' bits: the clock that the GPU holds under this load does."""
    _dev(operands)
    if operands.numel() * operands.element_size() < 16384 or not operands.is_contiguous():
        raise KernelError("probe_mfma: 16 KiB of operands")
    sink = _workspace(operands.device)
    _lib.call("sa_probe_mfma", _ptr(operands), int(iters), int(workgroups), _ptr(sink), _stream())
    return 2.0 * 16 * 16 * 32 * 16 * iters * 8 * workgroups


# --------------------------------------------------------------------------- sampling


SAMPLE_DRAWN, SAMPLE_TOP_K, SAMPLE_TOP_P = 1, 2, 4


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           seed: torch.Tensor, counter: torch.Tensor, tokens: torch.Tensor | None = None,
           logprobs: torch.Tensor | None = None, modes: int = 7) -> tuple[torch.Tensor, torch.Tensor]:
    """One token per row.  All per-row parameter tensors are on the device, [R].  modes: what some row may ask
    for (SAMPLE_DRAWN + SAMPLE_TOP_K + SAMPLE_TOP_P); the kernels for what no row asks for are left out."""
    _dev(logits, temperature, top_k, top_p, seed, counter, tokens, logprobs)
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    stride = _rows(logits, "sample: logits")
    R, V = logits.shape
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p"), (seed, torch.int64, "seed"), (counter, torch.int32, "counter")):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be a contiguous {dt} tensor with one entry per row")
    if tokens is None:
        tokens = torch.empty(R, dtype=torch.int32, device=logits.device)
    if logprobs is None:
        logprobs = torch.empty(R, dtype=torch.float32, device=logits.device)
    _i32(tokens, "sample: tokens", R)
    ws = _workspace(logits.device)
    _lib.call("sa_sample", _ptr(logits), stride, R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seed),
              _ptr(counter), _ptr(tokens), _ptr(logprobs), int(modes), _ptr(ws), ws.numel(), _stream())
    return tokens, logprobs


#: what `score` gives for a token that is left out (the reference's neg_inf for float32)
SCORE_MASKED = -0.5 * 3.4028234663852886e38


def score(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
          tokens: torch.Tensor, scores: torch.Tensor | None = None) -> torch.Tensor:
    """The log-probability of tokens[r] under row r's temperature, top-k and top-p, as `sample` reports it for the
    token it draws: greedy rows give 0 for the argmax and SCORE_MASKED otherwise, a token that the masks leave out
    gives SCORE_MASKED."""
    _dev(logits, temperature, top_k, top_p, tokens, scores)
    if logits.dtype != torch.float32:
        raise KernelError("score: logits must be float32")
    stride = _rows(logits, "score: logits")
    R, V = logits.shape
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p")):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"score: {name} must be a contiguous {dt} tensor with one entry per row")
    _i32(tokens, "score: tokens", R)
    if scores is None:
        scores = torch.empty(R, dtype=torch.float32, device=logits.device)
    if scores.dtype != torch.float32 or scores.numel() < R or not scores.is_contiguous():
        raise KernelError("score: scores must be a contiguous float32 tensor with one entry per row")
    _lib.call("sa_score", _ptr(logits), stride, R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(tokens),
              _ptr(scores), _stream())
    return scores


def philox4x32_10(counter: tuple[int, int, int, int], key: tuple[int, int]) -> tuple[int, int, int, int]:
    """Host function: one block of the generator that `sample` uses."""
    c = (ctypes.c_uint32 * 4)(*counter)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    _lib.load().sa_philox4x32_10(c, k, o)
    return tuple(int(v) for v in o)
