"""The tiled layout of bfloat16 weight matrices.

A matrix W[N, K] is cut into blocks of 16 rows by 32 columns; each block is stored as the 1 KiB that
one v_mfma_f32_16x16x32_bf16 operand occupies in registers: [lane 64][8], lane = (k % 32) // 8 * 16 +
n % 16, element k % 8.  Blocks follow each other along K, then along N; rows and columns beyond N and K
are zero.  A wavefront that streams a block therefore reads one contiguous KiB, where row-major rows
would give it sixteen 64-byte pieces (about half the bandwidth on MI355X).
"""
from __future__ import annotations

import dataclasses

import torch


@dataclasses.dataclass
class TiledWeight:
    data: torch.Tensor   # [ceil(N / 16), ceil(K / 32), 64, 8] bfloat16, contiguous ([2 * ceil(N / 16), ...] if paired)
    rows: int            # N
    cols: int            # K
    paired: bool = False  # two matrices [N, K], their 16-row tiles in turn (gate, factor, gate, factor, ...)

    @property
    def shape(self) -> tuple[int, int]:
        return (self.rows, self.cols)

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype

    @property
    def device(self):
        return self.data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()


_cache: dict[tuple, tuple[torch.Tensor, TiledWeight]] = {}   # the source is kept alive so that its address stays its own


def pack_tiles(w: torch.Tensor, cached: bool = False) -> TiledWeight:
    """Row-major [N, K] bfloat16 -> tiled.  With `cached`, the same storage is packed once (a tied
    embedding table that is also the head); `clear_cache()` ends the sharing."""
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise ValueError(f"pack_tiles: expected a 2-D bfloat16 tensor, got {tuple(w.shape)} {w.dtype}")
    key = (w.data_ptr(), tuple(w.shape), str(w.device))
    if cached and key in _cache:
        return _cache[key][1]
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        padded = torch.zeros((Np, Kp), dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
    else:
        padded = w
    # [N/16, 16 rows, K/32, 4 kq, 8] -> [N/16, K/32, 4 kq, 16 rows, 8]
    data = padded.view(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(Np // 16, Kp // 32, 64, 8)
    tw = TiledWeight(data, N, K)
    if cached:
        _cache[key] = (w, tw)
    return tw


def pack_gate_up(gate: torch.Tensor, up: torch.Tensor) -> TiledWeight:
    """Both factors of a gated product as one tiled weight whose 16-row tiles alternate (gate tile i, then the
    other factor's tile i): a wave that computes 16 output columns streams 2 KiB contiguous blocks, and gate and
    factor of a column meet in one lane's registers."""
    if gate.shape != up.shape:
        raise ValueError("pack_gate_up: the two matrices differ in shape")
    g, u = pack_tiles(gate).data, pack_tiles(up).data
    data = torch.stack([g, u], dim=1).reshape(2 * g.shape[0], *g.shape[1:]).contiguous()
    return TiledWeight(data, gate.shape[0], gate.shape[1], paired=True)


def unpack_gate_up(tw: TiledWeight) -> tuple[torch.Tensor, torch.Tensor]:
    d = tw.data.view(tw.data.shape[0] // 2, 2, *tw.data.shape[1:])
    return (unpack_tiles(TiledWeight(d[:, 0].contiguous(), tw.rows, tw.cols)),
            unpack_tiles(TiledWeight(d[:, 1].contiguous(), tw.rows, tw.cols)))


def unpack_tiles(tw: TiledWeight) -> torch.Tensor:
    if tw.paired:
        raise ValueError("unpack_tiles: a paired weight holds two matrices (unpack_gate_up)")
    nt, nc = tw.data.shape[:2]
    full = tw.data.view(nt, nc, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nt * 16, nc * 32)
    return full[:tw.rows, :tw.cols].contiguous()


def clear_cache() -> None:
    _cache.clear()


def concat_rows(*ws: torch.Tensor) -> torch.Tensor:
    return torch.cat(ws, dim=0).contiguous()


# ---- pages of keys

def keys_tiled(page_size: int, head_dim: int) -> bool:
    """Whether the kernels keep a page of keys in 16-key x 32-dimension blocks of MFMA operand order
    ([page_size / 16][head_dim / 32][64][8]) rather than row-major [page_size][head_dim]."""
    return page_size % 16 == 0 and head_dim % 32 == 0


def keys_to_rows(k_pages: torch.Tensor) -> torch.Tensor:
    """[pages, heads, page_size, head_dim] as the kernels store it -> row-major copy (tests, inspection)."""
    n, h, P, hd = k_pages.shape
    if not keys_tiled(P, hd):
        return k_pages.clone()
    return k_pages.reshape(n, h, P // 16, hd // 32, 4, 16, 8).permute(0, 1, 2, 5, 3, 4, 6).reshape(n, h, P, hd).contiguous()


def rows_to_keys(rows: torch.Tensor) -> torch.Tensor:
    """Row-major [pages, heads, page_size, head_dim] -> the kernels' storage order (same shape)."""
    n, h, P, hd = rows.shape
    if not keys_tiled(P, hd):
        return rows.clone()
    return rows.reshape(n, h, P // 16, 16, hd // 32, 4, 8).permute(0, 1, 2, 4, 5, 3, 6).reshape(n, h, P, hd).contiguous()
