"""Numpy restatement of the reference's BCSR/BCSC index semantics.

Canonical order: within a block-row the live block columns ascend (BCSR);
within a block-column the live block rows ascend (BCSC).  The reference
assigns slots with atomics, so any within-row order is a legal output of it;
the ascending one is the deterministic representative used for bit-exact
comparison.

Follows sparta/tesa/block_compressed.py:23-196,242-309 and
sparta/tesa/templates/block_compressed.cu.j2:138-220 (index bit fields and the
compressed value layout).
"""
import numpy as np


def reduce_block_mask(mask: np.ndarray, BH: int, BW: int) -> np.ndarray:
    """Block liveness = any non-zero byte in the tile.

    test/unit/test_tesa.py:11-17 (reduce_mask_ref) and
    block_compressed.cu.j2:86-100.
    """
    H, W = mask.shape
    assert H % BH == 0 and W % BW == 0
    tiles = mask.reshape(H // BH, BH, W // BW, BW)
    return (tiles != 0).any(axis=(1, 3))


def build_bcsr(mask: np.ndarray, BH: int, BW: int):
    """row_ptr int32[R+1], BCSR_idx int32[nnz] = (row << 16) | col.

    block_compressed.py:267-287, block_compressed.cu.j2:151.
    """
    live = reduce_block_mask(mask, BH, BW)
    rows, cols = np.nonzero(live)  # row-major order == canonical BCSR order
    row_ptr = np.zeros(live.shape[0] + 1, dtype=np.int32)
    np.cumsum(live.sum(axis=1), out=row_ptr[1:])
    idx = ((rows.astype(np.int64) << 16) | cols.astype(np.int64)).astype(np.int32)
    return row_ptr, idx, int(rows.size)


def build_bcsc(mask: np.ndarray, BH: int, BW: int):
    """col_ptr int32[Cn+1], BCSC_idx int32[nnz] = (col << 16) | row.

    block_compressed.py:289-309, block_compressed.cu.j2:166.
    """
    live = reduce_block_mask(mask, BH, BW)
    cols, rows = np.nonzero(live.T)  # column-major order == canonical BCSC order
    col_ptr = np.zeros(live.shape[1] + 1, dtype=np.int32)
    np.cumsum(live.sum(axis=0), out=col_ptr[1:])
    idx = ((cols.astype(np.int64) << 16) | rows.astype(np.int64)).astype(np.int32)
    return col_ptr, idx, int(rows.size)


def build_bcsrc(mask: np.ndarray, BH: int, BW: int):
    """Both indexes; BCSC_idx is int64 = (bcsr_pos << 32) | (col << 16) | row.

    block_compressed.py:242-265, block_compressed.cu.j2:163-164.
    """
    live = reduce_block_mask(mask, BH, BW)
    row_ptr, bcsr_idx, nnz = build_bcsr(mask, BH, BW)
    col_ptr, _, _ = build_bcsc(mask, BH, BW)
    pos = np.full(live.shape, -1, dtype=np.int64)
    rows, cols = np.nonzero(live)
    pos[rows, cols] = np.arange(nnz)
    ccols, crows = np.nonzero(live.T)
    bcsc_idx = (pos[crows, ccols] << 32) | (ccols.astype(np.int64) << 16) | crows.astype(np.int64)
    return row_ptr, bcsr_idx, col_ptr, bcsc_idx.astype(np.int64), nnz


def block_coords(idx: np.ndarray, fmt: str):
    """Decode (block_row, block_col) of every entry. fmt in {'bcsr','bcsc'}."""
    lo = (idx.astype(np.int64) & 0xffff)
    hi = ((idx.astype(np.int64) >> 16) & 0xffff)
    return (hi, lo) if fmt == 'bcsr' else (lo, hi)


def convert(dense: np.ndarray, idx: np.ndarray, fmt: str, BH: int, BW: int) -> np.ndarray:
    """dense [..., H, W] -> compressed [..., nnz*BH*BW]; block i at i*BH*BW,
    row-major inside the block, *not* multiplied by the element mask.

    block_compressed.cu.j2:172-195 (sparse[b, i*BH*BW + r*BW + c] =
    dense[b, by*BH + r, bx*BW + c]).
    """
    br, bc = block_coords(idx, fmt)
    lead = dense.shape[:-2]
    H, W = dense.shape[-2:]
    tiles = dense.reshape(lead + (H // BH, BH, W // BW, BW))
    tiles = np.moveaxis(tiles, -3, -2)  # [..., R, Cn, BH, BW]
    out = tiles[..., br, bc, :, :]      # [..., nnz, BH, BW]
    return np.ascontiguousarray(out).reshape(lead + (-1,))


def inverse(sparse: np.ndarray, idx: np.ndarray, fmt: str, BH: int, BW: int, H: int, W: int) -> np.ndarray:
    """compressed -> zero-filled dense. block_compressed.cu.j2:197-220."""
    br, bc = block_coords(idx, fmt)
    lead = sparse.shape[:-1]
    nnz = idx.shape[0]
    tiles = np.zeros(lead + (H // BH, W // BW, BH, BW), dtype=sparse.dtype)
    tiles[..., br, bc, :, :] = sparse.reshape(lead + (nnz, BH, BW))
    return np.ascontiguousarray(np.moveaxis(tiles, -2, -3)).reshape(lead + (H, W))


def expand_block_mask(live: np.ndarray, BH: int, BW: int) -> np.ndarray:
    """Block mask -> element mask (block_compressed.py:47-50)."""
    return np.kron(live.astype(np.uint8), np.ones((BH, BW), dtype=np.uint8))
