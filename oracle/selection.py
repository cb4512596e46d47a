"""Oracle for retained-mass tile selection and key-mask tile metadata.

Restates csrc/kernels/sparse_selection.cu and csrc/kernels/key_mask_tiles.cu
(test infrastructure only).
"""

from __future__ import annotations

import numpy as np


def select_retained_mass(masses: np.ndarray, theta: float, order: np.ndarray | None = None):
    """Shortest descending prefix whose FP64 mass reaches theta * total, as CSR.

    ``masses`` is float32 [rows, tiles].  ``order`` optionally fixes the
    descending permutation (the reference takes it from an unstable
    ``torch.sort``, src/risa_attention/sparse.py:24); by default a stable
    descending sort is used.  Returns ``(row_offsets int32 [rows+1],
    block_indices int32 [nnz], measured_mass float, counts int32 [rows])``.

    Follows select_mass_rows_kernel (sparse_selection.cu:9-67): lane-strided
    FP64 total reduced by a shuffle-down tree, Hillis-Steele inclusive scans
    over chunks of 32 ranks, first rank with ``cumulative + prefix >= target``.
    """
    masses = np.asarray(masses, dtype=np.float32)
    rows, tiles = masses.shape
    if order is None:
        order = np.argsort(-masses, axis=1, kind="stable")
    sorted_mass = np.take_along_axis(masses, order, axis=1).astype(np.float64)

    counts = np.zeros(rows, np.int32)
    selected_mass = np.zeros(rows, np.float64)
    total_mass = np.zeros(rows, np.float64)
    support = np.zeros((rows, tiles), bool)
    for r in range(rows):
        row = sorted_mass[r]
        lanes = np.zeros(32, np.float64)
        for rank in range(tiles):
            lanes[rank % 32] += row[rank]
        off = 16
        while off:
            lanes[:off] = lanes[:off] + lanes[off : 2 * off]
            off >>= 1
        total = lanes[0]
        target = theta * total
        cumulative = 0.0
        count = tiles
        selected = total
        for chunk in range(0, tiles, 32):
            prefix = np.zeros(32, np.float64)
            width = min(32, tiles - chunk)
            prefix[:width] = row[chunk : chunk + width]
            off = 1
            while off < 32:
                shifted = prefix.copy()
                shifted[off:] = prefix[off:] + prefix[:-off]
                prefix = shifted
                off <<= 1
            reaches = (np.arange(32) < width) & (cumulative + prefix >= target)
            if reaches.any():
                first = int(np.argmax(reaches))
                count = chunk + first + 1
                selected = cumulative + prefix[first]
                break
            cumulative += prefix[31]
        counts[r] = count
        selected_mass[r] = selected
        total_mass[r] = total
        support[r, order[r, :count]] = True

    row_offsets = np.zeros(rows + 1, np.int32)
    row_offsets[1:] = np.cumsum(counts)
    block_indices = np.nonzero(support)[1].astype(np.int32)  # ascending inside each row
    measured = float(selected_mass.sum() / max(total_mass.sum(), 1e-20))
    return row_offsets, block_indices, measured, counts


def key_mask_tiles(mask: np.ndarray, key_block: int) -> np.ndarray:
    """Active key tiles of a broadcast key mask [B,H,1,Lk] (key_mask_tiles.cu:10-43).

    Returns int32 [B,H,tiles+1]: ascending ids of the tiles holding at least one
    visible key, then unspecified leftovers (set to -1 here), and the count of
    active tiles in the last slot.  A key is visible when a bool mask is
    non-zero or a floating bias is finite.
    """
    batch, heads, _, length = mask.shape
    tiles = (length + key_block - 1) // key_block
    visible = mask[:, :, 0] if mask.dtype == np.bool_ else np.isfinite(mask[:, :, 0].astype(np.float32))
    out = np.full((batch, heads, tiles + 1), -1, np.int32)
    for b in range(batch):
        for h in range(heads):
            active = [t for t in range(tiles) if visible[b, h, t * key_block : (t + 1) * key_block].any()]
            out[b, h, : len(active)] = active
            out[b, h, tiles] = len(active)
    return out
