"""Oracle for the fused INT8 attention kernel (test infrastructure only).

Restates csrc/kernels/attention_int8.cuh, attention_softmax.cuh,
attention_value.cuh, attention_masks.cuh and the path selection of
attention_dispatch.cu.  One call processes prepared tensors exactly as the
kernel does: per 128-query block, key tile by key tile, with FP32 online
softmax in the exp2 domain, U8 probabilities quantised relative to each tile's
own maximum and integer P·V per tile.

Differences from the CUDA kernel that do not change the definition of the
result: the denominator is kept as one FP32 value per row instead of four
per-lane partials (O(1e-7) relative), and exp2/log2/reciprocal are correctly
rounded instead of the approximate PTX instructions.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .ieee import F32, LOG2E, ROW_FLOOR, U8_OFFSET, exp2_32, f32, fma32, log2_32, rni_sat, round_to_dtype

QUERY_BLOCK = 128


@dataclass
class Captured:
    """Per-row, per-tile statistics stored when block mass is captured.

    ``numerator[row, tile]`` is the integer sum of the tile's U8 probabilities,
    ``tile_max[row, tile]`` the tile's own shifted maximum, ``state`` the final
    (m, d) of the row (attention_int8.cuh:51-143, 769-848, 871-898).
    """

    numerator: np.ndarray
    tile_max: np.ndarray
    state_m: np.ndarray
    state_d: np.ndarray


def _mask_values(mask, b, h, rows, keys):
    """Returns (keep bool [R,C], bias*log2e f32 [R,C]) for mask[b,h,rows,keys]."""
    plane = mask[b, h]
    row_index = rows if plane.shape[0] > 1 else np.zeros(len(rows), dtype=np.int64)
    block = plane[row_index][:, keys]
    if block.dtype == np.bool_:
        return block, np.zeros(block.shape, F32)
    bias = block.astype(F32)
    keep = np.isfinite(bias)
    with np.errstate(invalid="ignore"):
        shifted = (np.where(keep, bias, F32(0)) * LOG2E).astype(F32)
    return keep, shifted


def attend(
    q_codes: np.ndarray,
    k_codes: np.ndarray,
    v_codes: np.ndarray,
    q_scale: np.ndarray,
    k_scale: np.ndarray,
    v_scale: np.ndarray,
    v_center: np.ndarray,
    *,
    key_block: int,
    sm_scale: float,
    mask: np.ndarray | None = None,
    is_causal: bool = False,
    row_offsets: np.ndarray | None = None,
    block_indices: np.ndarray | None = None,
    key_mask_tiles: np.ndarray | None = None,
    capture: bool = False,
    out_dtype: str = "bfloat16",
):
    """Run the quantised attention pipeline.

    ``q_codes`` [B,Hq,Lq,Dk] int8, ``k_codes`` [B,Hkv,Lk,Dk] int8, ``v_codes``
    [B*Hkv*Dk, Lpad] int8 in token order, scales as produced by
    ``oracle.prepare``.  ``mask`` is already broadcast to [B,Hq,Lq|1,Lk] (a
    query extent of 1 means a key-only mask).  Returns ``(out f32 rounded to
    out_dtype [B,Hq,Lq,Dk], lse f32 [B,Hq,Lq], Captured | None)``.
    """
    batch, q_heads, q_len, dim = q_codes.shape
    kv_heads, k_len = k_codes.shape[1], k_codes.shape[2]
    group = q_heads // kv_heads
    padded = v_codes.shape[1]
    n_kb = (k_len + key_block - 1) // key_block
    n_qb = (q_len + QUERY_BLOCK - 1) // QUERY_BLOCK
    assert padded == n_kb * key_block
    sparse = row_offsets is not None
    if mask is not None:
        mask = np.broadcast_to(mask, (batch, q_heads) + tuple(mask.shape[2:]))
    indexed_mask = key_mask_tiles is not None
    assert not (sparse and capture)

    # attention_int8.cuh:196 — custom masks, causal and non-positive scale keep
    # pre-scaled FP32 scores; the rest is the raw-score fast path.
    pre = mask is not None or is_causal or not (sm_scale > 0.0)
    guard_empty = mask is not None or is_causal  # :902-912
    sm2 = F32(F32(sm_scale) * LOG2E)  # :209
    width = 16 if dim == 256 else 32
    qf = q_codes.astype(F32)
    kf = k_codes.astype(F32)
    vf = v_codes.astype(F32).reshape(batch, kv_heads, dim, padded)

    out = np.zeros((batch, q_heads, q_len, dim), F32)
    lse = np.zeros((batch, q_heads, q_len), F32)
    cap = None
    if capture:
        cap = Captured(
            np.zeros((batch * q_heads * q_len, n_kb), np.int64),
            np.zeros((batch * q_heads * q_len, n_kb), F32),
            np.zeros(batch * q_heads * q_len, F32),
            np.zeros(batch * q_heads * q_len, F32),
        )

    for b in range(batch):
        for h in range(q_heads):
            hk = h // group
            vsc = v_scale.reshape(batch, kv_heads, dim)[b, hk]
            vce = v_center.reshape(batch, kv_heads, dim)[b, hk]
            # Dense non-causal calls give every query block the same tile list;
            # process all rows of the head at once in that case.
            uniform = not sparse and not (is_causal and not capture)
            blocks = [None] if uniform else list(range(n_qb))
            for qb in blocks:
                if qb is None:
                    rows = np.arange(q_len)
                else:
                    rows = np.arange(qb * QUERY_BLOCK, min(q_len, (qb + 1) * QUERY_BLOCK))
                if sparse:
                    r = (b * q_heads + h) * n_qb + qb
                    tiles = [int(t) for t in block_indices[row_offsets[r] : row_offsets[r + 1]]]
                elif indexed_mask:
                    count = int(key_mask_tiles[b, h, n_kb])
                    tiles = [int(t) for t in key_mask_tiles[b, h, :count]]
                elif is_causal and not capture:
                    limit = min(k_len, (qb + 1) * QUERY_BLOCK)
                    tiles = list(range((limit + key_block - 1) // key_block))
                else:
                    tiles = list(range(n_kb))

                qs = q_scale[b, h][(rows // width) * 8 + rows % 8]  # [R]
                q_rows = qf[b, h, rows]
                m = np.full(len(rows), ROW_FLOOR, F32)
                d = np.zeros(len(rows), F32)
                acc = np.zeros((len(rows), dim), F32)

                for it, t in enumerate(tiles):
                    last = it == len(tiles) - 1
                    k0 = t * key_block
                    keys = np.arange(k0, k0 + key_block)
                    inb = keys < k_len
                    k_tile = np.zeros((key_block, dim), F32)
                    k_tile[inb] = kf[b, hk, keys[inb]]
                    scores = q_rows @ k_tile.T  # exact: |S| <= 256*127^2 < 2^24
                    kgroup = (keys % 8) // 2
                    ks = k_scale[b, hk][t * 4 + kgroup]  # [C]
                    s = (sm2 * (qs[:, None] * ks[None, :]).astype(F32)).astype(F32)  # :439-442

                    if pre:
                        x = (scores * s).astype(F32)  # :497-499
                        keep = np.ones(x.shape, bool)
                        if mask is not None:
                            safe_keys = np.where(inb, keys, 0)
                            mkeep, mbias = _mask_values(mask, b, h, rows, safe_keys)
                            mkeep = mkeep & inb[None, :]
                            x = np.where(mkeep, (x + mbias).astype(F32), -np.inf)  # attention_masks.cuh:88
                            keep &= mkeep
                        if is_causal:
                            future = keys[None, :] > rows[:, None]  # attention_masks.cuh:27-47
                            x = np.where(future, -np.inf, x)
                        if last:
                            x = np.where(inb[None, :], x, -np.inf)  # :733-734
                        x = x.astype(F32)
                        tile_m = (np.maximum(ROW_FLOOR, x.max(axis=1)) - U8_OFFSET).astype(F32)
                        with np.errstate(invalid="ignore"):
                            p = exp2_32((x - tile_m[:, None]).astype(F32))
                    elif not last:
                        # update_online_softmax_i32, attention_softmax.cuh:121-183
                        tile_m = fma32(scores, s, -U8_OFFSET).max(axis=1)
                        p = exp2_32(fma32(scores, s, -tile_m[:, None]))
                    else:
                        # generic last tile on raw scores, attention_int8.cuh:721-734,
                        # attention_softmax.cuh:27-100: per-lane maxima start at -50000.
                        raw = np.where(inb[None, :], scores, F32(-1.0e30)).astype(F32)
                        tile_m = np.full(len(rows), -np.inf, F32)
                        for g in range(4):
                            sel = kgroup == g
                            lane_max = np.maximum(ROW_FLOOR, raw[:, sel].max(axis=1))
                            # every key of the group shares one k scale
                            s_lane = s[:, np.argmax(sel)]
                            tile_m = np.maximum(tile_m, fma32(lane_max, s_lane, -U8_OFFSET))
                        p = exp2_32(fma32(raw, s, -tile_m[:, None]))

                    p8 = rni_sat(p, 0, 255)
                    numer = p8.sum(axis=1, dtype=np.float64)  # exact integer <= 128*255
                    # online update, attention_softmax.cuh:60-76 / 148-158
                    with np.errstate(invalid="ignore"):
                        alpha = exp2_32(-np.abs(m - tile_m))
                    o_s = np.where(m < tile_m, alpha, F32(1)).astype(F32)
                    t_s = np.where(tile_m < m, alpha, F32(1)).astype(F32)
                    m = np.maximum(m, tile_m)
                    d = (d * o_s + numer.astype(F32) * t_s).astype(F32)
                    v_tile = vf[b, hk][:, k0 : k0 + key_block]  # [D, C], padding already 0
                    pv = p8 @ v_tile.T  # exact: <= 128*255*127 < 2^24
                    acc = fma32(pv, t_s[:, None], (acc * o_s[:, None]).astype(F32))  # attention_value.cuh:143-146
                    if capture:
                        rr = (b * q_heads + h) * q_len + rows
                        cap.numerator[rr, t] = numer.astype(np.int64)
                        cap.tile_max[rr, t] = tile_m

                # epilogue, attention_value.cuh:31-66, attention_int8.cuh:902-943, 1010-1025
                with np.errstate(divide="ignore", invalid="ignore"):
                    normalised = (acc * (F32(1) / d)[:, None]).astype(F32)
                    result = fma32(normalised, vsc[None, :], vce[None, :])
                    row_lse = ((log2_32(d) + m) / LOG2E).astype(F32)
                valid = d > 0
                if guard_empty:
                    result = np.where(valid[:, None], result, F32(0))
                out[b, h, rows] = result
                lse[b, h, rows] = np.where(valid, row_lse, -np.inf)
                if capture:
                    rr = (b * q_heads + h) * q_len + rows
                    cap.state_m[rr] = m
                    cap.state_d[rr] = d
    return round_to_dtype(out, out_dtype), lse, cap


def block_mass(cap: Captured, batch: int, q_heads: int, q_len: int) -> np.ndarray:
    """captured_block_mass_kernel (attention_int8.cuh:1028-1088).

    mass[row_block, tile] = sum over the block's queries of
    numerator * 2^(tile_max - m) / d (0 when d == 0), summed by a 32-lane
    shuffle-down tree per warp and a second tree over the four warp sums.
    """
    n_kb = cap.numerator.shape[1]
    n_qb = (q_len + QUERY_BLOCK - 1) // QUERY_BLOCK
    mass = np.zeros((batch * q_heads * n_qb, n_kb), F32)
    num = cap.numerator.astype(F32)
    for bh in range(batch * q_heads):
        for qb in range(n_qb):
            lo = bh * q_len + qb * QUERY_BLOCK
            hi = bh * q_len + min(q_len, (qb + 1) * QUERY_BLOCK)
            m = cap.state_m[lo:hi, None]
            d = cap.state_d[lo:hi, None]
            with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
                per_query = (num[lo:hi] * exp2_32((cap.tile_max[lo:hi] - m).astype(F32))).astype(F32) / d
            per_query = np.where(d > 0, per_query, F32(0)).astype(F32)
            lanes = np.zeros((QUERY_BLOCK, n_kb), F32)
            lanes[: hi - lo] = per_query
            lanes = lanes.reshape(4, 32, n_kb)
            off = 16
            while off:
                lanes[:, :off] = lanes[:, :off] + lanes[:, off : 2 * off]
                off >>= 1
            w = lanes[:, 0]
            mass[bh * n_qb + qb] = (w[0] + w[2]) + (w[1] + w[3])
    return mass
