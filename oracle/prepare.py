"""Oracle for the Q/K/V preparation kernels (test infrastructure only).

Restates csrc/kernels/quantize_qk_impl.cuh, csrc/kernels/quantize_v_impl.cuh,
csrc/kernels/lse_correction.cu and the tile policy of
src/risa_attention/_validation.py / _quantization.py in numpy.  All tensor
arguments are binary32 arrays that already hold the (exactly converted) values
of the fp16/bf16/fp32 inputs.
"""

from __future__ import annotations

import numpy as np

from .ieee import F32, f32, fma32, rni_sat

# ---------------------------------------------------------------------------
# Tile policy
# ---------------------------------------------------------------------------


def kernel_head_dim(head_dim: int) -> int:
    """src/risa_attention/_quantization.py:67-73."""
    return 64 if head_dim <= 64 else 128 if head_dim <= 128 else 256


def select_key_block_size(kernel_dim: int, key_length: int, has_query_mask: bool) -> int:
    """src/risa_attention/_validation.py:64-72."""
    if not has_query_mask and kernel_dim >= 128 and key_length > 1024:
        return 128
    return 64


def pad_key_length(length: int, key_block: int) -> int:
    """src/risa_attention/_validation.py:60-61."""
    return (length + key_block - 1) // key_block * key_block


def rotation_mode(kernel_dim: int, key_length: int) -> str:
    """Rotation chosen by launch_quantize_qk (quantize_qk_impl.cuh:769-811).

    Both Q and K use the mode keyed on the *key* length.
    """
    if key_length <= 256:
        return "h4"
    return {64: "h64", 128: "h128_signed", 256: "h128_plain"}[kernel_dim]


def pad_channels(x: np.ndarray, kernel_dim: int) -> np.ndarray:
    x = f32(x)
    if x.shape[-1] == kernel_dim:
        return x
    pad = [(0, 0)] * (x.ndim - 1) + [(0, kernel_dim - x.shape[-1])]
    return np.pad(x, pad)


# ---------------------------------------------------------------------------
# Rotation (quantize_qk_impl.cuh:69-147)
# ---------------------------------------------------------------------------

SIGN_WORDS = (0x1035997B, 0x8087F5EE, 0xEE2E4E1A, 0x71132418)  # quantize_qk_impl.cuh:89-92


def sign_diagonal() -> np.ndarray:
    """+1/-1 per channel of a 128-channel row: bit c%32 of word c//32, 1 -> +, 0 -> -."""
    signs = np.empty(128, dtype=F32)
    for c in range(128):
        bit = (SIGN_WORDS[c // 32] >> (c % 32)) & 1
        signs[c] = 1.0 if bit else -1.0
    return signs


def _h4(x: np.ndarray) -> np.ndarray:
    """convrot4 on every aligned group of four channels (quantize_qk_impl.cuh:69-82)."""
    g = x.reshape(*x.shape[:-1], -1, 4)
    a0 = g[..., 0] + g[..., 1]
    a1 = g[..., 0] - g[..., 1]
    a2 = g[..., 2] + g[..., 3]
    a3 = g[..., 2] - g[..., 3]
    half = F32(0.5)
    y = np.stack(((a0 + a2) * half, (a1 + a3) * half, (a0 - a2) * half, (a1 - a3) * half), axis=-1)
    return y.astype(F32)


def _lane_butterflies(g: np.ndarray, lanes: int) -> np.ndarray:
    """Shuffle butterflies over ``lanes`` four-channel groups (…:108-139).

    ``g`` has shape [..., lanes, 4].  Stage ``bit``: the lane with the bit set
    computes other - mine, the lane without it computes mine + other.
    """
    index = np.arange(lanes)
    bit = 1
    while bit < lanes:
        other = g[..., index ^ bit, :]
        upper = ((index & bit) != 0)[:, None]
        g = np.where(upper, other - g, g + other).astype(F32)
        bit <<= 1
    return g


def rotate(x: np.ndarray, mode: str) -> np.ndarray:
    """Apply the Q/K rotation to the last axis (length 64, 128 or 256)."""
    x = f32(x)
    dim = x.shape[-1]
    if mode == "h4":
        return _h4(x).reshape(x.shape)
    if mode == "h64":
        assert dim == 64
        g = _lane_butterflies(_h4(x), 16)
        return (g * F32(0.25)).astype(F32).reshape(x.shape)
    if mode in ("h128_signed", "h128_plain"):
        assert dim % 128 == 0 and (mode == "h128_plain" or dim == 128)
        t = x.reshape(*x.shape[:-1], dim // 128, 128)
        if mode == "h128_signed":
            # Sign flip is exact (IEEE sign bit), quantize_qk_impl.cuh:88-100.
            t = t * sign_diagonal()
        g = _lane_butterflies(_h4(t), 32)
        return (g * F32(0.1767766952966369)).astype(F32).reshape(x.shape)
    raise ValueError(mode)


# ---------------------------------------------------------------------------
# K anchor (quantize_qk_impl.cuh:442-577)
# ---------------------------------------------------------------------------


def _shfl_down_sum(v: np.ndarray) -> np.ndarray:
    """Lane 0 of the 32-lane ``v += shfl_down(v, off)`` tree, off = 16..1; v[..., 32]."""
    v = v.copy()
    off = 16
    while off:
        v[..., :off] = v[..., :off] + v[..., off : 2 * off]
        off >>= 1
    return v[..., 0]


def _shfl_down_max(v: np.ndarray) -> np.ndarray:
    return v.max(axis=-1)


def detect_key_anchor(k: np.ndarray) -> np.ndarray:
    """Anchor row per (batch, kv head) or -1; ``k`` is [B, Hkv, Lk, Dk] (padded)."""
    k = f32(k)
    batch, heads, length, dim = k.shape
    rows = np.array([s * (length - 1) // 8 for s in range(9)])
    samples = k[:, :, rows, :]  # [B,H,9,D]
    threads = 128
    e0 = np.zeros((batch, heads, threads), F32)
    m0 = np.zeros((batch, heads, threads), F32)
    dist = np.zeros((batch, heads, 9, threads), F32)
    # Thread t owns channels t, t+128 in that order.
    for base in range(0, dim, threads):
        width = min(threads, dim - base)
        x = samples[..., base : base + width]  # [B,H,9,w]
        csum = np.zeros((batch, heads, width), F32)
        for s in range(9):
            v = x[:, :, s]
            e0[..., :width] = fma32(v, v, e0[..., :width])
            m0[..., :width] = np.maximum(m0[..., :width], np.abs(v))
            csum = csum + v
        for c in range(9):
            d = F32(9.0) * x[:, :, c] - csum
            dist[:, :, c, :width] = fma32(d, d, dist[:, :, c, :width])

    def block_sum(v):  # v[..., 128] -> warp trees then warps 0..3 in order
        warps = _shfl_down_sum(v.reshape(*v.shape[:-1], 4, 32))
        total = np.zeros(v.shape[:-1], F32)
        for w in range(4):
            total = total + warps[..., w]
        return total

    total_dist = np.stack([block_sum(dist[:, :, c]) for c in range(9)], axis=-1)  # [B,H,9]
    best = np.zeros((batch, heads), np.int64)
    best_d = np.full((batch, heads), F32(3.402823466e38))
    for c in range(9):
        better = total_dist[..., c] < best_d
        best = np.where(better, c, best)
        best_d = np.where(better, total_dist[..., c], best_d)

    e1 = np.zeros((batch, heads, threads), F32)
    m1 = np.zeros((batch, heads, threads), F32)
    anchor_rows = np.take_along_axis(samples, best[:, :, None, None], axis=2)  # [B,H,1,D]
    for base in range(0, dim, threads):
        width = min(threads, dim - base)
        x = samples[..., base : base + width]
        a = anchor_rows[:, :, 0, base : base + width]
        for s in range(9):
            r = x[:, :, s] - a
            e1[..., :width] = fma32(r, r, e1[..., :width])
            m1[..., :width] = np.maximum(m1[..., :width], np.abs(r))
    te0, te1 = block_sum(e0), block_sum(e1)
    tm0, tm1 = m0.max(-1), m1.max(-1)
    improves = (te1 < te0) & (tm1 <= tm0 * F32(1.125))
    return np.where(improves, rows[best], -1).astype(np.int32)


# ---------------------------------------------------------------------------
# Q/K quantisation (quantize_qk_impl.cuh:153-426)
# ---------------------------------------------------------------------------


def _quantize_groups(y: np.ndarray, group_axes: tuple[int, ...]):
    mx = np.abs(y).max(axis=group_axes, keepdims=True)
    scale = (mx / F32(127.0) + F32(1e-7)).astype(F32)
    inverse = (F32(1.0) / scale).astype(F32)
    codes = rni_sat(y * inverse, -128, 127).astype(np.int8)
    return codes, scale


def quantize_queries(q: np.ndarray, key_length: int):
    """[B,Hq,Lq,Dk] -> (codes int8 same shape, scales [B,Hq,ceil(Lq/128)*S*8]).

    Group of token n: all channels of the tokens congruent to n mod 8 inside
    the W-row slice holding n; (S, W) = (4, 32) for Dk <= 128, (8, 16) for 256
    (process_q, quantize_qk_impl.cuh:158-165, 232-236).
    """
    q = f32(q)
    batch, heads, length, dim = q.shape
    y = rotate(q, rotation_mode(dim, key_length))
    width = 16 if dim == 256 else 32
    padded = (length + 127) // 128 * 128
    y = np.pad(y, ((0, 0), (0, 0), (0, padded - length), (0, 0)))
    g = y.reshape(batch, heads, padded // width, width // 8, 8, dim)
    codes, scale = _quantize_groups(g, (3, 5))
    codes = codes.reshape(batch, heads, padded, dim)[:, :, :length]
    return np.ascontiguousarray(codes), scale.reshape(batch, heads, padded // width * 8)


def quantize_keys(k: np.ndarray, key_block: int, anchor: np.ndarray | None = None):
    """[B,Hkv,Lk,Dk] -> (codes, scales [B,Hkv,ceil(Lk/cta_k)*4], anchor int32 [B,Hkv]).

    Group of token n: all channels of the tokens of tile n//cta_k with the
    same (n % 8)//2 (process_k, quantize_qk_impl.cuh:283-285, 325, 388).
    """
    k = f32(k)
    batch, heads, length, dim = k.shape
    if anchor is None:
        anchor = detect_key_anchor(k)
    shifted = k.copy()
    for b in range(batch):
        for h in range(heads):
            if anchor[b, h] >= 0:
                shifted[b, h] = k[b, h] - k[b, h, int(anchor[b, h])]
    y = rotate(shifted, rotation_mode(dim, length))
    padded = pad_key_length(length, key_block)
    y = np.pad(y, ((0, 0), (0, 0), (0, padded - length), (0, 0)))
    g = y.reshape(batch, heads, padded // key_block, key_block // 8, 4, 2, dim)
    codes, scale = _quantize_groups(g, (3, 5, 6))
    codes = codes.reshape(batch, heads, padded, dim)[:, :, :length]
    return (
        np.ascontiguousarray(codes),
        scale.reshape(batch, heads, padded // key_block * 4),
        anchor.astype(np.int32),
    )


# ---------------------------------------------------------------------------
# V quantisation (quantize_v_impl.cuh:83-292)
# ---------------------------------------------------------------------------


def _xor_tree_sum(v: np.ndarray) -> np.ndarray:
    """``v += shfl_xor(v, off)`` for off = 16..1 over the last axis of length 32."""
    index = np.arange(32)
    off = 16
    while off:
        v = v + v[..., index ^ off]
        off >>= 1
    return v[..., 0]


def quantize_values(v: np.ndarray, key_block: int, midpoint_affine: bool):
    """[B,Hkv,L,Dk] -> (codes int8 [B*Hkv*Dk, Lpad] in token order, scale, center).

    The code matrix is *logical*: column n is token n, padding columns are 0.
    Physical orders (the reference's 16-token permutation and the MFMA order of
    the HIP kernels) are applied by :func:`reference_value_order` and
    ``risaattention_amd.layout``.
    """
    v = f32(v)
    batch, heads, length, dim = v.shape
    padded = pad_key_length(length, key_block)
    vt = np.ascontiguousarray(v.transpose(0, 1, 3, 2)).reshape(batch * heads * dim, length)
    if midpoint_affine:
        mn, mx = vt.min(axis=1), vt.max(axis=1)
        center0 = (F32(0.5) * (mn + mx)).astype(F32)
        radius = (F32(0.5) * (mx - mn)).astype(F32)
    else:
        center0 = np.zeros(vt.shape[0], F32)
        radius = np.abs(vt).max(axis=1)
    scale = np.maximum(radius * (F32(1.0) / F32(127.0)), F32(1e-12)).astype(F32)
    inverse = (F32(1.0) / scale).astype(F32)
    normalized = ((vt - center0[:, None]) * inverse[:, None]).astype(F32)
    codes_f = rni_sat(normalized, -128, 127)
    codes = np.zeros((vt.shape[0], padded), np.int8)
    codes[:, :length] = codes_f.astype(np.int8)
    if not midpoint_affine:
        return codes, scale, np.zeros_like(scale)

    # Residual sum in the order of the 512-thread (128 for L <= 256) schedule:
    # thread t adds tokens L-1-t, L-1-t-T, ...; 32-lane xor tree; warps in order
    # (quantize_v_impl.cuh:233-275, launch_quantize_v :356-401).
    threads = 128 if length <= 256 else 512
    residual = (normalized - codes_f.astype(F32)).astype(F32)
    reverse = residual[:, ::-1]
    steps = (length + threads - 1) // threads
    reverse = np.pad(reverse, ((0, 0), (0, steps * threads - length)))
    per_thread = np.zeros((vt.shape[0], threads), F32)
    for step in range(steps):
        per_thread = per_thread + reverse[:, step * threads : (step + 1) * threads]
    warps = _xor_tree_sum(per_thread.reshape(vt.shape[0], threads // 32, 32))
    total = np.zeros(vt.shape[0], F32)
    for w in range(threads // 32):
        total = total + warps[:, w]
    restored_scale = (F32(1.0) / inverse).astype(F32)
    center = (center0 + restored_scale * (total / F32(length))).astype(F32)
    return codes, scale, center


def value_tile_sums(codes: np.ndarray, key_block: int) -> np.ndarray:
    """Per (row, key tile) integer sum of V codes (zero-point term of the HIP P·V)."""
    rows, padded = codes.shape
    return codes.reshape(rows, padded // key_block, key_block).astype(np.int32).sum(-1)


REFERENCE_ORDER_16 = (0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15)


def reference_value_order(codes: np.ndarray) -> np.ndarray:
    """Token order -> the reference's packed order (quantize_v_impl.cuh:47-52).

    Position p of each 16-token group holds token REFERENCE_ORDER_16[p]
    (tests/cuda/test_value_quantization.py:42).
    """
    rows, padded = codes.shape
    return codes.reshape(rows, padded // 16, 16)[..., list(REFERENCE_ORDER_16)].reshape(rows, padded)


# ---------------------------------------------------------------------------
# LSE anchor correction (lse_correction.cu:4-28)
# ---------------------------------------------------------------------------


def lse_shift(q: np.ndarray, k: np.ndarray, anchor: np.ndarray, scale: float) -> np.ndarray:
    """scale * <q[b,h,i], k[b,h//G,anchor]> with the kernel's summation order."""
    q, k = f32(q), f32(k)
    batch, q_heads, q_len, dim = q.shape
    group = q_heads // k.shape[1]
    out = np.zeros((batch, q_heads, q_len), F32)
    for b in range(batch):
        for h in range(q_heads):
            a = int(anchor[b, h // group])
            if a < 0:
                continue
            prod = (q[b, h] * k[b, h // group, a]).astype(F32)  # [Lq, D]
            lanes = np.zeros((q_len, 32), F32)
            for d0 in range(0, dim, 32):
                lanes = lanes + prod[:, d0 : d0 + 32]
            out[b, h] = _shfl_down_sum(lanes) * F32(scale)
    return out
