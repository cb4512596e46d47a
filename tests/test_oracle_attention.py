"""Pins for the attention, block-mass and selection oracle (CPU): the closed forms and
invariants the reference's own CUDA tests assert, evaluated against the oracle."""

import numpy as np
import pytest
import torch

from oracle import attention, pipeline, prepare, selection

rng = np.random.default_rng(11)


def fp32_attention(q, k, v, mask=None, causal=False, scale=None):
    group = q.shape[1] // k.shape[1]
    qf, kf, vf = (torch.from_numpy(np.asarray(t, np.float32)) for t in (q, k, v))
    kf, vf = kf.repeat_interleave(group, 1), vf.repeat_interleave(group, 1)
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    scores = qf @ kf.transpose(-1, -2) * scale
    if mask is not None:
        m = torch.from_numpy(np.asarray(mask))
        m = torch.broadcast_to(m, scores.shape)
        scores = scores.masked_fill(~m, -torch.inf) if m.dtype == torch.bool else scores + m
    if causal:
        qi = torch.arange(scores.shape[-2])[:, None]
        ki = torch.arange(scores.shape[-1])[None, :]
        scores = scores.masked_fill(ki > qi, -torch.inf)
    out = torch.softmax(scores, -1).nan_to_num(nan=0) @ vf
    return out.numpy(), scores.logsumexp(-1).numpy()


def half(x):
    return torch.from_numpy(x).to(torch.float16).float().numpy()


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("length", [63, 65, 193, 1153])
def test_tile_max_known_answer_and_capture(dim, length):
    """Packed Q=1, K=+3/-2 per tile, scales 1, scale 1/128: the captured tile maximum is
    float(level*D*log2e/128 - 7.9943534) exactly (reference tests/cuda/test_risa_attention.py:20-92)."""
    q = np.zeros((1, 2, 137, dim), np.float32)
    k = np.zeros((1, 1, length, dim), np.float32)
    v = half(rng.standard_normal((1, 1, length, dim)).astype(np.float32) + 2)
    p = pipeline.prequantize(q, k, v, scale=1 / 128, dtype_name="float16")
    p.q[:] = 1
    p.q_scale[:] = 1
    p.k_scale[:] = 1
    blocks = (length + p.cta_k - 1) // p.cta_k
    levels = np.array([3 if i % 2 == 0 else -2 for i in range(blocks)])
    for i in range(blocks):
        p.k[:, :, i * p.cta_k : (i + 1) * p.cta_k] = levels[i]
    plain, _, _ = pipeline.attend(p)
    captured, _, cap = pipeline.attend(p, capture=True)
    np.testing.assert_array_equal(plain, captured)
    expected = (levels.astype(np.float64) * dim * (np.float64(np.float32(1.44269504088896340736)) / 128)
                - np.float64(np.float32(7.9943534))).astype(np.float32)
    if blocks > 1:
        np.testing.assert_array_equal(cap.tile_max[:, :-1], np.broadcast_to(expected[:-1], (274, blocks - 1)))
    masses = attention.block_mass(cap, 1, 2, 137)
    np.testing.assert_allclose(masses.sum(1), [128, 9, 128, 9], atol=2e-4)
    # all-hidden mask: exact zeros even with a non-zero V centre
    p.mask = np.zeros((1, 2, 137, length), bool)
    empty, lse, _ = pipeline.attend(p)
    assert not empty.any() and np.isneginf(lse).all()


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("k_len", [512, 1025])
@pytest.mark.parametrize("scale", [None, 0.0, -0.125])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_constant_values_preserve_probability_mass(dim, k_len, scale, mode):
    """reference tests/cuda/test_probability_mass.py:21-34."""
    q = half(rng.standard_normal((1, 2, 33, dim)).astype(np.float32))
    k = half(rng.standard_normal((1, 1, k_len, dim)).astype(np.float32))
    values = half(np.linspace(-3, 5, dim, dtype=np.float32))
    v = np.broadcast_to(values, k.shape).copy()
    out = pipeline.int8_attention(q, k, v, scale=scale, v_quantization=mode, dtype_name="float16")
    np.testing.assert_array_equal(out, np.broadcast_to(values, out.shape))


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("mask_kind", ["none", "key_bias", "row_mask"])
def test_dense_close_to_fp32(mode, dim, causal, mask_kind):
    """reference tests/cuda/test_risa_attention.py:94-149 (atol 0.10, rtol 0.03)."""
    q = half(rng.standard_normal((1, 2, 137, dim)).astype(np.float32))
    k = half(rng.standard_normal((1, 1, 263, dim)).astype(np.float32))
    v = half(rng.standard_normal((1, 1, 263, dim)).astype(np.float32) + 2)
    mask = None
    if mask_kind == "key_bias":
        mask = np.linspace(-2, 0, 263, dtype=np.float32)[None, None, None, :]
    elif mask_kind == "row_mask":
        mask = np.ones((137, 263), bool)
        mask[0] = False
    out, lse = pipeline.int8_attention(q, k, v, mask=mask, is_causal=causal, v_quantization=mode,
                                       dtype_name="float16", return_lse=True)
    ref, ref_lse = fp32_attention(q, k, v, mask, causal)
    np.testing.assert_allclose(out, ref, atol=0.10, rtol=0.03)
    if mask_kind == "row_mask":
        assert not out[:, :, 0].any() and np.isneginf(lse[:, :, 0]).all()
        np.testing.assert_allclose(lse[:, :, 1:], ref_lse[:, :, 1:], atol=0.05)
    else:
        np.testing.assert_allclose(lse, ref_lse, atol=0.05)


def test_causal_future_values_are_invisible():
    """reference tests/cuda/test_risa_attention.py:151-165."""
    q = np.zeros((1, 1, 193, 64), np.float32)
    v = np.zeros_like(q)
    v[:, :, 128:] = 100
    for mode in ("midpoint_affine", "absmax"):
        out, pattern, _, _ = pipeline.construct_sparse(q, q, v, theta=1.0, is_causal=True,
                                                       v_quantization=mode, dtype_name="float16")
        np.testing.assert_allclose(out[:, :, :128], 0, atol=0.01)
        p = pipeline.prequantize(q, q, v, is_causal=True, v_quantization=mode, dtype_name="float16")
        sparse, _, _ = pipeline.attend(p, pattern=pattern)
        np.testing.assert_allclose(sparse, out, atol=0.05, rtol=0.01)


def test_key_bias_large_tile_and_lse():
    """reference tests/cuda/test_risa_attention.py:167-179."""
    q = np.zeros((1, 2, 17, 128), np.float32)
    k = np.zeros((1, 1, 1153, 128), np.float32)
    v = np.full_like(k, 3)
    mask = np.linspace(-3, 0, 1153, dtype=np.float32)[None, None, None, :]
    for mode in ("midpoint_affine", "absmax"):
        p = pipeline.prequantize(q, k, v, mask=mask, return_lse=True, v_quantization=mode, dtype_name="float16")
        assert p.cta_k == 128
        out, lse, _ = pipeline.attend(p, return_lse=True)
        np.testing.assert_allclose(out, 3, atol=0.03)
        expected = torch.from_numpy(mask).logsumexp(-1).numpy()
        np.testing.assert_allclose(lse, np.broadcast_to(expected, (1, 2, 17)), atol=0.01)


def test_lse_restores_shifted_keys_and_empty_rows():
    """reference tests/cuda/test_risa_attention.py:181-193."""
    r = np.random.default_rng(29)
    q = half(r.standard_normal((1, 2, 19, 128)).astype(np.float32))
    k = half((r.standard_normal((1, 1, 257, 128)) * 0.1 + 4).astype(np.float32))
    v = half(r.standard_normal((1, 1, 257, 128)).astype(np.float32))
    mask = np.ones((19, 257), bool)
    mask[0] = False
    p = pipeline.prequantize(q, k, v, mask=mask, is_causal=True, return_lse=True, dtype_name="float16")
    assert (p.anchor >= 0).all()
    out, lse, _ = pipeline.attend(p, return_lse=True)
    _, expected = fp32_attention(q, k, v, mask, True)
    assert np.isneginf(lse[:, :, 0]).all() and not out[:, :, 0].any()
    np.testing.assert_allclose(lse[:, :, 1:], expected[:, :, 1:], atol=0.15, rtol=0.02)


@pytest.mark.parametrize("scale", [0.0, -0.125])
def test_signed_scale_tail_masks_and_lse(scale):
    """reference tests/cuda/test_probability_mass.py:37-70 (scale 0 -> LSE = log #visible)."""
    q = half(rng.standard_normal((1, 2, 129, 128)).astype(np.float32))
    k = half(rng.standard_normal((1, 1, 512, 128)).astype(np.float32))
    v = np.full_like(k, 3)
    mask = np.ones((129, 512), bool)
    mask[0] = False
    mask[1:, 7::9] = False
    out, lse = pipeline.int8_attention(q, k, v, scale=scale, mask=mask, is_causal=True, return_lse=True,
                                       dtype_name="bfloat16")
    np.testing.assert_array_equal(out[:, :, 1:], 3)
    assert not out[:, :, 0].any() and np.isneginf(lse[:, :, 0]).all()
    if scale == 0:
        visible = mask & (np.arange(512)[None, :] <= np.arange(129)[:, None])
        np.testing.assert_allclose(lse, np.broadcast_to(np.log(visible.sum(-1).astype(np.float32)), lse.shape), atol=2e-5)


def test_single_key_mass_and_output():
    """Single key: output == V and every block-mass row sums to its query count
    (reference tests/cuda/test_large_offsets.py:63-72)."""
    q = np.zeros((1, 3, 300, 64), np.float32)
    k = np.zeros((1, 1, 1, 64), np.float32)
    v = np.full((1, 1, 1, 64), 20.0, np.float32)
    p = pipeline.prequantize(q, k, v, scale=0.125, dtype_name="float16")
    out, _, cap = pipeline.attend(p, capture=True)
    np.testing.assert_array_equal(out, 20.0)
    masses = attention.block_mass(cap, 1, 3, 300)
    np.testing.assert_allclose(masses[:, 0], [128, 128, 44] * 3, atol=2e-5)


@pytest.mark.parametrize("theta", [0.5, 0.9, 0.99, 1.0])
def test_selector_matches_sort_cumsum_rule(theta):
    """counts = #(cumsum(sorted) < theta*total) + 1, clamped (reference src/risa_attention/reference.py:115-131)."""
    masses = rng.random((37, 70)).astype(np.float32) ** 4
    masses[3] = 0
    masses[4, :] = 1.0
    row_offsets, block_indices, measured, counts = selection.select_retained_mass(masses, theta)
    t = torch.from_numpy(masses)
    ordered, order = t.double().sort(dim=-1, descending=True, stable=True)
    target = theta * ordered.sum(-1, keepdim=True)
    expected = ((ordered.cumsum(-1) < target).sum(-1) + 1).clamp_(max=70).numpy()
    close = np.abs(ordered.cumsum(-1) - target).min(-1).values.numpy() < 1e-9 * np.maximum(ordered.sum(-1).numpy(), 1e-30)
    assert np.array_equal(counts[~close], expected[~close])
    assert row_offsets[-1] == counts.sum() == len(block_indices)
    for r in range(37):
        row = block_indices[row_offsets[r] : row_offsets[r + 1]]
        assert np.all(np.diff(row) > 0)
        if not close[r]:
            assert set(row) == set(order[r, : counts[r]].numpy())
    if theta == 1.0:
        assert measured == pytest.approx(1.0)
    assert 0 < measured <= 1.0 + 1e-12


def test_key_mask_tiles_known_answer():
    """reference tests/cuda/test_key_mask_tiles.py:78-104: first 512 of 1153 keys hidden, 128-key tiles."""
    mask = np.ones((1, 4, 1, 1153), bool)
    mask[..., :512] = False
    tiles = selection.key_mask_tiles(mask, 128)
    assert tiles.shape == (1, 4, 11)
    np.testing.assert_array_equal(tiles[..., :6], np.broadcast_to([4, 5, 6, 7, 8, 9], (1, 4, 6)))
    assert (tiles[..., -1] == 6).all()
    bias = np.where(mask, 0.5, -np.inf).astype(np.float32)
    np.testing.assert_array_equal(selection.key_mask_tiles(bias, 128), tiles)


def test_key_mask_tile_skipping_equals_generic_mask():
    """reference tests/cuda/test_key_mask_tiles.py:16-54."""
    r = np.random.default_rng(74)
    q = half(r.standard_normal((1, 2, 257, 64)).astype(np.float32))
    k = half(r.standard_normal((1, 1, 1153, 64)).astype(np.float32))
    v = half(r.standard_normal((1, 1, 1153, 64)).astype(np.float32) + 3)
    visible = np.ones((1, 2, 1, 1153), bool)
    visible[..., :128] = False
    visible[..., 384:768] = False
    visible[0, 1] = False
    p = pipeline.prequantize(q, k, v, mask=visible, return_lse=True, dtype_name="bfloat16")
    assert pipeline.key_mask_tile_list(p) is not None
    fast, fast_lse, _ = pipeline.attend(p, return_lse=True)
    generic, generic_lse, _ = pipeline.attend(p, return_lse=True, use_key_mask_tiles=False)
    np.testing.assert_allclose(fast, generic, atol=0.002, rtol=0.01)
    finite = np.isfinite(generic_lse)
    np.testing.assert_allclose(fast_lse[finite], generic_lse[finite], atol=2e-4)
    assert not fast[0, 1].any() and np.isneginf(fast_lse[0, 1]).all()


def test_cpu_plumbing_config():
    """The CPU plumbing configuration (N=1024, D=128, bf16, absmax) at reduced head count:
    NRMSE vs FP32 SDPA in the range of the reference README."""
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 4, 1024, 128, generator=g, dtype=torch.bfloat16).float().numpy()
    k = torch.randn(1, 1, 1024, 128, generator=g, dtype=torch.bfloat16).float().numpy()
    v = torch.randn(1, 1, 1024, 128, generator=g, dtype=torch.bfloat16).float().numpy()
    out, lse = pipeline.int8_attention(q, k, v, return_lse=True)
    ref, ref_lse = fp32_attention(q, k, v)
    nrmse = np.sqrt(((out - ref) ** 2).mean()) / np.sqrt((ref**2).mean())
    assert nrmse < 0.0175
    np.testing.assert_allclose(lse, ref_lse, atol=0.02)
