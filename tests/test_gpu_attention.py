"""Parity of the HIP attention kernel with the oracle: outputs and LSE within 1e-3
relative L2 (the tolerance the task states for floating-point results), plus the
closed-form contracts of the reference's own CUDA tests."""

from dataclasses import replace
import math

import numpy as np
import pytest
import torch

from oracle import pipeline as oracle_pipeline
from tests.helpers import oracle_prequantize, relative_l2, seeded, to_numpy

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-3


def mask_variants(q_len, k_len, device="cuda"):
    key_bias = torch.linspace(-2, 0, k_len, device=device)[None, None, None, :]
    row_mask = torch.ones(q_len, k_len, device=device, dtype=torch.bool)
    row_mask[0] = False
    row_mask[1:, 7::9] = False
    return {"none": None, "key_bias": key_bias, "row_mask": row_mask}


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("mask_name", ["none", "key_bias", "row_mask"])
def test_dense_matches_oracle(risa, mode, dim, causal, mask_name):
    q = seeded((1, 2, 137, dim), torch.float16, 17)
    k = seeded((1, 1, 263, dim), torch.float16, 18)
    v = seeded((1, 1, 263, dim), torch.float16, 19, offset=2.0)
    mask = mask_variants(137, 263)[mask_name]
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, v_quantization=mode,
                                   return_lse=True)
    prepared = oracle_prequantize(q, k, v, attn_mask=mask, is_causal=causal, v_quantization=mode,
                                  return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse), expected_lse) < TOLERANCE
    # FP32 SDPA bound of reference tests/cuda/test_risa_attention.py:118-132
    from risaattention_amd.policy import apply_score_mask

    scores = q.float() @ k.float().repeat_interleave(2, 1).transpose(-1, -2) / dim**0.5
    expanded = None if mask is None else torch.broadcast_to(mask, scores.shape)
    scores = apply_score_mask(scores, expanded, causal, 0)
    reference = scores.softmax(-1).nan_to_num(nan=0) @ v.float().repeat_interleave(2, 1)
    torch.testing.assert_close(out.float(), reference, atol=0.10, rtol=0.03)


@pytest.mark.parametrize("dim,heads,k_len", [(128, 4, 1300), (64, 4, 700), (256, 2, 1300), (128, 144, 1300)])
@pytest.mark.parametrize("variant", ["plain", "causal", "row_mask", "key_bias"])
def test_outlier_channels_match_oracle(risa, dim, heads, k_len, variant):
    """One channel in a hundred scaled by 20: near one-hot attention rows, large score
    scales.  144 heads x 3 query blocks take the 32-query kernel, the others the 16-query one."""
    generator = torch.Generator().manual_seed(23)
    q_len = 300
    q = torch.randn(1, heads, q_len, dim, generator=generator)
    k = torch.randn(1, 2, k_len, dim, generator=generator)
    v = torch.randn(1, 2, k_len, dim, generator=generator)
    hot = torch.randperm(dim, generator=generator)[: max(1, dim // 100)]
    for tensor in (q, k, v):
        tensor[..., hot] *= 20.0
    q, k, v = (t.to(torch.bfloat16).cuda() for t in (q, k, v))
    masks = mask_variants(q_len, k_len)
    mask = masks.get(variant)
    causal = variant == "causal"
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, return_lse=True)
    oracle_heads = slice(0, min(heads, 8))  # the oracle on a slice of whole KV groups
    kv = slice(0, 1) if heads > 8 else slice(0, 2)
    prepared = oracle_prequantize(q[:, oracle_heads], k[:, kv], v[:, kv], attn_mask=mask, is_causal=causal,
                                  return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[:, oracle_heads]), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse[:, oracle_heads]), expected_lse) < TOLERANCE


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("k_len", [1153, 2304])
def test_large_tile_dense_and_scale_signs(risa, dtype, k_len):
    q = seeded((1, 4, 300, 128), dtype, 5)
    k = seeded((1, 2, k_len, 128), dtype, 6)
    v = seeded((1, 2, k_len, 128), dtype, 7)
    for scale in (None, 0.0, -0.125):
        out, lse = risa.int8_attention(q, k, v, scale=scale, return_lse=True)
        prepared = oracle_prequantize(q, k, v, scale=scale, return_lse=True)
        assert prepared.cta_k == 128
        expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
        assert relative_l2(to_numpy(out), expected) < TOLERANCE
        assert relative_l2(to_numpy(lse), expected_lse) < TOLERANCE


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("k_len", [512, 1025])
@pytest.mark.parametrize("scale", [None, 0.0, -0.125])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_constant_values_preserve_probability_mass(risa, dtype, dim, k_len, scale, mode):
    """reference tests/cuda/test_probability_mass.py:21-34."""
    torch.manual_seed(41)
    q = torch.randn(1, 4, 129, dim, device="cuda", dtype=dtype)
    k = torch.randn(1, 2, k_len, dim, device="cuda", dtype=dtype)
    values = torch.linspace(-3, 5, dim, device="cuda", dtype=dtype)
    v = values.expand_as(k).contiguous()
    out = risa.int8_attention(q, k, v, scale=scale, v_quantization=mode)
    torch.testing.assert_close(out, values.expand_as(out), atol=0, rtol=0)


@pytest.mark.parametrize("k_len", [512, 1025])
@pytest.mark.parametrize("scale", [0.0, -0.125])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_signed_scale_tail_masks_and_lse(risa, k_len, scale, mode):
    """reference tests/cuda/test_probability_mass.py:37-70."""
    torch.manual_seed(43)
    q = torch.randn(1, 4, 129, 128, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(1, 2, k_len, 128, device="cuda", dtype=q.dtype)
    v = torch.full_like(k, 3)
    mask = torch.ones(129, k_len, device="cuda", dtype=torch.bool)
    mask[0] = False
    mask[1:, 7::9] = False
    out, lse = risa.int8_attention(q, k, v, scale=scale, attn_mask=mask, is_causal=True,
                                   v_quantization=mode, return_lse=True)
    torch.testing.assert_close(out[:, :, 1:], torch.full_like(out[:, :, 1:], 3), atol=0, rtol=0)
    assert torch.count_nonzero(out[:, :, 0]) == 0
    assert torch.isneginf(lse[:, :, 0]).all()
    assert torch.isfinite(lse[:, :, 1:]).all()
    if scale == 0:
        visible = mask & (torch.arange(k_len, device="cuda")[None, :] <= torch.arange(129, device="cuda")[:, None])
        expected = visible.sum(-1).float().log().expand_as(lse)
        torch.testing.assert_close(lse, expected, atol=2e-5, rtol=0)


def test_residual_center_preserves_uniform_attention_mean(risa):
    """reference tests/cuda/test_probability_mass.py:148-155."""
    torch.manual_seed(3)
    q = torch.zeros(1, 2, 129, 128, device="cuda", dtype=torch.bfloat16)
    k = torch.zeros(1, 1, 512, 128, device="cuda", dtype=q.dtype)
    v = torch.randn_like(k) + 3
    v[..., ::53, :] += 12
    out = risa.int8_attention(q, k, v, v_quantization="midpoint_affine")
    expected = v.float().mean(-2, keepdim=True).to(v.dtype).expand_as(out)
    torch.testing.assert_close(out, expected, atol=0, rtol=0)


@pytest.mark.parametrize("mode", ["midpoint_affine", "absmax"])
@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("length", [63, 65, 193, 1153])
def test_capture_tile_max_known_answer(risa, mode, dim, length):
    """reference tests/cuda/test_risa_attention.py:20-92: packed Q=1, K=+3/-2 per tile."""
    q = torch.zeros(1, 2, 137, dim, device="cuda", dtype=torch.float16)
    k = torch.zeros(1, 1, length, dim, device="cuda", dtype=torch.float16)
    torch.manual_seed(length)
    packed = risa.prequantize_int8_attention(q, k, torch.randn_like(k) + 2, scale=1 / 128, v_quantization=mode)
    packed.q.fill_(1)
    packed.q_scale.fill_(1)
    packed.k_scale.fill_(1)
    blocks = (length + packed.cta_k - 1) // packed.cta_k
    levels = torch.tensor([3 if i % 2 == 0 else -2 for i in range(blocks)], dtype=torch.int8, device="cuda")
    for i in range(blocks):
        packed.k[:, :, i * packed.cta_k : (i + 1) * packed.cta_k].fill_(3 if i % 2 == 0 else -2)
    batch, heads, queries, _ = packed.q.shape
    mass_elements = batch * heads * ((queries + 127) // 128) * blocks
    rows = batch * heads * queries
    workspace = torch.empty(mass_elements + rows * (blocks * 2 + 2), device="cuda", dtype=torch.float32)
    plain = risa.int8_attention_from_prequantized(packed)
    captured = risa.int8_attention_from_prequantized(packed, _block_mass=workspace)
    assert torch.equal(plain.view(torch.int16), captured.view(torch.int16))
    if blocks > 1:
        full_stats = workspace[mass_elements : mass_elements + rows * (blocks - 1) * 2]
        maxima = full_stats.reshape(batch * heads, blocks - 1, queries, 2)[..., 1].transpose(1, 2).reshape(rows, blocks - 1)
        scale = torch.tensor(1.44269504088896340736, device="cuda", dtype=torch.float32) / 128
        offset = torch.tensor(7.9943534, device="cuda", dtype=torch.float32)
        expected = (levels[:-1].double() * dim * scale.double() - offset.double()).float()
        assert torch.equal(maxima, expected.expand_as(maxima))
    masses = workspace[:mass_elements].view(-1, blocks)
    per_block = torch.tensor([128.0, 9.0] * heads, device="cuda")
    torch.testing.assert_close(masses.sum(-1), per_block, atol=2e-4, rtol=0)
    hidden = torch.zeros(batch, heads, queries, length, device="cuda", dtype=torch.bool)
    empty = risa.int8_attention_from_prequantized(replace(packed, attn_mask=hidden))
    assert torch.count_nonzero(empty) == 0


def test_causal_future_values_are_invisible(risa):
    """reference tests/cuda/test_risa_attention.py:151-165."""
    q = torch.zeros(1, 1, 193, 64, device="cuda", dtype=torch.float16)
    v = torch.zeros_like(q)
    v[:, :, 128:] = 100
    for mode in ("midpoint_affine", "absmax"):
        out, pattern = risa.construct_sparse_int8_attention(q, q, v, is_causal=True, theta=1.0, v_quantization=mode)
        sparse = risa.sparse_int8_attention(q, q, v, pattern, is_causal=True, v_quantization=mode)
        torch.testing.assert_close(out[:, :, :128], torch.zeros_like(out[:, :, :128]), atol=0.01, rtol=0)
        torch.testing.assert_close(sparse, out, atol=0.05, rtol=0.01)


def test_key_bias_large_tile_and_lse(risa):
    """reference tests/cuda/test_risa_attention.py:167-179."""
    q = torch.zeros(1, 2, 17, 128, device="cuda", dtype=torch.float16)
    k = torch.zeros(1, 1, 1153, 128, device="cuda", dtype=torch.float16)
    v = torch.ones_like(k) * 3
    mask = torch.linspace(-3, 0, 1153, device="cuda")[None, None, None, :]
    for mode in ("midpoint_affine", "absmax"):
        packed = risa.prequantize_int8_attention(q, k, v, attn_mask=mask, return_lse=True, v_quantization=mode)
        assert packed.cta_k == 128
        out, lse = risa.int8_attention_from_prequantized(packed, return_lse=True)
        torch.testing.assert_close(out, torch.full_like(out, 3), atol=0.03, rtol=0)
        torch.testing.assert_close(lse, mask.logsumexp(-1).expand(1, 2, 17), atol=0.01, rtol=0)


@pytest.mark.parametrize("dim,heads,q_len,k_len", [(128, 40, 1024, 1500), (128, 2, 200, 1500), (64, 48, 900, 700),
                                                   (256, 4, 300, 1500), (64, 2, 100, 330)])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("kind", ["padding", "bias"])
def test_key_only_masks_with_untouched_tiles(risa, dim, heads, q_len, k_len, causal, kind):
    """A key-only mask that leaves whole key tiles untouched (an additive row of zeros there: the
    kernels skip the addition for such a tile) beside tiles with hidden keys, with finite terms,
    and a hidden tail; 32-query and 16-query kernels, 64- and 128-key tiles, every head dim."""
    q = seeded((1, heads, q_len, dim), torch.bfloat16, 41, scale=1.5)
    k = seeded((1, 2, k_len, dim), torch.bfloat16, 42, scale=1.5)
    v = seeded((1, 2, k_len, dim), torch.bfloat16, 43, offset=0.5)
    if kind == "padding":
        mask = torch.ones(1, 1, 1, k_len, dtype=torch.bool, device="cuda")
        mask[..., k_len - k_len // 7:] = False
        mask[..., 70:75] = False
    else:
        mask = torch.zeros(1, 1, 1, k_len, device="cuda")
        mask[..., 130:190] = seeded((60,), torch.float32, 44)
        mask[..., 3] = -0.0
        mask[..., k_len - 77:] = float("-inf")
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, return_lse=True)
    checked = slice(heads - 1, heads)
    prepared = oracle_prequantize(q[:, checked], k[:, 1:], v[:, 1:], attn_mask=mask, is_causal=causal, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[:, checked]), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse[:, checked]), expected_lse) < TOLERANCE


def test_lse_restores_shifted_keys_and_empty_rows(risa):
    """reference tests/cuda/test_risa_attention.py:181-193."""
    from risaattention_amd.policy import apply_score_mask

    torch.manual_seed(29)
    q = torch.randn(1, 2, 19, 128, device="cuda", dtype=torch.float16)
    k = torch.randn(1, 1, 257, 128, device="cuda", dtype=torch.float16) * 0.1 + 4
    v = torch.randn_like(k)
    mask = torch.ones(19, 257, dtype=torch.bool, device="cuda")
    mask[0] = False
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=True, return_lse=True)
    scores = q.float() @ k.float().transpose(-1, -2) / 128**0.5
    expected = apply_score_mask(scores, mask, True, 0).logsumexp(-1)
    assert torch.isneginf(lse[:, :, 0]).all()
    assert out[:, :, 0].count_nonzero().item() == 0
    torch.testing.assert_close(lse[:, :, 1:], expected[:, :, 1:], atol=0.15, rtol=0.02)


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("k_len", [264, 263, 1284])
@pytest.mark.parametrize("key_only", [False, True])
def test_mask_types_vector_and_scalar_loads(risa, mask_dtype, k_len, key_only):
    """Every mask element type through both load paths of the kernel: rows of 264 and
    1284 keys are aligned for one load per four keys, rows of 263 keys are not; a
    key-only mask over more than 1024 keys selects the 128-key tile."""
    dim, q_len = 128, 70
    q = seeded((1, 2, q_len, dim), torch.bfloat16, 41)
    k = seeded((1, 2, k_len, dim), torch.bfloat16, 42)
    v = seeded((1, 2, k_len, dim), torch.bfloat16, 43)
    generator = torch.Generator(device="cpu").manual_seed(44)
    shape = (1, 1, 1 if key_only else q_len, k_len)
    if mask_dtype == torch.bool:
        mask = torch.rand(shape, generator=generator) > 0.3
        mask[..., -5:] = False
        if not key_only:
            mask[:, :, 3] = False  # a fully hidden row
    else:
        mask = torch.randn(shape, generator=generator).to(mask_dtype)
        mask[..., 5::11] = float("-inf")
    mask = mask.cuda()
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, return_lse=True)
    prepared = oracle_prequantize(q, k, v, attn_mask=mask, return_lse=True)
    assert prepared.cta_k == (128 if key_only and k_len > 1024 else 64)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse), expected_lse) < TOLERANCE


def test_causal_launch_order_covers_every_block(risa):
    """Causal launches walk the query blocks longest first; every block of every head
    and batch entry must still be written exactly as the dense causal oracle says."""
    q = seeded((2, 3, 700, 64), torch.float16, 51)
    k = seeded((2, 3, 700, 64), torch.float16, 52)
    v = seeded((2, 3, 700, 64), torch.float16, 53)
    out = risa.int8_attention(q, k, v, is_causal=True)
    prepared = oracle_prequantize(q, k, v, is_causal=True)
    expected, _, _ = oracle_pipeline.attend(prepared)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("k_len", [263, 1153])
def test_both_unmasked_kernels_match_oracle(risa, dim, k_len):
    """Unmasked launches with no more workgroups than the GPU has compute units run
    sixteen queries per wavefront, larger ones thirty-two.  264 query heads go through
    the second kernel, a slice of 66 of them through the first; both must agree with
    the oracle on that slice and with each other everywhere."""
    heads, kv_heads, q_len = 264, 4, 40
    group = heads // kv_heads
    assert heads > torch.cuda.get_device_properties(0).multi_processor_count >= group
    q = seeded((1, heads, q_len, dim), torch.bfloat16, 61)
    k = seeded((1, kv_heads, k_len, dim), torch.bfloat16, 62)
    v = seeded((1, kv_heads, k_len, dim), torch.bfloat16, 63, offset=0.5)
    wide, wide_lse = risa.int8_attention(q, k, v, return_lse=True)
    for kv in range(kv_heads):
        rows = slice(kv * group, (kv + 1) * group)
        narrow, narrow_lse = risa.int8_attention(q[:, rows], k[:, kv:kv + 1], v[:, kv:kv + 1], return_lse=True)
        assert relative_l2(to_numpy(narrow), to_numpy(wide[:, rows])) < 1e-4
        assert relative_l2(to_numpy(narrow_lse), to_numpy(wide_lse[:, rows])) < 1e-6
    prepared = oracle_prequantize(q[:, :group], k[:, :1], v[:, :1], return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(wide[:, :group]), expected) < TOLERANCE
    assert relative_l2(to_numpy(wide_lse[:, :group]), expected_lse) < TOLERANCE


@pytest.mark.parametrize("length,heads", [(4096, 16), (4422, 30), (4608, 32)])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_lse_request_does_not_change_outputs(risa, length, heads, mode):
    """reference tests/cuda/test_probability_mass.py:158-170 (image-sized query tiles):
    the same packed tensors give bit-identical outputs with and without the LSE."""
    torch.manual_seed(59)
    q = torch.randn(1, heads, length, 128, device="cuda", dtype=torch.bfloat16)
    k, v = [torch.randn(1, 2, length, 128, device="cuda", dtype=q.dtype) for _ in range(2)]
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode, return_lse=True)
    plain = risa.int8_attention_from_prequantized(packed)
    with_lse, lse = risa.int8_attention_from_prequantized(packed, return_lse=True)
    assert torch.equal(plain, with_lse)
    assert torch.isfinite(lse).all()
    assert torch.equal(plain, risa.int8_attention(q, k, v, v_quantization=mode))


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_staged_mask_tiles_match_oracle(risa, mask_dtype, dim, causal):
    """Query-dependent masks whose rows are 16-byte aligned are copied to LDS tile by
    tile.  330 queries (a ragged last query block) x 400 keys (a ragged last key tile),
    two batch entries with a mask per batch entry and head; a mask view with an
    unaligned base takes the other load path and must give the same answer."""
    q_len, k_len = 330, 400
    q = seeded((2, 2, q_len, dim), torch.float16, 71)
    k = seeded((2, 1, k_len, dim), torch.float16, 72)
    v = seeded((2, 1, k_len, dim), torch.float16, 73)
    generator = torch.Generator(device="cpu").manual_seed(74)
    if mask_dtype == torch.bool:
        mask = torch.rand((2, 2, q_len, k_len), generator=generator) > 0.4
        mask[0, 1, 129] = False  # a fully hidden row
    else:
        mask = torch.randn((2, 2, q_len, k_len), generator=generator).to(mask_dtype)
        mask[..., 3::7] = float("-inf")
    mask = mask.cuda()
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, return_lse=True)
    prepared = oracle_prequantize(q, k, v, attn_mask=mask, is_causal=causal, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE
    finite = np.isfinite(expected_lse)
    assert np.array_equal(np.isfinite(to_numpy(lse)), finite)
    assert relative_l2(to_numpy(lse)[finite], expected_lse[finite]) < TOLERANCE
    # same values behind a base address that is not 16-byte aligned
    storage = torch.empty(mask.numel() + 16, dtype=mask.dtype, device="cuda")
    shifted = storage[4:4 + mask.numel()].view_as(mask).copy_(mask)
    assert shifted.data_ptr() % 16 != 0 or mask.element_size() == 4
    out_shifted, lse_shifted = risa.int8_attention(q, k, v, attn_mask=shifted, is_causal=causal, return_lse=True)
    assert torch.equal(out_shifted, out)
    assert torch.equal(lse_shifted, lse)


@pytest.mark.parametrize("heads", [4, 80, 200])
@pytest.mark.parametrize("dim,k_len", [(64, 500), (128, 500), (128, 1400), (256, 444), (128, 1100), (64, 180)])
def test_small_launches_match_oracle(risa, heads, dim, k_len):
    """Unmasked launches below one workgroup per compute unit: 4 heads run 32 queries per
    workgroup and 80 heads 64, both with four or more key tiles split over two sets of
    wavefronts (8, 22 and 8 tiles with a ragged last tile; 7 and 9 tiles: the second set
    walks one tile less; 3 tiles are not split); 200 heads run 128 queries per workgroup
    without the split."""
    assert 128 < torch.cuda.get_device_properties(0).multi_processor_count <= 256
    q = seeded((1, heads, 100, dim), torch.bfloat16, 91)
    k = seeded((1, 4, k_len, dim), torch.bfloat16, 92)
    v = seeded((1, 4, k_len, dim), torch.bfloat16, 93, offset=-0.5)
    out, lse = risa.int8_attention(q, k, v, return_lse=True)
    keep = slice(0, heads, max(1, heads // 8))  # the oracle checks every eighth head
    group = heads // 4
    kv_of = [h // group for h in range(heads)][keep]
    picked_k = k[:, kv_of]
    picked_v = v[:, kv_of]
    prepared = oracle_prequantize(q[:, keep], picked_k, picked_v, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[:, keep]), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse[:, keep]), expected_lse) < TOLERANCE


def test_concurrent_host_threads_on_their_own_streams(risa):
    """The C ABI keeps no shared mutable state (per-thread error text and device caches):
    two host threads, each on its own stream and with its own shapes, get the bits a
    single thread gets.  ctypes releases the interpreter lock during the native calls."""
    import threading

    problems = []
    for index, (heads, q_len, k_len, dim) in enumerate([(4, 300, 1300, 128), (6, 129, 700, 64)]):
        q = seeded((1, heads, q_len, dim), torch.bfloat16, 400 + 3 * index)
        k = seeded((1, 2, k_len, dim), torch.bfloat16, 401 + 3 * index)
        v = seeded((1, 2, k_len, dim), torch.bfloat16, 402 + 3 * index, offset=0.5)
        causal = bool(index)
        expected = risa.int8_attention(q, k, v, is_causal=causal, v_quantization="midpoint_affine")
        problems.append((q, k, v, causal, expected))
    torch.cuda.synchronize()
    failures = []

    def worker(problem):
        q, k, v, causal, expected = problem
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(25):
                    out = risa.int8_attention(q, k, v, is_causal=causal, v_quantization="midpoint_affine")
                    if not torch.equal(out, expected):
                        failures.append("outputs differ")
                        break
            stream.synchronize()
        except Exception as error:  # noqa: BLE001 - reported by the main thread
            failures.append(repr(error))

    threads = [threading.Thread(target=worker, args=(problem,)) for problem in problems]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join(timeout=100)
    assert not any(thread.is_alive() for thread in threads)
    assert not failures, failures


def expected_lane_words(mask, q_len, k_len):
    """Lane words of a [planes, q_len, k_len] boolean array, element by element: word
    (plane, w, t, 16*rb + i) has bit l set when query 32*w + l % 32 may attend to key
    64*t + 32*rb + 8*(i // 4) + 4*(l // 32) + i % 4."""
    planes = mask.shape[0]
    query_waves = -(-q_len // 128) * 4
    key_tiles = -(-k_len // 64)
    padded = np.zeros((planes, query_waves * 32, key_tiles * 64), dtype=bool)
    padded[:, :q_len, :k_len] = mask
    lane = np.arange(64)
    slot = np.arange(32)
    rows = lane % 32                                           # [64]
    keys = (slot[:, None] // 16) * 32 + ((slot[:, None] % 16) // 4) * 8 + (lane[None, :] // 32) * 4 + slot[:, None] % 4
    blocks = padded.reshape(planes, query_waves, 32, key_tiles, 64)
    bits = blocks[:, :, rows[None, :], :, keys]                # [slot, lane, planes, waves, tiles]
    bits = np.moveaxis(bits, (0, 1), (3, 4))                   # [planes, waves, tiles, slot, lane]
    weights = (np.uint64(1) << lane.astype(np.uint64))
    return (bits.astype(np.uint64) * weights).sum(-1, dtype=np.uint64)


@pytest.mark.parametrize("q_len,k_len,aligned", [(300, 704, True), (300, 700, False), (129, 263, False), (64, 64, True)])
def test_lane_words_of_a_boolean_mask(risa, q_len, k_len, aligned):
    """The conversion a boolean mask shared by several heads goes through, bit for bit."""
    from risaattention_amd.key_mask import prepare_mask_lanes

    generator = torch.Generator().manual_seed(q_len + k_len)
    planes = torch.rand((2, 1, q_len, k_len), generator=generator) > 0.5
    planes[1, 0, 5] = False
    mask = planes.cuda()
    assert (mask.stride(2) % 16 == 0) == aligned  # rows the conversion can read 16 bytes at a time
    heads = 264  # more than 256 workgroups of 128 queries: smaller launches read the mask themselves
    words, stride_b, stride_h = prepare_mask_lanes(mask.expand(2, heads, q_len, k_len), 64, 128)
    expected = expected_lane_words(planes[:, 0].numpy(), q_len, k_len)
    assert stride_h == 0 and stride_b == expected[0].size
    buffer = words.cpu().numpy().view(np.uint64)
    assert np.array_equal(buffer[: expected.size].reshape(expected.shape), expected)
    # behind the words: per (plane, block of 32 queries, tile) 1 = every bit set, 2 = none, 0 = neither
    classes = buffer[expected.size:].view(np.int32)[: expected.size // 32].reshape(expected.shape[:3])
    every = (expected == np.uint64(0xFFFFFFFFFFFFFFFF)).all(-1)
    none = (expected == 0).all(-1)
    assert np.array_equal(classes, np.where(every, 1, np.where(none, 2, 0)))
    # not for small launches, a plane per head, other tile sizes, head dim 256 or other dtypes
    assert prepare_mask_lanes(mask.expand(2, 8, q_len, k_len), 64, 128) is None
    assert prepare_mask_lanes(mask.expand(2, heads, q_len, k_len).contiguous(), 64, 128) is None
    assert prepare_mask_lanes(mask.expand(2, heads, q_len, k_len), 128, 128) is None
    assert prepare_mask_lanes(mask.expand(2, heads, q_len, k_len), 64, 256) is None
    assert prepare_mask_lanes(mask.expand(2, heads, q_len, k_len).float(), 64, 128) is None


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("q_len,k_len", [(330, 400), (257, 263)])
def test_shared_boolean_mask_equals_the_mask_per_head(risa, dim, causal, q_len, k_len):
    """A boolean mask that broadcasts over heads is applied from lane words; the same mask
    materialised per head is read element by element.  Same decisions, same arithmetic:
    outputs and LSE are equal bit for bit, and both match the oracle.  48 heads x 2 batch
    entries x 3 query blocks: launches of at most 256 workgroups read the mask themselves."""
    heads = 48
    q = seeded((2, heads, q_len, dim), torch.float16, 171)
    k = seeded((2, 2, k_len, dim), torch.float16, 172)
    v = seeded((2, 2, k_len, dim), torch.float16, 173)
    generator = torch.Generator().manual_seed(174)
    shared = (torch.rand((2, 1, q_len, k_len), generator=generator) > 0.4).cuda()
    shared[0, 0, 129] = False  # a fully hidden row
    shared[1, 0, :, 64:128] = False  # a fully hidden key tile
    per_head = shared.expand(2, heads, q_len, k_len).contiguous()
    out, lse = risa.int8_attention(q, k, v, attn_mask=shared, is_causal=causal, return_lse=True)
    out_heads, lse_heads = risa.int8_attention(q, k, v, attn_mask=per_head, is_causal=causal, return_lse=True)
    assert torch.equal(out, out_heads)
    assert torch.equal(lse, lse_heads)
    # the same mask as a window of a wider tensor: rows 13 elements apart from a multiple of
    # 16, base address odd (the conversion then reads it element by element)
    wider = torch.zeros((2, 1, q_len, k_len + 13), dtype=torch.bool, device="cuda")
    window = wider[..., 5:5 + k_len]
    window.copy_(shared)
    assert window.data_ptr() % 2 == 1 and not window.is_contiguous()
    out_window, lse_window = risa.int8_attention(q, k, v, attn_mask=window, is_causal=causal, return_lse=True)
    assert torch.equal(out_window, out)
    assert torch.equal(lse_window, lse)
    assert torch.equal(out, risa.int8_attention(q, k, v, attn_mask=shared, is_causal=causal))  # the one-call route
    prepared = oracle_prequantize(q[:1, :2], k[:1, :1], v[:1, :1], attn_mask=shared[:1], is_causal=causal,
                                  return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[:1, :2]), expected) < TOLERANCE
    finite = np.isfinite(expected_lse)
    assert np.array_equal(np.isfinite(to_numpy(lse[:1, :2])), finite)
    assert relative_l2(to_numpy(lse[:1, :2])[finite], expected_lse[finite]) < TOLERANCE


@pytest.mark.parametrize("dim", [128, 256])
def test_shared_boolean_mask_in_the_sparse_path(risa, dim):
    """Pattern construction (capturing kernel) and reuse (tile lists) under a query-dependent
    boolean mask: shared over heads (lane words up to head dim 128) they give what they give
    with the mask read per head, and both follow the oracle walking the same lists."""
    heads, q_len, k_len = 72, 512, 1500  # 288 workgroups: beyond the small-launch kernel
    q = seeded((1, heads, q_len, dim), torch.bfloat16, 181, scale=2.0)
    k = seeded((1, 2, k_len, dim), torch.bfloat16, 182, scale=2.0)
    v = seeded((1, 2, k_len, dim), torch.bfloat16, 183)
    generator = torch.Generator().manual_seed(184)
    shared = (torch.rand((1, 1, q_len, k_len), generator=generator) > 0.3).cuda()
    per_head = shared.expand(1, heads, q_len, k_len).contiguous()
    out, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.9, attn_mask=shared)
    out_heads, pattern_heads = risa.construct_sparse_int8_attention(q, k, v, theta=0.9, attn_mask=per_head)
    assert torch.equal(out, out_heads)
    assert torch.equal(pattern.row_offsets, pattern_heads.row_offsets)
    assert torch.equal(pattern.block_indices, pattern_heads.block_indices)
    assert 0.05 < pattern.sparsity < 0.95
    reuse = risa.sparse_int8_attention(q, k, v, pattern, attn_mask=shared)
    reuse_heads = risa.sparse_int8_attention(q, k, v, pattern_heads, attn_mask=per_head)
    assert torch.equal(reuse, reuse_heads)
    # the oracle on the first four query heads (they share the first KV head): same codes and
    # scales as in the whole problem, and the first 16 rows of the tile lists
    prepared = oracle_prequantize(q[:, :4], k[:, :1], v[:, :1], attn_mask=shared)
    expected, _, _ = oracle_pipeline.attend(prepared)
    assert relative_l2(to_numpy(out[:, :4]), expected) < TOLERANCE
    rows = 4 * (q_len // 128)
    row_offsets = pattern.row_offsets.cpu().numpy()[:rows + 1]
    lists = (row_offsets, pattern.block_indices.cpu().numpy()[:row_offsets[-1]])
    expected_reuse, _, _ = oracle_pipeline.attend(prepared, pattern=lists)
    assert relative_l2(to_numpy(reuse[:, :4]), expected_reuse) < TOLERANCE


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("heads,q_len", [(3, 77), (130, 200)])
def test_output_rows_in_both_layouts_and_misaligned_outputs(risa, dim, heads, q_len):
    """Output rows are written 16 bytes per lane, whole rows at a time (both kernels:
    the few-workgroup launch and the large one).  The sequence-major layout must hold the
    same values as the head-major one, rows past a ragged query length must stay untouched,
    and an output that is not 16-byte aligned is refused instead of written."""
    from risaattention_amd.attend import launch_attention

    q = seeded((2, heads, q_len, dim), torch.bfloat16, 71)
    k = seeded((2, 1, 300, dim), torch.bfloat16, 72)
    v = seeded((2, 1, 300, dim), torch.bfloat16, 73, offset=0.25)
    packed = risa.prequantize_int8_attention(q, k, v)
    head_major = risa.int8_attention_from_prequantized(packed)
    sequence_major = risa.int8_attention_from_prequantized(packed, output_layout="nhd")
    assert sequence_major.transpose(1, 2).is_contiguous()
    assert torch.equal(head_major, sequence_major)
    expected, _, _ = oracle_pipeline.attend(oracle_prequantize(q[:1, :2], k[:1], v[:1]))
    assert relative_l2(to_numpy(head_major[:1, :2]), expected) < TOLERANCE

    # written through the wrapper into a buffer with a sentinel tail: nothing lands past the
    # last row, and the same buffer shifted by 8 bytes is refused
    shape = tuple(head_major.shape[:3]) + (packed.q.shape[-1],)
    count = math.prod(shape)
    buffer = torch.full((count + 64,), 7.0, dtype=torch.bfloat16, device="cuda")
    arguments = dict(q_codes=packed.q, k_codes=packed.k, v_codes=packed.v, q_scale=packed.q_scale,
                     k_scale=packed.k_scale, v_scale=packed.v_scale, v_center=packed.v_center, v_tile_sum=None,
                     cta_k=packed.cta_k, sm_scale=packed.attention_scale)
    launch_attention(output=buffer[:count].view(shape), **arguments)
    assert torch.equal(buffer[:count].view(shape)[..., : head_major.shape[-1]], head_major)
    assert torch.equal(buffer[count:], torch.full_like(buffer[count:], 7.0))
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        launch_attention(output=buffer[4 : count + 4].view(shape), **arguments)


@pytest.mark.parametrize("dim", [64, 128])
@pytest.mark.parametrize("pattern", ["block_diagonal", "lower_triangle", "all_true"])
def test_structured_shared_masks_skip_and_pass_whole_tiles(risa, dim, pattern):
    """A boolean mask that many heads share is classified per (32 queries, 64 keys): tiles
    without a visible key are skipped and tiles without a hidden key take no select.  Both
    must be invisible in the results: equal to the same mask given per head (which reads
    the mask elements) bit for bit, and to the oracle on a slice."""
    q_len, k_len, heads = 640, 700, 72
    q = seeded((1, heads, q_len, dim), torch.bfloat16, 91)
    k = seeded((1, 1, k_len, dim), torch.bfloat16, 92)
    v = seeded((1, 1, k_len, dim), torch.bfloat16, 93, offset=0.5)
    rows = torch.arange(q_len)[:, None]
    keys = torch.arange(k_len)[None, :]
    if pattern == "block_diagonal":
        shared = (rows // 200) == (keys // 220)          # documents of unequal lengths
    elif pattern == "lower_triangle":
        shared = keys <= rows + 37
    else:
        shared = torch.ones(q_len, k_len, dtype=torch.bool)
        shared[3] = False                                 # one row without any key
    shared = shared.cuda()[None, None]
    per_head = shared.expand(1, heads, q_len, k_len).contiguous()
    from risaattention_amd.key_mask import prepare_mask_lanes
    assert prepare_mask_lanes(shared.expand(1, heads, q_len, k_len), 64, dim) is not None
    out, lse = risa.int8_attention(q, k, v, attn_mask=shared, return_lse=True)
    out_heads, lse_heads = risa.int8_attention(q, k, v, attn_mask=per_head, return_lse=True)
    assert torch.equal(out, out_heads)
    assert torch.equal(lse, lse_heads)
    checked = 2
    prepared = oracle_prequantize(q[:, :checked], k, v, attn_mask=shared, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[:, :checked]), expected) < TOLERANCE
    assert relative_l2(to_numpy(lse[:, :checked]), expected_lse) < TOLERANCE
