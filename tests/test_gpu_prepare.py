"""Bit-exact parity of the HIP preparation kernels with the oracle (through the C ABI)."""

import numpy as np
import pytest
import torch

from oracle import prepare as oracle_prepare
from tests.helpers import oracle_prequantize, seeded, to_numpy

pytestmark = pytest.mark.gpu

CASES = [
    # (dtype, head_dim, Lq, Lk, Hq, Hkv, mode, key offset)
    (torch.bfloat16, 128, 257, 1153, 4, 2, "absmax", 0.0),
    (torch.float16, 128, 137, 263, 2, 1, "midpoint_affine", 0.0),
    (torch.float32, 128, 64, 200, 2, 2, "midpoint_affine", 0.0),
    (torch.bfloat16, 64, 193, 700, 2, 1, "absmax", 0.0),
    (torch.float16, 64, 33, 129, 2, 2, "midpoint_affine", 0.0),
    (torch.bfloat16, 256, 130, 1100, 2, 1, "midpoint_affine", 0.0),
    (torch.float16, 256, 40, 250, 2, 2, "absmax", 0.0),
    (torch.bfloat16, 80, 100, 300, 2, 2, "absmax", 0.0),  # padded head dim
    (torch.float16, 128, 19, 257, 2, 1, "absmax", 4.0),  # anchor fires
    (torch.bfloat16, 128, 300, 2049, 4, 1, "midpoint_affine", 0.0),
    # beyond 4096 keys the residual-corrected centre comes from the two-kernel path
    (torch.bfloat16, 128, 40, 4611, 2, 2, "midpoint_affine", 0.0),
    (torch.float16, 64, 40, 9000, 2, 1, "midpoint_affine", 0.0),
    (torch.float32, 256, 40, 4200, 1, 1, "midpoint_affine", 0.0),
    # long absmax self-attention shapes take at most 64 partial V ranges and no parameter launch
    (torch.bfloat16, 128, 5000, 5000, 2, 1, "absmax", 0.0),
    (torch.float16, 64, 9100, 9100, 1, 1, "absmax", 0.0),
]


@pytest.mark.parametrize("dtype,dim,q_len,k_len,q_heads,kv_heads,mode,offset", CASES)
def test_prepared_tensors_match_oracle_bit_for_bit(risa, dtype, dim, q_len, k_len, q_heads, kv_heads, mode, offset):
    from risaattention_amd.layout import unpack_values

    q = seeded((2, q_heads, q_len, dim), dtype, 1)
    k = seeded((2, kv_heads, k_len, dim), dtype, 2, offset=offset, scale=0.1 if offset else 1.0)
    v = seeded((2, kv_heads, k_len, dim), dtype, 3, offset=1.5)
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode, return_lse=True)
    expected = oracle_prequantize(q, k, v, v_quantization=mode, return_lse=True)
    assert packed.cta_k == expected.cta_k
    if offset:
        assert (expected.anchor >= 0).all(), "test input should trigger the anchor"
    np.testing.assert_array_equal(packed.q.cpu().numpy(), expected.q)
    np.testing.assert_array_equal(packed.q_scale.cpu().numpy(), expected.q_scale)
    np.testing.assert_array_equal(packed.k.cpu().numpy(), expected.k)
    np.testing.assert_array_equal(packed.k_scale.cpu().numpy(), expected.k_scale)
    np.testing.assert_array_equal(unpack_values(packed.v).cpu().numpy(), expected.v)
    np.testing.assert_array_equal(packed.v_scale.cpu().numpy(), expected.v_scale)
    np.testing.assert_array_equal(packed.v_center.cpu().numpy(), expected.v_center)
    sums = oracle_prepare.value_tile_sums(expected.v, expected.cta_k)
    rows = expected.v.shape[0]
    kernel_dim = packed.q.shape[-1]
    got = packed.v_tile_sum.cpu().numpy().transpose(0, 2, 1).reshape(rows, -1)
    np.testing.assert_array_equal(got, sums * 128 + 0x4B400000)
    np.testing.assert_array_equal(to_numpy(packed.lse_shift), expected.lse_shift)
    assert kernel_dim in (64, 128, 256)


@pytest.mark.parametrize("dim,k_len,mode", [(128, 1300, "absmax"), (64, 700, "midpoint_affine"),
                                            (256, 1100, "midpoint_affine"), (128, 200, "absmax")])
@pytest.mark.parametrize("shifted", [False, True])
def test_outlier_channels_bit_for_bit(risa, dim, k_len, mode, shifted):
    """One channel in a hundred scaled by 20 (the masked benchmark configuration's inputs): the
    case the rotation spreads over the block and, with a common key offset on top, the anchor
    removes.  Codes, scales, centres, anchors and the LSE shift equal the oracle's bit for bit."""
    from risaattention_amd.layout import unpack_values

    generator = torch.Generator().manual_seed(11)
    q = torch.randn(2, 4, 150, dim, generator=generator)
    k = torch.randn(2, 2, k_len, dim, generator=generator)
    v = torch.randn(2, 2, k_len, dim, generator=generator)
    hot = torch.randperm(dim, generator=generator)[: max(1, dim // 100)]
    for tensor in (q, k, v):
        tensor[..., hot] *= 20.0
    if shifted:
        k = k * 0.1 + 5.0 * torch.randn(1, 1, 1, dim, generator=generator)
    q, k, v = (t.to(torch.bfloat16).cuda() for t in (q, k, v))
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode, return_lse=True)
    expected = oracle_prequantize(q, k, v, v_quantization=mode, return_lse=True)
    if shifted:
        assert (expected.anchor >= 0).all(), "a common key offset should trigger the anchor"
    np.testing.assert_array_equal(packed.q.cpu().numpy(), expected.q)
    np.testing.assert_array_equal(packed.q_scale.cpu().numpy(), expected.q_scale)
    np.testing.assert_array_equal(packed.k.cpu().numpy(), expected.k)
    np.testing.assert_array_equal(packed.k_scale.cpu().numpy(), expected.k_scale)
    np.testing.assert_array_equal(unpack_values(packed.v).cpu().numpy(), expected.v)
    np.testing.assert_array_equal(packed.v_scale.cpu().numpy(), expected.v_scale)
    np.testing.assert_array_equal(packed.v_center.cpu().numpy(), expected.v_center)
    np.testing.assert_array_equal(to_numpy(packed.lse_shift), expected.lse_shift)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["hnd", "nhd", "interleaved"])
@pytest.mark.parametrize("length", [1025, 2048, 2049, 4097])
def test_absmax_values_known_answer(risa, dtype, layout, length):
    """Power-of-two scales make codes and scales exact (reference
    tests/cuda/test_value_quantization.py:18-52, modulo the packed order)."""
    from risaattention_amd.layout import unpack_values

    batch, heads, channels = 2, 3, 128
    tokens = torch.arange(length, device="cuda")[None, None, :, None]
    head_offsets = torch.arange(batch * heads, device="cuda").reshape(batch, heads, 1, 1)
    codes = ((tokens + head_offsets) % 255 - 127).expand(batch, heads, length, channels)
    scales = 2.0 ** ((torch.arange(channels, device="cuda") % 4).float() - 2)
    v = (codes * scales).to(dtype)
    if layout == "nhd":
        v = v.transpose(1, 2).contiguous().transpose(1, 2)
    elif layout == "interleaved":
        storage = torch.empty(batch, length, 3, heads, channels, device="cuda", dtype=dtype)
        v = storage[:, :, 1].transpose(1, 2).copy_(v)
    q = torch.zeros(batch, heads * 2, 3, channels, device="cuda", dtype=dtype)
    k = torch.zeros_like(v)
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization="absmax")
    padded = packed.v.shape[-1]
    expected = torch.zeros(batch, heads, channels, padded, device="cuda", dtype=torch.int8)
    expected[..., :length] = codes.transpose(2, 3).to(torch.int8)
    logical = unpack_values(packed.v).reshape(batch, heads, channels, padded)
    assert torch.equal(logical, expected)
    assert torch.equal(packed.v_scale.reshape(batch, heads, channels), scales.expand(batch, heads, channels))
    assert torch.count_nonzero(packed.v_center) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_lse_shift_closed_form(risa, dtype, dim):
    """reference tests/cuda/test_lse_correction.py:9-31 through the C ABI."""
    from risaattention_amd import native

    torch.manual_seed(35)
    q = torch.randn(2, 17, 4, dim, device="cuda", dtype=dtype).transpose(1, 2)
    k = torch.randn(2, 9, 2, dim, device="cuda", dtype=dtype).transpose(1, 2)
    anchors = torch.tensor([[-1, 0], [3, 2]], device="cuda", dtype=torch.int32)
    out = torch.empty(2, 4, 17, device="cuda")
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    native.check(
        native.library().risa_lse_shift(
            q.data_ptr(), k.data_ptr(), anchors.data_ptr(), out.data_ptr(), 2, 4, 2, 17, dim,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            dim**-0.5, code, torch.cuda.current_stream().cuda_stream,
        )
    )
    selected = k.gather(2, anchors.clamp_min(0).long()[..., None, None].expand(2, 2, 1, dim))
    selected = selected.float() * (anchors >= 0)[..., None, None]
    reference = (q.float() * selected.repeat_interleave(2, 1)).sum(-1) * dim**-0.5
    torch.testing.assert_close(out, reference, rtol=2e-5, atol=5e-6)
    assert torch.count_nonzero(out[0, :2]) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["hnd", "nhd", "interleaved"])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_fused_permutation_matches_materialized_gather(risa, dtype, layout, mode):
    """reference tests/cuda/test_value_quantization.py:55-72, extended to K, the anchor,
    both V modes and the accumulator seeds: reading through the permutation inside
    the quantisation kernels gives the tensors of an eager gather, bit for bit."""
    torch.manual_seed(5)
    q = torch.randn(1, 4, 17, 128, device="cuda", dtype=dtype)
    k = torch.randn(1, 2, 2049, 128, device="cuda", dtype=dtype) * 0.1 + 3.0  # the anchor fires
    v = torch.randn(1, 2, 2049, 128, device="cuda", dtype=dtype) + 1.5
    if layout == "nhd":
        v = v.transpose(1, 2).contiguous().transpose(1, 2)
        k = k.transpose(1, 2).contiguous().transpose(1, 2)
    elif layout == "interleaved":
        storage = torch.empty(1, 2049, 3, 2, 128, device="cuda", dtype=dtype)
        v = storage[:, :, 1].transpose(1, 2).copy_(v)
    indices = torch.stack([torch.randperm(2049, device="cuda") for _ in range(2)])[None]
    permutation = risa.prepare_kv_permutation(indices)
    fused = risa.prequantize_int8_attention(q, k, v, kv_permutation=permutation, fuse_gather=True,
                                            v_quantization=mode)
    eager = risa.prequantize_int8_attention(q, k, v, kv_permutation=permutation, fuse_gather=False,
                                            v_quantization=mode)
    assert fused.kv_permuted and eager.kv_permuted
    for attribute in ("q", "q_scale", "k", "k_scale", "v", "v_scale", "v_center", "v_tile_sum"):
        assert torch.equal(getattr(fused, attribute), getattr(eager, attribute)), attribute
    # and the eager route is the plain path on gathered tensors
    index = indices[..., None].expand_as(k)
    plain = risa.prequantize_int8_attention(q, k.gather(2, index), v.gather(2, index), v_quantization=mode)
    assert torch.equal(plain.k, fused.k) and torch.equal(plain.v, fused.v)
    # the oracle on the materialised gather pins the fused path outside the library
    from risaattention_amd.layout import unpack_values

    expected = oracle_prequantize(q, k.gather(2, index), v.gather(2, index), v_quantization=mode)
    assert (expected.anchor >= 0).all()
    np.testing.assert_array_equal(fused.k.cpu().numpy(), expected.k)
    np.testing.assert_array_equal(fused.k_scale.cpu().numpy(), expected.k_scale)
    np.testing.assert_array_equal(unpack_values(fused.v).cpu().numpy(), expected.v)
    np.testing.assert_array_equal(fused.v_scale.cpu().numpy(), expected.v_scale)
    np.testing.assert_array_equal(fused.v_center.cpu().numpy(), expected.v_center)
    sums = oracle_prepare.value_tile_sums(expected.v, expected.cta_k)
    got = fused.v_tile_sum.cpu().numpy().transpose(0, 2, 1).reshape(expected.v.shape[0], -1)
    np.testing.assert_array_equal(got, sums * 128 + 0x4B400000)
    out = risa.int8_attention(q, k, v, kv_permutation=permutation, v_quantization=mode)
    expected = risa.int8_attention_from_prequantized(plain)
    assert torch.equal(out, expected)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["hnd", "token_major", "interleaved"])
@pytest.mark.parametrize("length", [1490, 14850])
def test_value_codes_do_not_depend_on_schedule(risa, dtype, layout, length):
    """reference tests/cuda/test_probability_mass.py:111-145: V codes and scales of one
    head are the same whether it is quantised alone or among 56 heads, for every memory
    layout; the two lengths take the one-pass and the chunked range reduction."""
    heads, channels = 56, 128
    q = torch.randn(1, heads, 17, channels, device="cuda", dtype=dtype)
    if layout == "hnd":
        k, v = [torch.randn(1, heads, length, channels, device="cuda", dtype=dtype) for _ in range(2)]
    elif layout == "token_major":
        k, v = [torch.randn(1, length, heads, channels, device="cuda", dtype=dtype).transpose(1, 2)
                for _ in range(2)]
    else:
        combined = torch.randn(1, length, 3, heads, channels, device="cuda", dtype=dtype)
        k, v = (combined[:, :, index].transpose(1, 2) for index in (1, 2))
    for mode in ("absmax", "midpoint_affine"):
        wide = risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
        narrow = risa.prequantize_int8_attention(q[:, :1], k[:, :1], v[:, :1], v_quantization=mode)
        padded = wide.v.shape[-1]
        assert torch.equal(wide.v.reshape(1, heads, channels, padded)[:, :1],
                           narrow.v.reshape(1, 1, channels, padded))
        assert torch.equal(wide.v_scale.reshape(1, heads, channels)[:, :1],
                           narrow.v_scale.reshape(1, 1, channels))
        assert torch.equal(wide.v_center.reshape(1, heads, channels)[:, :1],
                           narrow.v_center.reshape(1, 1, channels))
        assert torch.equal(wide.k[:, :1], narrow.k)
        assert torch.equal(wide.k_scale[:, :1], narrow.k_scale)


@pytest.mark.parametrize("permuted", [False, True])
@pytest.mark.parametrize("dtype,dim,length,mode", [
    (torch.bfloat16, 128, 1500, "absmax"),
    (torch.float16, 128, 6000, "midpoint_affine"),
    (torch.bfloat16, 64, 700, "midpoint_affine"),
    (torch.float32, 256, 4300, "absmax"),
])
def test_separate_entry_points_match_one_call_preparation(risa, dtype, dim, length, mode, permuted):
    """risa_quantize_qk + risa_quantize_v (one launch per kernel) against
    risa_sdpa_quantize (merged launches) on the same inputs, with and without a K/V
    permutation: every output bit-equal."""
    from risaattention_amd import native
    from risaattention_amd.policy import DTYPE_CODES

    q = seeded((2, 4, 333, dim), dtype, 81)
    k = seeded((2, 2, length, dim), dtype, 82, offset=3.0)
    v = seeded((2, 2, length, dim), dtype, 83, offset=-1.0)
    extra, order = {}, None
    if permuted:
        generator = torch.Generator(device="cpu").manual_seed(84)
        order = torch.stack([torch.randperm(length, generator=generator) for _ in range(4)])
        order = order.reshape(2, 2, length).to("cuda", torch.int32)
        extra = {"kv_permutation": risa.prepare_kv_permutation(order), "fuse_gather": True}
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode, **extra)
    lib = native.library()
    affine = int(mode == "midpoint_affine")
    q_codes, k_codes, v_codes = (torch.empty_like(t) for t in (packed.q, packed.k, packed.v))
    q_scale, k_scale, v_scale, v_center, tile_sum = (
        torch.empty_like(t) for t in (packed.q_scale, packed.k_scale, packed.v_scale, packed.v_center,
                                      packed.v_tile_sum))
    anchors = torch.empty(2, 2, dtype=torch.int32, device="cuda")
    workspace = torch.empty(max(1, lib.risa_quantize_v_workspace_bytes(2, 2, length, dim, affine)),
                            dtype=torch.uint8, device="cuda")
    stream = native.current_stream(q.device)
    code = DTYPE_CODES[dtype]
    native.check(lib.risa_quantize_qk(
        q.data_ptr(), q_codes.data_ptr(), q_scale.data_ptr(), k.data_ptr(), k_codes.data_ptr(),
        k_scale.data_ptr(), 2, 4, 333, 2, length, dim, packed.cta_k, *q.stride()[:3], *k.stride()[:3],
        code, anchors.data_ptr(), native.pointer(order), stream))
    native.check(lib.risa_quantize_v(
        v.data_ptr(), v_codes.data_ptr(), v_scale.data_ptr(), v_center.data_ptr(), tile_sum.data_ptr(),
        workspace.data_ptr(), workspace.numel(), 2, 2, length, dim, packed.v.shape[-1], packed.cta_k,
        *v.stride()[:3], code, affine, native.pointer(order), stream))
    for ours, theirs in ((q_codes, packed.q), (k_codes, packed.k), (v_codes, packed.v),
                         (q_scale, packed.q_scale), (k_scale, packed.k_scale), (v_scale, packed.v_scale),
                         (v_center, packed.v_center), (tile_sum, packed.v_tile_sum)):
        assert torch.equal(ours, theirs)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_infinite_inputs_bit_for_bit(risa, dtype, mode):
    """One infinite element in Q, K and V.  Its scale group's maximum is infinite, the
    reciprocal of the scale zero, every product 0 or NaN (inf * 0), and the saturating
    conversion of the reference turns NaN into code 0 (float_utils.cuh:23-31): the whole group
    gets zero codes and an infinite scale, everything else is untouched.  The add-a-constant
    conversion used here reads the low byte of the NaN that 0 * inf produces, which is zero."""
    from risaattention_amd.layout import unpack_values

    q = seeded((1, 2, 70, 128), dtype, 21)
    k = seeded((1, 1, 300, 128), dtype, 22)
    v = seeded((1, 1, 300, 128), dtype, 23)
    q[0, 0, 5, 7] = float("inf")
    k[0, 0, 130, 9] = float("-inf")
    v[0, 0, 17, 3] = float("inf")
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
    with np.errstate(all="ignore"):
        expected = oracle_prequantize(q, k, v, v_quantization=mode)
    assert np.isinf(expected.q_scale).sum() == 1 and np.isinf(expected.k_scale).sum() == 1
    np.testing.assert_array_equal(packed.q.cpu().numpy(), expected.q)
    np.testing.assert_array_equal(packed.q_scale.cpu().numpy(), expected.q_scale)
    np.testing.assert_array_equal(packed.k.cpu().numpy(), expected.k)
    np.testing.assert_array_equal(packed.k_scale.cpu().numpy(), expected.k_scale)
    np.testing.assert_array_equal(unpack_values(packed.v).cpu().numpy(), expected.v)
    np.testing.assert_array_equal(packed.v_scale.cpu().numpy(), expected.v_scale)
    np.testing.assert_array_equal(packed.v_center.cpu().numpy(), expected.v_center)  # NaN == NaN here
