"""GPU parity of capture, block mass, retained-mass selection, sparse reuse, key-mask tile
skipping, streams/graphs and full-size invariants (all through the C ABI)."""

from dataclasses import replace

import numpy as np
import pytest
import torch

from oracle import attention as oracle_attention
from oracle import pipeline as oracle_pipeline
from oracle import selection as oracle_selection
from tests.helpers import oracle_prequantize, relative_l2, seeded, to_numpy

pytestmark = pytest.mark.gpu


def block_structured(batch, q_heads, kv_heads, length, dim, groups, seed, dtype=torch.bfloat16):
    """Per-group centroid*3 plus unit noise for Q/K, unit-noise V (the block-structured
    inputs of the sparse-reuse benchmark)."""
    g = torch.Generator().manual_seed(seed)
    centroids = torch.randn(batch, kv_heads, groups, dim, generator=g) * 3
    per_token = centroids.repeat_interleave(length // groups, dim=2)
    k = (per_token + torch.randn(batch, kv_heads, length, dim, generator=g)).to(dtype).cuda()
    q = (per_token.repeat_interleave(q_heads // kv_heads, dim=1)
         + torch.randn(batch, q_heads, length, dim, generator=g)).to(dtype).cuda()
    v = torch.randn(batch, kv_heads, length, dim, generator=g).to(dtype).cuda()
    return q, k, v


def rows_of(row_offsets, block_indices):
    ro = np.asarray(row_offsets)
    bi = np.asarray(block_indices)
    return [set(bi[ro[r] : ro[r + 1]].tolist()) for r in range(len(ro) - 1)]


@pytest.mark.parametrize("length,theta", [(1024, 0.99), (2048, 0.9)])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_constructed_tile_sets_match_oracle(risa, length, theta, mode):
    q, k, v = block_structured(1, 4, 2, length, 128, 16, seed=length)
    out, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=theta, v_quantization=mode)
    prepared = oracle_prequantize(q, k, v, v_quantization=mode)
    expected_out, _, cap = oracle_pipeline.attend(prepared, capture=True)
    masses = oracle_attention.block_mass(cap, 1, 4, length)
    ro, bi, measured, _ = oracle_selection.select_retained_mass(masses, theta)
    assert relative_l2(to_numpy(out), expected_out) < 1e-3
    got = rows_of(pattern.row_offsets.cpu().numpy(), pattern.block_indices.cpu().numpy())
    want = rows_of(ro, bi)
    assert len(got) == len(want)
    for r, (g_set, w_set) in enumerate(zip(got, want)):
        if g_set == w_set:
            continue
        # Documented tie: the symmetric difference may only hold tiles whose mass is within
        # FP32 reduction noise of the cut (the smallest selected mass of the oracle row).
        cut = min(masses[r, t] for t in w_set)
        for t in g_set ^ w_set:
            assert abs(masses[r, t] - cut) <= 1e-4 * max(cut, 1e-6) + 1e-6, (r, t, masses[r, t], cut)
    assert pattern.measured_retained_mass == pytest.approx(measured, abs=1e-4)
    assert 0 < pattern.coverage < 1
    # reuse with the oracle's own pattern gives the oracle's sparse output
    oracle_pattern = replace(
        pattern,
        row_offsets=torch.from_numpy(ro).cuda(),
        block_indices=torch.from_numpy(bi).cuda(),
    )
    sparse = risa.sparse_int8_attention(q, k, v, oracle_pattern, v_quantization=mode)
    expected_sparse, _, _ = oracle_pipeline.attend(prepared, pattern=(ro, bi))
    assert relative_l2(to_numpy(sparse), expected_sparse) < 1e-3


def test_block_mass_values_match_oracle(risa):
    q, k, v = block_structured(1, 2, 1, 1280, 128, 8, seed=5)
    packed = risa.prequantize_int8_attention(q, k, v)
    blocks = 1280 // packed.cta_k
    mass_elements = 2 * 10 * blocks
    workspace = torch.empty(mass_elements + 2 * 1280 * (blocks * 2 + 2), device="cuda")
    risa.int8_attention_from_prequantized(packed, _block_mass=workspace)
    prepared = oracle_prequantize(q, k, v)
    _, _, cap = oracle_pipeline.attend(prepared, capture=True)
    expected = oracle_attention.block_mass(cap, 1, 2, 1280)
    got = workspace[:mass_elements].view(-1, blocks).cpu().numpy()
    np.testing.assert_allclose(got, expected, rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(got.sum(1), 128.0, atol=1e-3)


@pytest.mark.parametrize("theta", [0.5, 0.99, 1.0])
@pytest.mark.parametrize("rows,tiles", [(531, 257), (40, 1), (9, 2), (77, 64), (33, 1000), (5, 4096)])
def test_selector_kernel_matches_oracle_exactly(risa, theta, rows, tiles):
    """Rows of up to 4096 tiles are sorted inside the library, ties by ascending tile id: the
    order of the oracle's stable descending sort, so the CSR is equal entry for entry even with
    repeated masses (a row of zeros, a row of one value, masses drawn from eight levels)."""
    from risaattention_amd.patterns import select_retained_mass_csr

    g = torch.Generator().manual_seed(1)
    masses = (torch.rand(rows, tiles, generator=g) ** 6)
    masses[rows // 2] = 0
    masses[rows // 3] = 0.25
    masses[1] = (masses[1] * 8).floor() / 8
    masses = masses.cuda()
    row_offsets, block_indices, measured = select_retained_mass_csr(masses, theta)
    ro, bi, expected_measured, _ = oracle_selection.select_retained_mass(masses.cpu().numpy(), theta)
    np.testing.assert_array_equal(row_offsets.cpu().numpy(), ro)
    np.testing.assert_array_equal(block_indices.cpu().numpy(), bi)
    assert measured == pytest.approx(expected_measured, rel=1e-12)


@pytest.mark.parametrize("theta", [0.5, 0.99])
def test_selector_kernel_over_an_outside_sort(risa, theta):
    """Rows longer than the library sorts take torch.sort, as in the reference: the CSR equals the
    oracle's for that permutation."""
    from risaattention_amd.patterns import select_retained_mass_csr

    g = torch.Generator().manual_seed(2)
    masses = (torch.rand(6, 4100, generator=g) ** 6).cuda()
    row_offsets, block_indices, measured = select_retained_mass_csr(masses, theta)
    order = masses.sort(dim=-1, descending=True).indices.cpu().numpy()
    ro, bi, expected_measured, _ = oracle_selection.select_retained_mass(masses.cpu().numpy(), theta, order=order)
    np.testing.assert_array_equal(row_offsets.cpu().numpy(), ro)
    np.testing.assert_array_equal(block_indices.cpu().numpy(), bi)
    assert measured == pytest.approx(expected_measured, rel=1e-12)


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_key_mask_tile_skipping_matches_generic_mask(risa, mask_dtype, dim):
    """reference tests/cuda/test_key_mask_tiles.py:16-54."""
    torch.manual_seed(74)
    q = torch.randn(2, 4, 257, dim, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(2, 2, 1153, dim, device="cuda", dtype=q.dtype)
    v = torch.randn_like(k) + 3
    storage = torch.zeros(2, 4, 1, 2306, device="cuda", dtype=mask_dtype)
    mask = storage[..., ::2]
    visible = torch.ones(2, 4, 1, 1153, device="cuda", dtype=torch.bool)
    visible[..., :128] = False
    visible[..., 384:768] = False
    visible[0, 1] = False
    visible[1, 2, :, -1] = False
    visible[..., 897:913] = False
    if mask_dtype == torch.bool:
        mask.copy_(visible)
    else:
        mask.copy_(torch.linspace(-1, 2, 1153, device="cuda"))
        mask.masked_fill_(~visible, -torch.inf)
    packed = risa.prequantize_int8_attention(q, k, v, attn_mask=mask, return_lse=True)
    generic = replace(packed, attn_mask=packed.attn_mask.clone())
    actual, lse = risa.int8_attention_from_prequantized(packed, return_lse=True)
    expected, expected_lse = risa.int8_attention_from_prequantized(generic, return_lse=True)
    torch.testing.assert_close(actual, expected, atol=0.002, rtol=0.01)
    torch.testing.assert_close(lse, expected_lse, atol=2e-4, rtol=2e-6)
    assert torch.count_nonzero(actual[0, 1]) == 0
    assert torch.isneginf(lse[0, 1]).all()
    torch.testing.assert_close(risa.int8_attention(q, k, v, attn_mask=mask), actual, atol=0, rtol=0)
    # and against the oracle
    prepared = oracle_prequantize(q, k, v, attn_mask=mask, return_lse=True)
    want, want_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(actual), want) < 1e-3
    assert relative_l2(to_numpy(lse), want_lse) < 1e-3


def test_key_mask_tiles_known_answer(risa):
    """reference tests/cuda/test_key_mask_tiles.py:78-104."""
    from risaattention_amd.key_mask import prepare_key_mask_tiles

    q = torch.randn(1, 4, 257, 128, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(1, 2, 1153, 128, device="cuda", dtype=q.dtype)
    v = torch.randn_like(k)
    mask = torch.ones(1, 1, 1, 1153, device="cuda", dtype=torch.bool)
    mask[..., :512] = False
    packed = risa.prequantize_int8_attention(q, k, v, attn_mask=mask)
    tiles = prepare_key_mask_tiles(packed.attn_mask, packed.cta_k, 257, packed.attention_scale, False)
    expected = torch.tensor([4, 5, 6, 7, 8, 9], device="cuda", dtype=torch.int32)
    assert torch.equal(tiles[..., :6], expected.expand(1, 4, 6))
    assert (tiles[..., -1] == 6).all()
    assert prepare_key_mask_tiles(packed.attn_mask, packed.cta_k, 255, packed.attention_scale, False) is None
    assert prepare_key_mask_tiles(packed.attn_mask, packed.cta_k, 257, packed.attention_scale, True) is None
    assert prepare_key_mask_tiles(packed.attn_mask, packed.cta_k, 257, 0.0, False) is None


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_nondefault_stream_and_graph_replay(risa, mode):
    """reference tests/cuda/test_probability_mass.py:94-108 and test_value_quantization.py:75-90."""
    q = torch.randn(1, 4, 2049, 128, device="cuda", dtype=torch.bfloat16)
    k, v = [torch.randn(1, 2, 2049, 128, device="cuda", dtype=q.dtype) for _ in range(2)]
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode)
        expected = risa.int8_attention_from_prequantized(packed)
        expected_full = risa.int8_attention(q, k, v, v_quantization=mode)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            actual = risa.int8_attention_from_prequantized(packed)
            actual_full = risa.int8_attention(q, k, v, v_quantization=mode)
        for _ in range(3):
            actual.zero_()
            actual_full.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(actual, expected)
            assert torch.equal(actual_full, expected_full)
    torch.cuda.current_stream().wait_stream(stream)
    assert torch.equal(expected, expected_full)


def test_prequantized_nhd_layout_and_head_dim_padding(risa):
    q = seeded((2, 4, 150, 80), torch.float16, 1)
    k = seeded((2, 2, 333, 80), torch.float16, 2)
    v = seeded((2, 2, 333, 80), torch.float16, 3)
    packed = risa.prequantize_int8_attention(q, k, v)
    hnd = risa.int8_attention_from_prequantized(packed)
    nhd = risa.int8_attention_from_prequantized(packed, output_layout="nhd")
    assert hnd.shape == nhd.shape == (2, 4, 150, 80)
    assert nhd.transpose(1, 2).reshape(2, 150, -1).shape == (2, 150, 320)
    assert torch.equal(hnd, nhd)
    assert torch.equal(hnd, risa.int8_attention(q, k, v))


def test_input_strides_do_not_change_results(risa):
    base = seeded((1, 300, 3, 4, 128), torch.bfloat16, 9)
    q = base[:, :, 0].transpose(1, 2)
    k = base[:, :, 1, :2].transpose(1, 2)
    v = base[:, :, 2, :2].transpose(1, 2)
    strided = risa.int8_attention(q, k, v, v_quantization="midpoint_affine")
    dense = risa.int8_attention(q.contiguous(), k.contiguous(), v.contiguous(), v_quantization="midpoint_affine")
    assert torch.equal(strided, dense)


def test_dense_fallback_for_nearly_dense_pattern(risa):
    q = seeded((1, 2, 512, 128), torch.bfloat16, 3)
    k = seeded((1, 1, 512, 128), torch.bfloat16, 4)
    v = seeded((1, 1, 512, 128), torch.bfloat16, 5)
    built, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=1.0)
    assert pattern.sparsity < 0.05
    sparse = risa.sparse_int8_attention(q, k, v, pattern)
    assert torch.equal(sparse, risa.int8_attention(q, k, v))
    with pytest.raises(ValueError, match="is_causal"):
        risa.sparse_int8_attention(q, k, v, pattern, is_causal=True)


def test_full_size_invariants(risa):
    """Headline shape (N=32K, Hq16/Hkv4/D128, bf16): properties that need no oracle run."""
    length = 32768
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(1, 16, length, 128, generator=g, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(1, 4, length, 128, generator=g, device="cuda", dtype=torch.bfloat16)
    values = torch.linspace(-3, 5, 128, device="cuda", dtype=torch.bfloat16)
    v = values.expand_as(k).contiguous()
    out, lse = risa.int8_attention(q, k, v, return_lse=True)
    assert torch.equal(out, values.expand_as(out))
    zero_scale, lse0 = risa.int8_attention(q, k, v, scale=0.0, return_lse=True)
    assert torch.equal(zero_scale, values.expand_as(out))
    torch.testing.assert_close(lse0, torch.full_like(lse0, float(np.log(length))), atol=2e-5, rtol=0)
    # LSE against FP32 on a slice of queries
    rows = slice(1000, 1128)
    scores = q[:, :4, rows].float() @ k[:, :1].float().transpose(-1, -2) / 128**0.5
    torch.testing.assert_close(lse[:, :4, rows], scores.logsumexp(-1), atol=0.02, rtol=0)


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_key_mask_skipping_stream_and_graph(risa, mode):
    """reference tests/cuda/test_key_mask_tiles.py:57-76: constant V under a key mask that
    hides whole tiles, on a side stream, eagerly and from a captured graph."""
    q = torch.randn(1, 4, 513, 128, device="cuda", dtype=torch.float16)
    k = torch.randn(1, 2, 2049, 128, device="cuda", dtype=q.dtype)
    v = torch.full_like(k, 2.75)
    mask = torch.ones(1, 1, 1, 2049, device="cuda", dtype=torch.bool)
    mask[..., 128:1536] = False
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for _ in range(3):
            output = risa.int8_attention(q, k, v, attn_mask=mask, v_quantization=mode)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            captured = risa.int8_attention(q, k, v, attn_mask=mask, v_quantization=mode)
        for _ in range(3):
            captured.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(captured, output)
    torch.cuda.current_stream().wait_stream(stream)
    assert torch.equal(output, v[..., :513, :].repeat_interleave(2, dim=1))


@pytest.mark.parametrize("inference", [False, True])
def test_key_mask_metadata_and_mask_mutation(risa, inference):
    """reference tests/cuda/test_key_mask_tiles.py:79-104: the packed container keeps the
    caller's mask tensor, not a copy; the tile list is rebuilt from its current
    contents on every call."""
    from risaattention_amd.key_mask import prepare_key_mask_tiles

    q = torch.randn(1, 4, 257, 128, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(1, 2, 1153, 128, device="cuda", dtype=q.dtype)
    v = torch.randn_like(k)
    mask = torch.ones(1, 1, 1, 1153, device="cuda", dtype=torch.bool)
    if inference:
        with torch.inference_mode():
            mask = mask.clone()
    with torch.inference_mode():
        mask[..., :512] = False
    packed = risa.prequantize_int8_attention(q, k, v, attn_mask=mask)
    tiles = prepare_key_mask_tiles(packed.attn_mask, packed.cta_k, 257, packed.attention_scale, False)
    expected = torch.tensor([4, 5, 6, 7, 8, 9], device="cuda", dtype=torch.int32)
    assert torch.equal(tiles[..., :6], expected.expand(1, 4, 6))
    assert (tiles[..., -1] == 6).all()
    with torch.inference_mode():
        mask.fill_(True)
    actual = risa.int8_attention_from_prequantized(packed)
    generic = risa.int8_attention_from_prequantized(replace(packed, attn_mask=packed.attn_mask.clone()))
    assert torch.equal(actual, generic)
    # An all-true mask takes the pre-scaled path, no mask the raw-score path: same
    # codes, different FP32 rounding order.
    unmasked = risa.int8_attention_from_prequantized(replace(packed, attn_mask=None))
    assert relative_l2(to_numpy(actual), to_numpy(unmasked)) < 1e-2


@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_prequantized_mask_mutation_during_graph_replay(risa, mode):
    """reference tests/cuda/test_key_mask_tiles.py:107-123: a mask emptied after capture
    empties the replayed output."""
    with torch.inference_mode():
        q = torch.randn(1, 4, 257, 128, device="cuda", dtype=torch.bfloat16)
        k = torch.randn(1, 2, 1153, 128, device="cuda", dtype=q.dtype)
        v = torch.full_like(k, 2.75)
        mask = torch.ones(1, 1, 1, 1153, device="cuda", dtype=torch.bool)
        mask[..., :768] = False
        packed = risa.prequantize_int8_attention(q, k, v, attn_mask=mask, v_quantization=mode)
        for _ in range(3):
            eager = risa.int8_attention_from_prequantized(packed)
        assert torch.equal(eager, v[..., :257, :].repeat_interleave(2, dim=1))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = risa.int8_attention_from_prequantized(packed)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager)
        mask.fill_(False)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.count_nonzero(captured) == 0
        mask[..., 900:] = True
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager)


@pytest.mark.parametrize("dim,k_len", [(128, 1300), (64, 700), (256, 1300)])
def test_reuse_matches_oracle_at_every_launch_size(risa, dim, k_len):
    """Unmasked reuse runs sixteen queries per wavefront in workgroups of 32, 64 or 128
    queries when the launch is small (and always for head dim 256), thirty-two per wavefront
    otherwise: 16, 48, 96 and 160 query heads over two query blocks go through each of them.
    The first eight heads are checked against the oracle walking the same lists, and every
    launch against the largest one on the heads they share."""
    q_len, oracle_heads = 200, 8
    q_all = seeded((1, 160, q_len, dim), torch.bfloat16, 301, scale=2.0)
    k = seeded((1, 1, k_len, dim), torch.bfloat16, 302, scale=2.0)
    v = seeded((1, 1, k_len, dim), torch.bfloat16, 303, offset=0.25)
    _, pattern_all = risa.construct_sparse_int8_attention(q_all, k, v, theta=0.9)
    assert 0.0 < pattern_all.coverage < 1.0
    query_blocks = -(-q_len // 128)
    offsets_all = pattern_all.row_offsets.cpu().numpy()
    indices_all = pattern_all.block_indices.cpu().numpy()

    def pattern_for(heads):
        rows = heads * query_blocks
        return replace(pattern_all, q_heads=heads,
                       row_offsets=torch.from_numpy(offsets_all[:rows + 1].copy()).cuda(),
                       block_indices=torch.from_numpy(indices_all[:offsets_all[rows]].copy()).cuda())

    largest = risa.sparse_int8_attention(q_all, k, v, pattern_for(160))
    prepared = oracle_prequantize(q_all[:, :oracle_heads], k, v)
    rows = oracle_heads * query_blocks
    expected, _, _ = oracle_pipeline.attend(
        prepared, pattern=(offsets_all[:rows + 1], indices_all[:offsets_all[rows]]))
    assert relative_l2(to_numpy(largest[:, :oracle_heads]), expected) < 1e-3
    for heads in (16, 48, 96):
        out = risa.sparse_int8_attention(q_all[:, :heads], k, v, pattern_for(heads))
        assert relative_l2(to_numpy(out[:, :oracle_heads]), expected) < 1e-3, heads
        assert relative_l2(to_numpy(out), to_numpy(largest[:, :heads])) < 1e-4, heads


@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("heads,output_dtype", [(2, torch.bfloat16), (130, torch.float16)])
def test_short_tile_lists_match_oracle(risa, dim, heads, output_dtype):
    """Hand-made lists of one to three tiles per query block, the partial tail tile among
    them (always last: lists are ascending), through both kernels (few and many workgroups):
    the listed tile after the next one is read a tile ahead, the last listed tile takes the
    last-tile formulas, and keys past the end must not count."""
    from risaattention_amd.types import RetainedMassPattern

    q_len, k_len = 300, 1100
    q = seeded((1, heads, q_len, dim), output_dtype, 81)
    k = seeded((1, 1, k_len, dim), output_dtype, 82)
    v = seeded((1, 1, k_len, dim), output_dtype, 83, offset=0.5)
    packed = risa.prequantize_int8_attention(q, k, v, return_lse=True)
    tiles = -(-k_len // packed.cta_k)
    choices = [[tiles - 1], [0], [0, tiles - 1], [1, 2, tiles - 1], [tiles - 3, tiles - 2], [2]]
    query_blocks = -(-q_len // 128)
    lists = [choices[(head * query_blocks + block) % len(choices)] for head in range(heads) for block in range(query_blocks)]
    offsets = np.cumsum([0] + [len(entry) for entry in lists]).astype(np.int32)
    indices = np.concatenate(lists).astype(np.int32)
    pattern = RetainedMassPattern(torch.from_numpy(offsets).cuda(), torch.from_numpy(indices).cuda(), 1, heads, q_len,
                                  k_len, 128, packed.cta_k, packed.attention_scale, 0.5, 0.5)
    out, lse = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern, return_lse=True)
    checked = 2  # heads compared with the oracle
    rows = checked * query_blocks
    prepared = oracle_prequantize(q[:, :checked], k, v, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, pattern=(offsets[: rows + 1], indices[: offsets[rows]]),
                                                       return_lse=True)
    assert relative_l2(to_numpy(out[:, :checked]), expected) < 1e-3
    assert relative_l2(to_numpy(lse[:, :checked]), expected_lse) < 1e-3
    # heads with the same lists and inputs give the same rows whichever kernel ran
    period = len(choices)
    if heads > period * 2:
        twin = risa.int8_attention_from_prequantized(
            risa.prequantize_int8_attention(q[:, :2], k, v),
            sparse_pattern=RetainedMassPattern(pattern.row_offsets[: rows + 1].clone(),
                                               pattern.block_indices[: int(offsets[rows])].clone(), 1, 2, q_len, k_len,
                                               128, packed.cta_k, packed.attention_scale, 0.5, 0.5))
        assert relative_l2(to_numpy(twin), to_numpy(out[:, :2])) < 1e-4
