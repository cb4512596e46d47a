"""The hand-scheduled tile loops of the raw-score kernels (head dim 128, 128-key tiles, more
workgroups than compute units: dense, over tile lists, capturing) against the loop the compiler
schedules, which RISA_COMPILED_LOOP=1 selects at every launch: same arithmetic in the same order,
so outputs, log-sum-exp rows and the constructed pattern are equal bit for bit.  Tile lists are
also compared with the dense launch where they name every tile, and with the oracle walking the
same lists otherwise."""

import os
from contextlib import contextmanager

import numpy as np
import pytest
import torch

from oracle import pipeline as oracle_pipeline
from tests.helpers import oracle_prequantize, relative_l2, seeded, to_numpy

pytestmark = pytest.mark.gpu


@contextmanager
def compiled_loop():
    """Launches inside go through the compiler-scheduled tile loop."""
    before = os.environ.get("RISA_COMPILED_LOOP")
    os.environ["RISA_COMPILED_LOOP"] = "1"
    try:
        yield
    finally:
        if before is None:
            del os.environ["RISA_COMPILED_LOOP"]
        else:
            os.environ["RISA_COMPILED_LOOP"] = before


@pytest.mark.parametrize("length", [2048, 2049, 2304, 4096, 4190])
@pytest.mark.parametrize("mode", ["absmax", "midpoint_affine"])
def test_dense_and_capturing_loops_equal_the_compiled_loop_bit_for_bit(risa, length, mode):
    """Odd and even tile counts (the loop is unrolled by two and leaves from either half), a last
    tile of one key, of half a tile, a whole one."""
    heads = 20  # x 17..33 query blocks: above the small-launch limit of a 256-CU part
    q = seeded((1, heads, length, 128), torch.bfloat16, length, scale=1.5)
    k = seeded((1, 4, length, 128), torch.bfloat16, length + 1, scale=1.5)
    v = seeded((1, 4, length, 128), torch.bfloat16, length + 2, offset=0.25)
    dense, dense_lse = risa.int8_attention(q, k, v, v_quantization=mode, return_lse=True)
    captured, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.95, v_quantization=mode)
    with compiled_loop():
        compiled, compiled_lse = risa.int8_attention(q, k, v, v_quantization=mode, return_lse=True)
        compiled_captured, compiled_pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.95, v_quantization=mode)
    assert torch.equal(dense, compiled) and torch.equal(dense_lse, compiled_lse)
    assert torch.equal(captured, compiled_captured) and torch.equal(dense, captured)
    # the statistics the capturing loop stores decide the pattern: same rows, same tiles, same mass
    assert torch.equal(pattern.row_offsets, compiled_pattern.row_offsets)
    assert torch.equal(pattern.block_indices, compiled_pattern.block_indices)
    assert pattern.measured_retained_mass == compiled_pattern.measured_retained_mass
    checked = 2
    prepared = oracle_prequantize(q[:, :checked], k[:, :1], v[:, :1], v_quantization=mode, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(dense[:, :checked]), expected) < 1e-3
    assert relative_l2(to_numpy(dense_lse[:, :checked]), expected_lse) < 1e-3


@pytest.mark.parametrize("k_len", [2304, 2300])
def test_listed_loop_with_every_tile_equals_the_dense_launch(risa, k_len):
    from risaattention_amd.types import RetainedMassPattern

    heads, q_len = 40, 1024
    q = seeded((1, heads, q_len, 128), torch.float16, 11)
    k = seeded((1, 2, k_len, 128), torch.float16, 12)
    v = seeded((1, 2, k_len, 128), torch.float16, 13, offset=-0.5)
    packed = risa.prequantize_int8_attention(q, k, v, return_lse=True)
    assert packed.cta_k == 128
    tiles, rows = -(-k_len // 128), heads * (q_len // 128)
    offsets = (np.arange(rows + 1) * tiles).astype(np.int32)
    indices = np.tile(np.arange(tiles, dtype=np.int32), rows)
    pattern = RetainedMassPattern(torch.from_numpy(offsets).cuda(), torch.from_numpy(indices).cuda(), 1, heads, q_len,
                                  k_len, 128, 128, packed.attention_scale, 1.0, 1.0)
    listed, listed_lse = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern, return_lse=True)
    dense, dense_lse = risa.int8_attention_from_prequantized(packed, return_lse=True)
    assert torch.equal(listed, dense)
    assert torch.equal(listed_lse, dense_lse)


@pytest.mark.parametrize("seed", [0, 1])
def test_listed_loop_with_random_lists_matches_oracle(risa, seed):
    """Lists of one to nineteen tiles, each an ascending random subset (with and without the
    partial last tile), different for every query block."""
    from risaattention_amd.types import RetainedMassPattern

    heads, q_len, k_len = 36, 1000, 2350
    q = seeded((1, heads, q_len, 128), torch.bfloat16, 21 + seed)
    k = seeded((1, 1, k_len, 128), torch.bfloat16, 22 + seed)
    v = seeded((1, 1, k_len, 128), torch.bfloat16, 23 + seed, offset=0.5)
    packed = risa.prequantize_int8_attention(q, k, v, return_lse=True)
    tiles, query_blocks = -(-k_len // 128), -(-q_len // 128)
    rng = np.random.default_rng(seed)
    lists = [np.sort(rng.choice(tiles, size=1 + (row * 7 + seed) % tiles, replace=False)) for row in range(heads * query_blocks)]
    offsets = np.cumsum([0] + [len(entry) for entry in lists]).astype(np.int32)
    indices = np.concatenate(lists).astype(np.int32)
    pattern = RetainedMassPattern(torch.from_numpy(offsets).cuda(), torch.from_numpy(indices).cuda(), 1, heads, q_len,
                                  k_len, 128, 128, packed.attention_scale, 0.5, 0.5)
    out, lse = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern, return_lse=True)
    with compiled_loop():
        compiled, compiled_lse = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern, return_lse=True)
    assert torch.equal(out, compiled) and torch.equal(lse, compiled_lse)
    checked = 3
    rows = checked * query_blocks
    prepared = oracle_prequantize(q[:, :checked], k, v, return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, pattern=(offsets[: rows + 1], indices[: offsets[rows]]),
                                                       return_lse=True)
    assert relative_l2(to_numpy(out[:, :checked]), expected) < 1e-3
    assert relative_l2(to_numpy(lse[:, :checked]), expected_lse) < 1e-3


@pytest.mark.parametrize("k_len", [1025, 1152, 1153, 1280])
def test_shortest_dense_walks_and_two_batches(risa, k_len):
    """The shortest dense walks of the hand-scheduled loop (128-key tiles start above 1024 keys:
    nine or ten tiles, the last of one key or whole), cross attention, two batches of grouped
    heads."""
    q = seeded((2, 24, 1024, 128), torch.bfloat16, k_len, scale=2.0)
    k = seeded((2, 8, k_len, 128), torch.bfloat16, k_len + 1, scale=2.0)
    v = seeded((2, 8, k_len, 128), torch.bfloat16, k_len + 2, offset=-0.25)
    out, lse = risa.int8_attention(q, k, v, return_lse=True)
    with compiled_loop():
        compiled, compiled_lse = risa.int8_attention(q, k, v, return_lse=True)
    assert torch.equal(out, compiled) and torch.equal(lse, compiled_lse)
    assert risa.prequantize_int8_attention(q, k, v).cta_k == 128
    prepared = oracle_prequantize(q[1:, 21:], k[1:, 7:], v[1:, 7:], return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out[1:, 21:]), expected) < 1e-3
    assert relative_l2(to_numpy(lse[1:, 21:]), expected_lse) < 1e-3


@pytest.mark.parametrize("seed", range(8))
def test_random_shapes_equal_the_compiled_loop(risa, seed):
    """Random batch, head grouping, lengths, dtype and V mode (always more workgroups than a
    256-CU part has compute units): dense, capturing and list-walking launches of the
    hand-scheduled loops against the compiled loop, bit for bit."""
    from risaattention_amd.types import RetainedMassPattern

    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.integers(1, 3))
    kv_heads = int(rng.integers(1, 5))
    q_heads = kv_heads * int(rng.integers(1, 5))
    q_len = int(rng.integers(129, 1500))
    while batch * q_heads * -(-q_len // 128) <= 300:
        q_heads += kv_heads
    k_len = int(rng.integers(257, 3000))
    dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
    mode = ("absmax", "midpoint_affine")[seed % 2]
    q = seeded((batch, q_heads, q_len, 128), dtype, 3 * seed, scale=1.0 + seed % 3)
    k = seeded((batch, kv_heads, k_len, 128), dtype, 3 * seed + 1, scale=1.0 + seed % 2)
    v = seeded((batch, kv_heads, k_len, 128), dtype, 3 * seed + 2, offset=0.1 * seed)
    packed = risa.prequantize_int8_attention(q, k, v, v_quantization=mode, return_lse=True)
    # (the tile policy gives short key ranges 64-key tiles: those launches keep the compiled loop)
    tiles, query_blocks = -(-k_len // packed.cta_k), -(-q_len // 128)
    lists = [np.sort(rng.choice(tiles, size=int(rng.integers(1, tiles + 1)), replace=False))
             for _ in range(batch * q_heads * query_blocks)]
    offsets = np.cumsum([0] + [len(entry) for entry in lists]).astype(np.int32)
    pattern = RetainedMassPattern(torch.from_numpy(offsets).cuda(), torch.from_numpy(np.concatenate(lists).astype(np.int32)).cuda(),
                                  batch, q_heads, q_len, k_len, 128, packed.cta_k, packed.attention_scale, 0.5, 0.5)

    def run():
        dense = risa.int8_attention_from_prequantized(packed, return_lse=True)
        listed = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern, return_lse=True)
        captured, built = risa.construct_sparse_int8_attention(q, k, v, theta=0.9, v_quantization=mode)
        return [*dense, *listed, captured, built.row_offsets, built.block_indices]

    scheduled = run()
    with compiled_loop():
        compiled = run()
    for index, (mine, theirs) in enumerate(zip(scheduled, compiled)):
        assert torch.equal(mine, theirs), (index, batch, q_heads, kv_heads, q_len, k_len, dtype, mode)
