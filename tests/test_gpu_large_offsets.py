"""Addressing beyond 4 GiB, after reference tests/cuda/test_large_offsets.py:1-72: five
query heads of 2^24 + 128 tokens put the last head's codes, outputs and capture rows
past a 32-bit byte offset.  A single visible key makes every output row equal to V."""

import math

import pytest
import torch

from risaattention_amd.attend import launch_attention

pytestmark = pytest.mark.gpu

HEADS, DIM = 5, 64
# 2^24 + 128 queries of 64 one-byte channels are 1 GiB + 8 KiB per head: from the fifth head on,
# byte offsets of the codes need 33 bits, those of the fp16 output and of the capture rows more.
QUERIES = 2**24 + 128
MEMORY_NEEDED = 18 << 30


@pytest.fixture(scope="module")
def wide_buffers(risa):
    """Prepared operands built by hand: all-zero Q and K codes (every score is 0), unit Q/K
    scales, and a packed V matrix of one 64-key tile whose only non-zero column is token 0
    (byte 0 of its 32-token group) with code 100 and scale 0.2, so a row that sees just that
    key is exactly 20."""
    free_bytes, _ = torch.cuda.mem_get_info()
    if free_bytes < MEMORY_NEEDED:
        pytest.skip("large-offset checks need 18 GiB of free device memory")
    device = torch.device("cuda")
    operands = {
        "q": torch.zeros(1, HEADS, QUERIES, DIM, dtype=torch.int8, device=device),
        "k": torch.zeros(1, 1, 1, DIM, dtype=torch.int8, device=device),
        "v": torch.zeros(DIM, 64, dtype=torch.int8, device=device),
        "q_scale": torch.ones(1, HEADS, -(-QUERIES // 128) * 32, device=device),
        "k_scale": torch.ones(1, 1, 4, device=device),
        "v_scale": torch.full((DIM,), 0.2, device=device),
        "v_center": torch.zeros(DIM, device=device),
    }
    operands["v"][:, 0] = 100
    last_head_offset = (HEADS - 1) * operands["q"].stride(1)
    assert last_head_offset >= 2**32
    yield tuple(operands[name] for name in ("q", "k", "v", "q_scale", "k_scale", "v_scale", "v_center"))
    operands.clear()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("route", ["dense", "sparse", "capture"])
def test_real_wide_head_offsets(wide_buffers, route):
    q, k, v, q_scale, k_scale, v_scale, center = wide_buffers
    output = torch.empty(q.shape, dtype=torch.float16, device="cuda")
    rows = q.shape[1] * math.ceil(q.shape[2] / 128)
    extra = {}
    if route == "sparse":
        extra["row_offsets"] = torch.arange(rows + 1, device="cuda", dtype=torch.int32)
        extra["block_indices"] = torch.zeros(rows, device="cuda", dtype=torch.int32)
    elif route == "capture":
        extra["block_mass"] = torch.empty(rows + q.shape[1] * q.shape[2] * 4, device="cuda")
    launch_attention(q_codes=q, k_codes=k, v_codes=v, output=output, q_scale=q_scale, k_scale=k_scale,
                     v_scale=v_scale, v_center=center, v_tile_sum=None, cta_k=64, sm_scale=0.125, **extra)
    # Reductions over the whole tensor check every output write, including the head
    # whose base address is beyond 32 bits.
    assert output.amin().item() == 20.0
    assert output.amax().item() == 20.0
    if route == "capture":
        # The reciprocal of the row denominator may leave a mass one ULP below 128.
        mass = extra["block_mass"][:rows]
        torch.testing.assert_close(mass, torch.full_like(mass, 128.0), rtol=0.0, atol=2e-5)
