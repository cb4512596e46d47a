"""Addressing beyond 4 GiB, after reference tests/cuda/test_large_offsets.py:1-72: five
query heads of 2^24 + 128 tokens put the last head's codes, outputs and capture rows
past a 32-bit byte offset.  A single visible key makes every output row equal to V."""

import math

import pytest
import torch

from risaattention_amd.attend import launch_attention

pytestmark = pytest.mark.gpu

REQUIRED_BYTES = 18 * 1024**3


@pytest.fixture(scope="module")
def wide_buffers(risa):
    if torch.cuda.mem_get_info()[0] < REQUIRED_BYTES:
        pytest.skip("large-offset checks need 18 GiB of free device memory")
    length = (1 << 30) // 64 + 128
    heads, dim = 5, 64
    q = torch.zeros((1, heads, length, dim), dtype=torch.int8, device="cuda")
    k = torch.zeros((1, 1, 1, dim), dtype=torch.int8, device="cuda")
    v = torch.zeros((dim, 64), dtype=torch.int8, device="cuda")
    v[:, 0] = 100  # token 0 sits at position 0 of its packed group
    q_scale = torch.ones((1, heads, math.ceil(length / 128) * 32), device="cuda")
    k_scale = torch.ones((1, 1, 4), device="cuda")
    v_scale = torch.full((dim,), 0.2, device="cuda")
    assert (heads - 1) * q.stride(1) > (1 << 32) - 1
    yield q, k, v, q_scale, k_scale, v_scale, torch.zeros_like(v_scale)
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
