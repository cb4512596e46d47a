"""Seeded sweep over ragged shapes: every case draws its batch, head counts, lengths,
head dim, dtype, V mode and mask kind from one generator and is checked against the
oracle (outputs and LSE within 1e-3 relative L2).  The draw covers single-query and
single-key problems, lengths around the 64/128-key tile edges and the 16/32/128-query
workgroup edges, grouped heads, padded head dims and every mask element type."""

import numpy as np
import pytest
import torch

from oracle import pipeline as oracle_pipeline
from tests.helpers import oracle_prequantize, relative_l2, seeded, to_numpy

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-3
EDGE_LENGTHS = (1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 127, 128, 129, 191, 256, 257, 320)
KEY_LENGTHS = EDGE_LENGTHS + (511, 512, 640, 1023, 1024, 1025, 1100, 1152, 1217)


def draw_case(seed):
    rng = np.random.default_rng(seed)
    dim = int(rng.choice([64, 128, 256, 40, 80, 200]))
    kv_heads = int(rng.choice([1, 2, 3]))
    group = int(rng.choice([1, 2, 4]))
    case = {
        "batch": int(rng.choice([1, 2])),
        "kv_heads": kv_heads,
        "q_heads": kv_heads * group,
        "q_len": int(rng.choice(EDGE_LENGTHS)),
        "k_len": int(rng.choice(KEY_LENGTHS)),
        "dim": dim,
        "dtype": [torch.float16, torch.bfloat16, torch.float32][int(rng.integers(3))],
        "mode": ["absmax", "midpoint_affine"][int(rng.integers(2))],
        "mask": ["none", "none", "causal", "key_bool", "key_float", "full_bool", "full_float", "full_half"][
            int(rng.integers(8))],
        "offset": float(rng.choice([0.0, 0.0, 3.0])),
    }
    if case["mask"] == "causal":
        case["k_len"] = case["q_len"] if rng.integers(2) else case["k_len"]
    return case


def build_mask(case, seed):
    kind, q_len, k_len = case["mask"], case["q_len"], case["k_len"]
    if kind in ("none", "causal"):
        return None
    generator = torch.Generator(device="cpu").manual_seed(seed)
    rows = 1 if kind.startswith("key") else q_len
    shape = (case["batch"], 1, rows, k_len) if seed % 2 else (1, case["q_heads"], rows, k_len)
    if kind.endswith("bool"):
        mask = torch.rand(shape, generator=generator) > 0.35
        mask[..., 0] = True  # no row is hidden entirely by construction of this column
        if rows > 2:
            mask[:, :, 1] = False  # ... except this one
        return mask.cuda()
    dtype = torch.float16 if kind.endswith("half") else torch.float32
    mask = torch.randn(shape, generator=generator)
    mask[..., 2::5] = float("-inf")
    return mask.to(dtype).cuda()


@pytest.mark.parametrize("seed", range(48))
def test_random_shape_matches_oracle(risa, seed):
    case = draw_case(1000 + seed)
    q = seeded((case["batch"], case["q_heads"], case["q_len"], case["dim"]), case["dtype"], 3 * seed)
    k = seeded((case["batch"], case["kv_heads"], case["k_len"], case["dim"]), case["dtype"], 3 * seed + 1,
               offset=case["offset"])
    v = seeded((case["batch"], case["kv_heads"], case["k_len"], case["dim"]), case["dtype"], 3 * seed + 2,
               offset=0.25)
    mask = build_mask(case, seed)
    causal = case["mask"] == "causal"
    out, lse = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, v_quantization=case["mode"],
                                   return_lse=True)
    plain = risa.int8_attention(q, k, v, attn_mask=mask, is_causal=causal, v_quantization=case["mode"])
    prepared = oracle_prequantize(q, k, v, attn_mask=mask, is_causal=causal, v_quantization=case["mode"],
                                  return_lse=True)
    expected, expected_lse, _ = oracle_pipeline.attend(prepared, return_lse=True)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE, case
    assert relative_l2(to_numpy(plain), expected) < TOLERANCE, case
    finite = np.isfinite(expected_lse)
    assert np.array_equal(np.isfinite(to_numpy(lse)), finite), case
    if finite.any():
        assert relative_l2(to_numpy(lse)[finite], expected_lse[finite]) < TOLERANCE, case
    if case["mask"] == "none":
        # Unmasked launches with more workgroups than compute units run the other kernel
        # (32 queries per wavefront): repeat every query head until the launch is that large;
        # copy r of head h still reads KV head h // group.
        blocks = case["batch"] * case["q_heads"] * -(-case["q_len"] // 128)
        repeat = torch.cuda.get_device_properties(0).multi_processor_count // blocks + 1
        wide, wide_lse = risa.int8_attention(q.repeat_interleave(repeat, dim=1), k, v,
                                             v_quantization=case["mode"], return_lse=True)
        assert relative_l2(to_numpy(wide[:, ::repeat]), expected) < TOLERANCE, case
        assert relative_l2(to_numpy(wide[:, repeat - 1::repeat]), expected) < TOLERANCE, case
        assert relative_l2(to_numpy(wide_lse[:, ::repeat]), expected_lse) < TOLERANCE, case


def draw_sparse_case(seed):
    rng = np.random.default_rng(seed)
    kv_heads = int(rng.choice([1, 2]))
    case = {
        "batch": int(rng.choice([1, 2])),
        "kv_heads": kv_heads,
        "q_heads": kv_heads * int(rng.choice([1, 2, 4])),
        "q_len": int(rng.choice([1, 17, 128, 129, 200, 256, 300, 515])),
        "k_len": int(rng.choice([1, 63, 64, 65, 200, 512, 1000, 1024, 1025, 1300, 2050])),
        "dim": int(rng.choice([64, 128, 256, 80])),
        "dtype": [torch.float16, torch.bfloat16][int(rng.integers(2))],
        "mode": ["absmax", "midpoint_affine"][int(rng.integers(2))],
        "mask": ["none", "none", "causal", "key_bool", "key_float"][int(rng.integers(5))],
        "theta": float(rng.choice([0.5, 0.9, 0.99, 1.0])),
    }
    # Key-only masks over more than 1024 keys and at least 256 queries also carry a list of
    # unmasked key tiles; the pattern's lists take its place during reuse.
    case.update(KEY_MASK_LIST_CASES.get(seed, {}))
    return case


KEY_MASK_LIST_CASES = {
    5032: {"q_len": 300, "k_len": 1300, "dim": 128, "mask": "key_bool", "theta": 0.9},
    5033: {"q_len": 515, "k_len": 2050, "dim": 64, "mask": "key_float", "theta": 0.5},
    5034: {"q_len": 256, "k_len": 1025, "dim": 256, "mask": "key_bool", "theta": 0.99},
    5035: {"q_len": 300, "k_len": 2050, "dim": 80, "mask": "key_float", "theta": 1.0},
}


@pytest.mark.parametrize("seed", range(36))
def test_random_sparse_shape_matches_oracle(risa, seed):
    """Construction on ragged shapes, then reuse of the constructed tile lists: the dense
    output, the CSR structure and the sparse output (both reuse entry points) against the
    oracle walking the same lists."""
    case = draw_sparse_case(5000 + seed)
    generator = torch.Generator(device="cpu").manual_seed(seed)
    # a few dominant keys per query block make the retained sets proper subsets
    q = seeded((case["batch"], case["q_heads"], case["q_len"], case["dim"]), case["dtype"], 7 * seed, scale=2.0)
    k = seeded((case["batch"], case["kv_heads"], case["k_len"], case["dim"]), case["dtype"], 7 * seed + 1, scale=2.0)
    v = seeded((case["batch"], case["kv_heads"], case["k_len"], case["dim"]), case["dtype"], 7 * seed + 2, offset=0.25)
    mask = None
    if case["mask"] == "key_bool":
        mask = (torch.rand((case["batch"], 1, 1, case["k_len"]), generator=generator) > 0.3)
        mask[..., 0] = True
        mask = mask.cuda()
    elif case["mask"] == "key_float":
        mask = torch.randn((1, 1, 1, case["k_len"]), generator=generator)
        mask[..., 3::7] = float("-inf")
        mask = mask.cuda()
    causal = case["mask"] == "causal"
    common = dict(attn_mask=mask, is_causal=causal, v_quantization=case["mode"])

    out, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=case["theta"], **common)
    prepared = oracle_prequantize(q, k, v, **common)
    expected, _, _ = oracle_pipeline.attend(prepared)
    assert relative_l2(to_numpy(out), expected) < TOLERANCE, case

    row_offsets = pattern.row_offsets.cpu().numpy()
    block_indices = pattern.block_indices.cpu().numpy()
    key_blocks = -(-case["k_len"] // prepared.cta_k)
    rows = case["batch"] * case["q_heads"] * -(-case["q_len"] // 128)
    assert row_offsets.shape == (rows + 1,) and row_offsets[0] == 0, case
    assert row_offsets[-1] == block_indices.shape[0], case
    for r in range(rows):
        tiles = block_indices[row_offsets[r]:row_offsets[r + 1]]
        assert np.all(np.diff(tiles) > 0) and (tiles.size == 0 or (tiles[0] >= 0 and tiles[-1] < key_blocks)), case

    expected_sparse, _, _ = oracle_pipeline.attend(prepared, pattern=(row_offsets, block_indices))
    sparse = risa.sparse_int8_attention(q, k, v, pattern, **common)
    assert relative_l2(to_numpy(sparse), expected_sparse) < TOLERANCE, case
    packed = risa.prequantize_int8_attention(q, k, v, **common)
    replay = risa.int8_attention_from_prequantized(packed, sparse_pattern=pattern)
    assert relative_l2(to_numpy(replay), expected_sparse) < TOLERANCE, case
