"""The frozen vectors of tests/golden/vectors.npz (written by tests/golden/make_vectors.py):
the oracle must still compute them on the CPU, and the HIP path must reproduce them through
the C ABI (codes, scales, centres, anchors and LSE shift bit for bit; outputs and LSE within
1e-3 relative L2; block masses within FP32 reduction noise; selected tiles exactly for these
inputs, which hold no tie at the cut)."""

import numpy as np
import pytest

from oracle import attention as oracle_attention
from oracle import pipeline as oracle_pipeline
from oracle import selection as oracle_selection
from tests.golden.make_vectors import CASES
from tests.helpers import load_vectors, relative_l2

VECTORS = load_vectors()
EXACT_FIELDS = ("q_codes", "k_codes", "v_codes", "q_scale", "k_scale", "v_scale", "v_center", "anchor", "lse_shift")
PREPARED_NAMES = {"q_codes": "q", "k_codes": "k", "v_codes": "v"}


def test_every_case_has_vectors():
    assert set(VECTORS) == set(CASES)


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_still_computes_the_frozen_vectors(name):
    vector, case = VECTORS[name], CASES[name]
    prepared = oracle_pipeline.prequantize(vector["q"], vector["k"], vector["v"], mask=vector.get("mask"),
                                           v_quantization=case[5], is_causal=case[6], return_lse=True,
                                           dtype_name="bfloat16")
    assert prepared.cta_k == int(vector["cta_k"])
    for field in EXACT_FIELDS:
        np.testing.assert_array_equal(getattr(prepared, PREPARED_NAMES.get(field, field)), vector[field], err_msg=field)
    out, lse, captured = oracle_pipeline.attend(prepared, return_lse=True, capture="block_mass" in vector)
    np.testing.assert_array_equal(out.astype(np.float32), vector["out"])
    np.testing.assert_array_equal(lse.astype(np.float32), vector["lse"])
    if captured is not None:
        masses = oracle_attention.block_mass(captured, 1, case[0], case[2])
        np.testing.assert_array_equal(masses.astype(np.float32), vector["block_mass"])
        row_offsets, block_indices, measured, _ = oracle_selection.select_retained_mass(masses, 0.9)
        np.testing.assert_array_equal(row_offsets, vector["row_offsets"])
        np.testing.assert_array_equal(block_indices, vector["block_indices"])
        assert measured == float(vector["measured"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_path_reproduces_the_frozen_vectors(risa, name):
    import torch

    from risaattention_amd.layout import unpack_values

    vector, case = VECTORS[name], CASES[name]
    q, k, v = (torch.from_numpy(vector[key].copy()).to(torch.bfloat16).cuda() for key in ("q", "k", "v"))
    mask = None if "mask" not in vector else torch.from_numpy(vector["mask"].copy()).cuda()
    options = dict(attn_mask=mask, is_causal=case[6], v_quantization=case[5])
    packed = risa.prequantize_int8_attention(q, k, v, return_lse=True, **options)
    assert packed.cta_k == int(vector["cta_k"])
    kernel_dim = packed.q.shape[-1]
    pad = kernel_dim - case[4]
    got = {
        "q_codes": packed.q.cpu().numpy(), "k_codes": packed.k.cpu().numpy(),
        "v_codes": unpack_values(packed.v).cpu().numpy(), "q_scale": packed.q_scale.cpu().numpy(),
        "k_scale": packed.k_scale.cpu().numpy(), "v_scale": packed.v_scale.cpu().numpy(),
        "v_center": packed.v_center.cpu().numpy(), "lse_shift": packed.lse_shift.cpu().numpy(),
    }
    assert pad == vector["q_codes"].shape[-1] - case[4]
    for field, value in got.items():
        np.testing.assert_array_equal(value.reshape(vector[field].shape), vector[field], err_msg=field)
    out, lse = risa.int8_attention(q, k, v, return_lse=True, **options)
    assert relative_l2(out.float().cpu().numpy(), vector["out"]) < 1e-3
    finite = np.isfinite(vector["lse"])
    assert np.array_equal(np.isfinite(lse.cpu().numpy()), finite)
    assert relative_l2(lse.cpu().numpy()[finite], vector["lse"][finite]) < 1e-3
    if "block_mass" in vector:
        built, pattern = risa.construct_sparse_int8_attention(q, k, v, theta=0.9, **options)
        assert relative_l2(built.float().cpu().numpy(), vector["out"]) < 1e-3
        np.testing.assert_array_equal(pattern.row_offsets.cpu().numpy(), vector["row_offsets"])
        np.testing.assert_array_equal(pattern.block_indices.cpu().numpy(), vector["block_indices"])
        assert pattern.measured_retained_mass == pytest.approx(float(vector["measured"]), abs=1e-4)
