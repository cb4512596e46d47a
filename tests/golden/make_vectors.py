"""Writes tests/golden/vectors.npz: small inputs and what the oracle computes for them.

    python tests/golden/make_vectors.py

The reference ships no golden files for this path (its tests are closed-form and tolerance
checks), so these vectors do not come from it: they freeze the oracle's answers once the
oracle has passed its own pins, so that a later change of the oracle, of numpy or of the
kernels that moves a single code, scale or output shows up against a fixed target.  Inputs
are stored explicitly (the 16 bits of each bfloat16 value), not as seeds; ``load_vectors`` in
tests/helpers.py turns them back into float32.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import attention as oracle_attention  # noqa: E402
from oracle import pipeline  # noqa: E402
from oracle import selection  # noqa: E402

CASES = {
    # name: (Hq, Hkv, Lq, Lk, D, mode, causal, mask kind, key offset)
    "dense_d64_absmax": (2, 1, 40, 150, 64, "absmax", False, None, 0.0),
    "dense_d128_affine_anchor": (2, 1, 33, 96, 128, "midpoint_affine", False, None, 3.0),
    "causal_d64_affine": (2, 1, 70, 70, 64, "midpoint_affine", True, None, 0.0),
    "bias_d128_absmax": (2, 1, 20, 80, 128, "absmax", False, "bias", 0.0),
    "padded_d40_keymask": (2, 2, 17, 90, 40, "absmax", False, "key", 0.0),
}


def to_bfloat16(values: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bfloat16 (ties to even), returned as float32."""
    bits = values.astype(np.float32).view(np.uint32)
    rounded = bits + 0x7FFF + ((bits >> 16) & 1)
    return (rounded & 0xFFFF0000).astype(np.uint32).view(np.float32)


def bfloat16_bits(values: np.ndarray) -> np.ndarray:
    """The upper 16 bits of float32 values that are exactly representable in bfloat16."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    assert not (bits & 0xFFFF).any(), "value is not a bfloat16"
    return (bits >> 16).astype(np.uint16)


def inputs_for(index: int, case):
    q_heads, kv_heads, q_len, k_len, dim, _, _, mask_kind, offset = case
    rng = np.random.default_rng(20240 + index)
    q = to_bfloat16(rng.standard_normal((1, q_heads, q_len, dim)))
    k = to_bfloat16(rng.standard_normal((1, kv_heads, k_len, dim)) * (0.1 if offset else 1.0) + offset)
    v = to_bfloat16(rng.standard_normal((1, kv_heads, k_len, dim)) + 0.5)
    mask = None
    if mask_kind == "bias":
        mask = rng.standard_normal((1, 1, q_len, k_len)).astype(np.float32)
        mask[..., 3::7] = -np.inf
    elif mask_kind == "key":
        mask = rng.random((1, 1, 1, k_len)) > 0.3
        mask[..., 0] = True
    return q, k, v, mask


def main() -> None:
    arrays = {}
    for index, (name, case) in enumerate(CASES.items()):
        q, k, v, mask = inputs_for(index, case)
        mode, causal = case[5], case[6]
        prepared = pipeline.prequantize(q, k, v, mask=mask, v_quantization=mode, is_causal=causal,
                                        return_lse=True, dtype_name="bfloat16")
        out, lse, captured = pipeline.attend(prepared, return_lse=True, capture=mask is None and not causal)
        arrays.update({
            f"{name}.q": bfloat16_bits(q), f"{name}.k": bfloat16_bits(k), f"{name}.v": bfloat16_bits(v),
            f"{name}.q_codes": prepared.q, f"{name}.k_codes": prepared.k, f"{name}.v_codes": prepared.v,
            f"{name}.q_scale": prepared.q_scale, f"{name}.k_scale": prepared.k_scale,
            f"{name}.v_scale": prepared.v_scale, f"{name}.v_center": prepared.v_center,
            f"{name}.anchor": prepared.anchor, f"{name}.lse_shift": prepared.lse_shift,
            f"{name}.cta_k": np.int32(prepared.cta_k), f"{name}.out": bfloat16_bits(out.astype(np.float32)),
            f"{name}.lse": lse.astype(np.float32),
        })
        if mask is not None:
            arrays[f"{name}.mask"] = mask
        if captured is not None:
            masses = oracle_attention.block_mass(captured, 1, case[0], case[2])
            row_offsets, block_indices, measured, _ = selection.select_retained_mass(masses, 0.9)
            arrays.update({f"{name}.block_mass": masses.astype(np.float32), f"{name}.row_offsets": row_offsets,
                           f"{name}.block_indices": block_indices, f"{name}.measured": np.float64(measured)})
    target = Path(__file__).with_name("vectors.npz")
    np.savez_compressed(target, **arrays)
    print(f"wrote {target} ({target.stat().st_size} bytes, {len(arrays)} arrays)")


if __name__ == "__main__":
    main()
