"""Shared helpers for the parity tests (oracle on CPU vs HIP kernels on the GPU)."""

from __future__ import annotations

import numpy as np
import torch

from oracle import pipeline as oracle_pipeline

DTYPE_NAMES = {torch.float32: "float32", torch.float16: "float16", torch.bfloat16: "bfloat16"}


def to_numpy(tensor: torch.Tensor) -> np.ndarray:
    if tensor.dtype == torch.bool:
        return tensor.detach().cpu().numpy()
    return tensor.detach().float().cpu().numpy()


def mask_to_numpy(mask: torch.Tensor | None):
    """Keep a key-only mask's query extent at 1 so the oracle sees it as key-only."""
    if mask is None:
        return None
    while mask.ndim < 4:
        mask = mask[None]
    if mask.dtype == torch.bool:
        return mask.detach().cpu().numpy()
    return mask.detach().float().cpu().numpy()


def oracle_prequantize(q, k, v, *, attn_mask=None, **kwargs):
    if attn_mask is not None and "query_dependent_mask" not in kwargs:
        # The key tile policy looks at the broadcast view's query stride (reference
        # src/risa_attention/_quantization.py:90), which numpy's copy of the mask loses: a
        # contiguous [..., 1, Lk] mask over a single query keeps a non-zero stride there.
        view = attn_mask.broadcast_to((q.shape[0], q.shape[1], q.shape[2], k.shape[2]))
        kwargs["query_dependent_mask"] = view.stride(-2) != 0
    return oracle_pipeline.prequantize(
        to_numpy(q), to_numpy(k), to_numpy(v), mask=mask_to_numpy(attn_mask),
        dtype_name=DTYPE_NAMES[q.dtype], **kwargs,
    )


def relative_l2(actual, expected) -> float:
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    finite = np.isfinite(expected)
    assert np.array_equal(np.isfinite(actual), finite), "finite patterns differ"
    if not finite.any():
        return 0.0
    denominator = np.sqrt((expected[finite] ** 2).sum())
    return float(np.sqrt(((actual[finite] - expected[finite]) ** 2).sum()) / max(denominator, 1e-30))


def seeded(shape, dtype, seed, device="cuda", offset=0.0, scale=1.0):
    generator = torch.Generator(device="cpu").manual_seed(seed)
    values = torch.randn(shape, generator=generator, dtype=torch.float32) * scale + offset
    return values.to(dtype).to(device)


def load_vectors():
    """tests/golden/vectors.npz as {case: {field: array}}; 16-bit words become the float32
    values of the bfloat16 numbers they hold."""
    from pathlib import Path

    archive = np.load(Path(__file__).with_name("golden") / "vectors.npz")
    cases: dict[str, dict[str, np.ndarray]] = {}
    for key in archive.files:
        case, field = key.split(".", 1)
        value = archive[key]
        if value.dtype == np.uint16:
            value = (value.astype(np.uint32) << 16).view(np.float32)
        cases.setdefault(case, {})[field] = value
    return cases
