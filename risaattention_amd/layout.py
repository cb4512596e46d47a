"""Physical order of the packed V matrix.

``v`` of :class:`PrequantizedInt8Attention` is ``[B*Hkv*D, padded_keys]`` int8.
Inside every aligned group of 32 tokens, byte ``16*h + 4*b + r`` holds token
``8*b + 4*h + r`` (``h`` in 0..1, ``b``, ``r`` in 0..3).  A lane of the
32x32x32 INT8 matrix instruction that belongs to half ``h`` of the wavefront
owns exactly those sixteen keys of a transposed score tile, so the sixteen
bytes it reads from a V row are the ones its probabilities multiply.  (The
reference stores a 16-token order derived from the NVIDIA mma fragment,
csrc/kernels/quantize_v_impl.cuh:47-52; the codes themselves are identical.)
"""

from __future__ import annotations

import torch

GROUP = 32


def position_to_token() -> list[int]:
    order = [0] * GROUP
    for token in range(GROUP):
        b, h, r = token >> 3, (token >> 2) & 1, token & 3
        order[16 * h + 4 * b + r] = token
    return order


def unpack_values(packed: torch.Tensor) -> torch.Tensor:
    """Packed V -> token order (column n is token n)."""
    rows, padded = packed.shape
    tokens = torch.tensor(position_to_token(), device=packed.device)
    out = torch.empty_like(packed).view(rows, padded // GROUP, GROUP)
    out[..., tokens] = packed.view(rows, padded // GROUP, GROUP)
    return out.view(rows, padded)


def pack_values(logical: torch.Tensor) -> torch.Tensor:
    """Token order -> packed V."""
    rows, padded = logical.shape
    tokens = torch.tensor(position_to_token(), device=logical.device)
    return logical.view(rows, padded // GROUP, GROUP)[..., tokens].reshape(rows, padded).contiguous()
