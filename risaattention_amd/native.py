"""ctypes binding of the gfx950 C-ABI library and the device availability gate.

Takes the place of the reference's nanobind module ``risa_attention._C`` and of
its CUDA gate (reference src/risa_attention/_backend.py:9-32, which refuses HIP
builds of PyTorch): here the gate requires a ROCm build of PyTorch, the in-tree
shared library and a gfx950 device.  Tensors cross the boundary as raw device
pointers plus element strides, so no DLPack capsule is involved.
"""

from __future__ import annotations

import contextlib
import ctypes
import os
from pathlib import Path

import torch

LIBRARY_NAME = "_risa_hip.so"
REQUIRED_ARCH = "gfx950"

_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_c_ptr = ctypes.c_void_p
_c_f32 = ctypes.c_float
_c_f64 = ctypes.c_double
_c_size = ctypes.c_size_t

# name -> (restype, argtypes); must stay in step with include/risa_hip.h
SIGNATURES = {
    "risa_last_error": (ctypes.c_char_p, []),
    "risa_abi_version": (_c_int, []),
    "risa_quantize_qk": (
        _c_int,
        [_c_ptr] * 6 + [_c_int] * 7 + [_c_i64] * 6 + [_c_int, _c_ptr, _c_ptr, _c_ptr],
    ),
    "risa_quantize_v_workspace_bytes": (_c_size, [_c_int] * 5),
    "risa_quantize_v": (
        _c_int,
        [_c_ptr] * 6 + [_c_size] + [_c_int] * 6 + [_c_i64] * 3 + [_c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "risa_quantize_v_noalloc": (
        _c_int,
        [_c_ptr] * 5 + [_c_int] * 6 + [_c_i64] * 3 + [_c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "risa_sdpa_quantize": (
        _c_int,
        [_c_ptr] * 12 + [_c_size] + [_c_int] * 7 + [_c_i64] * 9 + [_c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    ),
    "risa_value_tile_sums": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr]),
    "risa_unpack_order": (None, [_c_ptr]),
    "risa_attention": (
        _c_int,
        [_c_ptr] * 10
        + [_c_i64] * 4
        + [_c_int] * 8
        + [_c_i64] * 3
        + [_c_f32, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr]
        + [_c_ptr, _c_i64, _c_i64, _c_ptr, _c_i64, _c_i64, _c_ptr],
    ),
    "risa_mask_lanes_bytes": (_c_size, [_c_int, _c_int, _c_int, _c_i64, _c_i64] + [_c_int] * 6),
    "risa_prepare_mask_lanes": (
        _c_int,
        [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_ptr],
    ),
    "risa_prepare_key_bias": (
        _c_int,
        [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr],
    ),
    "risa_sdpa_workspace_bytes": (_c_size, [_c_int] * 9 + [_c_i64, _c_i64, _c_int, _c_int]),
    "risa_sdpa": (
        _c_int,
        [_c_ptr] * 5 + [_c_size] + [_c_int] * 7 + [_c_i64] * 12 + [_c_f32, _c_int, _c_int, _c_int]
        + [_c_ptr] + [_c_i64] * 4 + [_c_int] * 4 + [_c_ptr, _c_ptr, _c_ptr],
    ),
    "risa_selector_workspace_size": (_c_size, [_c_int]),
    "risa_select_retained_mass": (_c_int, [_c_ptr] * 8 + [_c_int, _c_int, _c_f64, _c_ptr]),
    "risa_sortable_key_blocks": (_c_int, []),
    "risa_sort_select_retained_mass": (_c_int, [_c_ptr] * 9 + [_c_int, _c_int, _c_f64, _c_ptr]),
    "risa_prepare_key_mask_tiles": (
        _c_int,
        [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr],
    ),
    "risa_lse_shift": (
        _c_int,
        [_c_ptr] * 4 + [_c_int] * 5 + [_c_i64] * 6 + [_c_f32, _c_int, _c_ptr],
    ),
}

_LIBRARY: ctypes.CDLL | None = None
_LOAD_ERROR: Exception | None = None


def library_path() -> Path:
    override = os.environ.get("RISA_HIP_LIBRARY")
    return Path(override) if override else Path(__file__).resolve().parent / LIBRARY_NAME


def load_library(path: Path | str) -> ctypes.CDLL:
    """Another build of the C-ABI library (same entry points), with its signatures bound.
    Raises OSError / AttributeError when the file cannot be loaded or lacks an entry point."""
    loaded = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in SIGNATURES.items():
        function = getattr(loaded, name)
        function.restype = restype
        function.argtypes = argtypes
    return loaded


def _load() -> ctypes.CDLL | None:
    global _LIBRARY, _LOAD_ERROR
    if _LIBRARY is not None or _LOAD_ERROR is not None:
        return _LIBRARY
    try:
        _LIBRARY = load_library(library_path())
    except (OSError, AttributeError) as error:
        _LOAD_ERROR = error
    return _LIBRARY


@contextlib.contextmanager
def using_library(other: ctypes.CDLL):
    """Route every call made inside the block to *other* (from ``load_library``): the paired
    comparison of two builds in one process that the reference's benchmark runners do by
    swapping ``_backend._C`` (reference benchmarks/compare_native.py:40-53).  Sizes cached per
    shape are dropped on the way in and out, since two builds may lay out workspaces differently."""
    global _LIBRARY
    from . import attend

    previous = _load()
    attend.forget_cached_sizes()
    _LIBRARY = other
    try:
        yield other
    finally:
        _LIBRARY = previous
        attend.forget_cached_sizes()


def library() -> ctypes.CDLL:
    """The loaded library; raises when it was not built (there is no fallback)."""
    loaded = _load()
    if loaded is None:
        detail = f": {_LOAD_ERROR}" if _LOAD_ERROR is not None else ""
        raise RuntimeError(
            f"RISA attention HIP extension {library_path()} is not available{detail}; "
            "build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C risaattention_amd/csrc`"
        )
    return loaded


def require_extension() -> None:
    library()


def is_available(device: torch.device | int | str | None = None) -> bool:
    """Whether the HIP kernels can run on *device* (a gfx950 GPU under PyTorch-ROCm)."""
    if not getattr(torch.version, "hip", None) or _load() is None or not torch.cuda.is_available():
        return False
    try:
        resolved = None
        if device is not None:
            resolved = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
            if resolved.type != "cuda":
                return False
        arch = torch.cuda.get_device_properties(resolved).gcnArchName
        return arch.split(":")[0] == REQUIRED_ARCH
    except (AssertionError, RuntimeError, ValueError, AttributeError):
        return False


def check(status: int) -> None:
    """Turn a non-zero status into the RuntimeError the reference binding raises."""
    if status != 0:
        message = library().risa_last_error()
        raise RuntimeError(message.decode("utf-8", "replace") if message else "RISA HIP call failed")


def pointer(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> int:
    """Handle of the device's current stream (the raw query costs a tenth of building a
    ``torch.cuda.Stream`` object, which matters for calls of a few microseconds)."""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


def unpack_order() -> list[int]:
    """Token held at each byte position of a 32-token group of packed V."""
    buffer = (ctypes.c_int32 * 32)()
    library().risa_unpack_order(ctypes.cast(buffer, _c_ptr))
    return list(buffer)
