"""ComfyUI adapter for ``risaattention_amd`` (MI355X / gfx950).

Behaviour follows reference comfyui-risa-attention/node.py:1-379 and docs/comfyui.md:
one node clones a MODEL and installs an optimized-attention callable in one of three
modes; the sparse mode keeps frozen retained-mass patterns for the duration of one
sampling run, one per (conditioning branch, attention call ordinal, tensor
configuration), builds each on its first eligible call and reuses it afterwards.
Calls the sparse path cannot serve (masks, cross-attention, compilation) run dense
INT8 attention, never PyTorch attention.
"""

from __future__ import annotations

import importlib
import threading
from typing import NamedTuple

import torch

_ATTENTION_MODES = ["pytorch_attention", "int8_attention", "sparse_int8_attention"]
_WRAPPER_KEY = "risa_sparse_attention"
# A pattern that drops fewer tiles than this does not repay its index traversal.
_MIN_PATTERN_SPARSITY = 0.05

_MISSING = object()     # no pattern stored under the key yet
_DENSE_ONLY = object()  # the key is served by dense attention for the rest of the run

_backend_module = None


def _load_risa_attention():
    """The attention library, imported once and checked against the active GPU."""
    global _backend_module
    if _backend_module is None:
        try:
            module = importlib.import_module("risaattention_amd")
        except (ImportError, OSError) as error:
            raise RuntimeError(
                "risaattention_amd is not importable from ComfyUI's Python environment. "
                "Put the repository on its path and build the HIP library once with "
                "`make -C risaattention_amd/csrc` (hipcc, --offload-arch=gfx950)."
            ) from error
        if not module.int8_attention_is_available():
            raise RuntimeError(
                "risaattention_amd needs PyTorch-ROCm, its built HIP library and a gfx950 GPU "
                "(MI355X); at least one of them is missing here."
            )
        _backend_module = module
    return _backend_module


# ---------------------------------------------------------------------------
# ComfyUI tensor convention <-> [batch, heads, tokens, channels]
# ---------------------------------------------------------------------------
class _Heads(NamedTuple):
    batch: int
    heads: int
    channels: int
    merge: bool  # ComfyUI wants [batch, tokens, heads * channels] back

    def restore(self, output):
        if not self.merge:
            return output
        return output.transpose(1, 2).reshape(self.batch, -1, self.heads * self.channels)

    @property
    def output_layout(self):
        # Token-major storage makes the merge above a view instead of a copy.
        return "nhd" if self.merge else "hnd"


def _split(tensor, batch, heads, channels):
    return tensor.unsqueeze(3).reshape(batch, -1, heads, channels).transpose(1, 2)


def _to_head_major(q, k, v, heads, mask, skip_reshape, skip_output_reshape, enable_gqa):
    batch = q.shape[0]
    if skip_reshape:
        channels = q.shape[-1]
    else:
        channels = q.shape[-1] // heads
        # Under grouped-query attention K and V carry fewer heads than Q.
        k_heads = k.shape[-1] // channels if enable_gqa else heads
        v_heads = v.shape[-1] // channels if enable_gqa else heads
        q = _split(q, batch, heads, channels)
        k = _split(k, batch, k_heads, channels)
        v = _split(v, batch, v_heads, channels)
    if mask is not None:
        if mask.ndim == 2:  # [queries, keys]
            mask = mask.unsqueeze(0)
        if mask.ndim == 3:  # [batch, queries, keys]
            mask = mask.unsqueeze(1)
    return q, k, v, mask, _Heads(batch, heads, channels, not skip_output_reshape)


def _hashable(value):
    if value is None:
        return ()
    items = tuple(value) if isinstance(value, (list, tuple)) else (value,)
    try:
        hash(items)
    except TypeError:
        items = tuple(id(item) for item in items)
    return items


def _transformer_options(args, kwargs):
    options = kwargs.get("transformer_options")
    if isinstance(options, dict):
        return options
    marks = ("sigmas", "sample_sigmas", "optimized_attention_override")
    for candidate in reversed(args):
        if isinstance(candidate, dict) and any(mark in candidate for mark in marks):
            return candidate
    return {}


# ---------------------------------------------------------------------------
# Pattern store of one sampling run
# ---------------------------------------------------------------------------
class _SparsePatternState:
    """Patterns of one sampling run, keyed by conditioning branch and call ordinal.

    ``OUTER_SAMPLE`` opens and closes the store (nested runs share it; it is emptied
    when the outermost one begins and ends, also on exceptions); ``DIFFUSION_MODEL``
    pushes a frame per transformer forward, which numbers the attention calls made
    inside it.  Frames are per thread.
    """

    def __init__(self, theta: float):
        self.theta = float(theta)
        self.patterns = {}
        self._open_sessions = 0
        self._thread = threading.local()

    # -- scopes ------------------------------------------------------------
    def begin_session(self):
        if self._open_sessions == 0:
            self.patterns.clear()
        self._open_sessions += 1

    def end_session(self):
        if self._open_sessions > 0:
            self._open_sessions -= 1
        if self._open_sessions == 0:
            self.patterns.clear()

    def _frames(self):
        frames = getattr(self._thread, "frames", None)
        if frames is None:
            frames = self._thread.frames = []
        return frames

    def begin_forward(self, transformer_options):
        branch = (_hashable(transformer_options.get("uuids")),
                  _hashable(transformer_options.get("cond_or_uncond")))
        self._frames().append({"branch": branch, "ordinal": 0})

    def end_forward(self):
        frames = self._frames()
        if frames:
            frames.pop()

    def outer_sample_wrapper(self, executor, *args, **kwargs):
        self.begin_session()
        try:
            return executor(*args, **kwargs)
        finally:
            self.end_session()

    def diffusion_model_wrapper(self, executor, *args, **kwargs):
        self.begin_forward(_transformer_options(args, kwargs))
        try:
            return executor(*args, **kwargs)
        finally:
            self.end_forward()

    # -- lookup --------------------------------------------------------------
    def next_pattern_key(self, q, k, v, mask, scale):
        """Key of this attention call, or None when it must run dense.

        The ordinal advances for every call inside a forward, eligible or not, so
        the numbering of a layer does not depend on what other layers were given.
        """
        frames = self._frames()
        if self._open_sessions == 0 or not frames:
            return None
        frame = frames[-1]
        ordinal = frame["ordinal"]
        frame["ordinal"] = ordinal + 1
        self_attention = q.ndim == k.ndim == v.ndim == 4 and q.shape[2] == k.shape[2]
        if mask is not None or not self_attention or torch.compiler.is_compiling():
            return None
        return (frame["branch"], ordinal, q.device.type, q.device.index, q.dtype,
                tuple(q.shape), tuple(k.shape), tuple(v.shape),
                None if scale is None else float(scale))

    def get(self, key):
        return self.patterns.get(key, _MISSING)

    def put(self, key, pattern):
        self.patterns[key] = pattern if pattern.sparsity >= _MIN_PATTERN_SPARSITY else _DENSE_ONLY


# ---------------------------------------------------------------------------
# Attention callables with ComfyUI's optimized-attention signature
# ---------------------------------------------------------------------------
def make_int8_attention_function(backend):
    """Dense INT8 attention; carries no sampling state."""
    dense = backend.int8_attention
    prequantize = backend.prequantize_int8_attention
    attend = backend.int8_attention_from_prequantized

    def risa_int8_attention(q, k, v, heads, mask=None, attn_precision=None, skip_reshape=False,
                            skip_output_reshape=False, **kwargs):
        q, k, v, mask, shape = _to_head_major(q, k, v, heads, mask, skip_reshape, skip_output_reshape,
                                              kwargs.get("enable_gqa", False))
        return shape.restore(dense(q, k, v, scale=kwargs.get("scale"), attn_mask=mask))

    def risa_int8_attention_containers(q, k, v, heads, mask=None, attn_precision=None, skip_reshape=False,
                                       skip_output_reshape=False, **kwargs):
        # Tensor containers hand over ownership: quantise first, then let the
        # floating-point tensors go before the attention output is allocated.
        q, k, v = q.take(), k.take(), v.take()
        q, k, v, mask, shape = _to_head_major(q, k, v, heads, mask, skip_reshape, skip_output_reshape,
                                              kwargs.get("enable_gqa", False))
        packed = prequantize(q, k, v, scale=kwargs.get("scale"), attn_mask=mask)
        del q, k, v
        return shape.restore(attend(packed, output_layout=shape.output_layout))

    risa_int8_attention.container_function = risa_int8_attention_containers
    return risa_int8_attention


def make_sparse_attention_function(backend, state=None):
    """Retained-mass sparse INT8 attention with patterns frozen per sampling run."""
    state = state if state is not None else _SparsePatternState(theta=0.99)
    dense = backend.int8_attention
    reuse = backend.sparse_int8_attention
    construct = backend.construct_sparse_int8_attention
    prequantize = backend.prequantize_int8_attention
    attend = backend.int8_attention_from_prequantized
    construct_packed = backend.construct_sparse_int8_attention_from_prequantized

    def lookup(q, k, v, mask, scale):
        key = state.next_pattern_key(q, k, v, mask, scale)
        return key, (_DENSE_ONLY if key is None else state.get(key))

    def risa_sparse_attention(q, k, v, heads, mask=None, attn_precision=None, skip_reshape=False,
                              skip_output_reshape=False, **kwargs):
        q, k, v, mask, shape = _to_head_major(q, k, v, heads, mask, skip_reshape, skip_output_reshape,
                                              kwargs.get("enable_gqa", False))
        scale = kwargs.get("scale")
        key, pattern = lookup(q, k, v, mask, scale)
        if pattern is _DENSE_ONLY:
            output = dense(q, k, v, scale=scale, attn_mask=mask)
        elif pattern is _MISSING:
            output, pattern = construct(q, k, v, theta=state.theta, scale=scale,
                                        output_layout=shape.output_layout)
            state.put(key, pattern)
        else:
            output = reuse(q, k, v, pattern, scale=scale, output_layout=shape.output_layout)
        return shape.restore(output)

    def risa_sparse_attention_containers(q, k, v, heads, mask=None, attn_precision=None, skip_reshape=False,
                                         skip_output_reshape=False, **kwargs):
        q, k, v = q.take(), k.take(), v.take()
        q, k, v, mask, shape = _to_head_major(q, k, v, heads, mask, skip_reshape, skip_output_reshape,
                                              kwargs.get("enable_gqa", False))
        scale = kwargs.get("scale")
        key, pattern = lookup(q, k, v, mask, scale)
        packed = prequantize(q, k, v, scale=scale, attn_mask=mask)
        del q, k, v
        if pattern is _MISSING:
            output, pattern = construct_packed(packed, theta=state.theta, output_layout=shape.output_layout)
            state.put(key, pattern)
        else:
            output = attend(packed, sparse_pattern=None if pattern is _DENSE_ONLY else pattern,
                            output_layout=shape.output_layout)
        return shape.restore(output)

    risa_sparse_attention.container_function = risa_sparse_attention_containers
    risa_sparse_attention.sparse_state = state
    return risa_sparse_attention


# ---------------------------------------------------------------------------
# The node
# ---------------------------------------------------------------------------
class RISAAttentionNode:
    """Returns a clone of the MODEL with the chosen attention installed."""

    RETURN_TYPES = ("MODEL",)
    RETURN_NAMES = ("model",)
    FUNCTION = "patch_model"
    CATEGORY = "RISA Attention"
    DESCRIPTION = "PyTorch attention, dense RISA INT8 attention, or retained-mass sparse RISA attention."

    @classmethod
    def INPUT_TYPES(cls):
        theta = {
            "default": 0.99,
            "min": 0.9,
            "max": 1.0,
            "step": 0.001,
            "tooltip": "Share of the attention mass every frozen pattern keeps per query block.",
        }
        return {
            "required": {
                "model": ("MODEL",),
                "attention": (_ATTENTION_MODES, {"default": "sparse_int8_attention"}),
                "theta": ("FLOAT", theta),
            }
        }

    def patch_model(self, model, attention, theta):
        if attention not in _ATTENTION_MODES:
            raise ValueError(f"Unsupported attention mode: {attention}")
        patched = model.clone()
        if attention == "pytorch_attention":
            # The attention library is not imported in this mode.
            function = importlib.import_module("comfy.ldm.modules.attention").attention_pytorch
        elif attention == "int8_attention":
            function = make_int8_attention_function(_load_risa_attention())
        else:
            scopes = importlib.import_module("comfy.patcher_extension").WrappersMP
            state = _SparsePatternState(theta=theta)
            function = make_sparse_attention_function(_load_risa_attention(), state)
            patched.add_wrapper_with_key(scopes.OUTER_SAMPLE, _WRAPPER_KEY, state.outer_sample_wrapper)
            patched.add_wrapper_with_key(scopes.DIFFUSION_MODEL, _WRAPPER_KEY, state.diffusion_model_wrapper)
        patched.set_model_optimized_attention(function)
        return (patched,)
