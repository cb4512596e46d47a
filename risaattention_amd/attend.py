"""Attention over prepared tensors: the fused one-call path and the split path.

Host-side counterpart of reference src/risa_attention/_execution.py:28-328.
"""

from __future__ import annotations

import functools
import math

import torch

from . import native
from .key_mask import prepare_key_bias, prepare_key_mask_tiles, prepare_mask_lanes
from .policy import (
    DTYPE_CODES,
    MASK_DTYPE_CODES,
    MIN_PATTERN_SPARSITY,
    OUTPUT_LAYOUTS,
    QUERY_BLOCK_SIZE,
    UNAVAILABLE,
    is_available,
    mask_signature,
    select_key_block_size,
    validate_inputs,
)
from .prepare import pad_head_dim, resolve_scale
from .types import PrequantizedInt8Attention, RetainedMassPattern


def output_dtype_for(input_dtype: torch.dtype) -> torch.dtype:
    return torch.bfloat16 if input_dtype == torch.float32 else input_dtype


def ensure_tile_sums(v_codes, v_tile_sum, batch_heads, dim, cta_k):
    """Tile sums of packed V; computed on the device when the caller has none."""
    if v_tile_sum is not None:
        return v_tile_sum
    padded = v_codes.shape[1]
    sums = torch.empty((batch_heads, padded // cta_k, dim), dtype=torch.int32, device=v_codes.device)
    native.check(
        native.library().risa_value_tile_sums(
            v_codes.data_ptr(), sums.data_ptr(), batch_heads, dim, padded, cta_k,
            native.current_stream(v_codes.device),
        )
    )
    return sums


def launch_attention(*, q_codes, k_codes, v_codes, output, q_scale, k_scale, v_scale, v_center,
                     v_tile_sum, cta_k, sm_scale, attn_mask=None, row_offsets=None,
                     block_indices=None, block_mass=None, is_causal=False, lse=None,
                     key_mask_tiles=None):
    """Shape/stride checks of the packed operands, then one ``risa_attention`` call."""
    if q_codes.ndim != 4 or k_codes.ndim != 4 or v_codes.ndim != 2 or output.ndim != 4:
        raise RuntimeError("risa_sdpa_prequantized: q/k/o must be 4D and packed v must be 2D")
    if cta_k not in (64, 128):
        raise RuntimeError("risa_sdpa_prequantized: cta_k must be 64 or 128")
    if output.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError("risa_sdpa_prequantized: output_dtype_code must be 1 (fp16) or 2 (bf16)")
    batch, q_heads, q_len, dim = q_codes.shape
    kv_heads, k_len = k_codes.shape[1], k_codes.shape[2]
    padded = -(-k_len // cta_k) * cta_k
    if cta_k == 128 and dim == 64:
        raise RuntimeError("risa_sdpa_prequantized: cta_k 128 requires head_dim 128 or 256")
    if (row_offsets is None) != (block_indices is None):
        raise RuntimeError(
            "risa_sdpa_prequantized: sparse row offsets and block indices must be provided together"
        )
    if block_mass is not None and row_offsets is not None:
        raise RuntimeError("risa_sdpa_prequantized: block mass requires dense attention")
    if (
        k_codes.shape[0] != batch
        or k_codes.shape[3] != dim
        or tuple(output.shape) != (batch, q_heads, q_len, dim)
        or tuple(v_codes.shape) != (batch * kv_heads * dim, padded)
    ):
        raise RuntimeError("risa_sdpa_prequantized: incompatible quantized tensor shapes")
    if lse is not None and (
        tuple(lse.shape) != (batch, q_heads, q_len) or lse.dtype != torch.float32 or not lse.is_contiguous()
    ):
        raise RuntimeError(
            "risa_sdpa_prequantized: LSE must be contiguous float32 [batch_size,Hq,query_length]"
        )
    hnd = (q_len <= 1 or output.stride(2) == dim) and (q_heads <= 1 or output.stride(1) == q_len * dim)
    nhd = (q_heads <= 1 or output.stride(1) == dim) and (q_len <= 1 or output.stride(2) == q_heads * dim)
    if (
        not q_codes.is_contiguous()
        or not k_codes.is_contiguous()
        or not v_codes.is_contiguous()
        or output.stride(3) != 1
        or not (hnd or nhd)
    ):
        raise RuntimeError(
            "risa_sdpa_prequantized: quantized tensors must be contiguous and "
            "output must use HND- or NHD-contiguous storage"
        )
    mask_args = (None, 0, 0, 0, 0, -1)
    if attn_mask is not None:
        if tuple(attn_mask.shape) != (batch, q_heads, q_len, k_len):
            raise RuntimeError(
                "risa_sdpa_prequantized: attention mask must be expanded to "
                "[batch_size,query_heads,query_length,key_length]"
            )
        if attn_mask.dtype not in MASK_DTYPE_CODES:
            raise RuntimeError(
                "risa_sdpa_prequantized: attention mask must be bool, float16, bfloat16, or float32"
            )
        mask_args = (attn_mask.data_ptr(), *attn_mask.stride(), MASK_DTYPE_CODES[attn_mask.dtype])
    n_qb = -(-q_len // QUERY_BLOCK_SIZE)
    n_kb = padded // cta_k
    if row_offsets is not None:
        if (
            row_offsets.ndim != 1
            or row_offsets.numel() != batch * q_heads * n_qb + 1
            or block_indices.ndim != 1
            or row_offsets.dtype != torch.int32
            or block_indices.dtype != torch.int32
        ):
            raise RuntimeError(
                "risa_sdpa_prequantized: sparse support must be contiguous int32 "
                "CSR with batch_size*Hq*ceil(query_length/128)+1 row offsets"
            )
        if not row_offsets.is_contiguous() or not block_indices.is_contiguous() or block_indices.numel() == 0:
            raise RuntimeError(
                "risa_sdpa_prequantized: sparse CSR tensors must be non-empty and contiguous"
            )
    if block_mass is not None:
        expected = batch * q_heads * n_qb * n_kb + batch * q_heads * q_len * (n_kb * 2 + 2)
        if (
            block_mass.ndim != 1
            or block_mass.numel() != expected
            or block_mass.dtype != torch.float32
            or not block_mass.is_contiguous()
        ):
            raise RuntimeError(
                "risa_sdpa_prequantized: block_mass workspace must contain "
                "mass rows followed by captured tile statistics and softmax state"
            )
    if key_mask_tiles is not None and (
        tuple(key_mask_tiles.shape) != (batch, q_heads, n_kb + 1)
        or key_mask_tiles.dtype != torch.int32
        or not key_mask_tiles.is_contiguous()
    ):
        raise RuntimeError("key mask tiles must be contiguous CUDA int32 [B,Hq,tiles+1]")
    sums = ensure_tile_sums(v_codes, v_tile_sum, batch * kv_heads, dim, cta_k)
    key_bias = prepare_key_bias(attn_mask, cta_k)
    bias_args = (None, 0, 0) if key_bias is None else (key_bias[0].data_ptr(), key_bias[1], key_bias[2])
    mask_lanes = prepare_mask_lanes(attn_mask, cta_k, dim)
    lane_args = (None, 0, 0) if mask_lanes is None else (mask_lanes[0].data_ptr(), mask_lanes[1], mask_lanes[2])
    out_b = output.stride(0) if batch > 1 else q_heads * q_len * dim
    out_n = output.stride(2) if q_len > 1 else dim
    out_h = output.stride(1) if q_heads > 1 else q_len * dim
    native.check(
        native.library().risa_attention(
            q_codes.data_ptr(), k_codes.data_ptr(), v_codes.data_ptr(), output.data_ptr(),
            q_scale.data_ptr(), k_scale.data_ptr(), v_scale.data_ptr(), v_center.data_ptr(),
            sums.data_ptr(), *mask_args, cta_k, batch, q_len, k_len, q_heads, kv_heads, dim,
            out_b, out_n, out_h, float(sm_scale), DTYPE_CODES[output.dtype],
            native.pointer(row_offsets), native.pointer(block_indices), native.pointer(block_mass),
            int(bool(is_causal)), native.pointer(lse), native.pointer(key_mask_tiles),
            *bias_args, *lane_args, native.current_stream(q_codes.device),
        )
    )


@functools.lru_cache(maxsize=256)
def sdpa_workspace_bytes(*extents) -> int:
    """``risa_sdpa_workspace_bytes`` of the library (a pure function of its integer
    arguments), remembered per argument tuple: serving loops ask for the same few shapes."""
    return native.library().risa_sdpa_workspace_bytes(*extents)


def forget_cached_sizes() -> None:
    """Drop the remembered workspace sizes (they belong to the library that computed them)."""
    sdpa_workspace_bytes.cache_clear()


def execute_dense_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    scale: float | None = None,
    attn_mask: torch.Tensor | None = None,
    use_midpoint_affine: bool = False,
    is_causal: bool = False,
    sparse_pattern: RetainedMassPattern | None = None,
    output_layout: str = "hnd",
) -> torch.Tensor:
    """Quantize and attend in one native call; the intermediate buffers are sections of
    one workspace that lives only for the call (reference _execution.py:28-134 over
    ``_C.risa_sdpa``).  With ``sparse_pattern`` the attention walks the pattern's key tiles
    (the reuse call of the sparse path); a pattern under 5 % sparsity runs dense."""
    if output_layout not in OUTPUT_LAYOUTS:
        raise ValueError(f"output_layout must be one of {OUTPUT_LAYOUTS}, got {output_layout!r}")
    attn_mask = validate_inputs(q, k, v, attn_mask)
    original_dim, input_dtype = q.shape[-1], q.dtype
    q, k, v, dim = pad_head_dim(q, k, v)
    attention_scale = resolve_scale(scale, original_dim)
    batch, q_heads, q_len, _ = q.shape
    kv_heads, k_len = k.shape[1], k.shape[2]
    query_mask = attn_mask is not None and attn_mask.stride(-2) != 0
    cta_k = select_key_block_size(dim, k_len, has_mask=query_mask)
    lib = native.library()
    csr = (None, None)
    if sparse_pattern is not None:
        check_pattern_for(sparse_pattern, batch=batch, q_heads=q_heads, q_len=q_len, k_len=k_len, cta_k=cta_k,
                          attention_scale=attention_scale, is_causal=bool(is_causal), attn_mask=attn_mask,
                          device=q.device)
        if sparse_pattern.sparsity >= MIN_PATTERN_SPARSITY:
            csr = (sparse_pattern.row_offsets.data_ptr(), sparse_pattern.block_indices.data_ptr())
    out_dtype = output_dtype_for(input_dtype)
    if output_layout == "nhd":
        output = torch.empty(batch, q_len, q_heads, dim, dtype=out_dtype, device=q.device).permute(0, 2, 1, 3)
    else:
        output = torch.empty(batch, q_heads, q_len, dim, dtype=out_dtype, device=q.device)
    if attn_mask is None:
        mask_args = (None, 0, 0, 0, 0, -1, 1, 1)
    else:
        mask_args = (attn_mask.data_ptr(), *attn_mask.stride(), MASK_DTYPE_CODES[attn_mask.dtype],
                     batch if attn_mask.stride(0) != 0 else 1, q_heads if attn_mask.stride(1) != 0 else 1)
    # the size query takes the mask's dtype, query and key strides and own extents
    workspace = torch.empty(
        sdpa_workspace_bytes(batch, q_heads, q_len, kv_heads, k_len, dim, cta_k, int(use_midpoint_affine),
                             mask_args[5], mask_args[3], mask_args[4], mask_args[6], mask_args[7]),
        dtype=torch.uint8, device=q.device)
    native.check(
        lib.risa_sdpa(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), output.data_ptr(), workspace.data_ptr(),
            workspace.numel(), batch, q_heads, q_len, kv_heads, k_len, dim, cta_k,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
            v.stride(0), v.stride(1), v.stride(2), output.stride(0), output.stride(2), output.stride(1),
            attention_scale, DTYPE_CODES[input_dtype], DTYPE_CODES[output.dtype],
            int(use_midpoint_affine), *mask_args, int(bool(is_causal)), *csr,
            native.current_stream(q.device),
        )
    )
    if original_dim != dim:
        output = output[..., :original_dim]
    return output.float() if input_dtype == torch.float32 else output


def check_pattern_for(pattern: RetainedMassPattern, *, batch, q_heads, q_len, k_len, cta_k,
                      attention_scale, is_causal, attn_mask, device) -> None:
    """A pattern may only drive the attention problem it was built for
    (reference _execution.py:180-228)."""
    if not isinstance(pattern, RetainedMassPattern):
        raise TypeError("sparse_pattern must be returned by build_retained_mass_pattern")
    if pattern.is_causal != is_causal:
        raise ValueError("sparse pattern and attention call must use the same is_causal")
    if pattern.mask_signature != mask_signature(attn_mask):
        raise ValueError("sparse pattern mask has changed; rebuild the pattern")
    expected = (batch, q_heads, q_len, k_len, QUERY_BLOCK_SIZE, cta_k)
    actual = (pattern.batch_size, pattern.q_heads, pattern.q_length, pattern.kv_length,
              pattern.query_block_size, pattern.key_block_size)
    if actual != expected:
        raise ValueError(
            f"sparse pattern metadata does not match packed attention: expected {expected}, got {actual}"
        )
    if not math.isclose(pattern.attention_scale, attention_scale, rel_tol=1e-7, abs_tol=0.0):
        raise ValueError("sparse pattern and attention call must use the same scale")
    if pattern.row_offsets.device != device or pattern.block_indices.device != device:
        raise ValueError("sparse pattern and packed tensors must be on the same CUDA device")
    for index in (pattern.row_offsets, pattern.block_indices):
        if index.dtype != torch.int32 or not index.is_contiguous():
            raise TypeError("sparse CSR row offsets and block indices must be contiguous int32")


def check_pattern(quantized: PrequantizedInt8Attention, pattern: RetainedMassPattern) -> None:
    batch, q_heads, q_len = quantized.q.shape[:3]
    check_pattern_for(pattern, batch=batch, q_heads=q_heads, q_len=q_len, k_len=quantized.k.shape[2],
                      cta_k=quantized.cta_k, attention_scale=quantized.attention_scale,
                      is_causal=quantized.is_causal, attn_mask=quantized.attn_mask,
                      device=quantized.q.device)


def int8_attention_from_prequantized(
    quantized: PrequantizedInt8Attention,
    *,
    sparse_pattern: RetainedMassPattern | None = None,
    output_layout: str = "hnd",
    _block_mass: torch.Tensor | None = None,
    return_lse: bool = False,
) -> torch.Tensor | tuple[torch.Tensor, torch.Tensor]:
    """Run INT8 attention on packed operands.

    The result is always logically ``[batch, heads, sequence, head_dim]``;
    ``output_layout="nhd"`` stores it sequence-major so that
    ``out.transpose(1, 2).reshape(batch, sequence, -1)`` is a view.  A sparse
    pattern that keeps more than 95% of the tiles is ignored (dense run).
    """
    if not isinstance(quantized, PrequantizedInt8Attention):
        raise TypeError(
            f"quantized must be returned by prequantize_int8_attention, got {type(quantized).__name__}"
        )
    if output_layout not in OUTPUT_LAYOUTS:
        raise ValueError(f"output_layout must be one of {OUTPUT_LAYOUTS}, got {output_layout!r}")
    if quantized.kv_permuted and (sparse_pattern is not None or _block_mass is not None):
        raise ValueError("permuted K/V is supported only by dense attention")
    if return_lse and quantized.lse_shift is None:
        raise ValueError("prequantize with return_lse=True to retain the K-anchor correction")
    device = quantized.q.device
    packed = (quantized.k, quantized.v, quantized.q_scale, quantized.k_scale, quantized.v_scale,
              quantized.v_center)
    if not quantized.q.is_cuda:
        raise ValueError("prequantized INT8 attention tensors must be on a CUDA device")
    if any(t.device != device for t in packed):
        raise ValueError("prequantized INT8 attention tensors must be on the same CUDA device")
    if quantized.attn_mask is not None and quantized.attn_mask.device != device:
        raise ValueError("attn_mask must be on the same CUDA device as the packed tensors")
    if sparse_pattern is not None:
        check_pattern(quantized, sparse_pattern)
        if sparse_pattern.sparsity < MIN_PATTERN_SPARSITY:
            sparse_pattern = None
    batch, q_heads, q_len, dim = quantized.q.shape
    if _block_mass is not None:
        if sparse_pattern is not None:
            raise ValueError("block mass requires dense attention")
        n_kb = math.ceil(quantized.k.shape[2] / quantized.cta_k)
        expected = batch * q_heads * math.ceil(q_len / QUERY_BLOCK_SIZE) * n_kb
        expected += batch * q_heads * q_len * (n_kb * 2 + 2)
        if (
            _block_mass.ndim != 1
            or _block_mass.numel() != expected
            or _block_mass.dtype != torch.float32
            or _block_mass.device != device
            or not _block_mass.is_contiguous()
        ):
            raise ValueError(
                f"block mass workspace must be contiguous CUDA float32 with {expected} elements"
            )
    if not is_available(device):
        raise RuntimeError(UNAVAILABLE)

    dtype = output_dtype_for(quantized.input_dtype)
    if output_layout == "nhd":
        output = torch.empty(batch, q_len, q_heads, dim, dtype=dtype, device=device).permute(0, 2, 1, 3)
    else:
        output = torch.empty(batch, q_heads, q_len, dim, dtype=dtype, device=device)
    lse = torch.empty((batch, q_heads, q_len), dtype=torch.float32, device=device) if return_lse else None
    tiles = None
    if sparse_pattern is None and _block_mass is None:
        tiles = prepare_key_mask_tiles(quantized.attn_mask, quantized.cta_k, q_len,
                                       quantized.attention_scale, quantized.is_causal)
    launch_attention(
        q_codes=quantized.q, k_codes=quantized.k, v_codes=quantized.v, output=output,
        q_scale=quantized.q_scale, k_scale=quantized.k_scale, v_scale=quantized.v_scale,
        v_center=quantized.v_center, v_tile_sum=quantized.v_tile_sum, cta_k=quantized.cta_k,
        sm_scale=quantized.attention_scale, attn_mask=quantized.attn_mask,
        row_offsets=None if sparse_pattern is None else sparse_pattern.row_offsets,
        block_indices=None if sparse_pattern is None else sparse_pattern.block_indices,
        block_mass=_block_mass, is_causal=quantized.is_causal, lse=lse, key_mask_tiles=tiles,
    )
    if quantized.original_head_dim != dim:
        output = output[..., : quantized.original_head_dim]
    if quantized.input_dtype == torch.float32:
        output = output.float()
    if return_lse:
        lse.add_(quantized.lse_shift)
        return output, lse
    return output
