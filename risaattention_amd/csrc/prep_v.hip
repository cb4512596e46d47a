// Launchers of the V preparation kernels (prep_v_kernels.hpp).

#include "prep_v_kernels.hpp"

namespace risa {
namespace {

template <int DT> int run(const ValueArgs& a, hipStream_t stream) {
  const Workspace w = carve(a.workspace, a.batch, a.heads, a.length, a.head_dim, a.midpoint_affine);
  const int bh = a.batch * a.heads;
  const int chunks = range_chunks(a.length);
  const int rows = bh * a.head_dim;
  const int groups = rows / 8;
  dim3 range_grid((chunks + 3) / 4, bh);
  // At most 64 partial ranges (sequences up to 4096 tokens): the code pass reduces
  // them itself and no separate parameter launch is needed.
  const bool fuse_params = chunks <= 64;
  const FusedParams fused{w.part_max, w.part_min, a.scale, a.center, w.inverse, w.midpoint, chunks};
  if (a.midpoint_affine) {
    value_range_kernel<DT, true><<<range_grid, 256, 0, stream>>>(
        a.v, w.part_max, w.part_min, a.length, a.head_dim, a.heads, chunks, a.stride_b, a.stride_h,
        a.stride_n);
    if (!fuse_params)
      value_params_kernel<true><<<(groups + 3) / 4, 256, 0, stream>>>(
          w.part_max, w.part_min, a.scale, a.center, w.inverse, w.midpoint, a.head_dim, chunks, groups);
  } else {
    value_range_kernel<DT, false><<<range_grid, 256, 0, stream>>>(
        a.v, w.part_max, w.part_min, a.length, a.head_dim, a.heads, chunks, a.stride_b, a.stride_h,
        a.stride_n);
    if (!fuse_params)
      value_params_kernel<false><<<(groups + 3) / 4, 256, 0, stream>>>(
          w.part_max, w.part_min, a.scale, a.center, w.inverse, w.midpoint, a.head_dim, chunks, groups);
  }
  const int position_blocks = (a.padded + kCodeBlockPositions - 1) / kCodeBlockPositions;
  const dim3 code_grid(static_cast<unsigned>(position_blocks) * bh);
#define RISA_CODES_DIM(TILE, PARAMS, DIM)                                                          \
  value_codes_kernel<DT, TILE, PARAMS, DIM><<<code_grid, 256, 0, stream>>>(                        \
      a.v, a.codes, a.tile_sum, w.inverse, w.midpoint, a.length, a.padded, a.heads, a.stride_b,    \
      a.stride_h, a.stride_n, a.permutation, fused, position_blocks)
#define RISA_CODES(TILE, PARAMS)                                                                   \
  do {                                                                                             \
    if (a.head_dim == 64)                                                                          \
      RISA_CODES_DIM(TILE, PARAMS, 64);                                                            \
    else if (a.head_dim == 128)                                                                    \
      RISA_CODES_DIM(TILE, PARAMS, 128);                                                           \
    else                                                                                           \
      RISA_CODES_DIM(TILE, PARAMS, 256);                                                           \
  } while (0)
  if (a.cta_k == 128) {
    if (!fuse_params)
      RISA_CODES(128, kParamsStored);
    else if (a.midpoint_affine)
      RISA_CODES(128, kParamsAffine);
    else
      RISA_CODES(128, kParamsAbsmax);
  } else {
    if (!fuse_params)
      RISA_CODES(64, kParamsStored);
    else if (a.midpoint_affine)
      RISA_CODES(64, kParamsAffine);
    else
      RISA_CODES(64, kParamsAbsmax);
  }
#undef RISA_CODES_DIM
#undef RISA_CODES
  if (a.midpoint_affine) {
    if (a.length <= kFusedCenterMaxLength) {
      dim3 center_grid(a.head_dim / 8, bh);
      value_center_fused_kernel<DT><<<center_grid, summation_threads(a.length), 0, stream>>>(
          a.v, w.inverse, w.midpoint, a.center, a.length, a.head_dim, a.heads, a.stride_b, a.stride_h,
          a.stride_n, a.permutation);
    } else {
      const int threads = summation_threads(a.length);
      const int per_block = 256 / (a.head_dim / 4);
      dim3 residual_grid(threads / per_block, bh);
      value_residual_kernel<DT><<<residual_grid, 256, 0, stream>>>(
          a.v, w.partial, w.inverse, w.midpoint, a.length, a.head_dim, a.heads, threads, a.stride_b,
          a.stride_h, a.stride_n, a.permutation);
      value_center_from_partials_kernel<<<rows, threads, 0, stream>>>(
          w.partial, w.inverse, w.midpoint, a.center, rows, threads, a.length);
    }
  }
  return check_launch("risa_quantize_v");
}

}  // namespace

size_t value_workspace_bytes(int batch, int heads, int length, int head_dim, bool midpoint_affine) {
  return carve(nullptr, batch, heads, length, head_dim, midpoint_affine).bytes;
}

int launch_quantize_v(const ValueArgs& a, hipStream_t stream) {
  if (a.workspace_bytes <
      value_workspace_bytes(a.batch, a.heads, a.length, a.head_dim, a.midpoint_affine)) {
    return fail("risa_quantize_v: workspace is too small");
  }
  if (a.dtype == kF32) return run<kF32>(a, stream);
  if (a.dtype == kF16) return run<kF16>(a, stream);
  return run<kBF16>(a, stream);
}

int launch_value_tile_sums(const int8_t* codes, int32_t* tile_sum, int rows_bh, int head_dim,
                           int padded, int cta_k, hipStream_t stream) {
  dim3 grid((padded + 255) / 256, rows_bh);
  if (cta_k == 128)
    value_tile_sum_kernel<128><<<grid, 256, 0, stream>>>(codes, tile_sum, head_dim, padded);
  else
    value_tile_sum_kernel<64><<<grid, 256, 0, stream>>>(codes, tile_sum, head_dim, padded);
  return check_launch("risa_value_tile_sums");
}

}  // namespace risa
