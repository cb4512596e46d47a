// Q/K/V preparation in two launches (three beyond 4096 tokens, one up to 1024 tokens).
//
// The separate preparation kernels (prep_qk.hip, prep_v.hip) are five to seven
// launches whose order is fixed by data: anchor -> K codes, V range -> V parameters
// -> V codes.  Up to a few thousand tokens every one of them runs for about five
// microseconds however little it does, and the chain is longer than the attention
// kernel; for long sequences the tail of each launch leaves most of the GPU idle.
// The work has only two levels of dependence, so two launches are enough:
//   stage 1  K anchor | Q codes | V partial ranges      (independent workgroups)
//   stage 2  K codes (needs the anchor) | V codes (reduce the partial ranges themselves)
// With more than 64 partial ranges per channel (beyond 4096 tokens) the small
// parameter kernel runs between the stages instead of inside every code workgroup.
// A workgroup finds its role from its index; every role runs the same device
// function as the stand-alone kernel, so results are bit-identical.  Used when K and V
// have the same extents (always, for callers of the attention API).

#include "prep_qk_kernels.hpp"
#include "prep_v_kernels.hpp"

namespace risa {
namespace {

struct FusedArgs {
  QkArgs qk;
  ValueArgs v;
  float* part_max;
  float* part_min;
  float* inverse;
  float* midpoint;
  float* partial;
  int q_slices, q_blocks, anchor_blocks, range_groups, chunks;
  int key_tiles, key_blocks, code_blocks_x, kv;
  int center_blocks;  // midpoint_affine centres computed inside the second launch (0: separate kernels)
  int residual_blocks_x;  // long midpoint_affine sequences: the residual pass rides in the second launch
  int q_wide, k_wide;
};

template <int DT, int DK, int ROT, bool AFFINE>
__global__ __launch_bounds__(256) void prepare_stage1_kernel(const FusedArgs a) {
  // The anchor detectors go first: each is one long-running workgroup.
  int block = blockIdx.x;
  if (block < a.anchor_blocks) {
    detect_anchor_block<DT>(a.qk.k, a.qk.anchors, a.qk.k_len, a.qk.head_dim, a.qk.kv_heads,
                            a.qk.k_stride_b, a.qk.k_stride_h, a.qk.k_stride_n, a.qk.permutation,
                            block % a.qk.kv_heads, block / a.qk.kv_heads);
    return;
  }
  block -= a.anchor_blocks;
  // then the V range walks (long chunks on long sequences), then the many short Q blocks
  const int range_blocks = a.range_groups * a.kv;
  if (block < range_blocks) {
    value_range_block<DT, AFFINE>(a.v.v, a.part_max, a.part_min, a.v.length, a.v.head_dim, a.v.heads,
                                  a.chunks, a.v.stride_b, a.v.stride_h, a.v.stride_n,
                                  block % a.range_groups, block / a.range_groups);
    return;
  }
  block -= range_blocks;
  const int slice = block % a.q_slices;
  const int rest = block / a.q_slices;
  quantize_q_block<DT, DK, ROT>(a.qk.q, a.qk.q_codes, a.qk.q_scale, a.qk.q_len, a.qk.q_heads,
                                a.q_slices * 8, a.qk.q_stride_b, a.qk.q_stride_h, a.qk.q_stride_n,
                                a.q_wide, slice, rest % a.qk.q_heads, rest / a.qk.q_heads);
}

template <int DT, int DK, int CTA_K, int ROT, int PARAMS>
__global__ __launch_bounds__(256) void prepare_stage2_kernel(const FusedArgs a) {
  int block = blockIdx.x;
  if (block < a.key_blocks) {
    // half a key tile per workgroup: two wavefronts for each of its two scale groups
    const int part = block & 1;
    const int tile = (block >> 1) % a.key_tiles;
    const int rest = (block >> 1) / a.key_tiles;
    quantize_k_block<DT, DK, CTA_K, ROT>(a.qk.k, a.qk.k_codes, a.qk.k_scale, a.qk.anchors[rest], a.qk.k_len,
                                         a.qk.kv_heads, a.key_tiles * 4, a.qk.k_stride_b, a.qk.k_stride_h,
                                         a.qk.k_stride_n, a.k_wide, a.qk.permutation, tile, part,
                                         rest % a.qk.kv_heads, rest / a.qk.kv_heads);
    return;
  }
  block -= a.key_blocks;
  const FusedParams fused{a.part_max, a.part_min, a.v.scale, a.v.center, a.inverse, a.midpoint, a.chunks};
  if constexpr (PARAMS == kParamsAffine) {
    // the centre blocks come first: each walks the whole sequence of its eight channels
    if (block < a.center_blocks) {
      const int octets = a.v.head_dim / 8;
      value_center_block<DT>(a.v.v, fused, a.v.length, a.v.head_dim, a.v.heads, a.v.stride_b, a.v.stride_h,
                             a.v.stride_n, a.v.permutation, block % octets, block / octets);
      return;
    }
    block -= a.center_blocks;
  }
  if constexpr (PARAMS == kParamsStored) {
    const int residual_blocks = a.residual_blocks_x * a.kv;
    if (block < residual_blocks) {
      value_residual_block<DT>(a.v.v, a.partial, a.inverse, a.midpoint, a.v.length, a.v.head_dim, a.v.heads,
                               summation_threads(a.v.length), a.v.stride_b, a.v.stride_h, a.v.stride_n,
                               a.v.permutation, block % a.residual_blocks_x, block / a.residual_blocks_x);
      return;
    }
    block -= residual_blocks;
  }
  value_codes_block<DT, CTA_K, PARAMS, DK>(a.v.v, a.v.codes, a.v.tile_sum, a.inverse, a.midpoint, a.v.length,
                                           a.v.padded, a.v.heads, a.v.stride_b, a.v.stride_h, a.v.stride_n,
                                           a.v.permutation, fused, block % a.code_blocks_x, block / a.code_blocks_x);
}

// Short problems in one launch: nothing waits for another workgroup.  A K workgroup
// finds the anchor of its (batch, head) itself (nine sampled rows), a V workgroup walks the
// whole sequence of its (batch, head) for the channel maxima; both repeat work that a first
// launch would do once, which at this size costs less than the launch (about 5 us between two
// dependent kernels).  Same device functions as the two-stage path: bit-identical tensors.
template <int DT, int DK, int CTA_K, int ROT, bool AFFINE>
__global__ __launch_bounds__(256) void prepare_single_kernel(const FusedArgs a) {
  int block = blockIdx.x;
  if (block < a.key_blocks) {
    const int part = block & 1;
    const int tile = (block >> 1) % a.key_tiles;
    const int rest = (block >> 1) / a.key_tiles;
    const int h = rest % a.qk.kv_heads, b = rest / a.qk.kv_heads;
    const int anchor = detect_anchor_value<DT>(a.qk.k, a.qk.k_len, a.qk.head_dim, a.qk.kv_heads, a.qk.k_stride_b,
                                               a.qk.k_stride_h, a.qk.k_stride_n, a.qk.permutation, h, b);
    if (tile == 0 && part == 0 && threadIdx.x == 0) a.qk.anchors[rest] = anchor;  // for the LSE shift
    quantize_k_block<DT, DK, CTA_K, ROT>(a.qk.k, a.qk.k_codes, a.qk.k_scale, anchor, a.qk.k_len, a.qk.kv_heads,
                                         a.key_tiles * 4, a.qk.k_stride_b, a.qk.k_stride_h, a.qk.k_stride_n,
                                         a.k_wide, a.qk.permutation, tile, part, h, b);
    return;
  }
  block -= a.key_blocks;
  const FusedParams fused{a.part_max, a.part_min, a.v.scale, a.v.center, a.inverse, a.midpoint, a.chunks};
  if constexpr (AFFINE) {
    // the centre blocks: each walks the whole sequence of its eight channels, twice
    if (block < a.center_blocks) {
      const int octets = a.v.head_dim / 8;
      value_center_block<DT, true>(a.v.v, fused, a.v.length, a.v.head_dim, a.v.heads, a.v.stride_b, a.v.stride_h,
                                   a.v.stride_n, a.v.permutation, block % octets, block / octets);
      return;
    }
    block -= a.center_blocks;
  }
  const int code_blocks = a.code_blocks_x * a.kv;
  if (block < code_blocks) {
    value_codes_block<DT, CTA_K, AFFINE ? kParamsWalkAffine : kParamsWalk, DK>(a.v.v, a.v.codes, a.v.tile_sum, a.inverse, a.midpoint, a.v.length,
                                                  a.v.padded, a.v.heads, a.v.stride_b, a.v.stride_h, a.v.stride_n,
                                                  a.v.permutation, fused, block % a.code_blocks_x,
                                                  block / a.code_blocks_x);
    return;
  }
  block -= code_blocks;
  const int slice = block % a.q_slices;
  const int rest = block / a.q_slices;
  quantize_q_block<DT, DK, ROT>(a.qk.q, a.qk.q_codes, a.qk.q_scale, a.qk.q_len, a.qk.q_heads,
                                a.q_slices * 8, a.qk.q_stride_b, a.qk.q_stride_h, a.qk.q_stride_n,
                                a.q_wide, slice, rest % a.qk.q_heads, rest / a.qk.q_heads);
}

// One launch while the repeated reads stay small: every V workgroup (128 positions) reads its
// whole (batch, head), so V is read once per position block; up to 1024 tokens and 16 MiB of
// such reads (out of L2) that is cheaper than a second launch.
constexpr int kSingleLaunchMaxLength = 1024;
constexpr int64_t kSingleLaunchMaxBytes = int64_t{16} << 20;

template <int DT, int DK, int CTA_K, int ROT>
void launch_stages(const FusedArgs& a, hipStream_t stream) {
  const int64_t walked_bytes = static_cast<int64_t>(a.kv) * a.v.length * DK * (DT == kF32 ? 4 : 2) * a.code_blocks_x;
  if (a.v.length <= kSingleLaunchMaxLength && walked_bytes <= kSingleLaunchMaxBytes) {
    if (a.v.midpoint_affine) {
      FusedArgs with_center = a;
      with_center.center_blocks = a.kv * (a.v.head_dim / 8);
      const int blocks = a.key_blocks + with_center.center_blocks + a.code_blocks_x * a.kv + a.q_blocks;
      prepare_single_kernel<DT, DK, CTA_K, ROT, true><<<blocks, 256, 0, stream>>>(with_center);
    } else {
      const int blocks = a.key_blocks + a.code_blocks_x * a.kv + a.q_blocks;
      prepare_single_kernel<DT, DK, CTA_K, ROT, false><<<blocks, 256, 0, stream>>>(a);
    }
    return;
  }
  const int stage1_blocks = a.q_blocks + a.anchor_blocks + a.range_groups * a.kv;
  const bool stored_params = a.chunks > 64;
  const bool merged_center = a.v.midpoint_affine && !stored_params && a.v.length <= kFusedCenterMaxLength;
  FusedArgs with_center = a;
  with_center.center_blocks = merged_center ? a.kv * (a.v.head_dim / 8) : 0;
  const bool merged_residual = a.v.midpoint_affine && stored_params && a.v.length > kFusedCenterMaxLength;
  with_center.residual_blocks_x =
      merged_residual ? summation_threads(a.v.length) / (256 / (a.v.head_dim / 4)) : 0;
  const int stage2_blocks = a.key_blocks + with_center.center_blocks + with_center.residual_blocks_x * a.kv +
                            a.code_blocks_x * a.kv;
  const int groups = a.kv * a.v.head_dim / 8;
  if (a.v.midpoint_affine) {
    prepare_stage1_kernel<DT, DK, ROT, true><<<stage1_blocks, 256, 0, stream>>>(a);
    if (stored_params) {
      value_params_kernel<true><<<(groups + 3) / 4, 256, 0, stream>>>(
          a.part_max, a.part_min, a.v.scale, a.v.center, a.inverse, a.midpoint, a.v.head_dim, a.chunks, groups);
      prepare_stage2_kernel<DT, DK, CTA_K, ROT, kParamsStored><<<stage2_blocks, 256, 0, stream>>>(with_center);
    } else {
      prepare_stage2_kernel<DT, DK, CTA_K, ROT, kParamsAffine><<<stage2_blocks, 256, 0, stream>>>(with_center);
    }
    if (merged_center) {
      // done inside the second launch
    } else if (a.v.length <= kFusedCenterMaxLength) {
      dim3 center_grid(a.v.head_dim / 8, a.kv);
      value_center_fused_kernel<DT><<<center_grid, summation_threads(a.v.length), 0, stream>>>(
          a.v.v, a.inverse, a.midpoint, a.v.center, a.v.length, a.v.head_dim, a.v.heads, a.v.stride_b,
          a.v.stride_h, a.v.stride_n, a.v.permutation);
    } else {
      const int threads = summation_threads(a.v.length);
      const int per_block = 256 / (a.v.head_dim / 4);
      const int rows = a.kv * a.v.head_dim;
      if (!merged_residual) {
        dim3 residual_grid(threads / per_block, a.kv);
        value_residual_kernel<DT><<<residual_grid, 256, 0, stream>>>(
            a.v.v, a.partial, a.inverse, a.midpoint, a.v.length, a.v.head_dim, a.v.heads, threads,
            a.v.stride_b, a.v.stride_h, a.v.stride_n, a.v.permutation);
      }
      value_center_from_partials_kernel<<<rows, threads, 0, stream>>>(
          a.partial, a.inverse, a.midpoint, a.v.center, rows, threads, a.v.length);
    }
  } else {
    prepare_stage1_kernel<DT, DK, ROT, false><<<stage1_blocks, 256, 0, stream>>>(a);
    if (stored_params) {
      value_params_kernel<false><<<(groups + 3) / 4, 256, 0, stream>>>(
          a.part_max, a.part_min, a.v.scale, a.v.center, a.inverse, a.midpoint, a.v.head_dim, a.chunks, groups);
      prepare_stage2_kernel<DT, DK, CTA_K, ROT, kParamsStored><<<stage2_blocks, 256, 0, stream>>>(with_center);
    } else {
      prepare_stage2_kernel<DT, DK, CTA_K, ROT, kParamsAbsmax><<<stage2_blocks, 256, 0, stream>>>(a);
    }
  }
}

template <int DT, int DK> void launch_by_rotation(const FusedArgs& a, hipStream_t stream) {
  const bool short_keys = a.qk.k_len <= 256;
  constexpr int LONG_ROT = DK == 64 ? kRot64 : DK == 128 ? kRot128Signed : kRot128Plain;
  if constexpr (DK == 64) {
    if (short_keys)
      launch_stages<DT, DK, 64, kRot4>(a, stream);
    else
      launch_stages<DT, DK, 64, LONG_ROT>(a, stream);
  } else {
    if (a.qk.cta_k == 128) {
      if (short_keys)
        launch_stages<DT, DK, 128, kRot4>(a, stream);
      else
        launch_stages<DT, DK, 128, LONG_ROT>(a, stream);
    } else {
      if (short_keys)
        launch_stages<DT, DK, 64, kRot4>(a, stream);
      else
        launch_stages<DT, DK, 64, LONG_ROT>(a, stream);
    }
  }
}

template <int DT> void launch_by_dim(const FusedArgs& a, hipStream_t stream) {
  if (a.qk.head_dim == 64)
    launch_by_rotation<DT, 64>(a, stream);
  else if (a.qk.head_dim == 128)
    launch_by_rotation<DT, 128>(a, stream);
  else
    launch_by_rotation<DT, 256>(a, stream);
}

}  // namespace

bool can_prepare_fused(const QkArgs& qk, const ValueArgs& v) {
  return qk.k_len == v.length &&
         qk.batch == v.batch && qk.kv_heads == v.heads && qk.head_dim == v.head_dim &&
         qk.cta_k == v.cta_k && qk.dtype == v.dtype;
}

int launch_prepare_fused(const QkArgs& qk, const ValueArgs& v, hipStream_t stream) {
  if (!can_prepare_fused(qk, v)) return fail("risa_sdpa: operands do not qualify for the fused preparation");
  if (v.workspace_bytes < value_workspace_bytes(v.batch, v.heads, v.length, v.head_dim, v.midpoint_affine))
    return fail("risa_quantize_v: workspace is too small");
  const Workspace w = carve(v.workspace, v.batch, v.heads, v.length, v.head_dim, v.midpoint_affine);
  FusedArgs a{};
  a.qk = qk;
  a.v = v;
  a.part_max = w.part_max;
  a.part_min = w.part_min;
  a.inverse = w.inverse;
  a.midpoint = w.midpoint;
  a.partial = w.partial;
  const int slice_rows = qk.head_dim == 256 ? 16 : 32;
  a.q_slices = (qk.q_len + 127) / 128 * (128 / slice_rows);
  a.q_blocks = a.q_slices * qk.q_heads * qk.batch;
  a.kv = qk.batch * qk.kv_heads;
  a.anchor_blocks = a.kv;
  a.chunks = range_chunks(v.length);
  // Long absmax sequences whose Q work covers the longer V range walks: fewer, longer chunks,
  // so that the code blocks reduce the partial ranges themselves (no parameter launch).  The
  // long midpoint_affine path keeps the stored parameters its residual blocks read.
  if (!v.midpoint_affine && static_cast<int64_t>(qk.q_len) * qk.q_heads >= static_cast<int64_t>(v.length) * v.heads)
    a.chunks = capped_range_chunks(v.length);
  a.range_groups = (a.chunks + 3) / 4;
  a.key_tiles = (qk.k_len + qk.cta_k - 1) / qk.cta_k;
  a.key_blocks = 2 * a.key_tiles * a.kv;  // half a tile per workgroup
  a.code_blocks_x = (v.padded + kCodeBlockPositions - 1) / kCodeBlockPositions;
  a.q_wide = rows_are_16_byte_aligned(qk.q, qk.q_stride_b, qk.q_stride_h, qk.q_stride_n, qk.dtype);
  a.k_wide = rows_are_16_byte_aligned(qk.k, qk.k_stride_b, qk.k_stride_h, qk.k_stride_n, qk.dtype);
  if (qk.dtype == kF32)
    launch_by_dim<kF32>(a, stream);
  else if (qk.dtype == kF16)
    launch_by_dim<kF16>(a, stream);
  else
    launch_by_dim<kBF16>(a, stream);
  return check_launch("risa_sdpa preparation");
}

}  // namespace risa
