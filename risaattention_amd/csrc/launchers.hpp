// Internal launch interfaces between the C entry points (c_api.hip) and the
// kernel translation units.  Every launcher enqueues on the given stream,
// never allocates or synchronises, and returns 0 or a non-zero error code with
// the message left in risa::last_error_storage().
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace risa {

struct QkArgs {
  const void* q;
  int8_t* q_codes;
  float* q_scale;
  const void* k;
  int8_t* k_codes;
  float* k_scale;
  int* anchors;
  const int32_t* permutation;  // [B,Hkv,Lk] source token of every key, or null
  int batch, q_heads, q_len, kv_heads, k_len, head_dim, cta_k, dtype;
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
};
int launch_quantize_qk(const QkArgs& args, hipStream_t stream);

struct LseShiftArgs {
  const void* q;
  const void* k;
  const int* anchors;
  float* out;
  int batch, q_heads, kv_heads, q_len, head_dim, dtype;
  int64_t q_stride_b, q_stride_h, q_stride_n;
  int64_t k_stride_b, k_stride_h, k_stride_n;
  float scale;
};
int launch_lse_shift(const LseShiftArgs& args, hipStream_t stream);

struct ValueArgs {
  const void* v;
  int8_t* codes;     // [B*H*D, padded] in packed MFMA order
  float* scale;      // [B*H*D]
  float* center;     // [B*H*D]
  int32_t* tile_sum; // [B*H, padded/cta_k, D], 128 x sum of codes
  void* workspace;
  size_t workspace_bytes;
  const int32_t* permutation;  // [B,H,L] source token of every value row, or null
  int batch, heads, length, head_dim, padded, cta_k, dtype;
  int64_t stride_b, stride_h, stride_n;
  bool midpoint_affine;
};
size_t value_workspace_bytes(int batch, int heads, int length, int head_dim, bool midpoint_affine);
int launch_quantize_v(const ValueArgs& args, hipStream_t stream);
int launch_value_tile_sums(const int8_t* codes, int32_t* tile_sum, int rows_bh, int head_dim,
                           int padded, int cta_k, hipStream_t stream);

struct AttentionArgs {
  const int8_t* q;
  const int8_t* k;
  const int8_t* v;
  void* out;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  const float* v_center;
  const int32_t* v_tile_sum;
  const void* mask;
  int64_t mask_stride_b, mask_stride_h, mask_stride_q, mask_stride_k;
  int mask_dtype;
  int cta_k, batch, q_len, k_len, q_heads, kv_heads, head_dim;
  int64_t out_stride_b, out_stride_n, out_stride_h;
  float sm_scale;
  int out_dtype;
  const int32_t* sparse_row_offsets;
  const int32_t* sparse_block_indices;
  float* block_mass;
  bool is_causal;
  float* lse;
  const int32_t* key_mask_tiles;
  const float* key_bias;  // [Bm,Hm,padded] from launch_key_bias, or null
  int64_t key_bias_stride_b, key_bias_stride_h;
  const uint64_t* mask_lanes;  // lane words from launch_mask_lanes, or null
  int64_t mask_lanes_stride_b, mask_lanes_stride_h;  // in words
};
int launch_attention(const AttentionArgs& args, hipStream_t stream);
// Number of 128-query workgroups up to which a launch takes the sixteen-query kernel: the
// compute units of the current device (the MI355X's 256 when no device can be queried).
int narrow_attention_limit();

struct SelectArgs {
  const float* sorted_mass;
  const int64_t* descending_indices;
  int32_t* counts;
  uint8_t* support;
  double* row_totals;
  int32_t* row_offsets;
  int32_t* block_indices;
  double* summary;
  int rows, tiles;
  double theta;
};
int launch_select_retained_mass(const SelectArgs& args, hipStream_t stream);
// Most key tiles a row may have for the in-library sort (one workgroup, 32 KB of LDS).
constexpr int kSortableTiles = 4096;
int launch_sort_rows(const float* masses, float* sorted_mass, int64_t* order, int rows, int tiles,
                     hipStream_t stream);

int launch_key_mask_tiles(const void* mask, int32_t* tiles, int batch, int heads, int length,
                          int tile_size, int64_t stride_b, int64_t stride_h, int64_t stride_k,
                          int dtype, hipStream_t stream);

// Q/K/V preparation in two launches (short sequences, no permutation).
bool can_prepare_fused(const QkArgs& qk, const ValueArgs& v);
int launch_prepare_fused(const QkArgs& qk, const ValueArgs& v, hipStream_t stream);

// Lane words of a boolean mask with 64-key tiles: [batch, heads, ceil(q_len/128)*4,
// ceil(k_len/64), 32] 64-bit words, batch and heads being the mask's own extents.
// What the 32 lane words of one (block of 32 queries, 64-key tile) have in common: every bit
// set (the tile needs no select), none set (the wavefront skips the tile: it would add nothing
// to the sums and leave the running maximum where it is), or neither.
constexpr int kLaneTileMixed = 0, kLaneTileVisible = 1, kLaneTileHidden = 2;
size_t mask_lane_words(int batch, int heads, int q_len, int k_len);
size_t mask_lane_bytes(int batch, int heads, int q_len, int k_len);  // words, classes and tile lists
size_t mask_tile_list_offset(int batch, int heads, int q_len, int k_len);  // of the lists, in bytes
int launch_mask_lanes(const void* mask, uint64_t* lanes, int batch, int heads, int q_len, int k_len,
                      int64_t stride_b, int64_t stride_h, int64_t stride_q, hipStream_t stream);

int launch_key_bias(const void* mask, float* bias, int batch, int heads, int length, int padded,
                    int64_t stride_b, int64_t stride_h, int64_t stride_k, int dtype,
                    hipStream_t stream);

}  // namespace risa
