// extern "C" entry points declared in include/risa_hip.h: argument checks that
// the reference performs in csrc/bindings.cpp and the launchers, then dispatch.

#include "../../include/risa_hip.h"

#include "common.hpp"
#include "launchers.hpp"

#include <mutex>

// Scratch memory of risa_quantize_v_noalloc: the V preparation's partial ranges, channel
// parameters and residual partial sums, for callers that cannot hand over a workspace.
// Every GPU the library runs on holds its own copy of this array until the process ends.
// In host code the name is only a handle for hipGetSymbolAddress; kernels get the address.
#define RISA_STATIC_SCRATCH_BYTES RISA_QUANTIZE_V_NOALLOC_MAX_BYTES
static __device__ __align__(256) unsigned char risa_static_scratch[RISA_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;

// Device address of risa_static_scratch on the device the stream belongs to (the current device
// for the null stream), resolved once per device with that device current.
int static_scratch_address(hipStream_t stream, void** address) {
  static std::mutex guard;
  static void* resolved[kMaxDevices] = {};
  int current = -1;
  if (hipGetDevice(&current) != hipSuccess || current < 0 || current >= kMaxDevices)
    return risa::fail("risa_quantize_v_noalloc: cannot identify the current device");
  int device = current;
  if (stream != nullptr && hipStreamGetDevice(stream, &device) != hipSuccess)
    return risa::fail("risa_quantize_v_noalloc: cannot identify the device of the stream");
  if (device != current)
    return risa::fail("risa_quantize_v_noalloc: the stream belongs to device " + std::to_string(device) +
                      " but device " + std::to_string(current) + " is current");
  std::lock_guard<std::mutex> lock(guard);
  if (resolved[device] == nullptr) {
    void* pointer = nullptr;
    const hipError_t status = hipGetSymbolAddress(&pointer, HIP_SYMBOL(risa_static_scratch));
    if (status != hipSuccess || pointer == nullptr)
      return risa::fail(std::string("risa_quantize_v_noalloc: hipGetSymbolAddress failed: ") +
                        hipGetErrorString(status));
    resolved[device] = pointer;
  }
  *address = resolved[device];
  return 0;
}

bool aligned(const void* pointer, size_t bytes) {
  return reinterpret_cast<uintptr_t>(pointer) % bytes == 0;
}

// A stride is irrelevant when the extent is below two.
bool stride_multiple(int64_t stride, int extent, int64_t multiple) {
  return extent < 2 || (stride > 0 && stride % multiple == 0);
}

// Validation and argument block shared by risa_quantize_qk and risa_sdpa.
int checked_qk_args(risa::QkArgs& a, const void* q, void* q_int8, float* q_scale, const void* k,
                    void* k_int8, float* k_scale, int batch, int q_heads, int q_len, int kv_heads,
                    int k_len, int head_dim, int cta_k, int64_t q_stride_b, int64_t q_stride_h,
                    int64_t q_stride_n, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                    int input_dtype, int32_t* anchor_indices, const int32_t* kv_permutation) {
  using risa::fail;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail("risa_quantize_qk: padded head_dim must be 64, 128, or 256");
  if ((cta_k != 64 && cta_k != 128) || (head_dim == 64 && cta_k != 64))
    return fail("risa_quantize_qk: unsupported key tile for this head_dim");
  if (input_dtype < 0 || input_dtype > 2)
    return fail("risa_quantize_qk: input dtype code must be 0 (fp32), 1 (fp16), or 2 (bf16)");
  if (anchor_indices == nullptr) return fail("risa_quantize_qk: anchor_indices scratch is required");
  if (batch <= 0 || q_heads <= 0 || kv_heads <= 0 || q_len <= 0 || k_len <= 0)
    return fail("risa_quantize_qk: extents must be positive");
  const size_t vector_bytes = 4 * (input_dtype == 0 ? 4 : 2);
  const bool q_ok = aligned(q, vector_bytes) && stride_multiple(q_stride_b, batch, 4) &&
                    stride_multiple(q_stride_h, q_heads, 4) && stride_multiple(q_stride_n, q_len, 4);
  const bool k_ok = aligned(k, vector_bytes) && stride_multiple(k_stride_b, batch, 4) &&
                    stride_multiple(k_stride_h, kv_heads, 4) && stride_multiple(k_stride_n, k_len, 4);
  if (!q_ok || !k_ok)
    return fail("risa_quantize_qk: Q/K base pointers and batch/head/sequence strides must "
                "preserve 4-element alignment");
  a.q = q;
  a.q_codes = static_cast<int8_t*>(q_int8);
  a.q_scale = q_scale;
  a.k = k;
  a.k_codes = static_cast<int8_t*>(k_int8);
  a.k_scale = k_scale;
  a.anchors = anchor_indices;
  a.permutation = kv_permutation;
  a.batch = batch;
  a.q_heads = q_heads;
  a.q_len = q_len;
  a.kv_heads = kv_heads;
  a.k_len = k_len;
  a.head_dim = head_dim;
  a.cta_k = cta_k;
  a.dtype = input_dtype;
  a.q_stride_b = q_stride_b;
  a.q_stride_h = q_stride_h;
  a.q_stride_n = q_stride_n;
  a.k_stride_b = k_stride_b;
  a.k_stride_h = k_stride_h;
  a.k_stride_n = k_stride_n;
  return 0;
}

// Validation and argument block shared by risa_quantize_v and risa_sdpa.
int checked_v_args(risa::ValueArgs& a, const void* v, void* out, float* scale, float* center,
                   int32_t* tile_sum, void* workspace, size_t workspace_bytes, int batch, int heads,
                   int length, int head_dim, int padded_length, int cta_k, int64_t stride_b,
                   int64_t stride_h, int64_t stride_n, int input_dtype, int midpoint_affine,
                   const int32_t* kv_permutation) {
  using risa::fail;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail("risa_quantize_v: padded head_dim must be 64, 128, or 256");
  if (cta_k != 64 && cta_k != 128) return fail("risa_quantize_v: cta_k must be 64 or 128");
  if (input_dtype < 0 || input_dtype > 2) return fail("risa_quantize_v: unsupported input dtype");
  if (batch <= 0 || heads <= 0 || length <= 0) return fail("risa_quantize_v: extents must be positive");
  if (padded_length != (length + cta_k - 1) / cta_k * cta_k)
    return fail("risa_quantize_v: padded length must round the sequence up to the key tile");
  const int64_t per_16_bytes = input_dtype == 0 ? 4 : 8;
  if (!aligned(v, 16) || !stride_multiple(stride_b, batch, per_16_bytes) ||
      !stride_multiple(stride_h, heads, per_16_bytes) ||
      !stride_multiple(stride_n, length, per_16_bytes))
    return fail("risa_quantize_v: V base pointer and batch/head/sequence strides must be "
                "16-byte aligned");
  if (tile_sum == nullptr || workspace == nullptr)
    return fail("risa_quantize_v: tile sums and workspace are required");
  a.v = v;
  a.codes = static_cast<int8_t*>(out);
  a.scale = scale;
  a.center = center;
  a.tile_sum = tile_sum;
  a.workspace = workspace;
  a.workspace_bytes = workspace_bytes;
  a.permutation = kv_permutation;
  a.batch = batch;
  a.heads = heads;
  a.length = length;
  a.head_dim = head_dim;
  a.padded = padded_length;
  a.cta_k = cta_k;
  a.dtype = input_dtype;
  a.stride_b = stride_b;
  a.stride_h = stride_h;
  a.stride_n = stride_n;
  a.midpoint_affine = midpoint_affine != 0;
  return 0;
}

}  // namespace

extern "C" {

const char* risa_last_error(void) { return risa::last_error_storage().c_str(); }

int risa_abi_version(void) { return 3; }

int risa_quantize_qk(const void* q, void* q_int8, float* q_scale, const void* k, void* k_int8,
                     float* k_scale, int batch, int q_heads, int q_len, int kv_heads, int k_len,
                     int head_dim, int cta_k, int64_t q_stride_b, int64_t q_stride_h,
                     int64_t q_stride_n, int64_t k_stride_b, int64_t k_stride_h,
                     int64_t k_stride_n, int input_dtype, int32_t* anchor_indices,
                     const int32_t* kv_permutation, void* stream) {
  risa::QkArgs a{};
  const int status = checked_qk_args(a, q, q_int8, q_scale, k, k_int8, k_scale, batch, q_heads, q_len,
                                     kv_heads, k_len, head_dim, cta_k, q_stride_b, q_stride_h,
                                     q_stride_n, k_stride_b, k_stride_h, k_stride_n, input_dtype,
                                     anchor_indices, kv_permutation);
  if (status != 0) return status;
  return risa::launch_quantize_qk(a, static_cast<hipStream_t>(stream));
}

size_t risa_quantize_v_workspace_bytes(int batch, int heads, int length, int head_dim,
                                       int midpoint_affine) {
  return risa::value_workspace_bytes(batch, heads, length, head_dim, midpoint_affine != 0);
}

int risa_quantize_v(const void* v, void* out, float* scale, float* center, int32_t* tile_sum,
                    void* workspace, size_t workspace_bytes, int batch, int heads, int length,
                    int head_dim, int padded_length, int cta_k, int64_t stride_b,
                    int64_t stride_h, int64_t stride_n, int input_dtype, int midpoint_affine,
                    const int32_t* kv_permutation, void* stream) {
  risa::ValueArgs a{};
  const int status = checked_v_args(a, v, out, scale, center, tile_sum, workspace, workspace_bytes,
                                    batch, heads, length, head_dim, padded_length, cta_k, stride_b,
                                    stride_h, stride_n, input_dtype, midpoint_affine, kv_permutation);
  if (status != 0) return status;
  return risa::launch_quantize_v(a, static_cast<hipStream_t>(stream));
}

int risa_quantize_v_noalloc(const void* v, void* out, float* scale, float* center, int32_t* tile_sum,
                            int batch, int heads, int length, int head_dim, int padded_length,
                            int cta_k, int64_t stride_b, int64_t stride_h, int64_t stride_n,
                            int input_dtype, int midpoint_affine, const int32_t* kv_permutation,
                            void* stream) {
  if (batch <= 0 || heads <= 0 || length <= 0 || (head_dim != 64 && head_dim != 128 && head_dim != 256))
    return risa::fail("risa_quantize_v_noalloc: extents must be positive and head_dim 64, 128, or 256");
  const size_t needed = risa::value_workspace_bytes(batch, heads, length, head_dim, midpoint_affine != 0);
  if (needed > RISA_STATIC_SCRATCH_BYTES)
    return risa::fail("risa_quantize_v_noalloc: this problem needs " + std::to_string(needed) +
                      " bytes of scratch memory, the built-in buffer holds " +
                      std::to_string(static_cast<size_t>(RISA_STATIC_SCRATCH_BYTES)) +
                      "; use risa_quantize_v with a caller-provided workspace");
  void* scratch = nullptr;
  int status = static_scratch_address(static_cast<hipStream_t>(stream), &scratch);
  if (status != 0) return status;
  risa::ValueArgs a{};
  status = checked_v_args(a, v, out, scale, center, tile_sum, scratch, RISA_STATIC_SCRATCH_BYTES, batch,
                          heads, length, head_dim, padded_length, cta_k, stride_b, stride_h, stride_n,
                          input_dtype, midpoint_affine, kv_permutation);
  if (status != 0) return status;
  return risa::launch_quantize_v(a, static_cast<hipStream_t>(stream));
}

int risa_sdpa_quantize(const void* q, void* q_int8, float* q_scale, const void* k, void* k_int8,
                       float* k_scale, const void* v, void* v_int8, float* v_scale, float* v_center,
                       int32_t* v_tile_sum, void* v_workspace, size_t v_workspace_bytes, int batch,
                       int q_heads, int q_len, int kv_heads, int k_len, int head_dim, int cta_k,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                       int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_b, int64_t v_stride_h,
                       int64_t v_stride_n, int input_dtype, int midpoint_affine,
                       int32_t* anchor_indices, const int32_t* kv_permutation, void* stream) {
  if (cta_k != 64 && cta_k != 128) return risa::fail("risa_sdpa_quantize: cta_k must be 64 or 128");
  const int padded = (k_len + cta_k - 1) / cta_k * cta_k;
  risa::QkArgs qk{};
  int status = checked_qk_args(qk, q, q_int8, q_scale, k, k_int8, k_scale, batch, q_heads, q_len, kv_heads,
                               k_len, head_dim, cta_k, q_stride_b, q_stride_h, q_stride_n, k_stride_b,
                               k_stride_h, k_stride_n, input_dtype, anchor_indices, kv_permutation);
  if (status != 0) return status;
  risa::ValueArgs value{};
  status = checked_v_args(value, v, v_int8, v_scale, v_center, v_tile_sum, v_workspace, v_workspace_bytes,
                          batch, kv_heads, k_len, head_dim, padded, cta_k, v_stride_b, v_stride_h,
                          v_stride_n, input_dtype, midpoint_affine, kv_permutation);
  if (status != 0) return status;
  hipStream_t hip_stream = static_cast<hipStream_t>(stream);
  if (risa::can_prepare_fused(qk, value)) return risa::launch_prepare_fused(qk, value, hip_stream);
  status = risa::launch_quantize_qk(qk, hip_stream);
  if (status != 0) return status;
  return risa::launch_quantize_v(value, hip_stream);
}

int risa_value_tile_sums(const void* v_int8, int32_t* tile_sum, int batch_heads, int head_dim,
                         int padded_length, int cta_k, void* stream) {
  if ((cta_k != 64 && cta_k != 128) || padded_length % cta_k != 0 || head_dim <= 0)
    return risa::fail("risa_value_tile_sums: unsupported tile or padding");
  return risa::launch_value_tile_sums(static_cast<const int8_t*>(v_int8), tile_sum, batch_heads,
                                      head_dim, padded_length, cta_k,
                                      static_cast<hipStream_t>(stream));
}

void risa_unpack_order(int32_t* order) {
  for (int token = 0; token < 32; ++token) order[risa::packed_value_position(token)] = token;
}

int risa_attention(const void* q_int8, const void* k_int8, const void* v_int8, void* out,
                   const float* q_scale, const float* k_scale, const float* v_scale,
                   const float* v_center, const int32_t* v_tile_sum, const void* mask,
                   int64_t mask_stride_b, int64_t mask_stride_h, int64_t mask_stride_q,
                   int64_t mask_stride_k, int mask_dtype, int cta_k, int batch, int q_len,
                   int k_len, int q_heads, int kv_heads, int head_dim, int64_t out_stride_b,
                   int64_t out_stride_n, int64_t out_stride_h, float sm_scale, int out_dtype,
                   const int32_t* sparse_row_offsets, const int32_t* sparse_block_indices,
                   float* block_mass, int is_causal, float* lse, const int32_t* key_mask_tiles,
                   const float* key_bias, int64_t key_bias_stride_b, int64_t key_bias_stride_h,
                   const uint64_t* mask_lanes, int64_t mask_lanes_stride_b,
                   int64_t mask_lanes_stride_h, void* stream) {
  using risa::fail;
  if (out_dtype != 1 && out_dtype != 2)
    return fail("risa_attention: output dtype code must be 1 (fp16) or 2 (bf16)");
  if (mask != nullptr && (mask_dtype < 0 || mask_dtype > 3))
    return fail("risa_attention: attention mask must be bool, float16, bfloat16, or float32");
  if (batch <= 0 || q_heads <= 0 || kv_heads <= 0 || q_len <= 0 || k_len <= 0)
    return fail("risa_attention: extents must be positive");
  // (the output's alignment rule is checked once, by the launcher)
  risa::AttentionArgs a{};
  a.q = static_cast<const int8_t*>(q_int8);
  a.k = static_cast<const int8_t*>(k_int8);
  a.v = static_cast<const int8_t*>(v_int8);
  a.out = out;
  a.q_scale = q_scale;
  a.k_scale = k_scale;
  a.v_scale = v_scale;
  a.v_center = v_center;
  a.v_tile_sum = v_tile_sum;
  a.mask = mask;
  a.mask_stride_b = mask_stride_b;
  a.mask_stride_h = mask_stride_h;
  a.mask_stride_q = mask_stride_q;
  a.mask_stride_k = mask_stride_k;
  a.mask_dtype = mask_dtype;
  a.cta_k = cta_k;
  a.batch = batch;
  a.q_len = q_len;
  a.k_len = k_len;
  a.q_heads = q_heads;
  a.kv_heads = kv_heads;
  a.head_dim = head_dim;
  a.out_stride_b = out_stride_b;
  a.out_stride_n = out_stride_n;
  a.out_stride_h = out_stride_h;
  a.sm_scale = sm_scale;
  a.out_dtype = out_dtype;
  a.sparse_row_offsets = sparse_row_offsets;
  a.sparse_block_indices = sparse_block_indices;
  a.block_mass = block_mass;
  a.is_causal = is_causal != 0;
  a.lse = lse;
  a.key_mask_tiles = key_mask_tiles;
  if (key_bias != nullptr && (mask == nullptr || mask_stride_q != 0))
    return fail("risa_attention: a key bias row goes with a key-only mask (query stride 0)");
  a.key_bias = key_bias;
  a.key_bias_stride_b = key_bias_stride_b;
  a.key_bias_stride_h = key_bias_stride_h;
  if (mask_lanes != nullptr && mask == nullptr)
    return fail("risa_attention: lane words go with the boolean mask they were made from");
  a.mask_lanes = mask_lanes;
  a.mask_lanes_stride_b = mask_lanes_stride_b;
  a.mask_lanes_stride_h = mask_lanes_stride_h;
  return risa::launch_attention(a, static_cast<hipStream_t>(stream));
}

size_t risa_selector_workspace_size(int) { return 0; }

int risa_select_retained_mass(const float* sorted_mass, const int64_t* descending_indices,
                              int32_t* counts, uint8_t* support, double* row_totals,
                              int32_t* row_offsets, int32_t* block_indices, double* summary,
                              int row_count, int key_blocks, double theta, void* stream) {
  if (row_count <= 0 || key_blocks <= 0)
    return risa::fail("risa_select_retained_mass: invalid shape, dtype, or stride");
  if (static_cast<int64_t>(row_count) * key_blocks > INT32_MAX)
    return risa::fail("risa_select_retained_mass: matrix is too large");
  risa::SelectArgs a{sorted_mass, descending_indices, counts,   support,    row_totals, row_offsets,
                     block_indices, summary,          row_count, key_blocks, theta};
  return risa::launch_select_retained_mass(a, static_cast<hipStream_t>(stream));
}

int risa_sort_select_retained_mass(const float* masses, float* sorted_mass, int64_t* descending_indices,
                                   int32_t* counts, uint8_t* support, double* row_totals,
                                   int32_t* row_offsets, int32_t* block_indices, double* summary,
                                   int row_count, int key_blocks, double theta, void* stream) {
  if (row_count <= 0 || key_blocks <= 0)
    return risa::fail("risa_sort_select_retained_mass: invalid shape, dtype, or stride");
  if (static_cast<int64_t>(row_count) * key_blocks > INT32_MAX)
    return risa::fail("risa_sort_select_retained_mass: matrix is too large");
  if (key_blocks > risa::kSortableTiles)
    return risa::fail("risa_sort_select_retained_mass: more than " + std::to_string(risa::kSortableTiles) +
                      " key tiles per row: sort outside and call risa_select_retained_mass");
  const int status = risa::launch_sort_rows(masses, sorted_mass, descending_indices, row_count, key_blocks,
                                            static_cast<hipStream_t>(stream));
  if (status != 0) return status;
  risa::SelectArgs a{sorted_mass, descending_indices, counts,   support,    row_totals, row_offsets,
                     block_indices, summary,          row_count, key_blocks, theta};
  return risa::launch_select_retained_mass(a, static_cast<hipStream_t>(stream));
}

int risa_sortable_key_blocks(void) { return risa::kSortableTiles; }

int risa_prepare_key_mask_tiles(const void* mask, int32_t* tiles, int batch, int q_heads,
                                int key_length, int tile_size, int64_t stride_b, int64_t stride_h,
                                int64_t stride_k, int mask_dtype, void* stream) {
  if (tile_size != 64 && tile_size != 128)
    return risa::fail("risa_prepare_key_mask_tiles requires an expanded broadcast key mask");
  if (mask_dtype < 0 || mask_dtype > 3)
    return risa::fail("risa_prepare_key_mask_tiles requires a supported mask dtype");
  return risa::launch_key_mask_tiles(mask, tiles, batch, q_heads, key_length, tile_size, stride_b,
                                     stride_h, stride_k, mask_dtype,
                                     static_cast<hipStream_t>(stream));
}

int risa_prepare_key_bias(const void* mask, float* bias, int batch, int heads, int key_length,
                          int padded_length, int64_t stride_b, int64_t stride_h, int64_t stride_k,
                          int mask_dtype, void* stream) {
  if (mask == nullptr || bias == nullptr || batch <= 0 || heads <= 0 || key_length <= 0 ||
      padded_length < key_length || padded_length % 64 != 0)
    return risa::fail("risa_prepare_key_bias: bad extents");
  if (mask_dtype < 0 || mask_dtype > 3)
    return risa::fail("risa_prepare_key_bias requires a supported mask dtype");
  return risa::launch_key_bias(mask, bias, batch, heads, key_length, padded_length, stride_b,
                               stride_h, stride_k, mask_dtype, static_cast<hipStream_t>(stream));
}

size_t risa_mask_lanes_bytes(int mask_dtype, int head_dim, int cta_k, int64_t mask_stride_q,
                             int64_t mask_stride_k, int batch, int q_heads, int mask_batch,
                             int mask_heads, int q_len, int k_len) {
  if (mask_dtype != risa::kBool || cta_k != 64 || mask_stride_q == 0 || mask_stride_k != 1) return 0;
  if (head_dim > 128) return 0;  // the sixteen-query kernel of head dim 256 has another score layout
  // A launch of at most one workgroup per compute unit runs the sixteen-query kernel (the same
  // limit the launcher applies), and the conversion would be a launch of its own next to a
  // short kernel.
  if (static_cast<int64_t>(batch) * q_heads * ((q_len + 127) / 128) <= risa::narrow_attention_limit()) return 0;
  // one conversion launch: blocks of 32 queries and mask planes are grid dimensions
  if ((static_cast<int64_t>(q_len) + 127) / 128 * 4 > 65535 || static_cast<int64_t>(mask_batch) * mask_heads > 65535)
    return 0;
  if (batch <= 0 || q_heads <= 0 || mask_batch <= 0 || mask_heads <= 0 || q_len <= 0 || k_len <= 0) return 0;
  // The conversion reads the mask once; it pays when several heads then share the words.
  if (static_cast<int64_t>(batch) * q_heads < int64_t{8} * mask_batch * mask_heads) return 0;
  return risa::mask_lane_bytes(mask_batch, mask_heads, q_len, k_len);
}

int risa_prepare_mask_lanes(const void* mask, uint64_t* lanes, int mask_batch, int mask_heads,
                            int q_len, int k_len, int64_t stride_b, int64_t stride_h,
                            int64_t stride_q, void* stream) {
  if (mask == nullptr || lanes == nullptr || mask_batch <= 0 || mask_heads <= 0 || q_len <= 0 || k_len <= 0)
    return risa::fail("risa_prepare_mask_lanes: bad extents");
  if (!aligned(lanes, 8)) return risa::fail("risa_prepare_mask_lanes: lane words must be 8-byte aligned");
  return risa::launch_mask_lanes(mask, lanes, mask_batch, mask_heads, q_len, k_len,
                                 mask_batch > 1 ? stride_b : 0, mask_heads > 1 ? stride_h : 0, stride_q,
                                 static_cast<hipStream_t>(stream));
}

int risa_lse_shift(const void* q, const void* k, const int32_t* anchors, float* out, int batch,
                   int q_heads, int kv_heads, int q_len, int head_dim, int64_t q_stride_b,
                   int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b, int64_t k_stride_h,
                   int64_t k_stride_n, float scale, int dtype, void* stream) {
  if (dtype < 0 || dtype > 2) return risa::fail("risa_lse_shift: unsupported dtype");
  risa::LseShiftArgs a{q,          k,          anchors,    out,        batch,      q_heads,
                       kv_heads,   q_len,      head_dim,   dtype,      q_stride_b, q_stride_h,
                       q_stride_n, k_stride_b, k_stride_h, k_stride_n, scale};
  return risa::launch_lse_shift(a, static_cast<hipStream_t>(stream));
}

}  // extern "C"

namespace {

// Sections of the risa_sdpa workspace, each aligned to 256 bytes.
struct SdpaLayout {
  size_t q_codes, k_codes, v_codes, q_scale, k_scale, v_scale, v_center, tile_sum, anchors,
      v_workspace, v_workspace_bytes, key_bias, key_tiles, mask_lanes, bytes;
};

SdpaLayout sdpa_layout(int batch, int q_heads, int q_len, int kv_heads, int k_len, int head_dim,
                       int cta_k, bool affine, bool key_only_mask, size_t mask_lanes_bytes) {
  SdpaLayout l{};
  size_t offset = 0;
  auto take = [&](size_t bytes) {
    const size_t at = offset;
    offset += (bytes + 255) / 256 * 256;
    return at;
  };
  const size_t tiles = (static_cast<size_t>(k_len) + cta_k - 1) / cta_k;
  const size_t padded = tiles * cta_k;
  const size_t kv = static_cast<size_t>(batch) * kv_heads;
  const size_t q_groups = (static_cast<size_t>(q_len) + 127) / 128 * (head_dim == 256 ? 64 : 32);
  l.q_codes = take(static_cast<size_t>(batch) * q_heads * q_len * head_dim);
  l.k_codes = take(kv * k_len * head_dim);
  l.v_codes = take(kv * head_dim * padded);
  l.q_scale = take(static_cast<size_t>(batch) * q_heads * q_groups * 4);
  l.k_scale = take(kv * tiles * 4 * 4);
  l.v_scale = take(kv * head_dim * 4);
  l.v_center = take(kv * head_dim * 4);
  l.tile_sum = take(kv * tiles * head_dim * 4);
  l.anchors = take(kv * 4);
  l.v_workspace_bytes = risa::value_workspace_bytes(batch, kv_heads, k_len, head_dim, affine);
  l.v_workspace = take(l.v_workspace_bytes);
  l.key_bias = key_only_mask ? take(static_cast<size_t>(batch) * q_heads * padded * 4) : 0;
  l.key_tiles = key_only_mask ? take(static_cast<size_t>(batch) * q_heads * (tiles + 1) * 4) : 0;
  l.mask_lanes = mask_lanes_bytes != 0 ? take(mask_lanes_bytes) : 0;
  l.bytes = offset;
  return l;
}

}  // namespace

extern "C" {

size_t risa_sdpa_workspace_bytes(int batch, int q_heads, int q_len, int kv_heads, int k_len,
                                 int head_dim, int cta_k, int midpoint_affine, int mask_dtype,
                                 int64_t mask_stride_q, int64_t mask_stride_k, int mask_batch,
                                 int mask_heads) {
  if (batch <= 0 || q_heads <= 0 || q_len <= 0 || kv_heads <= 0 || k_len <= 0 || head_dim <= 0 ||
      (cta_k != 64 && cta_k != 128))
    return 0;
  const bool key_only = mask_dtype >= 0 && mask_stride_q == 0;
  const size_t lanes = risa_mask_lanes_bytes(mask_dtype, head_dim, cta_k, mask_stride_q, mask_stride_k,
                                             batch, q_heads, mask_batch, mask_heads, q_len, k_len);
  return sdpa_layout(batch, q_heads, q_len, kv_heads, k_len, head_dim, cta_k, midpoint_affine != 0,
                     key_only, lanes)
      .bytes;
}

int risa_sdpa(const void* q, const void* k, const void* v, void* out, void* workspace,
              size_t workspace_bytes, int batch, int q_heads, int q_len, int kv_heads, int k_len,
              int head_dim, int cta_k, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
              int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_b,
              int64_t v_stride_h, int64_t v_stride_n, int64_t out_stride_b, int64_t out_stride_n,
              int64_t out_stride_h, float sm_scale, int input_dtype, int output_dtype,
              int midpoint_affine, const void* mask, int64_t mask_stride_b, int64_t mask_stride_h,
              int64_t mask_stride_q, int64_t mask_stride_k, int mask_dtype, int mask_batch,
              int mask_heads, int is_causal, const int32_t* sparse_row_offsets,
              const int32_t* sparse_block_indices, void* stream) {
  using risa::fail;
  if (batch <= 0 || q_heads <= 0 || q_len <= 0 || kv_heads <= 0 || k_len <= 0 ||
      (cta_k != 64 && cta_k != 128))
    return fail("risa_sdpa: extents must be positive and cta_k 64 or 128");
  const bool key_only = mask != nullptr && mask_stride_q == 0;
  if (mask != nullptr) {
    if (mask_batch != 1 && mask_batch != batch) return fail("risa_sdpa: mask batch extent");
    if (mask_heads != 1 && mask_heads != q_heads) return fail("risa_sdpa: mask head extent");
  }
  const size_t lanes_bytes =
      mask == nullptr ? 0
                      : risa_mask_lanes_bytes(mask_dtype, head_dim, cta_k, mask_stride_q, mask_stride_k,
                                              batch, q_heads, mask_batch, mask_heads, q_len, k_len);
  const SdpaLayout l = sdpa_layout(batch, q_heads, q_len, kv_heads, k_len, head_dim, cta_k,
                                   midpoint_affine != 0, key_only, lanes_bytes);
  if (workspace == nullptr || !aligned(workspace, 256) || workspace_bytes < l.bytes)
    return fail("risa_sdpa: workspace must be 256-byte aligned and hold risa_sdpa_workspace_bytes");
  auto* base = static_cast<unsigned char*>(workspace);
  auto* q_scale = reinterpret_cast<float*>(base + l.q_scale);
  auto* k_scale = reinterpret_cast<float*>(base + l.k_scale);
  auto* v_scale = reinterpret_cast<float*>(base + l.v_scale);
  auto* v_center = reinterpret_cast<float*>(base + l.v_center);
  auto* tile_sum = reinterpret_cast<int32_t*>(base + l.tile_sum);
  const int tiles = (k_len + cta_k - 1) / cta_k;
  const int padded = tiles * cta_k;
  risa::QkArgs qk{};
  int status = checked_qk_args(qk, q, base + l.q_codes, q_scale, k, base + l.k_codes, k_scale, batch,
                               q_heads, q_len, kv_heads, k_len, head_dim, cta_k, q_stride_b,
                               q_stride_h, q_stride_n, k_stride_b, k_stride_h, k_stride_n,
                               input_dtype, reinterpret_cast<int32_t*>(base + l.anchors), nullptr);
  if (status != 0) return status;
  risa::ValueArgs value{};
  status = checked_v_args(value, v, base + l.v_codes, v_scale, v_center, tile_sum,
                          base + l.v_workspace, l.v_workspace_bytes, batch, kv_heads, k_len, head_dim,
                          padded, cta_k, v_stride_b, v_stride_h, v_stride_n, input_dtype,
                          midpoint_affine, nullptr);
  if (status != 0) return status;
  hipStream_t hip_stream = static_cast<hipStream_t>(stream);
  if (risa::can_prepare_fused(qk, value)) {
    status = risa::launch_prepare_fused(qk, value, hip_stream);
  } else {
    status = risa::launch_quantize_qk(qk, hip_stream);
    if (status == 0) status = risa::launch_quantize_v(value, hip_stream);
  }
  if (status != 0) return status;
  const float* key_bias = nullptr;
  const int32_t* key_tiles = nullptr;
  int64_t bias_stride_b = 0, bias_stride_h = 0;
  const uint64_t* mask_lanes = nullptr;
  int64_t lanes_stride_b = 0, lanes_stride_h = 0;
  if (lanes_bytes != 0) {
    auto* words = reinterpret_cast<uint64_t*>(base + l.mask_lanes);
    status = risa_prepare_mask_lanes(mask, words, mask_batch, mask_heads, q_len, k_len, mask_stride_b,
                                     mask_stride_h, mask_stride_q, stream);
    if (status != 0) return status;
    mask_lanes = words;
    const int64_t plane = static_cast<int64_t>(risa::mask_lane_words(1, 1, q_len, k_len));
    lanes_stride_h = mask_heads > 1 ? plane : 0;
    lanes_stride_b = mask_batch > 1 ? plane * mask_heads : 0;
  }
  if (key_only) {
    auto* bias = reinterpret_cast<float*>(base + l.key_bias);
    status = risa_prepare_key_bias(mask, bias, mask_batch, mask_heads, k_len, padded,
                                   mask_batch > 1 ? mask_stride_b : 0,
                                   mask_heads > 1 ? mask_stride_h : 0, mask_stride_k, mask_dtype,
                                   stream);
    if (status != 0) return status;
    key_bias = bias;
    bias_stride_h = mask_heads > 1 ? padded : 0;
    bias_stride_b = mask_batch > 1 ? static_cast<int64_t>(mask_heads) * padded : 0;
    // tile lists pay off under the conditions of reference _key_mask.py:9-28
    if (k_len > 1024 && q_len >= 256 && sm_scale > 0.0f && is_causal == 0 && sparse_row_offsets == nullptr) {
      auto* list = reinterpret_cast<int32_t*>(base + l.key_tiles);
      status = risa_prepare_key_mask_tiles(mask, list, batch, q_heads, k_len, cta_k, mask_stride_b,
                                           mask_stride_h, mask_stride_k, mask_dtype, stream);
      if (status != 0) return status;
      key_tiles = list;
    }
  }
  return risa_attention(base + l.q_codes, base + l.k_codes, base + l.v_codes, out, q_scale, k_scale,
                        v_scale, v_center, tile_sum, mask, mask_stride_b, mask_stride_h,
                        mask_stride_q, mask_stride_k, mask_dtype, cta_k, batch, q_len, k_len,
                        q_heads, kv_heads, head_dim, out_stride_b, out_stride_n, out_stride_h,
                        sm_scale, output_dtype, sparse_row_offsets, sparse_block_indices, nullptr,
                        is_causal, nullptr, key_tiles, key_bias, bias_stride_b, bias_stride_h,
                        mask_lanes, lanes_stride_b, lanes_stride_h, stream);
}

}  // extern "C"
