// Host-side dispatch of the fused attention kernel and the block-mass
// reconstruction that follows a capturing run.
//
// Path selection follows reference csrc/kernels/attention_dispatch.cu:113-296:
// the raw-score path runs when there is no mask, no causal flag and a positive
// scale; custom and key-only masks share the pre-scaled path; sparse support
// and key-mask tile lists both iterate an index list.

#include "attention_dispatch.hpp"

namespace risa {

template <> int launch_attention_variant<64>(const KernelParams&, int, bool, bool, bool, hipStream_t);
template <> int launch_attention_variant<128>(const KernelParams&, int, bool, bool, bool, hipStream_t);
template <> int launch_attention_variant<256>(const KernelParams&, int, bool, bool, bool, hipStream_t);

namespace {

// One workgroup per 128-query block; thread r owns query row r and walks the
// key tiles.  mass[block, tile] = sum_r numerator * 2^(tile_max - m) / d,
// reduced by a shuffle-down tree per 32 rows and a second tree over the four
// partial sums (reference attention_int8.cuh:1028-1088).
__global__ __launch_bounds__(128) void block_mass_kernel(float* __restrict__ workspace, int q_len,
                                                         int n_kb, int n_qb, int q_heads, int batch) {
  __shared__ float partial[4];
  const int q_block = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x;
  const int query = q_block * kQueryBlock + tid;
  const uint64_t query_rows = static_cast<uint64_t>(batch) * q_heads * q_len;
  const uint64_t mass_elements = static_cast<uint64_t>(batch) * q_heads * n_qb * n_kb;
  const uint64_t full_words = query_rows * (n_kb - 1) * 2;
  const uint32_t* stats = reinterpret_cast<const uint32_t*>(workspace + mass_elements);
  const float* state = reinterpret_cast<const float*>(stats + full_words + query_rows * 2);
  const uint64_t row = (static_cast<uint64_t>(b) * q_heads + head) * q_len + query;
  const bool active = query < q_len;
  const float m = active ? state[row * 2] : 0.0f;
  const float d = active ? state[row * 2 + 1] : 0.0f;
  const uint64_t mass_row = (static_cast<uint64_t>(b) * q_heads + head) * n_qb + q_block;
  for (int tile = 0; tile < n_kb; ++tile) {
    float value = 0.0f;
    if (active && d > 0.0f) {
      float numerator, tile_max;
      if (tile + 1 < n_kb) {
        const uint64_t offset = (row * (n_kb - 1) + tile) * 2;
        numerator = static_cast<float>(stats[offset]);
        tile_max = __uint_as_float(stats[offset + 1]);
      } else {
        const uint64_t offset = full_words + row * 2;
        numerator = __uint_as_float(stats[offset]);
        tile_max = __uint_as_float(stats[offset + 1]);
      }
      value = numerator * __builtin_amdgcn_exp2f(tile_max - m) / d;
    }
#pragma unroll
    for (int offset = 16; offset > 0; offset >>= 1) value += __shfl_down(value, offset, 32);
    if ((tid & 31) == 0) partial[tid >> 5] = value;
    __syncthreads();
    if (tid == 0) {
      workspace[mass_row * n_kb + tile] = (partial[0] + partial[2]) + (partial[1] + partial[3]);
    }
    __syncthreads();
  }
}

}  // namespace

int launch_attention(const AttentionArgs& a, hipStream_t stream) {
  if (a.cta_k != 64 && a.cta_k != 128) return fail("risa_attention: cta_k must be 64 or 128");
  if (a.cta_k == 128 && a.head_dim == 64)
    return fail("risa_attention: cta_k 128 requires head_dim 128 or 256");
  const bool sparse = a.sparse_row_offsets != nullptr || a.sparse_block_indices != nullptr;
  if (sparse && (a.sparse_row_offsets == nullptr || a.sparse_block_indices == nullptr))
    return fail("risa_attention: sparse row offsets and block indices must be provided together");
  const bool capture = a.block_mass != nullptr;
  if (capture && sparse) return fail("risa_attention: block mass requires dense attention");
  if (a.v_tile_sum == nullptr) return fail("risa_attention: V tile sums are required");
  if (a.q_heads % a.kv_heads != 0) return fail("risa_attention: head counts are incompatible");
  const int64_t padded_keys = static_cast<int64_t>((a.k_len + a.cta_k - 1) / a.cta_k) * a.cta_k;
  if (padded_keys * a.head_dim >= (int64_t{1} << 32) || static_cast<int64_t>(a.k_len) * a.head_dim >= (int64_t{1} << 31))
    return fail("risa_attention: one head of K or V exceeds the 32-bit tile offsets of the kernel");

  KernelParams p{};
  p.q = a.q;
  p.k = a.k;
  p.v = a.v;
  p.out = a.out;
  p.q_scale = a.q_scale;
  p.k_scale = a.k_scale;
  p.v_scale = a.v_scale;
  p.v_center = a.v_center;
  p.v_tile_sum = a.v_tile_sum;
  p.mask = a.mask;
  p.mask_stride_b = a.mask_stride_b;
  p.mask_stride_h = a.mask_stride_h;
  p.mask_stride_q = a.mask_stride_q;
  p.mask_stride_k = a.mask_stride_k;
  p.mask_dtype = a.mask != nullptr ? a.mask_dtype : -1;
  p.q_len = a.q_len;
  p.k_len = a.k_len;
  p.q_heads = a.q_heads;
  p.kv_heads = a.kv_heads;
  p.n_kb = (a.k_len + a.cta_k - 1) / a.cta_k;
  p.n_qb = (a.q_len + kQueryBlock - 1) / kQueryBlock;
  p.padded = p.n_kb * a.cta_k;
  p.batch = a.batch;
  p.out_stride_b = a.out_stride_b;
  p.out_stride_n = a.out_stride_n;
  p.out_stride_h = a.out_stride_h;
  p.sm2 = a.sm_scale * kLog2e;
  p.out_dtype = a.out_dtype;
  p.workspace = a.block_mass;
  p.lse = a.lse;
  p.causal = a.is_causal ? 1 : 0;

  const bool use_key_tiles = a.key_mask_tiles != nullptr && a.mask != nullptr &&
                             a.mask_stride_q == 0 && !sparse && !capture && !a.is_causal;
  if (sparse) {
    p.index_mode = 1;
    p.row_offsets = a.sparse_row_offsets;
    p.tile_indices = a.sparse_block_indices;
  } else if (use_key_tiles) {
    p.index_mode = 2;
    p.tile_indices = a.key_mask_tiles;
  }
  const bool indexed = p.index_mode != 0;
  const bool fast = a.mask == nullptr && !a.is_causal && a.sm_scale > 0.0f;

  int status;
  if (a.head_dim == 64)
    status = launch_attention_variant<64>(p, a.cta_k, fast, indexed, capture, stream);
  else if (a.head_dim == 128)
    status = launch_attention_variant<128>(p, a.cta_k, fast, indexed, capture, stream);
  else if (a.head_dim == 256)
    status = launch_attention_variant<256>(p, a.cta_k, fast, indexed, capture, stream);
  else
    return fail("risa_attention: unsupported head_dim");
  if (status != 0) return status;
  if (capture) {
    const dim3 grid(p.n_qb, a.q_heads, a.batch);
    block_mass_kernel<<<grid, 128, 0, stream>>>(a.block_mass, a.q_len, p.n_kb, p.n_qb, a.q_heads,
                                                a.batch);
  }
  return check_launch("risa_attention");
}

}  // namespace risa
