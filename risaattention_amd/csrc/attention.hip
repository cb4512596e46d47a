// Host-side dispatch of the fused attention kernel and the block-mass
// reconstruction that follows a capturing run.
//
// Path selection follows reference csrc/kernels/attention_dispatch.cu:113-296:
// the raw-score path runs when there is no mask, no causal flag and a positive
// scale; custom and key-only masks share the pre-scaled path; sparse support
// and key-mask tile lists both iterate an index list.

#include "attention_dispatch.hpp"

#include <cstdlib>

namespace risa {

template <> int launch_attention_variant<64>(const KernelParams&, int, bool, bool, bool, int, hipStream_t);
template <> int launch_attention_variant<128>(const KernelParams&, int, bool, bool, bool, int, hipStream_t);
int launch_attention_narrow(const KernelParams& p, int head_dim, int cta_k, hipStream_t stream);
int launch_attention_narrow_general(const KernelParams& p, int head_dim, int cta_k, bool fast, bool indexed,
                                    bool capture, int mask_mode, hipStream_t stream);

namespace {

// mass[block, tile] = sum_r numerator * 2^(tile_max - m) / d over the 128 query
// rows r of the block, added in the order of the reference (attention_int8.cuh:
// 1028-1088): a shuffle-down tree per 32 rows (offsets 16, 8, 4, 2, 1), then
// (p0 + p2) + (p1 + p3) over the four partial sums.
//
// One workgroup per query block, one wavefront per key tile (strided).  Lane l
// owns rows 2l and 2l+1, so a tile's statistics of the whole block are one
// coalesced 1 KB load (the attention kernel stores them tile-major).  In the
// tree, rows 16, 8, 4, 2 apart are lanes 8, 4, 2, 1 apart within a 16-lane
// group and the last level adds a lane's own two rows.
__global__ __launch_bounds__(256) void block_mass_kernel(float* __restrict__ workspace, int q_len,
                                                         int n_kb, int n_qb, int q_heads, int batch) {
  const int q_block = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int query = q_block * kQueryBlock + 2 * lane;
  const uint64_t bhq = static_cast<uint64_t>(b) * q_heads + head;
  const uint64_t query_rows = static_cast<uint64_t>(batch) * q_heads * q_len;
  const uint64_t mass_elements = static_cast<uint64_t>(batch) * q_heads * n_qb * n_kb;
  const uint64_t full_words = query_rows * (n_kb - 1) * 2;
  const uint32_t* stats = reinterpret_cast<const uint32_t*>(workspace + mass_elements);
  const float* state = reinterpret_cast<const float*>(stats + full_words + query_rows * 2);
  const uint64_t row = bhq * q_len + query;
  // q_len may be odd: the second row of the last lane can be out of range.
  const bool active0 = query < q_len, active1 = query + 1 < q_len;
  float m[2] = {0.0f, 0.0f}, d[2] = {0.0f, 0.0f};
  if (active0) {
    m[0] = state[row * 2];
    d[0] = state[row * 2 + 1];
  }
  if (active1) {
    m[1] = state[row * 2 + 2];
    d[1] = state[row * 2 + 3];
  }
  const uint64_t mass_row = bhq * n_qb + q_block;
  for (int tile = wave; tile < n_kb; tile += 4) {
    const bool last = tile + 1 == n_kb;
    const uint64_t offset =
        last ? full_words + row * 2 : ((bhq * (n_kb - 1) + tile) * static_cast<uint64_t>(q_len) + query) * 2;
    float value[2] = {0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if ((j == 0 ? active0 : active1) && d[j] > 0.0f) {
        const uint32_t raw = stats[offset + 2 * j];
        const float numerator = last ? __uint_as_float(raw) : static_cast<float>(raw);
        const float tile_max = __uint_as_float(stats[offset + 2 * j + 1]);
        value[j] = numerator * __builtin_amdgcn_exp2f(tile_max - m[j]) / d[j];
      }
    }
#pragma unroll
    for (int step = 8; step > 0; step >>= 1) {
      value[0] += __shfl_down(value[0], step, 16);
      value[1] += __shfl_down(value[1], step, 16);
    }
    const float group = value[0] + value[1];              // lanes 0, 16, 32, 48: p0..p3
    const float pair = group + __shfl_down(group, 32);    // lane 0: p0 + p2, lane 16: p1 + p3
    const float total = pair + __shfl_down(pair, 16);
    if (lane == 0) workspace[mass_row * n_kb + tile] = total;
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
  // output rows leave the kernels in 16-byte pieces
  if (reinterpret_cast<uintptr_t>(a.out) % 16 != 0 || ((a.out_stride_b | a.out_stride_h | a.out_stride_n) & 7) != 0)
    return fail("risa_attention: the output must be 16-byte aligned, with strides that are multiples of 8 elements");
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
  int mask_mode = kMaskScalar;
  int lane_planes_b = 0, lane_planes_h = 0;  // mask planes behind the lane words
  if (a.mask != nullptr) {
    // Groups of four keys start at multiples of four, so one load per group needs
    // unit key stride, the other strides multiples of four elements and the base
    // aligned to four elements.  Staging the mask tile in LDS copies 16 bytes per lane:
    // everything 16-byte aligned, rows not overlapping backwards, and the 128 rows of a
    // query block within reach of a 32-bit byte offset.
    const int64_t element = mask_element_bytes(a.mask_dtype);
    const auto address = reinterpret_cast<uintptr_t>(a.mask);
    const int64_t strides = a.mask_stride_b | a.mask_stride_h | a.mask_stride_q;
    if (a.mask_stride_k == 1 && address % (4 * element) == 0 && (strides & 3) == 0) {
      mask_mode = kMaskVector;
      if (address % 16 == 0 && (strides * element) % 16 == 0 && a.mask_stride_q >= 0 &&
          a.mask_stride_q * element * kQueryBlock < (int64_t{1} << 31)) {
        mask_mode = kMaskStaged;
      }
    }
    if (a.mask_lanes != nullptr && a.head_dim <= 128) {  // the sixteen-query kernel of head dim 256 reads the mask itself
      if (a.mask_dtype != kBool || a.cta_k != 64 || a.mask_stride_q == 0 || a.mask_stride_k != 1)
        return fail("risa_attention: lane words go with a query-dependent boolean mask of unit key stride and 64-key tiles");
      // The strides say how many planes the buffer was made for: they are either zero or the
      // words of one plane (times the head planes for the batch stride).
      {
        const int64_t plane = static_cast<int64_t>(mask_lane_words(1, 1, a.q_len, a.k_len));
        const int64_t heads = a.mask_lanes_stride_h != 0 ? a.q_heads : 1;
        if ((a.mask_lanes_stride_h != 0 && a.mask_lanes_stride_h != plane) ||
            (a.mask_lanes_stride_b != 0 && a.mask_lanes_stride_b != plane * heads))
          return fail("risa_attention: lane word strides must be 0 or the plane sizes risa_prepare_mask_lanes uses");
      }
      if (reinterpret_cast<uintptr_t>(a.mask_lanes) % 8 != 0)
        return fail("risa_attention: lane words must be 8-byte aligned");
      mask_mode = kMaskLanes;
      p.mask_lanes = a.mask_lanes;
      p.mask_lanes_stride_b = a.mask_lanes_stride_b;
      p.mask_lanes_stride_h = a.mask_lanes_stride_h;
      lane_planes_b = a.mask_lanes_stride_b != 0 ? a.batch : 1;
      lane_planes_h = a.mask_lanes_stride_h != 0 ? a.q_heads : 1;
    }
    if (a.key_bias != nullptr) {
      if (a.mask_stride_q != 0) return fail("risa_attention: a key bias row needs a key-only mask");
      if (reinterpret_cast<uintptr_t>(a.key_bias) % 16 != 0 || (a.key_bias_stride_b | a.key_bias_stride_h) % 4 != 0)
        return fail("risa_attention: key bias rows must be 16-byte aligned");
      p.mask_dtype = kKeyBias;
      p.key_bias = a.key_bias;
      p.key_bias_stride_b = a.key_bias_stride_b;
      p.key_bias_stride_h = a.key_bias_stride_h;
    }
  }
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
  // Diagnostic switch, read at every launch: RISA_COMPILED_LOOP=1 sends the raw-score kernels of
  // head dim 128 through the tile loop the compiler schedules instead of the hand-scheduled one
  // (same results bit for bit; the tests compare the two).
  const char* compiled_loop = std::getenv("RISA_COMPILED_LOOP");
  p.compiled_loop = compiled_loop != nullptr && compiled_loop[0] != '\0' && compiled_loop[0] != '0';

  const bool use_key_tiles = a.key_mask_tiles != nullptr && a.mask != nullptr &&
                             a.mask_stride_q == 0 && !sparse && !capture && !a.is_causal;
  if (sparse) {
    p.index_mode = 1;
    p.row_offsets = a.sparse_row_offsets;
    p.tile_indices = a.sparse_block_indices;
  } else if (use_key_tiles) {
    p.index_mode = 2;
    p.tile_indices = a.key_mask_tiles;
  } else if (mask_mode == kMaskLanes && !capture && !a.is_causal) {
    // The buffer of the lane words also lists, per mask plane and query block, the tiles in
    // which the block sees a key at all: block-structured masks (documents, windows) skip
    // the rest the way a sparse pattern would; skipped tiles would have added zeros.
    p.index_mode = 3;
    p.tile_indices = reinterpret_cast<const int32_t*>(
        reinterpret_cast<const unsigned char*>(a.mask_lanes) +
        mask_tile_list_offset(lane_planes_b, lane_planes_h, a.q_len, a.k_len));
    const int64_t per_plane = static_cast<int64_t>(p.n_qb) * (p.n_kb + 1);
    p.tile_list_stride_h = lane_planes_h > 1 ? per_plane : 0;
    p.tile_list_stride_b = lane_planes_b > 1 ? per_plane * lane_planes_h : 0;
  }
  const bool indexed = p.index_mode != 0;
  const bool fast = a.mask == nullptr && !a.is_causal && a.sm_scale > 0.0f;

  // A launch that cannot give every compute unit more than one workgroup runs the
  // raw-score path with sixteen queries per wavefront (two wavefronts per SIMD).  So does
  // every launch with head dim 256, masked, causal and capturing ones included: thirty-two
  // queries of 256 channels per wavefront need some 380 registers, which leaves one
  // wavefront per SIMD (1200 against 1630 dense-equivalent TOPS at N=16K).
  const int64_t workgroups = static_cast<int64_t>(p.n_qb) * a.q_heads * a.batch;
  const bool narrow = fast && p.index_mode != 2 && !capture &&
                      (a.head_dim > 128 || workgroups <= narrow_attention_limit());

  // The other launches of that size (masked, causal, capturing, key-mask tile lists) and all of
  // head dim 256 take the same kernel with 128-query workgroups; lane words, when given, keep
  // the 32-query kernel that reads them.
  const bool narrow_general = !narrow && mask_mode != kMaskLanes &&
                              (a.head_dim > 128 || workgroups <= narrow_attention_limit());
  int status;
  if (narrow)
    status = launch_attention_narrow(p, a.head_dim, a.cta_k, stream);
  else if (narrow_general)
    status = launch_attention_narrow_general(p, a.head_dim, a.cta_k, fast, indexed, capture, mask_mode, stream);
  else if (a.head_dim == 64)
    status = launch_attention_variant<64>(p, a.cta_k, fast, indexed, capture, mask_mode, stream);
  else if (a.head_dim == 128)
    status = launch_attention_variant<128>(p, a.cta_k, fast, indexed, capture, mask_mode, stream);
  else
    return fail("risa_attention: unsupported head_dim");
  if (status != 0) return status;
  if (capture) {
    const dim3 grid(p.n_qb, a.q_heads, a.batch);
    block_mass_kernel<<<grid, 256, 0, stream>>>(a.block_mass, a.q_len, p.n_kb, p.n_qb, a.q_heads,
                                                a.batch);
  }
  return check_launch("risa_attention");
}

}  // namespace risa
