// Q/K preparation for gfx950: K anchor detection, sign-diagonal + Walsh-Hadamard
// rotation and per-group signed INT8 quantisation.
//
// Numerical contract (bit-exact): reference csrc/kernels/quantize_qk_impl.cuh
//   detect_k_anchor :442-577, rotations :69-147, process_q :153-269,
//   process_k :278-426, dispatch by (head_dim, key_length) :769-811.
// The reference assigns one scale group to a 32-lane warp in which every lane
// owns four adjacent channels.  Here one 32-lane half of a 64-wide wavefront
// plays that role, so a wavefront quantises two scale groups at once and the
// butterfly order (4-point local stage, then lane bits 1, 2, 4, 8, 16) is the
// reference's.  All arithmetic is IEEE binary32 without contraction.

#pragma once

#include "common.hpp"
#include "launchers.hpp"

#include <type_traits>

namespace risa {
namespace {

constexpr int kRot4 = 4;
constexpr int kRot64 = 64;
constexpr int kRot128Signed = 128;
constexpr int kRot128Plain = 129;

__device__ __forceinline__ void rotate4(float* v) {
  const float a0 = v[0] + v[1];
  const float a1 = v[0] - v[1];
  const float a2 = v[2] + v[3];
  const float a3 = v[2] - v[3];
  v[0] = (a0 + a2) * 0.5f;
  v[1] = (a1 + a3) * 0.5f;
  v[2] = (a0 - a2) * 0.5f;
  v[3] = (a1 - a3) * 0.5f;
}

// Channel c keeps its sign when bit c%32 of word c/32 is set and is negated
// otherwise; `sub` is the lane inside the 32-lane half, owning channels 4*sub..
__device__ __forceinline__ void apply_sign_diagonal(float* v, int sub) {
  const uint32_t words[4] = {0x1035997bu, 0x8087f5eeu, 0xee2e4e1au, 0x71132418u};
  const uint32_t word = words[sub >> 3];
  const int shift = (sub & 7) * 4;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint32_t flip = ((word >> (shift + c)) & 1u) ^ 1u;
    v[c] = __uint_as_float(__float_as_uint(v[c]) ^ (flip << 31));
  }
}

// Value of lane (l xor BIT) for BIT in {1, 2, 4, 8}, with DPP moves (no LDS
// traffic): quad permutations inside groups of four lanes, for BIT 4 two row shifts
// written under a bank mask (lanes whose partner is above take the left shift, the
// others the right shift), for BIT 8 one rotation of the row by eight lanes.
template <int BIT> __device__ __forceinline__ float dpp_partner(float value) {
  const int bits = __float_as_int(value);
  if constexpr (BIT == 1) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, bits, 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
  } else if constexpr (BIT == 2) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, bits, 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
  } else if constexpr (BIT == 4) {
    const int up = __builtin_amdgcn_update_dpp(0, bits, 0x104, 0xf, 0x5, true);      // row_shl:4 -> banks 0, 2
    return __int_as_float(__builtin_amdgcn_update_dpp(up, bits, 0x114, 0xf, 0xA, false));  // row_shr:4 -> banks 1, 3
  } else {
    static_assert(BIT == 8, "DPP reaches partners inside a row of sixteen lanes");
    // rotating a row of sixteen lanes by eight swaps its halves: lane l reads lane l xor 8
    return __int_as_float(__builtin_amdgcn_update_dpp(0, bits, 0x128, 0xf, 0xf, true));  // row_ror:8
  }
}

// One Hadamard butterfly level between lanes l and l xor BIT for COUNT values of a lane.  The
// reference keeps a + b on the lane with the bit clear and a - b on the other (a: the value of
// the lane with the bit clear).  Here every lane computes own + beta * partner in one fused
// multiply-add whose DPP operand is the partner (beta = -1 on the lanes with the bit set, a
// product that is exact): the lane with the bit set ends up with b - a, the exact negative of
// the reference's value (IEEE addition is symmetric in sign).  Partners of a later level differ
// in that level's bit only, so both carry the same sign and the recurrence holds at every
// level; after all levels lane j holds the reference's values times (-1)^popcount(j), which the
// caller folds into the final scaling.  All values of the lane pass a level together, so that
// the exchanges of one value (which must wait two cycles for the instruction that produced
// their operand) issue between those of the others.
//
// The multiply-adds are written out (four values per block): the compiler selects the VOP3
// form of a fused multiply-add, which takes no DPP operand, and would spend a separate move
// per exchange.  Every instruction of a block reads and writes its own value only, and a
// value was last written a whole level earlier, which is what an instruction with a DPP
// operand requires (two wait states after the write of its source); the s_nop in front of a
// level's first block covers whatever the compiler placed ahead of it.
#define RISA_BUTTERFLY_BLOCK(NOP, CONTROL)                                                   \
  asm volatile(NOP                                                                           \
               "v_fmac_f32_dpp %0, %0, %4 " CONTROL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
               "v_fmac_f32_dpp %1, %1, %4 " CONTROL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
               "v_fmac_f32_dpp %2, %2, %4 " CONTROL " row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t" \
               "v_fmac_f32_dpp %3, %3, %4 " CONTROL " row_mask:0xf bank_mask:0xf bound_ctrl:1"       \
               : "+v"(*values[n]), "+v"(*values[n + 1]), "+v"(*values[n + 2]), "+v"(*values[n + 3]) \
               : "v"(beta))
template <int BIT, int COUNT> __device__ __forceinline__ void butterfly_level(float* (&values)[COUNT], int sub) {
  static_assert(BIT == 1 || BIT == 2 || BIT == 4 || BIT == 8, "DPP reaches partners inside a row of sixteen lanes");
  static_assert(COUNT % 4 == 0, "values come in runs of four channels");
  const float beta = (sub & BIT) ? -1.0f : 1.0f;
#pragma unroll
  for (int n = 0; n < COUNT; n += 4) {
    if constexpr (BIT == 1) {
      if (n == 0) {
        RISA_BUTTERFLY_BLOCK("s_nop 1\n\t", "quad_perm:[1,0,3,2]");
      } else {
        RISA_BUTTERFLY_BLOCK("", "quad_perm:[1,0,3,2]");
      }
    } else if constexpr (BIT == 2) {
      if (n == 0) {
        RISA_BUTTERFLY_BLOCK("s_nop 1\n\t", "quad_perm:[2,3,0,1]");
      } else {
        RISA_BUTTERFLY_BLOCK("", "quad_perm:[2,3,0,1]");
      }
    } else if constexpr (BIT == 8) {
      // rotating a row of sixteen lanes by eight swaps its halves
      if (n == 0) {
        RISA_BUTTERFLY_BLOCK("s_nop 1\n\t", "row_ror:8");
      } else {
        RISA_BUTTERFLY_BLOCK("", "row_ror:8");
      }
    } else {
      // l xor 4 = (l xor 3) xor 7: the reversal of every quad, then the reversal of every eight
      // lanes; the second move joins the multiply-add.  (A row shift reaches l xor 4 only for
      // half of the lanes, which takes two moves that cannot join it.)
      float r0, r1, r2, r3;
      asm volatile("s_nop 1\n\t"
                   "v_mov_b32_dpp %4, %0 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %5, %1 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %6, %2 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_mov_b32_dpp %7, %3 quad_perm:[3,2,1,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %0, %4, %8 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %1, %5, %8 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %2, %6, %8 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
                   "v_fmac_f32_dpp %3, %7, %8 row_half_mirror row_mask:0xf bank_mask:0xf bound_ctrl:1"
                   : "+v"(*values[n]), "+v"(*values[n + 1]), "+v"(*values[n + 2]), "+v"(*values[n + 3]),
                     "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3)
                   : "v"(beta));
    }
  }
}
#undef RISA_BUTTERFLY_BLOCK

// Rotation of the channels one lane holds of SETS 128-channel blocks (64 channels for head
// dim 64), SETS = tokens x blocks the lane works on.  Sixteen lanes share a token; lane j
// owns GROUPS runs of four consecutive channels per block, 4*GROUPS*j + 4g .. +3, i.e. the
// channels of lanes 2j and 2j+1 (GROUPS 2) or of lane j (GROUPS 1) of the reference's 32-lane
// layout (csrc/kernels/quantize_qk.cuh).  The additions are the reference's, in its order for
// every value: 4-point transform per run, then one butterfly level per channel bit from bit 2
// up -- the first inside the lane when it holds two runs, the others between lanes with DPP
// moves, bits 1, 2, 4, 8 of the lane index in turn.
template <int ROT, int GROUPS, int SETS> __device__ __forceinline__ void rotate(float (*v[SETS])[4], int j) {
#pragma unroll
  for (int set = 0; set < SETS; ++set)
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      if constexpr (ROT == kRot128Signed) apply_sign_diagonal(v[set][g], GROUPS * j + g);
      rotate4(v[set][g]);
    }
  if constexpr (ROT == kRot4) return;
  if constexpr (GROUPS == 2) {
#pragma unroll
    for (int set = 0; set < SETS; ++set)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float low = v[set][0][c], high = v[set][1][c];
        v[set][0][c] = low + high;
        v[set][1][c] = low - high;
      }
  }
  constexpr int COUNT = SETS * GROUPS * 4;
  float* values[COUNT];
#pragma unroll
  for (int set = 0; set < SETS; ++set)
#pragma unroll
    for (int g = 0; g < GROUPS; ++g)
#pragma unroll
      for (int c = 0; c < 4; ++c) values[(set * GROUPS + g) * 4 + c] = &v[set][g][c];
  butterfly_level<1, COUNT>(values, j);
  butterfly_level<2, COUNT>(values, j);
  butterfly_level<4, COUNT>(values, j);
  butterfly_level<8, COUNT>(values, j);
  // the scaling of the transform, with the sign the butterfly levels left on this lane
  constexpr float factor = ROT == kRot64 ? 0.25f : 0.1767766952966369f;
  const float lane_factor = (__builtin_popcount(j & 15) & 1) ? -factor : factor;
#pragma unroll
  for (int n = 0; n < COUNT; ++n) *values[n] *= lane_factor;
}

// Maximum over the 32 lanes of a half wavefront, in every lane: one lane swap for the
// two 16-lane rows, DPP moves inside a row, no LDS round trips.
__device__ __forceinline__ float half_wave_max(float value) {
  value = max_across_row_pairs(value);
  value = __builtin_fmaxf(value, dpp_partner<8>(value));
  value = __builtin_fmaxf(value, dpp_partner<4>(value));
  value = __builtin_fmaxf(value, dpp_partner<2>(value));
  value = __builtin_fmaxf(value, dpp_partner<1>(value));
  return value;
}

// One scale group handled by LANES lanes (a 32-lane half or a whole wavefront): NTOK
// tokens x DK channels, LANES / 16 tokens at a time (one per 16-lane row).
// `token_of(i)` gives the i-th token of the group, `sub` the lane's index inside the
// LANES.  `wide` says rows are 16-byte aligned, so 16-bit inputs are read eight
// channels per load.
// `own_max` / `partner_max` (optional): LDS slots through which two wavefronts that share one
// scale group (each with NTOK of its tokens) exchange their maxima; `own_max` is written, a
// workgroup barrier follows, `partner_max` is read.  The maximum is order independent.
template <int DT, int DK, int ROT, int NTOK, int LANES = 32, typename TokenOf>
__device__ __forceinline__ void quantize_group(const void* in, int64_t in_base, int64_t stride_n,
                                               int8_t* out, float* scale_slot, int length, int sub,
                                               bool has_bias, int64_t bias_offset, bool wide, TokenOf token_of,
                                               const int32_t* source = nullptr, float* own_max = nullptr,
                                               const float* partner_max = nullptr) {
  constexpr int BLOCKS = DK == 256 ? 2 : 1;   // 128-channel rotation blocks
  constexpr int GROUPS = DK == 64 ? 1 : 2;    // runs of four channels per lane and block
  constexpr int PER_STEP = LANES / 16;
  constexpr int STEPS = NTOK / PER_STEP;
  static_assert(LANES == 32 || LANES == 64, "a half or a whole wavefront");
  static_assert(NTOK % PER_STEP == 0, "whole steps");
  const int j = sub & 15, row = sub >> 4;
  auto channel_of = [&](int block, int g) { return block * 128 + (GROUPS * j + g) * 4; };

  // Every load of the group is issued before any is consumed, and none sits inside a
  // branch (the compiler waits for each load of a conditional block before leaving it):
  // tokens past the end read the last row and are zeroed afterwards, the gather indices are
  // fetched as one batch, the row that stands in for a missing anchor row is ignored, and the
  // uniform choices (row width, permutation) are made once around the whole batch.
  float bias[BLOCKS][GROUPS][4];
  float v[STEPS][BLOCKS][GROUPS][4];
  int from[STEPS];
  bool valid[STEPS];
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    const int n = token_of(PER_STEP * i + row);
    valid[i] = n < length;
    from[i] = min(n, length - 1);
  }
  if (source != nullptr) {
    // with a permutation, token n of the gathered sequence is source row source[n]
#pragma unroll
    for (int i = 0; i < STEPS; ++i) from[i] = source[from[i]];
  }
  const int64_t bias_base =
      in_base + (has_bias ? bias_offset : static_cast<int64_t>(from[0]) * stride_n);
  auto load_all = [&](auto wide_tag) {
    constexpr bool EIGHT = GROUPS == 2 && DT != kF32 && decltype(wide_tag)::value;
    auto load_row = [&](int64_t row_base, float (&dst)[BLOCKS][GROUPS][4]) {
#pragma unroll
      for (int block = 0; block < BLOCKS; ++block) {
        if constexpr (EIGHT) {
          float eight[8];
          load8<DT>(in, row_base + channel_of(block, 0), eight);
#pragma unroll
          for (int c = 0; c < 8; ++c) dst[block][c / 4][c % 4] = eight[c];
        } else {
#pragma unroll
          for (int g = 0; g < GROUPS; ++g) load4<DT>(in, row_base + channel_of(block, g), dst[block][g]);
        }
      }
    };
    load_row(bias_base, bias);
#pragma unroll
    for (int i = 0; i < STEPS; ++i) load_row(in_base + static_cast<int64_t>(from[i]) * stride_n, v[i]);
  };
  if (wide) {
    load_all(std::true_type{});
  } else {
    load_all(std::false_type{});
  }
#pragma unroll
  for (int i = 0; i < STEPS; ++i)
#pragma unroll
    for (int block = 0; block < BLOCKS; ++block)
#pragma unroll
      for (int g = 0; g < GROUPS; ++g)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float shifted = has_bias ? v[i][block][g][c] - bias[block][g][c] : v[i][block][g][c];
          v[i][block][g][c] = valid[i] ? shifted : 0.0f;
        }
  float mx = 0.0f;
  {
    // Eight token-blocks (32 values of a lane) at a time through the butterfly levels: enough
    // independent exchanges to hide their operand latency, few enough to stay in registers.
    constexpr int SETS = STEPS * BLOCKS;
    constexpr int BATCH = SETS < 8 ? SETS : 8;
    static_assert(SETS % BATCH == 0, "whole batches");
#pragma unroll
    for (int first = 0; first < SETS; first += BATCH) {
      float (*sets[BATCH])[4];
#pragma unroll
      for (int n = 0; n < BATCH; ++n) sets[n] = v[(first + n) / BLOCKS][(first + n) % BLOCKS];
      rotate<ROT, GROUPS, BATCH>(sets, j);
    }
  }
#pragma unroll
  for (int i = 0; i < STEPS; ++i)
#pragma unroll
    for (int block = 0; block < BLOCKS; ++block)
#pragma unroll
      for (int g = 0; g < GROUPS; ++g)
#pragma unroll
        for (int c = 0; c < 4; ++c) mx = __builtin_fmaxf(mx, __builtin_fabsf(v[i][block][g][c]));
  mx = half_wave_max(mx);
  if constexpr (LANES == 64) mx = max_across_halves(mx);
  if (own_max != nullptr) {
    if (sub == 0) *own_max = mx;
    __syncthreads();
    mx = __builtin_fmaxf(mx, *partner_max);
  }
  const float scale = mx / 127.0f + 1e-7f;
  const float inverse = 1.0f / scale;
  if (sub == 0) *scale_slot = scale;
#pragma unroll
  for (int i = 0; i < STEPS; ++i) {
    const int n = token_of(PER_STEP * i + row);
    if (n < length) {
#pragma unroll
      for (int block = 0; block < BLOCKS; ++block) {
        uint32_t packed[GROUPS];
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
          packed[g] = pack_codes(round_to_code(v[i][block][g][0] * inverse), round_to_code(v[i][block][g][1] * inverse),
                                 round_to_code(v[i][block][g][2] * inverse), round_to_code(v[i][block][g][3] * inverse));
        }
        int8_t* at = out + static_cast<int64_t>(n) * DK + channel_of(block, 0);
        if constexpr (GROUPS == 2) {
          *reinterpret_cast<uint2*>(at) = make_uint2(packed[0], packed[1]);
        } else {
          *reinterpret_cast<uint32_t*>(at) = packed[0];
        }
      }
    }
  }
}

// One W-row slice of one (batch, head): eight 32-lane halves = the eight scale
// groups (token index mod 8), W = 32 (16 for head_dim 256).  256 threads.
template <int DT, int DK, int ROT>
__device__ __forceinline__ void quantize_q_block(const void* __restrict__ q, int8_t* __restrict__ codes,
                                                 float* __restrict__ scales, int length, int heads,
                                                 int scales_per_head, int64_t stride_b,
                                                 int64_t stride_h, int64_t stride_n, int wide,
                                                 int slice, int h, int b) {
  constexpr int W = DK == 256 ? 16 : 32;
  constexpr int NR = W / 8;
  const int sub = threadIdx.x & 31;
  const int group = threadIdx.x >> 5;
  const int64_t in_base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t bh = static_cast<int64_t>(b) * heads + h;
  const int base = slice * W + group;
  quantize_group<DT, DK, ROT, NR>(q, in_base, stride_n, codes + bh * length * DK,
                                  scales + bh * scales_per_head + slice * 8 + group, length, sub,
                                  false, 0, wide != 0, [base](int i) { return base + i * 8; });
}

// grid (slices, Hq, B), 256 threads.  One slice (8 KB of input) per workgroup: two or
// four slices per workgroup measure the same (52-54 us at 16 x 32768 tokens), workgroup
// launch is not what limits the kernel.
template <int DT, int DK, int ROT>
__global__ __launch_bounds__(256) void quantize_q_kernel(const void* __restrict__ q,
                                                         int8_t* __restrict__ codes,
                                                         float* __restrict__ scales, int length,
                                                         int heads, int scales_per_head,
                                                         int64_t stride_b, int64_t stride_h,
                                                         int64_t stride_n, int wide) {
  quantize_q_block<DT, DK, ROT>(q, codes, scales, length, heads, scales_per_head, stride_b, stride_h,
                                stride_n, wide, blockIdx.x, blockIdx.y, blockIdx.z);
}

// Half of key tile `tile` (`part` 0 or 1: its scale groups 2*part and 2*part + 1, scale group of
// a token = (token mod 8) / 2) by one workgroup of four wavefronts: two wavefronts per scale
// group, each with half of the group's tokens, four tokens per step; the two exchange their
// maxima through LDS.  A wavefront then keeps CTA_K / 8 rotated tokens in registers instead of
// CTA_K / 4, and twice as many wavefronts stand behind every tile.
template <int DT, int DK, int CTA_K, int ROT>
__device__ __forceinline__ void quantize_k_block(const void* __restrict__ k, int8_t* __restrict__ codes,
                                                 float* __restrict__ scales, int anchor, int length,
                                                 int heads, int scales_per_head, int64_t stride_b,
                                                 int64_t stride_h, int64_t stride_n, int wide,
                                                 const int32_t* __restrict__ permutation, int tile,
                                                 int part, int h, int b) {
  constexpr int NTOK = CTA_K / 8;  // tokens of the group held by one wavefront
  __shared__ float wave_max[4];
  const int sub = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int group = part * 2 + (wave >> 1);
  const int first_index = (wave & 1) * NTOK;  // this wavefront's share of the group's CTA_K / 4 tokens
  const int64_t in_base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t bh = static_cast<int64_t>(b) * heads + h;
  const int32_t* source = permutation != nullptr ? permutation + bh * length : nullptr;
  // element offset of the anchor row (subtracted from every key) when one was chosen
  const int anchor_row = anchor >= 0 && source != nullptr ? source[anchor] : anchor;
  const int64_t anchor_offset = static_cast<int64_t>(anchor_row) * stride_n;
  const int first = tile * CTA_K + group * 2;
  quantize_group<DT, DK, ROT, NTOK, 64>(
      k, in_base, stride_n, codes + bh * length * DK, scales + bh * scales_per_head + tile * 4 + group,
      length, sub, anchor >= 0, anchor_offset, wide != 0,
      [first, first_index](int i) { return first + ((i + first_index) >> 1) * 8 + ((i + first_index) & 1); },
      source, wave_max + wave, wave_max + (wave ^ 1));
}

// grid (2 * key tiles, Hkv, B), 256 threads: half a key tile of CTA_K tokens per workgroup.
template <int DT, int DK, int CTA_K, int ROT>
__global__ __launch_bounds__(256) void quantize_k_kernel(const void* __restrict__ k,
                                                         int8_t* __restrict__ codes,
                                                         float* __restrict__ scales,
                                                         const int* __restrict__ anchors, int length,
                                                         int heads, int scales_per_head,
                                                         int64_t stride_b, int64_t stride_h,
                                                         int64_t stride_n, int wide,
                                                         const int32_t* __restrict__ permutation) {
  quantize_k_block<DT, DK, CTA_K, ROT>(k, codes, scales, anchors[blockIdx.z * heads + blockIdx.y], length, heads,
                                       scales_per_head, stride_b, stride_h, stride_n, wide, permutation,
                                       blockIdx.x >> 1, blockIdx.x & 1, blockIdx.y, blockIdx.z);
}

// ---------------------------------------------------------------------------
// Anchor detector of one (batch, head).  The first 128 threads of the workgroup work
// (the others only take part in the barriers).  Thread t owns channels t and
// t+128; partial sums are combined by a 32-lane shuffle-down tree and then the
// four 32-lane segments are added in order, which is the reference's order.
// ---------------------------------------------------------------------------
constexpr int kSamples = 9;

// Sum / maximum of a 32-lane segment as lane 0 of the segment gets it from a
// shuffle-down tree with offsets 16, 8, 4, 2, 1 (the reference's order).  An exchange
// butterfly gives lane 0 the same additions in the same order (x + y = y + x exactly),
// and needs one lane swap plus four DPP moves instead of five trips through LDS.
__device__ __forceinline__ float segment_down_sum(float value) {
  const auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(value), __float_as_uint(value), false, false);
  value = __uint_as_float(rows[0]) + __uint_as_float(rows[1]);
  value += dpp_partner<8>(value);
  value += dpp_partner<4>(value);
  value += dpp_partner<2>(value);
  value += dpp_partner<1>(value);
  return value;
}
__device__ __forceinline__ float segment_down_max(float value) { return half_wave_max(value); }

// Returns the anchor row of (b, h), or -1, to every thread of the workgroup.
template <int DT>
__device__ __forceinline__ int detect_anchor_value(const void* __restrict__ k, int length, int dim, int heads,
                                                   int64_t stride_b, int64_t stride_h, int64_t stride_n,
                                                   const int32_t* __restrict__ permutation, int h, int b) {
  __shared__ float samples[kSamples * 256];
  __shared__ float seg_energy[4], seg_max[4], seg_dist[kSamples][4], seg_best_energy[4],
      seg_best_max[4];
  __shared__ int chosen;
  const int tid = threadIdx.x, sub = tid & 31, seg = tid >> 5;
  const bool working = tid < 128;
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  // Thread t fetches channels t and t + 128 of the nine sampled rows; every load is issued
  // before any is stored (the detector sits in front of the K quantisation of short problems,
  // where a loop of load-then-store round trips would be the longest chain of the launch).
  {
    int64_t rows[kSamples];
#pragma unroll
    for (int s = 0; s < kSamples; ++s) rows[s] = static_cast<int64_t>(s) * (length - 1) / (kSamples - 1);
    if (permutation != nullptr) {
#pragma unroll
      for (int s = 0; s < kSamples; ++s) rows[s] = permutation[(static_cast<int64_t>(b) * heads + h) * length + rows[s]];
    }
    float fetched[2][kSamples];
#pragma unroll
    for (int part = 0; part < 2; ++part) {
      // a channel past the head dim reads channel 0 (never stored)
      const int channel = tid + part * 128 < dim && working ? tid + part * 128 : 0;
#pragma unroll
      for (int s = 0; s < kSamples; ++s) fetched[part][s] = load1<DT>(k, base + rows[s] * stride_n + channel);
    }
#pragma unroll
    for (int part = 0; part < 2; ++part) {
      const int channel = tid + part * 128;
      if (working && channel < dim) {
#pragma unroll
        for (int s = 0; s < kSamples; ++s) samples[s * dim + channel] = fetched[part][s];
      }
    }
  }
  __syncthreads();

  float energy = 0.0f, peak = 0.0f, dist[kSamples];
#pragma unroll
  for (int c = 0; c < kSamples; ++c) dist[c] = 0.0f;
  for (int channel = working ? tid : dim; channel < dim; channel += 128) {
    float sum = 0.0f;
#pragma unroll
    for (int s = 0; s < kSamples; ++s) {
      const float value = samples[s * dim + channel];
      energy = __builtin_fmaf(value, value, energy);
      peak = __builtin_fmaxf(peak, __builtin_fabsf(value));
      sum += value;
    }
#pragma unroll
    for (int c = 0; c < kSamples; ++c) {
      const float d = 9.0f * samples[c * dim + channel] - sum;
      dist[c] = __builtin_fmaf(d, d, dist[c]);
    }
  }
  energy = segment_down_sum(energy);
  peak = segment_down_max(peak);
#pragma unroll
  for (int c = 0; c < kSamples; ++c) dist[c] = segment_down_sum(dist[c]);
  if (sub == 0 && working) {
    seg_energy[seg] = energy;
    seg_max[seg] = peak;
#pragma unroll
    for (int c = 0; c < kSamples; ++c) seg_dist[c][seg] = dist[c];
  }
  __syncthreads();
  if (tid == 0) {
    int best = 0;
    float best_distance = 3.402823466e+38f;
    for (int c = 0; c < kSamples; ++c) {
      float total = 0.0f;
      for (int w = 0; w < 4; ++w) total += seg_dist[c][w];
      if (total < best_distance) {
        best = c;
        best_distance = total;
      }
    }
    chosen = best;
  }
  __syncthreads();
  const int best = chosen;
  float best_energy = 0.0f, best_peak = 0.0f;
  for (int channel = working ? tid : dim; channel < dim; channel += 128) {
    const float anchor = samples[best * dim + channel];
#pragma unroll
    for (int s = 0; s < kSamples; ++s) {
      const float residual = samples[s * dim + channel] - anchor;
      best_energy = __builtin_fmaf(residual, residual, best_energy);
      best_peak = __builtin_fmaxf(best_peak, __builtin_fabsf(residual));
    }
  }
  best_energy = segment_down_sum(best_energy);
  best_peak = segment_down_max(best_peak);
  if (sub == 0 && working) {
    seg_best_energy[seg] = best_energy;
    seg_best_max[seg] = best_peak;
  }
  __syncthreads();
  if (tid == 0) {
    float e0 = 0.0f, m0 = 0.0f, e1 = 0.0f, m1 = 0.0f;
    for (int w = 0; w < 4; ++w) {
      e0 += seg_energy[w];
      m0 = __builtin_fmaxf(m0, seg_max[w]);
      e1 += seg_best_energy[w];
      m1 = __builtin_fmaxf(m1, seg_best_max[w]);
    }
    const bool improves = e1 < e0 && m1 <= m0 * 1.125f;
    chosen = improves ? static_cast<int>(static_cast<int64_t>(best) * (length - 1) / (kSamples - 1)) : -1;
  }
  __syncthreads();
  return chosen;
}

template <int DT>
__device__ __forceinline__ void detect_anchor_block(const void* __restrict__ k, int* __restrict__ anchors,
                                                    int length, int dim, int heads, int64_t stride_b,
                                                    int64_t stride_h, int64_t stride_n,
                                                    const int32_t* __restrict__ permutation, int h,
                                                    int b) {
  const int anchor = detect_anchor_value<DT>(k, length, dim, heads, stride_b, stride_h, stride_n, permutation, h, b);
  if (threadIdx.x == 0) anchors[b * heads + h] = anchor;
}


// grid (Hkv, B), 128 threads.
template <int DT>
__global__ __launch_bounds__(128) void detect_anchor_kernel(const void* __restrict__ k,
                                                            int* __restrict__ anchors, int length,
                                                            int dim, int heads, int64_t stride_b,
                                                            int64_t stride_h, int64_t stride_n,
                                                            const int32_t* __restrict__ permutation) {
  detect_anchor_block<DT>(k, anchors, length, dim, heads, stride_b, stride_h, stride_n, permutation,
                          blockIdx.x, blockIdx.y);
}

// 16-bit inputs can be read eight channels (16 bytes) per load when every row
// starts on a 16-byte boundary.
inline int rows_are_16_byte_aligned(const void* base, int64_t stride_b, int64_t stride_h,
                                    int64_t stride_n, int dtype) {
  if (dtype == kF32) return 1;
  return reinterpret_cast<uintptr_t>(base) % 16 == 0 && ((stride_b | stride_h | stride_n) & 7) == 0;
}

}  // namespace
}  // namespace risa
