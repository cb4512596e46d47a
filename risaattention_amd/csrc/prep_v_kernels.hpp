// V preparation for gfx950: per-channel range, signed INT8 codes in the packed
// MFMA order, accumulator seeds (128 x per-tile code sums, the zero-point term of the
// signed P·V product, plus risa::kAccumulatorSeedBits) and
// the residual-corrected centre of the midpoint_affine mode.
//
// Numerical contract (bit-exact): reference csrc/kernels/quantize_v_impl.cuh:83-292
// (range :104-186, codes :203-246, residual centre :248-275) and the schedule
// choice of launch_quantize_v :356-401 (512 summation threads, 128 when L <= 256).
//
// The reference runs one block per (batch, head, 8 channels) that walks the whole
// sequence twice; at 32K tokens and four KV heads that is 64 blocks.  Here the
// sequence axis is split across the grid:
//   1. value_range_kernel     partial min/max per (wavefront chunk of 64+ tokens, channel)
//   2. value_params_kernel    scale, midpoint and reciprocal per channel
//   3. value_codes_kernel     codes + packed transposed store + tile sums
//   4. value_center_kernel    (affine) per-summation-thread residual sums in the
//                             reference's order (thread t adds tokens L-1-t-k*T),
//                             tree per 32 threads, warps in order
// min/max are order independent, so 1-3 are exact for any split; 4-5 keep the
// floating-point summation order explicitly.

#pragma once

#include <type_traits>

#include "common.hpp"
#include "launchers.hpp"

#include <cfloat>

namespace risa {
namespace {

// The range pass gives every wavefront tokens_per_wave(length) consecutive tokens:
// 64 up to 32768 tokens, then whatever keeps the number of partial ranges per
// (batch, head) at 512, which one wavefront of the parameter pass reduces in eight
// loads per lane.
__host__ __device__ inline int tokens_per_wave(int length) { return 64 * ((length + 64 * 512 - 1) / (64 * 512)); }
__host__ __device__ inline int range_chunks(int length) {
  const int per_wave = tokens_per_wave(length);
  return (length + per_wave - 1) / per_wave;
}

// Whole 64-token groups per chunk when `length` tokens are split into `chunks` chunks.
__host__ __device__ inline int chunk_tokens(int length, int chunks) {
  return ((length + chunks - 1) / chunks + 63) / 64 * 64;
}
// At most 64 partial ranges per (batch, head): one wavefront of a code block reduces them
// itself and the parameter launch between the two stages is not needed.
__host__ __device__ inline int capped_range_chunks(int length) {
  const int per_wave = 64 * ((length + 4095) / 4096);
  return (length + per_wave - 1) / per_wave;
}

__host__ __device__ inline int summation_threads(int length) { return length <= 256 ? 128 : 512; }
// up to this many tokens the residual sums and the centre are one launch
constexpr int kFusedCenterMaxLength = 4096;

// Tokens held by the four consecutive packed positions starting at p0 (multiple of 4).
__device__ __forceinline__ int first_token_of_positions(int p0) {
  const int pos = p0 & 31;
  const int h = pos >> 4;
  const int b = (pos & 15) >> 2;
  return (p0 & ~31) + 8 * b + 4 * h;
}

// grid (ceil(chunks/4), B*H), 256 threads: one wavefront per chunk of
// tokens_per_wave(length) tokens.  A token row is dim/8 lanes wide (8 channels =
// 16 bytes of a 16-bit input per lane), so every load instruction of the wavefront
// covers whole consecutive rows; the lanes holding the same channels are combined
// with xor shuffles at the end.  min/max do not depend on the order.
template <int DT, bool AFFINE>
__device__ __forceinline__ void value_range_block(const void* __restrict__ v, float* __restrict__ part_max,
                                                  float* __restrict__ part_min, int length, int dim,
                                                  int heads, int chunks, int64_t stride_b,
                                                  int64_t stride_h, int64_t stride_n, int chunk_group,
                                                  int bh) {
  const int b = bh / heads, h = bh - b * heads;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = chunk_group * 4 + wave;
  if (chunk >= chunks) return;
  const int octets = dim / 8;
  const int octet = lane % octets, row = lane / octets, rows_per_load = 64 / octets;
  // tokens per chunk follow from the chunk count: tokens_per_wave(length) for the standard
  // count, more when the caller asked for fewer partial ranges
  const int per_wave = chunk_tokens(length, chunks);
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  float mx[8], mn[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    mx[i] = AFFINE ? -FLT_MAX : 0.0f;
    mn[i] = FLT_MAX;
  }
  const int first = chunk * per_wave;
#pragma unroll 8
  for (int t = row; t < per_wave; t += rows_per_load) {
    // Past the end the last token is read again (a repeated element changes neither a
    // minimum nor a maximum), which keeps the loads out of branches and lets the unrolled
    // loop keep eight of them in flight.
    const int n = min(first + t, length - 1);
    float x[8];
    load8<DT>(v, base + static_cast<int64_t>(n) * stride_n + octet * 8, x);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (AFFINE) {
        mx[i] = __builtin_fmaxf(mx[i], x[i]);
        mn[i] = __builtin_fminf(mn[i], x[i]);
      } else {
        mx[i] = __builtin_fmaxf(mx[i], __builtin_fabsf(x[i]));
      }
    }
  }
  for (int offset = octets; offset < 64; offset <<= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = __builtin_fmaxf(mx[i], __shfl_xor(mx[i], offset));
      if constexpr (AFFINE) mn[i] = __builtin_fminf(mn[i], __shfl_xor(mn[i], offset));
    }
  }
  if (lane < octets) {
    const int64_t slot = (static_cast<int64_t>(bh) * chunks + chunk) * dim + octet * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      part_max[slot + i] = mx[i];
      if constexpr (AFFINE) part_min[slot + i] = mn[i];
    }
  }
}

template <int DT, bool AFFINE>
__global__ __launch_bounds__(256) void value_range_kernel(const void* __restrict__ v,
                                                          float* __restrict__ part_max,
                                                          float* __restrict__ part_min, int length,
                                                          int dim, int heads, int chunks,
                                                          int64_t stride_b, int64_t stride_h,
                                                          int64_t stride_n) {
  value_range_block<DT, AFFINE>(v, part_max, part_min, length, dim, heads, chunks, stride_b, stride_h,
                                stride_n, blockIdx.x, blockIdx.y);
}

// grid (ceil(B*H*dim/8 / 4)), 256 threads: one wavefront per (batch, head, 8
// channels); lanes stride over the partial ranges, xor shuffles combine them.
template <bool AFFINE>
__global__ __launch_bounds__(256) void value_params_kernel(const float* __restrict__ part_max,
                                                           const float* __restrict__ part_min,
                                                           float* __restrict__ scale,
                                                           float* __restrict__ center,
                                                           float* __restrict__ inverse,
                                                           float* __restrict__ midpoint, int dim,
                                                           int chunks, int groups) {
  const int lane = threadIdx.x & 63;
  const int group = blockIdx.x * 4 + (threadIdx.x >> 6);  // (b*H + h) * dim/8 + octet
  if (group >= groups) return;
  const int octets = dim / 8;
  const int bh = group / octets, octet = group - bh * octets;
  float mx[8], mn[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    mx[i] = AFFINE ? -FLT_MAX : 0.0f;
    mn[i] = FLT_MAX;
  }
  for (int chunk = lane; chunk < chunks; chunk += 64) {
    const int64_t slot = (static_cast<int64_t>(bh) * chunks + chunk) * dim + octet * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = __builtin_fmaxf(mx[i], part_max[slot + i]);
      if constexpr (AFFINE) mn[i] = __builtin_fminf(mn[i], part_min[slot + i]);
    }
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = __builtin_fmaxf(mx[i], __shfl_xor(mx[i], offset));
      if constexpr (AFFINE) mn[i] = __builtin_fminf(mn[i], __shfl_xor(mn[i], offset));
    }
  }
  if (lane < 8) {
    const int row = group * 8 + lane;
    float hi = mx[0], lo = mn[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) {
      hi = lane == i ? mx[i] : hi;
      lo = lane == i ? mn[i] : lo;
    }
    const float mid = AFFINE ? 0.5f * (lo + hi) : 0.0f;
    const float radius = AFFINE ? 0.5f * (hi - lo) : hi;
    const float sc = __builtin_fmaxf(radius * (1.0f / 127.0f), 1e-12f);
    scale[row] = sc;
    inverse[row] = 1.0f / sc;
    midpoint[row] = mid;
    if constexpr (!AFFINE) center[row] = 0.0f;
  }
}

// grid (ceil(padded/128) * B*H), 256 threads: a workgroup turns 128 packed positions (128
// tokens) of every channel into codes.
//   * Loads cover whole token rows: the dim/8 lanes next to each other read the 16-byte
//     pieces of one row, so a load instruction of a wavefront touches 64/(dim/8) rows and
//     every cache line once (a lane-per-token mapping touches 64 rows for 16 bytes each and
//     is limited by the address rate of the load path: 4.0 TB/s where Q and K reach 5.7-6.1).
//     A thread owns four consecutive positions (four consecutive tokens) of eight channels,
//     32/(256/(dim/8)) such quads; all its loads are issued before any is used.
//   * The four codes of a channel become one 32-bit word, which goes to LDS at
//     [channel row][position quad]; after a barrier two threads per channel row read 64 bytes
//     each and store them: every store instruction of a wavefront writes whole cache lines of
//     the packed transposed matrix, and the same words give the accumulator seeds of the
//     tile(s) (a 128-key tile is the workgroup's 128 positions, a 64-key tile one half).
//   * LDS rows are 36 words apart and channel 8*o + i sits in row i*(dim/8) + o: the words a
//     wavefront writes at once (fixed i, all o, four quads) then fall into different banks
//     two by two, and so do the 16-byte reads of neighbouring rows.
//
// PARAMS says where the per-channel scale and midpoint come from: kParamsStored reads
// what value_params_kernel left; kParamsAbsmax / kParamsAffine reduce the partial
// ranges (at most 64 of them) inside every workgroup, one thread per channel, which saves a
// launch for short sequences; the workgroups of the first 128 positions also store
// the parameters for the kernels that follow.  kParamsWalk / kParamsWalkAffine (short
// sequences) take no partial ranges at all: every workgroup walks the whole sequence of its
// (batch, head) for the channel ranges itself, which leaves the preparation without a launch
// to wait for.
constexpr int kParamsStored = 0, kParamsAbsmax = 1, kParamsAffine = 2, kParamsWalk = 3, kParamsWalkAffine = 4;
constexpr int kCodeBlockPositions = 128;

struct FusedParams {
  const float* part_max;
  const float* part_min;
  float* scale;
  float* center;
  float* inverse;
  float* midpoint;
  int chunks;
};

template <int DT, int CTA_K, int PARAMS, int DK>
__device__ __forceinline__ void value_codes_block(const void* __restrict__ v, int8_t* __restrict__ codes,
                                                  int32_t* __restrict__ tile_sum,
                                                  const float* __restrict__ inverse,
                                                  const float* __restrict__ midpoint, int length,
                                                  int padded, int heads, int64_t stride_b,
                                                  int64_t stride_h, int64_t stride_n,
                                                  const int32_t* __restrict__ permutation,
                                                  const FusedParams& fused, int position_block, int bh) {
  constexpr int OCTETS = DK / 8;        // lanes per token row
  constexpr int SLOTS = 256 / OCTETS;   // quads of positions in flight per load
  constexpr int QUADS = 32 / SLOTS;     // quads per thread
  constexpr int BATCH = QUADS < 2 ? QUADS : 2;  // quads whose loads are in flight together
  constexpr int PITCH = 36;             // words between LDS rows (16-byte aligned, 4 banks apart)
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) uint32_t transposed[DK * PITCH];
  __shared__ float channel_inverse[DK], channel_midpoint[DK];
  [[maybe_unused]] __shared__ float partial_max[256 / DK][DK], partial_min[256 / DK][DK];
  constexpr bool WALK = PARAMS == kParamsWalk || PARAMS == kParamsWalkAffine;
  [[maybe_unused]] __shared__ float walked_max[WALK ? SLOTS : 1][DK];
  [[maybe_unused]] __shared__ float walked_min[PARAMS == kParamsWalkAffine ? SLOTS : 1][DK];
  const int b = bh / heads, h = bh - b * heads;
  const int tid = threadIdx.x;
  const int octet = tid % OCTETS, slot = tid / OCTETS;
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t row0 = static_cast<int64_t>(bh) * DK;
  const int tiles = padded / CTA_K;
  const int first_position = position_block * kCodeBlockPositions;

  float inv[8], mid[8];
  if constexpr (PARAMS == kParamsStored) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      inv[i] = inverse[row0 + octet * 8 + i];
      mid[i] = midpoint[row0 + octet * 8 + i];
    }
  } else if constexpr (WALK) {
    // Thread (octet, slot) takes the rows slot, slot + SLOTS, ... of the whole sequence; rows
    // past the end read the last one again (a repeated element changes neither a maximum nor
    // a minimum), so the loads sit in no branch.  Neither depends on the order.
    constexpr bool AFFINE = PARAMS == kParamsWalkAffine;
    float mx[8], mn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = AFFINE ? -FLT_MAX : 0.0f;
      mn[i] = FLT_MAX;
    }
    // sixteen rows in flight per thread: the walk is a chain of round trips, not of bytes
    constexpr int IN_FLIGHT = 16;
    const int passes = (length + SLOTS - 1) / SLOTS;
    for (int first_pass = 0; first_pass < passes; first_pass += IN_FLIGHT) {
      float rows_in_flight[IN_FLIGHT][8];
#pragma unroll
      for (int j = 0; j < IN_FLIGHT; ++j) {
        const int n = min((first_pass + j) * SLOTS + slot, length - 1);
        load8<DT>(v, base + static_cast<int64_t>(n) * stride_n + octet * 8, rows_in_flight[j]);
      }
#pragma unroll
      for (int j = 0; j < IN_FLIGHT; ++j) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float x = rows_in_flight[j][i];
          if constexpr (AFFINE) {
            mx[i] = __builtin_fmaxf(mx[i], x);
            mn[i] = __builtin_fminf(mn[i], x);
          } else {
            mx[i] = __builtin_fmaxf(mx[i], __builtin_fabsf(x));
          }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      walked_max[slot][octet * 8 + i] = mx[i];
      if constexpr (AFFINE) walked_min[slot][octet * 8 + i] = mn[i];
    }
    __syncthreads();
    if (tid < DK) {
      float top = walked_max[0][tid], bottom = AFFINE ? walked_min[0][tid] : FLT_MAX;
#pragma unroll
      for (int part = 1; part < SLOTS; ++part) {
        top = __builtin_fmaxf(top, walked_max[part][tid]);
        if constexpr (AFFINE) bottom = __builtin_fminf(bottom, walked_min[part][tid]);
      }
      const float middle = AFFINE ? 0.5f * (bottom + top) : 0.0f;
      const float radius = AFFINE ? 0.5f * (top - bottom) : top;
      const float sc = __builtin_fmaxf(radius * (1.0f / 127.0f), 1e-12f);
      const float reciprocal = 1.0f / sc;
      channel_inverse[tid] = reciprocal;
      channel_midpoint[tid] = middle;
      if (position_block == 0) {
        fused.scale[row0 + tid] = sc;
        fused.inverse[row0 + tid] = reciprocal;
        fused.midpoint[row0 + tid] = middle;
        if constexpr (!AFFINE) fused.center[row0 + tid] = 0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      inv[i] = channel_inverse[octet * 8 + i];
      mid[i] = channel_midpoint[octet * 8 + i];
    }
  } else {
    constexpr bool AFFINE = PARAMS == kParamsAffine;
    // All 256 threads walk the (at most 64) partial ranges: thread (channel, part) takes every
    // PARTS-th one.  The loads are independent of each other and of the token loads below and
    // sit in no branch (a range past the last one reads the last one again, which changes
    // neither a maximum nor a minimum), so all of them are in flight together.
    constexpr int PARTS = 256 / DK;
    constexpr int PER_PART = 64 / PARTS;
    {
      const int channel = tid % DK, part = tid / DK;
      float mx = AFFINE ? -FLT_MAX : 0.0f, mn = FLT_MAX;
#pragma unroll
      for (int k = 0; k < PER_PART; ++k) {
        const int chunk = min(k * PARTS + part, fused.chunks - 1);
        const int64_t at = (static_cast<int64_t>(bh) * fused.chunks + chunk) * DK + channel;
        mx = __builtin_fmaxf(mx, fused.part_max[at]);
        if constexpr (AFFINE) mn = __builtin_fminf(mn, fused.part_min[at]);
      }
      partial_max[part][channel] = mx;
      if constexpr (AFFINE) partial_min[part][channel] = mn;
    }
    __syncthreads();
    if (tid < DK) {
      float mx = partial_max[0][tid], mn = AFFINE ? partial_min[0][tid] : FLT_MAX;
#pragma unroll
      for (int part = 1; part < PARTS; ++part) {
        mx = __builtin_fmaxf(mx, partial_max[part][tid]);
        if constexpr (AFFINE) mn = __builtin_fminf(mn, partial_min[part][tid]);
      }
      const float middle = AFFINE ? 0.5f * (mn + mx) : 0.0f;
      const float radius = AFFINE ? 0.5f * (mx - mn) : mx;
      const float sc = __builtin_fmaxf(radius * (1.0f / 127.0f), 1e-12f);
      const float reciprocal = 1.0f / sc;
      channel_inverse[tid] = reciprocal;
      channel_midpoint[tid] = middle;
      if (position_block == 0) {
        fused.scale[row0 + tid] = sc;
        fused.inverse[row0 + tid] = reciprocal;
        fused.midpoint[row0 + tid] = middle;
        if constexpr (!AFFINE) fused.center[row0 + tid] = 0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      inv[i] = channel_inverse[octet * 8 + i];
      mid[i] = channel_midpoint[octet * 8 + i];
    }
  }

#pragma unroll
  for (int first = 0; first < QUADS; first += BATCH) {
    // The loads of a batch are issued together, outside any branch; tokens past the end
    // read the last row and their codes are zeroed.
    int from[BATCH][4];
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int n0 = first_token_of_positions(first_position + (slot + SLOTS * (first + j)) * 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) from[j][r] = min(n0 + r, length - 1);
    }
    if (permutation != nullptr) {
#pragma unroll
      for (int j = 0; j < BATCH; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) from[j][r] = permutation[static_cast<int64_t>(bh) * length + from[j][r]];
    }
    float x[BATCH][4][8];
#pragma unroll
    for (int j = 0; j < BATCH; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        load8<DT>(v, base + static_cast<int64_t>(from[j][r]) * stride_n + octet * 8, x[j][r]);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int quad = slot + SLOTS * (first + j);
      const int n0 = first_token_of_positions(first_position + quad * 4);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float q[4];  // codes as magic sums (round_to_code)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          q[r] = n0 + r < length ? round_to_code((x[j][r][i] - mid[i]) * inv[i]) : kRoundMagic;
        transposed[(i * OCTETS + octet) * PITCH + quad] = pack_codes(q[0], q[1], q[2], q[3]);
      }
    }
  }
  __syncthreads();

  // Two threads per LDS row: 64 positions (bytes) each.  Row r holds channel 8*(r % OCTETS) + r / OCTETS.
#pragma unroll
  for (int task = tid; task < DK * 2; task += 256) {
    const int row = task >> 1, half = task & 1;
    const int channel = (row % OCTETS) * 8 + row / OCTETS;
    const int position = first_position + half * 64;
    const v4u* source = reinterpret_cast<const v4u*>(transposed + row * PITCH + half * 16);
    v4u words[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) words[n] = source[n];
    int sum = 0;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int w = 0; w < 4; ++w) sum += sum_of_codes(words[n][w]);
    if constexpr (CTA_K == 128) sum += __shfl_xor(sum, 1);
    if (position < padded) {
      v4u* target = reinterpret_cast<v4u*>(codes + (row0 + channel) * padded + position);
#pragma unroll
      for (int n = 0; n < 4; ++n) target[n] = words[n];
      if (CTA_K == 64 || half == 0) {
        tile_sum[(static_cast<int64_t>(bh) * tiles + position / CTA_K) * DK + channel] =
            sum * 128 + kAccumulatorSeedBits;
      }
    }
  }
}

template <int DT, int CTA_K, int PARAMS, int DK>
__global__ __launch_bounds__(256) void value_codes_kernel(const void* __restrict__ v,
                                                          int8_t* __restrict__ codes,
                                                          int32_t* __restrict__ tile_sum,
                                                          const float* __restrict__ inverse,
                                                          const float* __restrict__ midpoint,
                                                          int length, int padded, int heads,
                                                          int64_t stride_b, int64_t stride_h,
                                                          int64_t stride_n,
                                                          const int32_t* __restrict__ permutation,
                                                          FusedParams fused, int position_blocks) {
  value_codes_block<DT, CTA_K, PARAMS, DK>(v, codes, tile_sum, inverse, midpoint, length, padded, heads,
                                           stride_b, stride_h, stride_n, permutation, fused,
                                           blockIdx.x % position_blocks, blockIdx.x / position_blocks);
}

// grid (T / (256/quads), B*H), 256 threads: thread = (summation thread t, four channels);
// four rather than eight channels per thread so that a long sequence fills every SIMD.
template <int DT>
__device__ __forceinline__ void value_residual_block(const void* __restrict__ v, float* __restrict__ partial,
                                                     const float* __restrict__ inverse,
                                                     const float* __restrict__ midpoint, int length,
                                                     int dim, int heads, int threads, int64_t stride_b,
                                                     int64_t stride_h, int64_t stride_n,
                                                     const int32_t* __restrict__ permutation,
                                                     int block, int bh) {
  const int b = bh / heads, h = bh - b * heads;
  const int quads = dim / 4;
  const int quad = threadIdx.x % quads;
  const int t = block * (256 / quads) + threadIdx.x / quads;
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t row0 = static_cast<int64_t>(bh) * dim + quad * 4;
  float inv[4], mid[4], residual[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    inv[i] = inverse[row0 + i];
    mid[i] = midpoint[row0 + i];
    residual[i] = 0.0f;
  }
  // The additions of one thread are sequential by contract; the loads are not: eight tokens
  // are requested before the first is consumed, which is what hides the memory latency with
  // only 512 summation threads per (batch, head).
  // Loads past the front of the sequence are clamped to token 0 and not accumulated, so
  // that no load sits inside a branch (the compiler would wait for each of those in turn).
  constexpr int kInFlight = 8;
  auto accumulate = [&](auto permuted_tag) {
    constexpr bool PERMUTED = decltype(permuted_tag)::value;
    const int32_t* order = PERMUTED ? permutation + static_cast<int64_t>(bh) * length : nullptr;
    for (int src0 = length - 1 - t; src0 >= 0; src0 -= threads * kInFlight) {
      int from[kInFlight];
      float x[kInFlight][4];
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        const int src = max(src0 - j * threads, 0);
        if constexpr (PERMUTED) {
          from[j] = order[src];
        } else {
          from[j] = src;
        }
      }
#pragma unroll
      for (int j = 0; j < kInFlight; ++j)
        load4<DT>(v, base + static_cast<int64_t>(from[j]) * stride_n + quad * 4, x[j]);
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        if (src0 - j * threads >= 0) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float normalized = (x[j][i] - mid[i]) * inv[i];
            const float code = code_value(round_to_code(normalized));
            residual[i] += normalized - code;
          }
        }
      }
    }
  };
  if (permutation != nullptr) {
    accumulate(std::true_type{});
  } else {
    accumulate(std::false_type{});
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) partial[(row0 + i) * threads + t] = residual[i];
}

template <int DT>
__global__ __launch_bounds__(256) void value_residual_kernel(const void* __restrict__ v,
                                                             float* __restrict__ partial,
                                                             const float* __restrict__ inverse,
                                                             const float* __restrict__ midpoint,
                                                             int length, int dim, int heads,
                                                             int threads, int64_t stride_b,
                                                             int64_t stride_h, int64_t stride_n,
                                                             const int32_t* __restrict__ permutation) {
  value_residual_block<DT>(v, partial, inverse, midpoint, length, dim, heads, threads, stride_b, stride_h,
                           stride_n, permutation, blockIdx.x, blockIdx.y);
}

// One workgroup of `threads` threads per row: every 32 partials combine with the reference's
// tree (t[i] += t[i+16], +8, +4, +2, +1: a shuffle-down) and the totals of the 32-thread
// groups are added in group order.
__global__ __launch_bounds__(512) void value_center_from_partials_kernel(
    const float* __restrict__ partial, const float* __restrict__ inverse,
    const float* __restrict__ midpoint, float* __restrict__ center, int rows, int threads, int length) {
  __shared__ float group_total[16];
  const int row = blockIdx.x;
  const int t = threadIdx.x;
  float value = partial[static_cast<int64_t>(row) * threads + t];
#pragma unroll
  for (int offset = 16; offset > 0; offset >>= 1) value += __shfl_down(value, offset, 32);
  if ((t & 31) == 0) group_total[t >> 5] = value;
  __syncthreads();
  if (t == 0) {
    float total = 0.0f;
    for (int w = 0; w < threads / 32; ++w) total += group_total[w];
    const float scale = 1.0f / inverse[row];
    const float mean = total / static_cast<float>(length);
    const float correction = scale * mean;
    center[row] = midpoint[row] + correction;
  }
}

// The centre of value_center_fused_kernel as a block of a 256-thread launch that also
// holds the code blocks: the parameters come from the partial ranges (the same reduction
// and arithmetic as value_codes_block, so the same bits), and thread t plays the summation
// threads t and t + 256 one after the other.  Warp totals land in the reference's order.
// WALK: the ranges of the block's eight channels come from a walk over the whole sequence
// instead of the partial ranges of an earlier launch.
template <int DT, bool WALK = false>
__device__ __forceinline__ void value_center_block(const void* __restrict__ v, const FusedParams& fused,
                                                   int length, int dim, int heads, int64_t stride_b,
                                                   int64_t stride_h, int64_t stride_n,
                                                   const int32_t* __restrict__ permutation, int octet,
                                                   int bh) {
  __shared__ float warp_total[8][16];
  __shared__ float parameters[2][8];
  const int b = bh / heads, h = bh - b * heads;
  const int t = threadIdx.x, lane = t & 63;
  const int threads = summation_threads(length);
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t row0 = static_cast<int64_t>(bh) * dim + octet * 8;
  float mx[8], mn[8], inv[8], mid[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    mx[i] = -FLT_MAX;
    mn[i] = FLT_MAX;
  }
  if constexpr (WALK) {
    // rows t, t + 256, ...; past the end the last row again (no effect on a range)
    const int passes = (length + 255) / 256;
#pragma unroll 4
    for (int pass = 0; pass < passes; ++pass) {
      float x[8];
      load8<DT>(v, base + static_cast<int64_t>(min(pass * 256 + t, length - 1)) * stride_n + octet * 8, x);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        mx[i] = __builtin_fmaxf(mx[i], x[i]);
        mn[i] = __builtin_fminf(mn[i], x[i]);
      }
    }
  } else if (lane < fused.chunks) {
    const int64_t slot = (static_cast<int64_t>(bh) * fused.chunks + lane) * dim + octet * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = fused.part_max[slot + i];
      mn[i] = fused.part_min[slot + i];
    }
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = __builtin_fmaxf(mx[i], __shfl_xor(mx[i], offset));
      mn[i] = __builtin_fminf(mn[i], __shfl_xor(mn[i], offset));
    }
  }
  if constexpr (WALK) {
    // the four wavefronts hold different rows: combine them through LDS
    __shared__ float wave_range[2][4][8];
    if (lane < 8) {
      float hi = mx[0], lo = mn[0];
#pragma unroll
      for (int i = 1; i < 8; ++i) {
        hi = lane == i ? mx[i] : hi;
        lo = lane == i ? mn[i] : lo;
      }
      wave_range[0][t >> 6][lane] = hi;
      wave_range[1][t >> 6][lane] = lo;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      mx[i] = __builtin_fmaxf(__builtin_fmaxf(wave_range[0][0][i], wave_range[0][1][i]),
                              __builtin_fmaxf(wave_range[0][2][i], wave_range[0][3][i]));
      mn[i] = __builtin_fminf(__builtin_fminf(wave_range[1][0][i], wave_range[1][1][i]),
                              __builtin_fminf(wave_range[1][2][i], wave_range[1][3][i]));
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    mid[i] = 0.5f * (mn[i] + mx[i]);
    const float radius = 0.5f * (mx[i] - mn[i]);
    const float sc = __builtin_fmaxf(radius * (1.0f / 127.0f), 1e-12f);
    inv[i] = 1.0f / sc;
    if (t == i) {
      parameters[0][i] = inv[i];
      parameters[1][i] = mid[i];
    }
  }
  constexpr int kInFlight = 8;
  for (int pass = 0; pass * 256 < threads; ++pass) {
    const int st = t + pass * 256;  // summation thread
    float residual[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) residual[i] = 0.0f;
    auto accumulate = [&](auto permuted_tag) {
      constexpr bool PERMUTED = decltype(permuted_tag)::value;
      const int32_t* order = PERMUTED ? permutation + static_cast<int64_t>(bh) * length : nullptr;
      for (int src0 = st < threads ? length - 1 - st : -1; src0 >= 0; src0 -= threads * kInFlight) {
        int from[kInFlight];
        float x[kInFlight][8];
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
          const int src = max(src0 - j * threads, 0);
          if constexpr (PERMUTED) {
            from[j] = order[src];
          } else {
            from[j] = src;
          }
        }
#pragma unroll
        for (int j = 0; j < kInFlight; ++j)
          load8<DT>(v, base + static_cast<int64_t>(from[j]) * stride_n + octet * 8, x[j]);
#pragma unroll
        for (int j = 0; j < kInFlight; ++j) {
          if (src0 - j * threads >= 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              const float normalized = (x[j][i] - mid[i]) * inv[i];
              const float code = code_value(round_to_code(normalized));
              residual[i] += normalized - code;
            }
          }
        }
      }
    };
    if (permutation != nullptr) {
      accumulate(std::true_type{});
    } else {
      accumulate(std::false_type{});
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int offset = 16; offset > 0; offset >>= 1) residual[i] += __shfl_down(residual[i], offset, 32);
      if ((t & 31) == 0 && st < threads) warp_total[i][st >> 5] = residual[i];
    }
  }
  __syncthreads();
  if (t < 8) {
    float total = 0.0f;
    for (int w = 0; w < threads / 32; ++w) total += warp_total[t][w];
    const float scale = 1.0f / parameters[0][t];
    const float mean = total / static_cast<float>(length);
    const float correction = scale * mean;
    fused.center[row0 + t] = parameters[1][t] + correction;
  }
}

// One-launch form of the two kernels above for short sequences (a workgroup reads 16
// bytes of every row, which wastes cache lines once the sequence is long).
// Residual-corrected centre of the midpoint_affine mode (reference
// quantize_v_impl.cuh:233-275).  grid (dim/8, B*H), `threads` threads (512, or 128
// for at most 256 tokens): thread t is the reference's summation thread t for the
// eight channels of the workgroup.  It adds the residuals of tokens L-1-t-k*threads
// (k ascending); every 32 threads combine with the reference's tree (t[i] += t[i+16],
// +8, +4, +2, +1: a shuffle-down), and the warp totals are added in warp order.
template <int DT>
__global__ __launch_bounds__(512) void value_center_fused_kernel(const void* __restrict__ v,
                                                           const float* __restrict__ inverse,
                                                           const float* __restrict__ midpoint,
                                                           float* __restrict__ center, int length,
                                                           int dim, int heads, int64_t stride_b,
                                                           int64_t stride_h, int64_t stride_n,
                                                           const int32_t* __restrict__ permutation) {
  __shared__ float warp_total[8][16];
  const int octet = blockIdx.x, bh = blockIdx.y;
  const int b = bh / heads, h = bh - b * heads;
  const int t = threadIdx.x, threads = blockDim.x;
  const int64_t base = static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(h) * stride_h;
  const int64_t row0 = static_cast<int64_t>(bh) * dim + octet * 8;
  float inv[8], mid[8], residual[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    inv[i] = inverse[row0 + i];
    mid[i] = midpoint[row0 + i];
    residual[i] = 0.0f;
  }
  // The additions of one thread are sequential by contract; the loads are not: eight tokens
  // are requested before the first is consumed, which is what hides the memory latency with
  // only 512 summation threads per (batch, head).
  // Loads past the front of the sequence are clamped to token 0 and not accumulated, so
  // that no load sits inside a branch (the compiler would wait for each of those in turn).
  constexpr int kInFlight = 8;
  auto accumulate = [&](auto permuted_tag) {
    constexpr bool PERMUTED = decltype(permuted_tag)::value;
    const int32_t* order = PERMUTED ? permutation + static_cast<int64_t>(bh) * length : nullptr;
    for (int src0 = length - 1 - t; src0 >= 0; src0 -= threads * kInFlight) {
      int from[kInFlight];
      float x[kInFlight][8];
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        const int src = max(src0 - j * threads, 0);
        if constexpr (PERMUTED) {
          from[j] = order[src];
        } else {
          from[j] = src;
        }
      }
#pragma unroll
      for (int j = 0; j < kInFlight; ++j)
        load8<DT>(v, base + static_cast<int64_t>(from[j]) * stride_n + octet * 8, x[j]);
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        if (src0 - j * threads >= 0) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float normalized = (x[j][i] - mid[i]) * inv[i];
            const float code = code_value(round_to_code(normalized));
            residual[i] += normalized - code;
          }
        }
      }
    }
  };
  if (permutation != nullptr) {
    accumulate(std::true_type{});
  } else {
    accumulate(std::false_type{});
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
#pragma unroll
    for (int offset = 16; offset > 0; offset >>= 1) residual[i] += __shfl_down(residual[i], offset, 32);
    if ((t & 31) == 0) warp_total[i][t >> 5] = residual[i];
  }
  __syncthreads();
  if (t < 8) {
    float total = 0.0f;
    for (int w = 0; w < threads / 32; ++w) total += warp_total[t][w];
    const float scale = 1.0f / inverse[row0 + t];
    const float mean = total / static_cast<float>(length);
    const float correction = scale * mean;
    center[row0 + t] = midpoint[row0 + t] + correction;
  }
}

// grid (ceil(padded/256), rows_bh), 256 threads: accumulator seeds of already packed codes.
template <int CTA_K>
__global__ __launch_bounds__(256) void value_tile_sum_kernel(const int8_t* __restrict__ codes,
                                                             int32_t* __restrict__ tile_sum, int dim,
                                                             int padded) {
  const int bh = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p0 = blockIdx.x * 256 + lane * 4;
  const int tiles = padded / CTA_K;
  for (int c = wave; c < dim; c += 4) {
    int sum = 0;
    if (p0 < padded) {
      const uint32_t word =
          *reinterpret_cast<const uint32_t*>(codes + (static_cast<int64_t>(bh) * dim + c) * padded + p0);
      sum = static_cast<int8_t>(word & 0xff) + static_cast<int8_t>((word >> 8) & 0xff) +
            static_cast<int8_t>((word >> 16) & 0xff) + static_cast<int8_t>(word >> 24);
    }
#pragma unroll
    for (int offset = CTA_K / 8; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset);
    if ((lane & (CTA_K / 4 - 1)) == 0 && p0 < padded) {
      tile_sum[(static_cast<int64_t>(bh) * tiles + p0 / CTA_K) * dim + c] = sum * 128 + kAccumulatorSeedBits;
    }
  }
}

struct Workspace {
  float* part_max;
  float* part_min;
  float* inverse;
  float* midpoint;
  float* partial;
  size_t bytes;
};

Workspace carve(void* base, int batch, int heads, int length, int dim, bool affine) {
  const size_t bh = static_cast<size_t>(batch) * heads;
  const size_t chunks = range_chunks(length);
  const size_t rows = bh * dim;
  float* p = static_cast<float*>(base);
  Workspace w{};
  size_t offset = 0;
  w.part_max = p + offset;
  offset += bh * chunks * dim;
  w.part_min = p + offset;
  offset += affine ? bh * chunks * dim : 0;
  w.inverse = p + offset;
  offset += rows;
  w.midpoint = p + offset;
  offset += rows;
  w.partial = p + offset;
  offset += affine ? rows * summation_threads(length) : 0;
  w.bytes = offset * sizeof(float);
  return w;
}

}  // namespace
}  // namespace risa
