// Fused INT8 attention for gfx950 (CDNA4), wave64 + INT8 MFMA.
//
// Numerical contract: reference csrc/kernels/attention_int8.cuh:145-1026 with
// attention_softmax.cuh (online softmax in the exp2 domain, U8 probabilities
// quantised against each tile's own maximum), attention_value.cuh (integer P·V
// per tile, one FP32 FMA per tile), attention_masks.cuh (custom / key / causal /
// out-of-bound masks) and the capture stores :51-143, :769-848, :871-898.
//
// Mapping onto the matrix cores (not the reference's):
//   * One workgroup = 128 queries of one (batch, query head) = 4 wavefronts of 32
//     queries.  K and V tiles of CTA_K keys are copied from HBM/L2 straight into
//     LDS (global_load_lds_dwordx4, no staging registers), double buffered; the
//     16-byte chunks of every row are XOR-swizzled by choosing which global
//     chunk each lane fetches, so the 16-byte operand reads are conflict free.
//   * Scores are computed transposed, S^T = K · Q^T, with v_mfma_i32_32x32x32_i8:
//     A = K tile rows from LDS, B = Q rows kept in registers for the whole kernel.
//     Lane l then holds query (l % 32) and, per 32-key block, the sixteen keys
//     8*b + 4*(l / 32) + r (b, r in 0..3): row maximum and row sum are in-lane
//     reductions plus one exchange between the two 32-lane halves.
//   * The sixteen U8 probabilities of a lane pack into four registers that are
//     already the B operand of O^T = V^T · P^T.  The V matrix is stored by the
//     preparation kernel with each 32-token group permuted accordingly
//     (risa::packed_value_position), so the A operand is one 16-byte LDS read.
//   * The MFMA multiplies signed bytes.  P_u8 = P_s8 + 128, hence
//     sum_j P_u8[j] V[c][j] = sum_j P_s8[j] V[c][j] + 128 * sum_j V[c][j]:
//     the accumulator of every tile starts from 128 * (tile sum of V codes of
//     channel c), which the preparation kernel provides, and P_s8 = P_u8 ^ 0x80.
//     The result is the exact integer the unsigned product would give.  The seed
//     also carries the bit pattern of 1.5 * 2^23, so the finished accumulator read
//     as a float is 12582912 + n exactly (risa::kAccumulatorSeedBits).
#pragma once

#include "common.hpp"
#include "launchers.hpp"

#include <type_traits>

namespace risa {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kU8Offset = 7.9943534f;
constexpr float kRowFloor = -50000.0f;
// The score accumulators start at the bit pattern of 1.5 * 2^23 instead of zero: with
// |Q.K| < 2^22 (at most 256 products of signed bytes) the INT32 result, read as FP32, is
// exactly 1.5 * 2^23 + Q.K, so one exact subtraction replaces the slower integer-to-float
// conversion.  Integer comparisons of seeded accumulators order like the raw scores.
constexpr int kScoreSeedBits = 0x4B400000;
constexpr float kScoreSeed = 12582912.0f;
__device__ __forceinline__ float score_value(int seeded) { return __int_as_float(seeded) - kScoreSeed; }
constexpr int kQueryBlock = 128;

struct KernelParams {
  const int8_t* q;
  const int8_t* k;
  const int8_t* v;
  void* out;
  const float* q_scale;
  const float* k_scale;
  const float* v_scale;
  const float* v_center;
  const int32_t* v_tile_sum;  // accumulator seeds per (kv head, key tile, channel)
  const void* mask;
  int64_t mask_stride_b, mask_stride_h, mask_stride_q, mask_stride_k;
  int mask_dtype;  // -1: no mask
  const float* key_bias;  // key-only mask as an additive row [Bm,Hm,padded] (mask_dtype kKeyBias)
  int64_t key_bias_stride_b, key_bias_stride_h;
  const uint64_t* mask_lanes;  // boolean mask as one 64-lane word per score slot (kMaskLanes)
  int64_t mask_lanes_stride_b, mask_lanes_stride_h;  // in words; 0 where the mask broadcasts
  int q_len, k_len, q_heads, kv_heads, padded, n_kb, n_qb, batch;
  int64_t out_stride_b, out_stride_n, out_stride_h;
  float sm2;  // sm_scale * log2(e)
  int out_dtype;
  const int32_t* row_offsets;   // sparse CSR (index_mode 1)
  const int32_t* tile_indices;  // sparse block indices (1), key-mask tiles (2) or mask tile lists (3)
  int index_mode;
  int64_t tile_list_stride_b, tile_list_stride_h;  // mode 3: elements between the lists of mask planes (0: shared)
  float* workspace;  // capture
  float* lse;
  int causal;
  int compiled_loop;  // non-zero: every tile through the loop the compiler schedules (see RISA_COMPILED_LOOP)
};

// Byte offset of 16-byte chunk `chunk` of row `row` in a swizzled LDS tile.
template <int ROWBYTES> __device__ __forceinline__ int swizzled(int row, int chunk) {
  constexpr int CH = ROWBYTES / 16;
  constexpr int ROWS_PER_256 = 256 / ROWBYTES;
  return row * ROWBYTES + ((chunk ^ ((row / ROWS_PER_256) & (CH - 1))) << 4);
}

// Two FP32 values as a pair of 16-bit floats in one word (first value in the low half), round
// to nearest even: one v_cvt_pk_bf16_f32 for bfloat16, two conversions and a pack for half.
__device__ __forceinline__ uint32_t to_bf16_pair(float low, float high) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const f32x2 values = {low, high};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(values, bf16x2));
}
__device__ __forceinline__ uint32_t to_f16_pair(float low, float high) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f16x2 values = {static_cast<_Float16>(low), static_cast<_Float16>(high)};
  return __builtin_bit_cast(uint32_t, values);
}
__device__ __forceinline__ uint32_t to_output_pair(float low, float high, int out_dtype) {
  return out_dtype == kF16 ? to_f16_pair(low, high) : to_bf16_pair(low, high);
}

// Copies 16 bytes per lane from global memory to LDS without touching VGPRs:
// lane l of the wavefront writes LDS bytes [lds_wave_base + 16*l, +16).
__device__ __forceinline__ void copy16_to_lds(const void* src, unsigned char* lds_wave_base) {
  typedef const __attribute__((address_space(1))) void* GlobalPointer;
  typedef __attribute__((address_space(3))) void* LdsPointer;
  __builtin_amdgcn_global_load_lds((GlobalPointer)src, (LdsPointer)lds_wave_base, 16, 0, 0);
}

// Same copy with the address given as a wave-uniform base plus a 32-bit byte
// offset per lane, the form the instruction takes without any vector ALU work
// (scalar base register pair + one offset register).  The empty asm keeps the
// zero extension of the offset next to the copy, where instruction selection
// can fold it; hoisted out of the loop it would cost a 64-bit vector add per copy.
__device__ __forceinline__ void copy16_to_lds_uniform(const int8_t* uniform_base, uint32_t lane_offset,
                                                      unsigned char* lds_wave_base) {
  asm volatile("" : "+v"(lane_offset));
  copy16_to_lds(uniform_base + static_cast<uint64_t>(lane_offset), lds_wave_base);
}

// Lane index computed where it is used (two instructions).  The masked kernels
// use it inside the tile loop instead of values derived from threadIdx before
// the loop, which the register allocator would otherwise spill.
__device__ __forceinline__ int fresh_lane() {
  int lane_id;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_id));
  return lane_id;
}

// MASK_BYTES: bytes of the mask tile kept next to K and V in each of the two stages;
// SHARED_MASK_BYTES: bytes of a single mask tile behind both stages (0 unless staged).
template <int D, int CTA_K, int MASK_BYTES = 0, int SHARED_MASK_BYTES = 0> struct TileShape {
  static constexpr int kTileBytes = CTA_K * D;
  static constexpr int kCopiesPerWave = kTileBytes / 16 / 256;  // 1 KB copy instructions per wave
  static constexpr int kSeedBytes = D * 4;                       // accumulator seeds of the tile
  static constexpr int kBiasBytes = CTA_K * 4;                   // key-only mask row of the tile
  static constexpr int kMaskOffset = 2 * kTileBytes + kSeedBytes + kBiasBytes;
  static constexpr int kStageBytes = kMaskOffset + MASK_BYTES;
  static constexpr int kSharedMaskOffset = 2 * kStageBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes + SHARED_MASK_BYTES;
};

// How the kernel reads a mask tensor (template parameter MASK_MODE).
constexpr int kMaskScalar = 0;  // element by element: any strides
constexpr int kMaskVector = 1;  // one load per four keys: unit key stride, aligned rows
constexpr int kMaskStaged = 2;  // mask tile copied to LDS with K and V: 16-byte aligned rows, 64-key tiles
// Boolean mask shared by several heads, turned beforehand into lane words: for every block
// of 32 queries, 64-key tile and score slot of the kernel's register layout, the 64 bits
// that say which lanes keep that score.  The words are wave-uniform, so they arrive through
// the scalar cache in scalar registers (no vector load, no LDS, no unpacking) and one
// v_cndmask per score applies them.
constexpr int kMaskLanes = 3;
constexpr int kLaneWordsPerTile = 32;  // 64-key tile: two 32-key blocks x 16 scores per lane

// Word index of (block of 32 queries, key tile) within one (batch, head) plane of lane words.
__host__ __device__ constexpr int64_t lane_word_offset(int64_t query_wave, int64_t key_tiles, int64_t tile) {
  return (query_wave * key_tiles + tile) * kLaneWordsPerTile;
}

constexpr int mask_element_bytes(int mask_dtype) { return mask_dtype == kF32 ? 4 : mask_dtype == kBool ? 1 : 2; }
// LDS bytes of a staged mask tile (128 queries x CTA_K keys).
// 1- and 2-byte masks keep one tile per stage (requested a tile ahead, like K and V).
// A 4-byte mask tile is 32 KB: it is kept once, which leaves room for two workgroups
// per compute unit, and is requested after the softmax of the previous tile.  That
// needs no barrier: every wavefront copies and reads only the rows of its own queries.
constexpr bool staged_mask_is_shared(int mask_dtype) { return mask_dtype == kF32; }
constexpr int staged_mask_bytes(int mask_dtype, int mask_mode, int cta_k, bool shared) {
  return mask_mode == kMaskStaged && staged_mask_is_shared(mask_dtype) == shared
             ? kQueryBlock * cta_k * mask_element_bytes(mask_dtype)
             : 0;
}
template <int D, int CTA_K, int MASK_DT, int MASK_MODE>
using AttentionTileShape = TileShape<D, CTA_K, staged_mask_bytes(MASK_DT, MASK_MODE, CTA_K, false),
                                     staged_mask_bytes(MASK_DT, MASK_MODE, CTA_K, true)>;

// MASK_DT: element type of the mask tensor (risa::kBool, kF32, kF16, kBF16), kKeyBias
// for a key-only mask prepared as an FP32 row, or -1 for none; FAST (raw-score path)
// implies -1.  MASK_MODE: kMaskScalar / kMaskVector / kMaskStaged; a template parameter
// and not a run-time branch so that the tile loop holds one unrolled mask path and
// stays inside the instruction cache.
template <int D, int CTA_K, bool FAST, bool INDEXED, bool CAPTURE, int MASK_DT, int MASK_MODE>
__global__ __launch_bounds__(256, (D == 256 ? 1 : D == 64 && MASK_MODE == kMaskLanes ? 4 : 2)) void attention_kernel(
    const KernelParams p) {
  // (lane words, head dim 64: 128 registers keep four workgroups per compute unit; the variant
  // that walks tile lists would otherwise take 130 and lose one)
  static_assert(!FAST || MASK_DT < 0, "the raw-score path takes no mask");
  static_assert(MASK_MODE == kMaskScalar || (MASK_DT >= 0 && MASK_DT != kKeyBias), "vector loads need a mask tensor");
  static_assert(MASK_MODE != kMaskStaged || CTA_K == 64, "staged masks: 64-key tiles");
  static_assert(MASK_MODE != kMaskLanes || (CTA_K == 64 && MASK_DT == kBool), "lane words: boolean masks, 64-key tiles");
  constexpr bool MASK_VEC = MASK_MODE != kMaskScalar;
  constexpr bool STAGED = MASK_MODE == kMaskStaged;
  constexpr bool LANES = MASK_MODE == kMaskLanes;
  constexpr bool SHARED_MASK = STAGED && staged_mask_is_shared(MASK_DT);
  using Shape = AttentionTileShape<D, CTA_K, MASK_DT, MASK_MODE>;
  constexpr int RB = CTA_K / 32;  // 32-key blocks per tile
  constexpr int CB = D / 32;      // 32-channel blocks
  constexpr int KK = D / 32;      // k-steps of the score product
  constexpr int NC = Shape::kCopiesPerWave;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x;
  // (not const: the hand-scheduled tile loop owns every vector register, and the values below are
  // formed again behind it rather than kept in scratch memory across it)
  int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int l32 = lane & 31, half = lane >> 5;

  // Workgroup order.  Without a causal mask the query blocks of one head are
  // neighbours, so co-resident workgroups walk the same K/V tiles and share them
  // in L2.  Under a causal mask the work per query block differs by up to the
  // number of key tiles: the launch then goes through all heads of the last query
  // block first and the first query block last (longest first keeps the tail short).
  int bx, head, batch;
  if (!FAST && (p.causal || p.index_mode == 3)) {
    // (tile lists of a mask: a lower-triangular mask given as a tensor is the common case of
    // lists that grow with the query block)
    const int heads = p.q_heads * p.batch;
    const int rest = blockIdx.x % heads;
    bx = p.n_qb - 1 - blockIdx.x / heads;
    head = rest % p.q_heads;
    batch = rest / p.q_heads;
  } else {
    bx = blockIdx.x % p.n_qb;
    const int rest = blockIdx.x / p.n_qb;
    head = rest % p.q_heads;
    batch = rest / p.q_heads;
  }
  const int kv_head = head / (p.q_heads / p.kv_heads);
  const int64_t bhk = static_cast<int64_t>(batch) * p.kv_heads + kv_head;
  const int64_t bhq = static_cast<int64_t>(batch) * p.q_heads + head;

  const int8_t* k_base = p.k + bhk * p.k_len * D;
  const int8_t* v_base = p.v + bhk * D * p.padded;
  const int32_t* sum_base = p.v_tile_sum + bhk * p.n_kb * D;
  const float* ks_base = p.k_scale + bhk * p.n_kb * 4;
  [[maybe_unused]] const float* bias_base = nullptr;
  if constexpr (MASK_DT == kKeyBias) {
    bias_base = p.key_bias + batch * p.key_bias_stride_b + head * p.key_bias_stride_h;
  }

  int query = bx * kQueryBlock + wave * 32 + l32;
  bool query_ok = query < p.q_len;

  // --- Q operand and scales ------------------------------------------------
  // Requested before the tile list is read: the list's first entries are needed at once and
  // would otherwise keep these loads waiting behind their round trip.
  v4i qreg[KK];
  {
    const int8_t* q_row = p.q + (bhq * p.q_len + query) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      qreg[kk] = query_ok ? *reinterpret_cast<const v4i*>(q_row + kk * 32 + half * 16) : v4i{0, 0, 0, 0};
    }
  }
  constexpr int W = D == 256 ? 16 : 32;
  const int q_groups = (p.q_len + 127) / 128 * (128 / W) * 8;
  const float q_scale = query_ok ? p.q_scale[bhq * q_groups + (query / W) * 8 + (query & 7)] : 1.0f;
  const float qs2 = p.sm2;

  // --- tile list -----------------------------------------------------------
  int n_it;
  const int32_t* indices = nullptr;
  if constexpr (INDEXED) {
    if (p.index_mode == 1) {
      const int64_t row = bhq * p.n_qb + bx;
      const int start = p.row_offsets[row];
      n_it = p.row_offsets[row + 1] - start;
      indices = p.tile_indices + start;
    } else if (p.index_mode == 3) {
      // lists of a boolean mask several heads share: per mask plane and query block, the
      // tiles in which the block sees at least one key
      indices = p.tile_indices + batch * p.tile_list_stride_b + head * p.tile_list_stride_h +
                static_cast<int64_t>(bx) * (p.n_kb + 1);
      n_it = indices[p.n_kb];
    } else {
      indices = p.tile_indices + bhq * (p.n_kb + 1);
      n_it = indices[p.n_kb];
    }
  } else {
    n_it = p.n_kb;
    if (!FAST && !CAPTURE && p.causal) {
      const int limit = min(p.k_len, (bx + 1) * kQueryBlock);
      n_it = (limit + CTA_K - 1) / CTA_K;
    }
  }
  n_it = __builtin_amdgcn_readfirstlane(n_it);
  // Lists are ascending without repeats: one that names every tile is 0, 1, 2, ... and is
  // walked without being read (a mask that hides no whole tile costs no list reads).
  [[maybe_unused]] const bool whole_list = INDEXED && n_it == p.n_kb;
  // Entry `it` of the tile list through the scalar cache (the address is uniform): the first
  // entries are needed before anything else can start, and as a vector load their wait would
  // include the Q rows requested above (vector memory returns in order).
  auto tile_at = [&](int it) -> int {
    if constexpr (INDEXED) {
      if (whole_list) return it;
      typedef const __attribute__((address_space(4))) int32_t* UniformEntries;
      return ((UniformEntries)(reinterpret_cast<uintptr_t>(indices)))[it];
    }
    return it;
  };

  // --- per-lane copy descriptors -------------------------------------------------
  // Copy instruction i of this wave fills LDS bytes [(wave*NC+i)*1024, +1024) of
  // a tile; this lane supplies chunk `lane` of that kilobyte.  The source offsets
  // are constant over tiles.  The raw-score kernels keep them in registers; the
  // masked kernels have none to spare (a spilled offset would be reloaded through
  // the same counter the LDS copies complete on, serialising them) and recompute
  // them per tile from a lane id the compiler cannot see through.
  // (The hand-scheduled tile loop issues its own copies and owns every vector register: kernels
  // that have it issue at most two tiles from here, and offsets kept for them would live in
  // scratch memory across the loop.)
  constexpr bool KEEP_OFFSETS = FAST && !(D == 128 && CTA_K == 128);
  auto k_source_offset = [&](int i, int lane_id) -> uint32_t {
    constexpr int CH = D / 16;
    const int slot = (wave * NC + i) * 64 + lane_id;
    const int row = slot / CH, phys = slot % CH;
    const int chunk = phys ^ ((row / (256 / D)) & (CH - 1));
    return row * D + chunk * 16;
  };
  auto v_source_offset = [&](int i, int lane_id) -> uint32_t {
    constexpr int CH = CTA_K / 16;
    const int slot = (wave * NC + i) * 64 + lane_id;
    const int row = slot / CH, phys = slot % CH;
    const int chunk = phys ^ ((row / (256 / CTA_K)) & (CH - 1));
    return static_cast<uint32_t>(row) * static_cast<uint32_t>(p.padded) + chunk * 16;
  };
  [[maybe_unused]] uint32_t k_kept[NC], v_kept[NC];
  if constexpr (KEEP_OFFSETS) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      k_kept[i] = k_source_offset(i, lane);
      v_kept[i] = v_source_offset(i, lane);
    }
  }
  // Staged masks: the mask tile of the workgroup's 128 queries (64 * ES bytes per row,
  // 16-byte chunks XOR-swizzled by row so that the 32 rows a half-wave reads spread over
  // the banks) is copied like K and V.  Source offsets are relative to the first row of
  // the query block; rows past the last query re-read the last one.
  constexpr int MASK_ES = MASK_DT >= 0 && MASK_DT != kKeyBias ? mask_element_bytes(MASK_DT) : 1;
  constexpr int MASK_ROW_BYTES = CTA_K * MASK_ES;
  constexpr int MASK_CH = MASK_ROW_BYTES / 16;                       // chunks per row
  constexpr int NM = STAGED ? kQueryBlock * MASK_CH / 256 : 1;       // copy instructions per wave
  constexpr int MASK_ROWS_PER_256 = MASK_ROW_BYTES >= 256 ? 1 : 256 / MASK_ROW_BYTES;
  auto mask_swizzle = [](int row) { return (row / MASK_ROWS_PER_256) & (MASK_CH - 1); };
  [[maybe_unused]] const int8_t* mask_block = nullptr;
  if constexpr (STAGED) {
    mask_block = static_cast<const int8_t*>(p.mask) +
                 (static_cast<int64_t>(batch) * p.mask_stride_b + static_cast<int64_t>(head) * p.mask_stride_h +
                  static_cast<int64_t>(bx) * kQueryBlock * p.mask_stride_q) * MASK_ES;
  }
  auto mask_region = [&](int stage) -> unsigned char* {
    if constexpr (SHARED_MASK) return lds + Shape::kSharedMaskOffset;
    return lds + stage * Shape::kStageBytes + Shape::kMaskOffset;
  };
  auto issue_mask_tile = [&](int tile, int stage) {
    if constexpr (STAGED) {
      unsigned char* slot = mask_region(stage) + wave * (NM * 1024);
      const int8_t* source = mask_block + static_cast<int64_t>(tile) * MASK_ROW_BYTES;
      const int lane_id = fresh_lane();
      const int last_row = p.q_len - 1 - bx * kQueryBlock;
#pragma unroll
      for (int i = 0; i < NM; ++i) {
        const int index = (wave * NM + i) * 64 + lane_id;
        const int row = index / MASK_CH, chunk = (index % MASK_CH) ^ mask_swizzle(row);
        const uint32_t offset = static_cast<uint32_t>(min(row, last_row)) *
                                    static_cast<uint32_t>(p.mask_stride_q * MASK_ES) + chunk * 16;
        copy16_to_lds_uniform(source, offset, slot + i * 1024);
      }
    }
  };
  auto issue_tile = [&](int tile, int stage) {
    unsigned char* k_slot = lds + stage * Shape::kStageBytes + wave * (NC * 1024);
    unsigned char* v_slot = k_slot + Shape::kTileBytes;
    unsigned char* sl = lds + stage * Shape::kStageBytes + 2 * Shape::kTileBytes;
    const int8_t* k_tile = k_base + static_cast<int64_t>(tile) * CTA_K * D;
    const int8_t* v_tile = v_base + static_cast<int64_t>(tile) * CTA_K;
    uint32_t k_src_offset[NC], v_src_offset[NC];
    if constexpr (KEEP_OFFSETS) {
#pragma unroll
      for (int i = 0; i < NC; ++i) k_src_offset[i] = k_kept[i], v_src_offset[i] = v_kept[i];
    } else {
      const int lane_id = fresh_lane();
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        k_src_offset[i] = k_source_offset(i, lane_id);
        v_src_offset[i] = v_source_offset(i, lane_id);
      }
    }
    const int keys_left = p.k_len - tile * CTA_K;
    if (keys_left >= CTA_K) {
#pragma unroll
      for (int i = 0; i < NC; ++i) copy16_to_lds_uniform(k_tile, k_src_offset[i], k_slot + i * 1024);
    } else {
      // Keys past the end exist only in the tail tile; their LDS rows keep stale
      // bytes, which is harmless because those scores are masked by index.
      const uint32_t bytes_left = static_cast<uint32_t>(keys_left) * D;
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        if (k_src_offset[i] < bytes_left) copy16_to_lds_uniform(k_tile, k_src_offset[i], k_slot + i * 1024);
      }
    }
#pragma unroll
    for (int i = 0; i < NC; ++i) copy16_to_lds_uniform(v_tile, v_src_offset[i], v_slot + i * 1024);
    if (wave == 0) {
      const int lane_id = KEEP_OFFSETS ? lane : fresh_lane();
      if (lane_id < D / 4) {
        copy16_to_lds_uniform(reinterpret_cast<const int8_t*>(sum_base + static_cast<int64_t>(tile) * D),
                              static_cast<uint32_t>(lane_id) * 16, sl);
      }
    }
    if constexpr (MASK_DT == kKeyBias) {
      if (wave == 1) {
        const int lane_id = fresh_lane();
        if (lane_id < CTA_K / 4) {
          copy16_to_lds_uniform(reinterpret_cast<const int8_t*>(bias_base + static_cast<int64_t>(tile) * CTA_K),
                                static_cast<uint32_t>(lane_id) * 16, sl + Shape::kSeedBytes);
        }
      }
    }
  };

  float o_acc[CB][16];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[cb][i] = 0.0f;
  float m_run = kRowFloor;
  float d_part = 0.0f;  // this lane's half of the row denominator
  // The float whose bits the P·V accumulators start from, kept in a vector
  // register: with a literal or scalar operand the subtraction that removes it
  // issues at half the rate.
  float seed_value;
  asm volatile("v_mov_b32 %0, %1" : "=v"(seed_value) : "s"(kAccumulatorSeedBits));

  // capture bookkeeping
  [[maybe_unused]] uint32_t* stats = nullptr;
  [[maybe_unused]] uint64_t full_words = 0;
  [[maybe_unused]] uint64_t stat_row = 0;
  if constexpr (CAPTURE) {
    const uint64_t mass_elements = static_cast<uint64_t>(p.batch) * p.q_heads * p.n_qb * p.n_kb;
    stats = reinterpret_cast<uint32_t*>(p.workspace + mass_elements);
    full_words = static_cast<uint64_t>(p.batch) * p.q_heads * p.q_len * (p.n_kb - 1) * 2;
    stat_row = static_cast<uint64_t>(bhq) * p.q_len + query;
  }

  const int64_t mask_row =
      (MASK_DT >= 0 && MASK_DT != kKeyBias)
          ? static_cast<int64_t>(batch) * p.mask_stride_b + static_cast<int64_t>(head) * p.mask_stride_h +
                static_cast<int64_t>(query) * p.mask_stride_q
          : 0;

  // Lane words of one tile: 16 scalar register pairs per 32-key block, loaded through the
  // scalar cache from a wave-uniform address.  The words of a tile's first key block are
  // requested a tile ahead, as soon as their predecessors have been applied; those of the
  // second block at the start of the softmax, where the first block's scores hide most of
  // the load (requested before the score product instead, the kernel is 1-4 % slower: more
  // scalar registers spilled).  All 32 requested a tile ahead do not fit the scalar registers.
  constexpr int kLaneWordsPerBlock = kLaneWordsPerTile / 2;
  [[maybe_unused]] uint64_t lane_words[2][LANES ? kLaneWordsPerBlock : 1];
  auto load_lane_words = [&](int tile, int key_block) {
    if constexpr (LANES) {
      typedef const __attribute__((address_space(4))) uint64_t* UniformWords;
      const uint64_t* at = p.mask_lanes + batch * p.mask_lanes_stride_b + head * p.mask_lanes_stride_h +
                           lane_word_offset(bx * 4 + wave, p.n_kb, tile) + key_block * kLaneWordsPerBlock;
      const UniformWords words = (UniformWords)(reinterpret_cast<uintptr_t>(at));
#pragma unroll
      for (int slot = 0; slot < kLaneWordsPerBlock; ++slot) lane_words[key_block][slot] = words[slot];
    }
  };

  // Mask elements of a full tile, requested before the next tile's copies.  Vector
  // memory operations complete in order: a mask load issued after the copies can only
  // be consumed once they have landed, which stalls the softmax of this tile on the
  // operands of the next one.  Requested first, it is waited for with the copies still
  // in flight.  Used for query-dependent masks (always 64-key tiles, where the
  // registers are there) that allow one load per group of four keys; not for FP32
  // masks with head dim 64, where the 32 extra registers cost a resident wavefront.
  constexpr bool PRELOAD = MASK_MODE == kMaskVector && CTA_K == 64 && !(MASK_DT == kF32 && D == 64);
  constexpr int WORDS = MASK_DT == kF32 ? 4 : MASK_DT == kBool ? 1 : 2;  // 32-bit words per four keys
  constexpr bool LATE_COPIES = PRELOAD;
  [[maybe_unused]] uint32_t mask_words[PRELOAD ? RB * 4 * WORDS : 1];
  auto load_mask_words = [&](int tile) {
    if constexpr (PRELOAD) {
      constexpr int ES = MASK_DT == kF32 ? 4 : MASK_DT == kBool ? 1 : 2;
      // Rows past the last query read the last row; their scores are discarded.
      const int64_t row = mask_row - static_cast<int64_t>(query_ok ? 0 : query - (p.q_len - 1)) * p.mask_stride_q;
      const unsigned char* base = static_cast<const unsigned char*>(p.mask) +
                                  (row + tile * CTA_K + half * 4) * ES;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          const unsigned char* at = base + (rb * 32 + b4 * 8) * ES;
          uint32_t* words = mask_words + (rb * 4 + b4) * WORDS;
          if constexpr (WORDS == 1) {
            words[0] = *reinterpret_cast<const uint32_t*>(at);
          } else if constexpr (WORDS == 2) {
            const uint2 w = *reinterpret_cast<const uint2*>(at);
            words[0] = w.x, words[1] = w.y;
          } else {
            const uint4 w = *reinterpret_cast<const uint4*>(at);
            words[0] = w.x, words[1] = w.y, words[2] = w.z, words[3] = w.w;
          }
        }
    }
  };

  // ---- S^T = K · Q^T for the tile staged in `stage` ---------------------------
  // The K fragments of k-step kk+1 are requested from LDS before the MFMAs of
  // k-step kk are issued, so the LDS latency hides behind RB matrix instructions.
  auto load_k_fragments = [&](const unsigned char* kl, int kk, v4i (&frag)[RB]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      frag[rb] = *reinterpret_cast<const v4i*>(kl + swizzled<D>(rb * 32 + l32, kk * 2 + half));
  };
  v16i score_seed;
#pragma unroll
  for (int i = 0; i < 16; ++i) score_seed[i] = kScoreSeedBits;
  auto score_tile = [&](int stage, v4i (&first)[RB], v16i (&s)[RB]) {
    const unsigned char* kl = lds + stage * Shape::kStageBytes;
    v4i frag[2][RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) frag[0][rb] = first[rb];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) load_k_fragments(kl, kk + 1, frag[(kk + 1) & 1]);
      __builtin_amdgcn_sched_group_barrier(0x100, RB, 0);  // RB LDS reads ...
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (kk == 0) {
          s[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[kk & 1][rb], qreg[kk], score_seed, 0, 0, 0);
        } else {
          s[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[kk & 1][rb], qreg[kk], s[rb], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);  // ... then RB MFMAs
    }
  };

  // ---- scores -> U8 probabilities (as signed bytes) and the online-softmax state.
  // LAST selects the formulas of the last listed tile.  Returns the factor the
  // tile's integer P·V is scaled by.
  //
  // The running reference m_run only moves when a tile maximum exceeds it by
  // more than kRescaleSlack: O and d are then relative to 2^m_run instead of
  // 2^(true running maximum), which cancels in O/d and in log2(d) + m_run and
  // changes FP32 rounding only, while the output accumulators are rescaled on
  // a handful of tiles instead of on every new maximum.
  constexpr float kRescaleSlack = 8.0f;
  auto softmax_tile = [&](auto last_tag, int it, int tile, int next_tile, float ks0, float ks1, v16i (&s)[RB],
                          v4i (&pk)[RB]) -> float {
    constexpr bool LAST = decltype(last_tag)::value;
    // K scale groups of this lane: keys 8b+4*half+r, group (key % 8) / 2 = 2*half + r/2.
    const float sc0 = qs2 * (q_scale * ks0);
    const float sc1 = qs2 * (q_scale * ks1);
    const int key0 = tile * CTA_K + half * 4;  // element (rb, i) is key key0 + rb*32 + (i>>2)*8 + (i&3)
    float tile_m;
    uint32_t row_sum = 0;

    // Raw scores of a tile without keys past the end: maxima of the seeded integers, one FMA
    // per score.  FLOORED applies the last-tile rule that a scale group's maximum starts from
    // -50000 (a clamp of the converted maximum: the conversion is exact and monotone).
    auto raw_score_tile = [&](auto floored_tag) {
      constexpr bool FLOORED = decltype(floored_tag)::value;
      int mx0 = s[0][0], mx1 = s[0][2];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (i & 2)
            mx1 = max(mx1, s[rb][i]);
          else
            mx0 = max(mx0, s[rb][i]);
        }
      float top0 = score_value(mx0), top1 = score_value(mx1);
      if constexpr (FLOORED) {
        top0 = __builtin_fmaxf(kRowFloor, top0);
        top1 = __builtin_fmaxf(kRowFloor, top1);
      }
      tile_m = __builtin_fmaxf(__builtin_fmaf(top0, sc0, -kU8Offset), __builtin_fmaf(top1, sc1, -kU8Offset));
      tile_m = max_across_halves(tile_m);
      const float neg_m = -tile_m;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          uint32_t packed = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x = __builtin_fmaf(score_value(s[rb][b4 * 4 + r]), (r & 2) ? sc1 : sc0, neg_m);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_exp2f(x), r, packed);
          }
          row_sum = __builtin_amdgcn_udot4(packed, 0x01010101u, row_sum, false);
          pk[rb][b4] = static_cast<int>(packed ^ 0x80808080u);
        }
    };
    if constexpr (FAST && !LAST) {
      raw_score_tile(std::false_type{});
    } else if constexpr (FAST) {
      // Last listed tile of the raw-score path: every scale group's maximum starts from
      // -50000, and keys past the end count as -1e30.  Their seeded scores are replaced by
      // the bit pattern of -1e30: a negative integer, so it never wins the integer maximum
      // (a group made of such keys alone ends at the -50000 clamp), and removing the seed
      // from it leaves -1e30 exactly.
      if ((tile + 1) * CTA_K > p.k_len) {
        constexpr int kPastEndBits = static_cast<int>(0xF149F2CAu);  // -1e30f
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = key0 + rb * 32 + (i >> 2) * 8 + (i & 3);
            s[rb][i] = key < p.k_len ? s[rb][i] : kPastEndBits;
          }
      }
      raw_score_tile(std::true_type{});
    } else {
      // Pre-scaled scores with masks.  Whether a tile needs any masking at all is
      // uniform over the wavefront: tiles below the causal diagonal, inside the key
      // range and without a mask tensor take the short loop.
      const float neg_inf = -__builtin_inff();
      constexpr bool has_mask = MASK_DT >= 0;
      const int first_query = bx * kQueryBlock + wave * 32;
      const bool on_diagonal = p.causal && tile * CTA_K + CTA_K - 1 > first_query;
      const bool partial = LAST && (tile + 1) * CTA_K > p.k_len;
      float mx = kRowFloor;
      // A key-only mask whose additive row is zero over this whole tile (a padding mask leaves
      // every tile but the one at its edge like that) changes nothing in it: x + 0 = x bit for
      // bit (a zero of either sign; only the sign of a zero sum can differ, which neither the
      // maximum nor the exponential sees).  One LDS read per wavefront and tile decides.
      [[maybe_unused]] bool zero_row = false;
      if constexpr (MASK_DT == kKeyBias) {
        if (!on_diagonal && !partial) {
          const float* bias_row = reinterpret_cast<const float*>(
              lds + (it & 1) * Shape::kStageBytes + 2 * Shape::kTileBytes + Shape::kSeedBytes);
          const v4i probe = *reinterpret_cast<const v4i*>(bias_row + (lane & (CTA_K / 4 - 1)) * 4);
          const bool nonzero = (static_cast<uint32_t>(probe[0] | probe[1] | probe[2] | probe[3]) << 1) != 0;
          zero_row = __builtin_amdgcn_ballot_w64(nonzero) == 0;
        }
      }
      if ((!has_mask || zero_row) && !on_diagonal && !partial) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float value = score_value(s[rb][i]) * ((i & 2) ? sc1 : sc0);
            s[rb][i] = __float_as_int(value);
            mx = __builtin_fmaxf(mx, value);
          }
      } else if constexpr (MASK_DT == kKeyBias) {
        // Key-only mask: the tile's row of additive terms (already in the exp2
        // domain, -inf for hidden and out-of-range keys) sits in LDS next to the
        // seeds; a lane reads the four consecutive keys of a group in one go.  The
        // causal comparison is only compiled into the pass for tiles on the diagonal.
        const float* bias_row = reinterpret_cast<const float*>(
            lds + (it & 1) * Shape::kStageBytes + 2 * Shape::kTileBytes + Shape::kSeedBytes);
        auto biased_scores = [&](auto diagonal_tag) {
          constexpr bool DIAGONAL = decltype(diagonal_tag)::value;
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
              const int local = rb * 32 + b4 * 8 + half * 4;
              // A plain vector type on purpose: the compiler orders an LDS read it cannot
              // classify (HIP's float4 is a struct) behind every outstanding copy into LDS,
              // which would wait for the next tile in the middle of this one.
              const v4f bias = *reinterpret_cast<const v4f*>(bias_row + local);
              const float terms[4] = {bias[0], bias[1], bias[2], bias[3]};
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float value = score_value(s[rb][b4 * 4 + r]) * ((r & 2) ? sc1 : sc0) + terms[r];
                if constexpr (DIAGONAL) {
                  if (tile * CTA_K + local + r > query) value = neg_inf;
                }
                s[rb][b4 * 4 + r] = __float_as_int(value);
                mx = __builtin_fmaxf(mx, value);
              }
            }
        };
        if (on_diagonal) {
          biased_scores(std::true_type{});
        } else {
          biased_scores(std::false_type{});
        }
      } else if constexpr (LANES) {
        // Lane words: bit l of word (rb, i) says whether lane l keeps score (rb, i); keys past
        // the end and rows past the last query have no bit set, so the last tile needs nothing else.
        auto lane_masked_scores = [&](auto diagonal_tag, auto block_tag) {
          constexpr bool DIAGONAL = decltype(diagonal_tag)::value;
          constexpr int rb = decltype(block_tag)::value;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            bool keep = __builtin_amdgcn_inverse_ballot_w64(lane_words[rb][i]);
            if constexpr (DIAGONAL) keep = keep && key0 + rb * 32 + (i >> 2) * 8 + (i & 3) <= query;
            const float scaled = score_value(s[rb][i]) * ((i & 2) ? sc1 : sc0);
            const float value = keep ? scaled : neg_inf;
            s[rb][i] = __float_as_int(value);
            mx = __builtin_fmaxf(mx, value);
          }
        };
        auto lane_pass = [&](auto diagonal_tag) {
          load_lane_words(tile, 1);
          __builtin_amdgcn_sched_barrier(0);
          lane_masked_scores(diagonal_tag, std::integral_constant<int, 0>{});
          lane_masked_scores(diagonal_tag, std::integral_constant<int, 1>{});
          __builtin_amdgcn_sched_barrier(0);
          if (!LAST) load_lane_words(next_tile, 0);
        };
        if (on_diagonal) {
          lane_pass(std::true_type{});
        } else {
          lane_pass(std::false_type{});
        }
      } else {
        // DT: mask element type (-1: none, only the causal / key-range tests);
        // VEC: one load per group of four consecutive keys.
        auto masked_scores = [&](auto dtype_tag, auto vector_tag, auto preloaded_tag, auto diagonal_tag) {
          constexpr bool DIAGONAL = decltype(diagonal_tag)::value;  // causal comparison per score
          constexpr int DT = decltype(dtype_tag)::value;
          constexpr bool VEC = decltype(vector_tag)::value;
          constexpr bool LOADED = decltype(preloaded_tag)::value;  // elements are in mask_words
          constexpr int ES = DT == kF32 ? 4 : DT == kBool ? 1 : 2;
          [[maybe_unused]] const unsigned char* lane_mask = nullptr;
          if constexpr (DT >= 0) {
            lane_mask = static_cast<const unsigned char*>(p.mask) +
                        (mask_row + static_cast<int64_t>(key0) * p.mask_stride_k) * ES;
          }
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int b4 = 0; b4 < 4; ++b4) {
              const int local = rb * 32 + b4 * 8;  // first of four consecutive keys of this lane
              const int key = key0 + local;
              bool keep[4] = {true, true, true, true};
              float bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
              if constexpr (DT >= 0) {
                if constexpr (LOADED) {
                  // Rows past the last query hold the last row's mask: they behave like
                  // a valid row and are never stored.
                  [[maybe_unused]] uint32_t staged_words[4];
                  const uint32_t* words = mask_words + (rb * 4 + b4) * WORDS;
                  if constexpr (STAGED) {
                    // This lane's four keys of the group: bytes [offset, offset + 4 * ES) of its row.
                    const int row = wave * 32 + l32;
                    const int offset = (local + half * 4) * MASK_ES;
                    const unsigned char* at = mask_region(it & 1) + row * MASK_ROW_BYTES +
                                              (((offset >> 4) ^ mask_swizzle(row)) << 4) + (offset & 15);
                    if constexpr (MASK_ES == 1) {
                      staged_words[0] = *reinterpret_cast<const uint32_t*>(at);
                    } else if constexpr (MASK_ES == 4) {
                      typedef uint32_t v4u __attribute__((ext_vector_type(4)));
                      const v4u quad = *reinterpret_cast<const v4u*>(at);
                      staged_words[0] = quad[0], staged_words[1] = quad[1];
                      staged_words[2] = quad[2], staged_words[3] = quad[3];
                    } else {
                      typedef uint32_t v2u __attribute__((ext_vector_type(2)));
                      const v2u pair = *reinterpret_cast<const v2u*>(at);
                      staged_words[0] = pair[0], staged_words[1] = pair[1];
                    }
                    words = staged_words;
                  }
                  if constexpr (DT == kBool) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) keep[r] = ((words[0] >> (8 * r)) & 0xffu) != 0;
                  } else if constexpr (DT == kF32) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) bias[r] = __uint_as_float(words[r]);
                  } else {
                    const uint32_t bits16[4] = {words[0] & 0xffffu, words[0] >> 16, words[1] & 0xffffu,
                                                words[1] >> 16};
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                      bias[r] = DT == kF16 ? static_cast<float>(__builtin_bit_cast(
                                                 _Float16, static_cast<uint16_t>(bits16[r])))
                                           : __uint_as_float(bits16[r] << 16);
                    }
                  }
                } else if (!query_ok) {
#pragma unroll
                  for (int r = 0; r < 4; ++r) keep[r] = false;
                } else if (VEC && key + 3 < p.k_len) {
                  const unsigned char* at = lane_mask + local * ES;
                  if constexpr (DT == kBool) {
                    const uint32_t word = *reinterpret_cast<const uint32_t*>(at);
#pragma unroll
                    for (int r = 0; r < 4; ++r) keep[r] = ((word >> (8 * r)) & 0xffu) != 0;
                  } else if constexpr (DT == kF32) {
                    const float4 w = *reinterpret_cast<const float4*>(at);
                    bias[0] = w.x, bias[1] = w.y, bias[2] = w.z, bias[3] = w.w;
                  } else {
                    const uint2 w = *reinterpret_cast<const uint2*>(at);
                    const uint32_t bits16[4] = {w.x & 0xffffu, w.x >> 16, w.y & 0xffffu, w.y >> 16};
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                      bias[r] = DT == kF16 ? static_cast<float>(__builtin_bit_cast(
                                                 _Float16, static_cast<uint16_t>(bits16[r])))
                                           : __uint_as_float(bits16[r] << 16);
                    }
                  }
                } else {
#pragma unroll
                  for (int r = 0; r < 4; ++r) {
                    keep[r] = key + r < p.k_len;
                    if (keep[r]) {
                      const unsigned char* at = lane_mask + (local + r) * p.mask_stride_k * ES;
                      if constexpr (DT == kBool) {
                        keep[r] = *at != 0;
                      } else {
                        bias[r] = load1<DT>(at, 0);
                      }
                    }
                  }
                }
                if constexpr (DT != kBool) {
#pragma unroll
                  for (int r = 0; r < 4; ++r) keep[r] = keep[r] && __builtin_isfinite(bias[r]);
                }
              }
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                float value = score_value(s[rb][b4 * 4 + r]) * ((r & 2) ? sc1 : sc0);
                if constexpr (DT >= 0) value = keep[r] ? value + bias[r] * kLog2e : neg_inf;
                if constexpr (DIAGONAL) {
                  if (key + r > query) value = neg_inf;
                }
                if (LAST && key + r >= p.k_len) value = neg_inf;
                s[rb][b4 * 4 + r] = __float_as_int(value);
                mx = __builtin_fmaxf(mx, value);
              }
              // The mask loads of one key block at a time: all of a tile in flight
              // at once do not fit the register file.
              if constexpr (DT >= 0 && !LOADED) {
                if (b4 == 3) {
                  asm volatile("" ::: "memory");
                  __builtin_amdgcn_sched_barrier(0);
                }
              }
            }
        };
        using MaskType = std::integral_constant<int, MASK_DT>;
        auto mask_pass = [&](auto diagonal_tag) {
          if constexpr ((PRELOAD || STAGED) && !LAST) {
            masked_scores(MaskType{}, std::true_type{}, std::true_type{}, diagonal_tag);
          } else if constexpr (MASK_VEC) {
            masked_scores(MaskType{}, std::true_type{}, std::false_type{}, diagonal_tag);
          } else {
            masked_scores(MaskType{}, std::false_type{}, std::false_type{}, diagonal_tag);
          }
        };
        if (on_diagonal) {
          mask_pass(std::true_type{});
        } else {
          mask_pass(std::false_type{});
        }
      }
      tile_m = mx - kU8Offset;
      tile_m = max_across_halves(tile_m);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          uint32_t packed = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            packed = __builtin_amdgcn_cvt_pk_u8_f32(
                __builtin_amdgcn_exp2f(__int_as_float(s[rb][b4 * 4 + r]) - tile_m), r, packed);
          }
          row_sum = __builtin_amdgcn_udot4(packed, 0x01010101u, row_sum, false);
          pk[rb][b4] = static_cast<int>(packed ^ 0x80808080u);
        }
    }

    // ---- online softmax state ----------------------------------------------
    const bool raise = tile_m > m_run + kRescaleSlack;
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float o_scale = raise ? __builtin_amdgcn_exp2f(m_run - tile_m) : 1.0f;
      m_run = raise ? tile_m : m_run;
      d_part *= o_scale;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[cb][i] *= o_scale;
    }
    const float t_scale = __builtin_amdgcn_exp2f(tile_m - m_run);
    d_part = __builtin_fmaf(static_cast<float>(row_sum), t_scale, d_part);

    if constexpr (CAPTURE) {
      const uint32_t numerator = sum_across_halves(row_sum);
      if (half == 0 && query_ok) {
        if constexpr (!LAST) {
          // Tile-major: the 32 queries of a half-wave store 256 contiguous bytes.
          const uint64_t offset = ((bhq * (p.n_kb - 1) + it) * static_cast<uint64_t>(p.q_len) + query) * 2;
          stats[offset] = numerator;
          stats[offset + 1] = __float_as_uint(tile_m);
        } else {
          const uint64_t offset = full_words + stat_row * 2;
          stats[offset] = __float_as_uint(static_cast<float>(numerator));
          stats[offset + 1] = __float_as_uint(tile_m);
        }
      }
    }
    return t_scale;
  };

  // ---- O^T += t_scale * (128*sum(V) + V^T · P_s8^T) -----------------------------
  // Channel blocks are processed in pairs (two independent MFMA chains keep the
  // matrix pipe busy).  LDS operands are requested ahead of use: the accumulator
  // seeds (zero-point terms) and first V fragments of the first pair before the
  // exponentials when PREFETCH is set, everything else one step ahead of its MFMAs.
  constexpr bool PREFETCH = FAST && D <= 128;
  auto load_seed_pair = [&](int stage, int cb, v16i (&acc)[2]) {
    const int* sl = reinterpret_cast<const int*>(lds + stage * Shape::kStageBytes + 2 * Shape::kTileBytes);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const v4i init = *reinterpret_cast<const v4i*>(sl + (cb + j) * 32 + b4 * 8 + half * 4);
        acc[j][b4 * 4 + 0] = init[0];
        acc[j][b4 * 4 + 1] = init[1];
        acc[j][b4 * 4 + 2] = init[2];
        acc[j][b4 * 4 + 3] = init[3];
      }
    }
  };
  auto load_v_pair = [&](int stage, int cb, int rb, v4i (&frag)[2]) {
    const unsigned char* vl = lds + stage * Shape::kStageBytes + Shape::kTileBytes;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      frag[j] = *reinterpret_cast<const v4i*>(vl + swizzled<CTA_K>((cb + j) * 32 + l32, rb * 2 + half));
  };
  auto unseed = [&](int bits) { return __int_as_float(bits) - seed_value; };
  auto value_tile = [&](int stage, const v4i (&pk)[RB], v16i (&seed0)[2], v4i (&first0)[2], float t_scale) {
    // Three accumulator sets rotate when there are more than two pairs: one being
    // seeded, one being multiplied, one being folded into the output.
    constexpr int SETS = CB / 2 > 2 ? 3 : 2;
    v16i acc[SETS][2];  // [pair % SETS][block of the pair]
    v4i frag[2][2];     // [step parity][block of the pair]
    acc[0][0] = seed0[0];
    acc[0][1] = seed0[1];
    frag[0][0] = first0[0];
    frag[0][1] = first0[1];
    int step = 0;
#pragma unroll
    for (int pair = 0; pair < CB / 2; ++pair) {
      const int cb = pair * 2;
      if (pair + 1 < CB / 2) load_seed_pair(stage, cb + 2, acc[(pair + 1) % SETS]);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb, ++step) {
        // request the operands of the next step before this step's MFMAs
        if (rb + 1 < RB) {
          load_v_pair(stage, cb, rb + 1, frag[(step + 1) & 1]);
        } else if (pair + 1 < CB / 2) {
          load_v_pair(stage, cb + 2, 0, frag[(step + 1) & 1]);
        }
        acc[pair % SETS][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[step & 1][0], pk[rb], acc[pair % SETS][0], 0, 0, 0);
        acc[pair % SETS][1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(frag[step & 1][1], pk[rb], acc[pair % SETS][1], 0, 0, 0);
      }
      if (pair > 0) {
        // fold the previous pair while this pair's MFMAs run
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          o_acc[cb - 2][i] = __builtin_fmaf(unseed(acc[(pair - 1) % SETS][0][i]), t_scale, o_acc[cb - 2][i]);
          o_acc[cb - 1][i] = __builtin_fmaf(unseed(acc[(pair - 1) % SETS][1][i]), t_scale, o_acc[cb - 1][i]);
        }
      }
    }
    constexpr int last_pair = CB / 2 - 1;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      o_acc[CB - 2][i] = __builtin_fmaf(unseed(acc[last_pair % SETS][0][i]), t_scale, o_acc[CB - 2][i]);
      o_acc[CB - 1][i] = __builtin_fmaf(unseed(acc[last_pair % SETS][1][i]), t_scale, o_acc[CB - 1][i]);
    }
  };

  // --- main loop: one barrier per tile -----------------------------------------
  // At the barrier of iteration t every wave has finished tile t-1 (so stage
  // (t+1)&1 may be overwritten) and has seen its own share of tile t land.
  // Raw-score launches with head dim 128 and 128-key tiles (dense, over a sparse pattern's tile
  // lists, or capturing the statistics of pattern construction) walk every tile but the last in
  // a hand-scheduled loop, written by gen_dense_loop.py into dense_, sparse_ and
  // capture_loop_d128.inc: same arithmetic in the same order as the loop below, bit-identical
  // results.  The loop owns the whole register file, so its operands are pinned to the registers
  // the generator chose; the last listed tile (the one that may be partial) and the epilogue
  // stay below.
  constexpr bool ASM_LOOP = FAST && D == 128 && CTA_K == 128;
  int first_tile = 0;
  if constexpr (ASM_LOOP) {
    if (n_it > 1 && !p.compiled_loop) {
      typedef __attribute__((address_space(3))) unsigned char* LdsBytes;
      const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((LdsBytes)lds));
      issue_tile(tile_at(0), 0);
      v16i out0 = {}, out1 = {}, out2 = {}, out3 = {};
      // this lane's fragment address per k-step (K) / key block (V): row l32 of a 32-row block
      const uint32_t a0 = lds_address + swizzled<128>(l32, 0 + half), a1 = lds_address + swizzled<128>(l32, 2 + half);
      const uint32_t a2 = lds_address + swizzled<128>(l32, 4 + half), a3 = lds_address + swizzled<128>(l32, 6 + half);
      const uint32_t seed_address = lds_address + half * 16 + 2048;  // (the generator's SEED_BIAS)
      // lane share of the copy source offsets: the rest, (wave * NC + i) KiB of K or that many
      // groups of eight V rows, is scalar arithmetic in the loop; the share repeats with period 2 in i
      const uint32_t kc0 = k_source_offset(0, lane) - static_cast<uint32_t>(wave * NC) * 1024u;
      const uint32_t kc1 = k_source_offset(1, lane) - static_cast<uint32_t>(wave * NC + 1) * 1024u;
      const uint32_t vc0 = v_source_offset(0, lane) - static_cast<uint32_t>(wave * NC) * 8u * static_cast<uint32_t>(p.padded);
      const uint32_t vc1 = v_source_offset(1, lane) - static_cast<uint32_t>(wave * NC + 1) * 8u * static_cast<uint32_t>(p.padded);
      // dense: sources of tile 1 (the loop advances them); sparse: bases of the head and the tile list
      const uint64_t k_source = reinterpret_cast<uint64_t>(INDEXED ? k_base : k_base + CTA_K * D);
      const uint64_t v_source = reinterpret_cast<uint64_t>(INDEXED ? v_base : v_base + CTA_K);
      const uint64_t sum_source = reinterpret_cast<uint64_t>(INDEXED ? sum_base : sum_base + D);
      const uint64_t ks_source = reinterpret_cast<uint64_t>(ks_base);
      const int count = n_it - 1;
      if constexpr (INDEXED) {
        const uint64_t list = reinterpret_cast<uint64_t>(indices);
        asm volatile(
#include "sparse_loop_d128.inc"
            : "+{v[128:143]}"(out0), "+{v[144:159]}"(out1), "+{v[160:175]}"(out2), "+{v[176:191]}"(out3),
              "+{v241}"(m_run), "+{v242}"(d_part)
            : "{v[192:195]}"(qreg[0]), "{v[196:199]}"(qreg[1]), "{v[200:203]}"(qreg[2]), "{v[204:207]}"(qreg[3]),
              "{v244}"(q_scale), "{v246}"(a0), "{v247}"(a1), "{v248}"(a2), "{v249}"(a3), "{v250}"(seed_address),
              "{v251}"(kc0), "{v252}"(kc1), "{v253}"(vc0), "{v254}"(vc1),
              [kptr] "s"(k_source), [vptr] "s"(v_source), [sumptr] "s"(sum_source), [ksptr] "s"(ks_source),
              [count] "s"(count), [wave] "s"(wave), [qs2] "s"(qs2), [padded] "s"(p.padded), [list] "s"(list)
            :
#include "sparse_loop_d128_clobbers.inc"
        );
      } else if constexpr (CAPTURE) {
        // statistics of tile 0 for this wavefront's first query; lanes 0..31 hold the queries that store
        const uint64_t stats_rows = reinterpret_cast<uint64_t>(
            stats + (bhq * static_cast<uint64_t>(p.n_kb - 1) * p.q_len + (bx * kQueryBlock + wave * 32)) * 2);
        const uint32_t tile_bytes = static_cast<uint32_t>(p.q_len) * 8u;
        const uint64_t storing = __builtin_amdgcn_ballot_w64(half == 0 && query_ok);
        asm volatile(
#include "capture_loop_d128.inc"
            : "+{v[128:143]}"(out0), "+{v[144:159]}"(out1), "+{v[160:175]}"(out2), "+{v[176:191]}"(out3),
              "+{v241}"(m_run), "+{v242}"(d_part)
            : "{v[192:195]}"(qreg[0]), "{v[196:199]}"(qreg[1]), "{v[200:203]}"(qreg[2]), "{v[204:207]}"(qreg[3]),
              "{v244}"(q_scale), "{v246}"(a0), "{v247}"(a1), "{v248}"(a2), "{v249}"(a3), "{v250}"(seed_address),
              "{v251}"(kc0), "{v252}"(kc1), "{v253}"(vc0), "{v254}"(vc1),
              [kptr] "s"(k_source), [vptr] "s"(v_source), [sumptr] "s"(sum_source), [ksptr] "s"(ks_source),
              [count] "s"(count), [wave] "s"(wave), [qs2] "s"(qs2), [padded] "s"(p.padded),
              [stats] "s"(stats_rows), [qlen8] "s"(tile_bytes), [capexec] "s"(storing)
            :
#include "capture_loop_d128_clobbers.inc"
        );
      } else {
        asm volatile(
#include "dense_loop_d128.inc"
            : "+{v[128:143]}"(out0), "+{v[144:159]}"(out1), "+{v[160:175]}"(out2), "+{v[176:191]}"(out3),
              "+{v241}"(m_run), "+{v242}"(d_part)
            : "{v[192:195]}"(qreg[0]), "{v[196:199]}"(qreg[1]), "{v[200:203]}"(qreg[2]), "{v[204:207]}"(qreg[3]),
              "{v244}"(q_scale), "{v246}"(a0), "{v247}"(a1), "{v248}"(a2), "{v249}"(a3), "{v250}"(seed_address),
              "{v251}"(kc0), "{v252}"(kc1), "{v253}"(vc0), "{v254}"(vc1),
              [kptr] "s"(k_source), [vptr] "s"(v_source), [sumptr] "s"(sum_source), [ksptr] "s"(ks_source),
              [count] "s"(count), [wave] "s"(wave), [qs2] "s"(qs2), [padded] "s"(p.padded)
            :
#include "dense_loop_d128_clobbers.inc"
        );
      }
      lane = fresh_lane();
      l32 = lane & 31;
      half = lane >> 5;
      query = bx * kQueryBlock + wave * 32 + l32;
      query_ok = query < p.q_len;
      if constexpr (CAPTURE) stat_row = static_cast<uint64_t>(bhq) * p.q_len + query;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        o_acc[0][i] = __int_as_float(out0[i]);
        o_acc[1][i] = __int_as_float(out1[i]);
        o_acc[2][i] = __int_as_float(out2[i]);
        o_acc[3][i] = __int_as_float(out3[i]);
      }
      first_tile = n_it - 1;
    }
  }
  if (n_it > 0) {
    v16i s[RB];
    v4i pk[RB];
    v4i k_first[RB];
    v4i v_first[2];
    v16i seed[2];
    int tile = tile_at(first_tile);
    if (first_tile == 0) issue_tile(tile, 0);
    // The last listed tile reads its mask elements directly (it may be partial).
    if (n_it > 1) issue_mask_tile(tile, 0);
    load_lane_words(tile, 0);
    float ks0 = ks_base[tile * 4 + 2 * half];
    float ks1 = ks_base[tile * 4 + 2 * half + 1];
    // Listed tiles: the entry after the next one is requested a whole tile before it is
    // needed, ahead of the copies (read where it is needed, its round trip would be
    // waited for in every tile).
    [[maybe_unused]] int listed_next = INDEXED && n_it > 1 ? tile_at(1) : 0;
    for (int it = first_tile; it < n_it - 1; ++it) {
      const int stage = it & 1;
      const int next_tile = INDEXED ? listed_next : it + 1;
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      [[maybe_unused]] int listed_after_next = 0;
      if constexpr (INDEXED) {
        listed_after_next = min(it + 2, n_it - 1);
        if (!whole_list) listed_after_next = indices[listed_after_next];
      }
      load_k_fragments(lds + stage * Shape::kStageBytes, 0, k_first);
      if constexpr (PRELOAD) {
        load_mask_words(tile);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (!LATE_COPIES) issue_tile(next_tile, stage ^ 1);
      if constexpr (!SHARED_MASK) {
        if (it + 2 < n_it) issue_mask_tile(next_tile, stage ^ 1);
      }
      const int scale_pair = KEEP_OFFSETS ? 2 * half : (fresh_lane() >> 5) * 2;
      const float next_ks0 = ks_base[next_tile * 4 + scale_pair];
      const float next_ks1 = ks_base[next_tile * 4 + scale_pair + 1];
      // Wave priorities by phase: when one wavefront of a SIMD is in its softmax and
      // the other in a matrix phase, the vector instructions go first.  Matrix and
      // vector instructions do not overlap on a SIMD; a matrix instruction issued
      // ahead of short vector work delays a whole dependent chain, the other way
      // round it costs the matrix phase one issue slot (3 % on the dense kernel).
      __builtin_amdgcn_s_setprio(0);
      score_tile(stage, k_first, s);
      if constexpr (PREFETCH) {
        load_seed_pair(stage, 0, seed);
        load_v_pair(stage, 0, 0, v_first);
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_s_setprio(2);
      const float t_scale = softmax_tile(std::false_type{}, it, tile, next_tile, ks0, ks1, s, pk);
      __builtin_amdgcn_s_setprio(1);
      if constexpr (LATE_COPIES) {
        __builtin_amdgcn_sched_barrier(0);
        issue_tile(next_tile, stage ^ 1);
      }
      if constexpr (SHARED_MASK) {
        // this wavefront has consumed its rows of the one mask tile: refill them
        __builtin_amdgcn_sched_barrier(0);
        if (it + 2 < n_it) issue_mask_tile(next_tile, stage ^ 1);
      }
      if constexpr (PREFETCH) {
        __builtin_amdgcn_sched_barrier(0);
      } else {
        load_seed_pair(stage, 0, seed);
        load_v_pair(stage, 0, 0, v_first);
      }
      value_tile(stage, pk, seed, v_first, t_scale);
      tile = next_tile;
      ks0 = next_ks0;
      ks1 = next_ks1;
      if constexpr (INDEXED) listed_next = __builtin_amdgcn_readfirstlane(listed_after_next);
    }
    const int stage = (n_it - 1) & 1;
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    load_k_fragments(lds + stage * Shape::kStageBytes, 0, k_first);
    score_tile(stage, k_first, s);
    const float t_scale = softmax_tile(std::true_type{}, n_it - 1, tile, tile, ks0, ks1, s, pk);
    load_seed_pair(stage, 0, seed);
    load_v_pair(stage, 0, 0, v_first);
    value_tile(stage, pk, seed, v_first, t_scale);
  }

  // ---- epilogue --------------------------------------------------------------
  if constexpr (CAPTURE) {
    const float d_total = d_part + __shfl_xor(d_part, 32);
    if (half == 0 && query_ok) {
      const uint64_t query_rows = static_cast<uint64_t>(p.batch) * p.q_heads * p.q_len;
      float* state = reinterpret_cast<float*>(stats + full_words + query_rows * 2);
      state[stat_row * 2] = m_run;
      state[stat_row * 2 + 1] = d_total;
    }
  }
  // A lane owns one query and, per instruction, four channels of it: stored from there, an
  // instruction would write 16 bytes into each of 32 rows, and a launch with short tile
  // lists spends more time on such stores than on its tiles (40 heads x 32K tokens, one
  // listed tile per query block: 155 of 264 us).  The rows go through LDS instead (every
  // wavefront has left the tiles by then; 64 * D bytes per wavefront) and leave as whole
  // rows, 16 bytes per lane.
  __syncthreads();  // no wavefront reads a tile any more
  constexpr int ROW_BYTES = D * 2;
  constexpr int CHUNKS = ROW_BYTES / 16;  // 16-byte pieces of a row
  constexpr int ROWS_PER_STORE = 64 / CHUNKS;
  constexpr int STORES = 32 / ROWS_PER_STORE;
  const float d_total = d_part + __shfl_xor(d_part, 32);
  const bool guard_empty = !FAST && (MASK_DT >= 0 || p.causal);
  const bool row_valid = d_total > 0.0f;
  const float inv_d = 1.0f / d_total;
  const bool zero_row = guard_empty && !row_valid;
  unsigned char* mine = lds + wave * (32 * ROW_BYTES);
  const int first_query = bx * kQueryBlock + wave * 32;
  unsigned char* out_block = static_cast<unsigned char*>(p.out) +
                             2 * (batch * p.out_stride_b + head * p.out_stride_h +
                                  static_cast<int64_t>(first_query) * p.out_stride_n);
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int b4 = 0; b4 < 4; ++b4) {
      const int c = cb * 32 + b4 * 8 + half * 4;
      const v4f scale4 = *reinterpret_cast<const v4f*>(p.v_scale + bhk * D + c);
      const v4f center4 = *reinterpret_cast<const v4f*>(p.v_center + bhk * D + c);
      float value[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        value[r] = __builtin_fmaf(o_acc[cb][b4 * 4 + r] * inv_d, scale4[r], center4[r]);
        value[r] = zero_row ? 0.0f : value[r];
      }
      typedef uint32_t v2u __attribute__((ext_vector_type(2)));
      v2u word;
      word.x = to_output_pair(value[0], value[1], p.out_dtype);
      word.y = to_output_pair(value[2], value[3], p.out_dtype);
      *reinterpret_cast<v2u*>(mine + swizzled<ROW_BYTES>(l32, cb * 4 + b4) + half * 8) = word;
    }
  asm volatile("" ::: "memory");  // the pieces below are read from other lanes' writes
#pragma unroll
  for (int i = 0; i < STORES; ++i) {
    const int row = i * ROWS_PER_STORE + lane / CHUNKS, chunk = lane % CHUNKS;
    const v4i piece = *reinterpret_cast<const v4i*>(mine + swizzled<ROW_BYTES>(row, chunk));
    if (first_query + row < p.q_len) {
      *reinterpret_cast<v4i*>(out_block + 2 * static_cast<int64_t>(row) * p.out_stride_n + chunk * 16) = piece;
    }
  }
  if (p.lse != nullptr && half == 0 && query_ok) {
    p.lse[bhq * p.q_len + query] =
        row_valid ? (__builtin_amdgcn_logf(d_total) + m_run) / kLog2e : -__builtin_inff();
  }
}

}  // namespace risa
