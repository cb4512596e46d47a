// Attention kernel with sixteen queries per wavefront: launches with fewer workgroups
// than compute units, and every launch with head dim 256.
//
// Same arithmetic as risa::attention_kernel (reference csrc/kernels/attention_int8.cuh:
// 145-1026; the raw-score path, and for head dim 256 also the pre-scaled path with masks,
// the causal rule and the capture stores) on the same operands, with the 128 queries of a
// workgroup spread over eight wavefronts of sixteen queries instead of four of thirty-two.  A lone 256-thread workgroup leaves
// one wavefront per SIMD, which issues a vector instruction only every other slot;
// eight wavefronts put two on every SIMD with half the work each.  Measured on
// B=1, H=16, D=128: 19 -> 17 us at 512 tokens, 29 -> 27.5 us at 1024, 47 -> 40.5 us at
// 2048; what remains per tile is the dependent chain barrier -> LDS -> MFMA -> row
// maximum -> exp2 -> MFMA.  On a full machine the wide kernel is the faster one (fewer
// vector instructions per score, half the LDS operand traffic).
//
// Matrix instruction: v_mfma_i32_16x16x64_i8.  Lane l = 16*g + c feeds row/column c
// with the sixteen bytes [16*g, 16*g + 16) of the 64-deep product and receives rows
// 4*g .. 4*g + 3 of column c.
//   * S^T = K · Q^T per 16-key block: A = 16 K rows from LDS, B = Q rows in registers.
//     Row r of block (s, b) (s: 64-key step, b: 0..3) is key 64*s + 8*b + 32*(r/8) + r%8,
//     so that lane group g ends up with keys 64*s + 32*(g/2) + 8*b + 4*(g%2) + i,
//     i = 0..3: packing the four blocks b of a step gives sixteen bytes that sit at
//     positions 16*g + 4*b + i of the step, exactly where the packed V matrix
//     (risa::packed_value_position) keeps those tokens.
//   * O^T = V^T · P^T per 16-channel block: A = 16 V rows (channels) from LDS, one
//     16-byte read per 64-key step, B = the packed probabilities, no shuffle.
#pragma once

#include "attention_kernel.hpp"

namespace risa {


// XOR applied to the 16-byte chunk index of K row `row` in LDS.  The sixteen rows a
// matrix instruction reads are two runs of eight consecutive keys 32 apart; folding
// bit 5 of the row into the swizzle keeps their sixteen chunks in distinct banks.
template <int ROWBYTES> __device__ __forceinline__ int narrow_key_swizzle(int row) {
  constexpr int CH = ROWBYTES / 16;
  constexpr int ROWS_PER_256 = 256 / ROWBYTES;
  return ((row / ROWS_PER_256) ^ ((row >> 5) * (8 / ROWS_PER_256))) & (CH - 1);
}

// WAVES wavefronts of sixteen queries per workgroup (8, 4 or 2: 128, 64 or 32 queries).
// The launcher picks the largest workgroup that still gives every compute unit one.
// KSPLIT = 2 doubles the wavefronts: two parts of WAVES wavefronts walk the first and the
// second half of the key tiles of the same queries (each with its own LDS stages) and
// the first part merges the two partial results through LDS at the end, which halves
// the chain of dependent tiles of a short sequence.  The merge is the online-softmax
// update applied once more, so only the FP32 rounding order differs.
// INDEXED walks the key tiles listed for the 128-query block of the workgroup's queries
// (the CSR pattern of the sparse path, or the active tiles of a key-only mask) instead of
// all of them; the last listed tile takes the last-tile formulas, as in the wide kernel.
//
// GENERAL is the pre-scaled path of the wide kernel (masks, causal, scale <= 0) with the
// same decisions and arithmetic per score, CAPTURE its statistics stores; both run with
// 128-query workgroups only.  MASK_DT as in the wide kernel (-1 none, kKeyBias for the
// additive row of a key-only mask, else the element type of the mask tensor); MASK_VEC:
// the four consecutive keys of a score group come from one load (unit key stride, aligned
// rows).  They exist for head dim 256, where thirty-two queries per wavefront leave one
// wavefront per SIMD.
template <int D, int CTA_K, int MASK_DT = -1> using NarrowTileShape = TileShape<D, CTA_K, MASK_DT == kKeyBias ? CTA_K * 4 : 0>;

__device__ __forceinline__ uint32_t sum_across_row_pairs(uint32_t x) {
  const auto both = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  return both[0] + both[1];
}

template <int D, int CTA_K, int WAVES, int KSPLIT = 1, bool INDEXED = false, bool GENERAL = false,
          bool CAPTURE = false, int MASK_DT = -1, bool MASK_VEC = false>
__global__ __launch_bounds__(64 * WAVES * KSPLIT) void attention_narrow_kernel(const KernelParams p) {
  static_assert(WAVES == 8 || WAVES == 4 || WAVES == 2, "seeds and scales are copied by two different wavefronts");
  static_assert(KSPLIT == 1 || (KSPLIT == 2 && WAVES <= 4), "at most eight wavefronts per workgroup");
  static_assert(!INDEXED || KSPLIT == 1, "tile lists are not split");
  static_assert(!(GENERAL || CAPTURE) || (WAVES == 8 && KSPLIT == 1), "masks and capture: 128-query workgroups");
  static_assert(GENERAL || MASK_DT < 0, "the raw-score path takes no mask");
  static_assert(!(CAPTURE && INDEXED), "statistics are captured on dense runs");
  constexpr bool TENSOR_MASK = MASK_DT >= 0 && MASK_DT != kKeyBias;
  constexpr int QUERIES = 16 * WAVES;
  using Shape = NarrowTileShape<D, CTA_K, MASK_DT>;
  constexpr int KB = CTA_K / 16;  // 16-key blocks per tile
  constexpr int SB = CTA_K / 64;  // 64-key steps of the P·V product
  constexpr int CB = D / 16;      // 16-channel blocks
  constexpr int KK = D / 64;      // 64-channel steps of the score product
  constexpr int COPIES = Shape::kTileBytes / 1024;  // 1 KB copy instructions per operand tile
  constexpr int NC = (COPIES + WAVES - 1) / WAVES;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_all[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int workgroup_wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int part = workgroup_wave / WAVES;  // which half of the key tiles (0 when KSPLIT == 1)
  const int wave = workgroup_wave % WAVES;  // which sixteen queries
  const int ql = lane & 15, grp = lane >> 4;
  unsigned char* lds = lds_all + part * Shape::kLdsBytes;

  const int query_blocks = (p.q_len + QUERIES - 1) / QUERIES;
  int bx, head, batch;
  if (GENERAL && p.causal) {
    // longest query blocks first, across all heads (as in the wide kernel)
    const int heads = p.q_heads * p.batch;
    const int rest = blockIdx.x % heads;
    bx = query_blocks - 1 - blockIdx.x / heads;
    head = rest % p.q_heads;
    batch = rest / p.q_heads;
  } else {
    bx = blockIdx.x % query_blocks;
    const int rest = blockIdx.x / query_blocks;
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

  const int query = bx * QUERIES + wave * 16 + ql;
  const bool query_ok = query < p.q_len;
  // KSPLIT == 2: the second part takes the last floor(n/2) tiles, the first part the rest.
  const int second_half = p.n_kb / 2;
  int n_it = KSPLIT == 1 ? p.n_kb : part == 0 ? p.n_kb - second_half : second_half;
  const int first_tile = part == 0 ? 0 : p.n_kb - second_half;
  [[maybe_unused]] const int32_t* indices = nullptr;
  if constexpr (INDEXED) {
    if (p.index_mode == 1) {
      const int64_t row = bhq * p.n_qb + (bx * QUERIES) / kQueryBlock;
      const int start = p.row_offsets[row];
      n_it = __builtin_amdgcn_readfirstlane(p.row_offsets[row + 1] - start);
      indices = p.tile_indices + start;
    } else {
      indices = p.tile_indices + bhq * (p.n_kb + 1);
      n_it = __builtin_amdgcn_readfirstlane(indices[p.n_kb]);
    }
  } else if constexpr (GENERAL && !CAPTURE) {
    if (p.causal) {
      const int limit = min(p.k_len, (bx + 1) * QUERIES);
      n_it = (limit + CTA_K - 1) / CTA_K;
    }
  }
  // listed tiles come through the scalar cache (uniform address; as vector loads their wait
  // would include every vector load requested before them)
  auto tile_at = [&](int step) -> int {
    if constexpr (INDEXED) {
      typedef const __attribute__((address_space(4))) int32_t* UniformEntries;
      return ((UniformEntries)(reinterpret_cast<uintptr_t>(indices)))[step];
    }
    return first_tile + step;
  };

  // --- copies HBM/L2 -> LDS ---------------------------------------------------------
  // Copy instruction (wave*NC + i) fills LDS bytes [(wave*NC + i)*1024, +1024) of a
  // tile; this lane supplies chunk `lane` of that kilobyte.
  uint32_t k_src_offset[NC], v_src_offset[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int slot = (wave * NC + i) * 64 + lane;
    {
      constexpr int CH = D / 16;
      const int row = slot / CH, phys = slot % CH;
      k_src_offset[i] = row * D + ((phys ^ narrow_key_swizzle<D>(row)) << 4);
    }
    {
      constexpr int CH = CTA_K / 16;
      const int row = slot / CH, phys = slot % CH;
      const int chunk = phys ^ ((row / (256 / CTA_K)) & (CH - 1));
      v_src_offset[i] = static_cast<uint32_t>(row) * static_cast<uint32_t>(p.padded) + chunk * 16;
    }
  }
  // The tail tile re-reads row 0 for keys past the end; those scores are masked by
  // index.  The last two wavefronts add one copy each: the accumulator seeds and the
  // four K scales of the tile.
  const bool copies_tiles = wave * NC < COPIES;
  auto issue_tile = [&](int tile, int stage) {
    unsigned char* k_slot = lds + stage * Shape::kStageBytes + wave * (NC * 1024);
    unsigned char* v_slot = k_slot + Shape::kTileBytes;
    unsigned char* sl = lds + stage * Shape::kStageBytes + 2 * Shape::kTileBytes;
    const int8_t* k_tile = k_base + static_cast<int64_t>(tile) * CTA_K * D;
    const int8_t* v_tile = v_base + static_cast<int64_t>(tile) * CTA_K;
    const int keys_left = p.k_len - tile * CTA_K;
    if (copies_tiles) {
      if (keys_left >= CTA_K) {
#pragma unroll
        for (int i = 0; i < NC; ++i) copy16_to_lds_uniform(k_tile, k_src_offset[i], k_slot + i * 1024);
      } else {
        const uint32_t bytes_left = static_cast<uint32_t>(keys_left) * D;
#pragma unroll
        for (int i = 0; i < NC; ++i) {
          const uint32_t offset = k_src_offset[i] < bytes_left ? k_src_offset[i] : (k_src_offset[i] & (D - 1));
          copy16_to_lds_uniform(k_tile, offset, k_slot + i * 1024);
        }
      }
#pragma unroll
      for (int i = 0; i < NC; ++i) copy16_to_lds_uniform(v_tile, v_src_offset[i], v_slot + i * 1024);
    }
    if (wave == WAVES - 1) {
      if (lane < D / 4) {
        copy16_to_lds_uniform(reinterpret_cast<const int8_t*>(sum_base + static_cast<int64_t>(tile) * D),
                              static_cast<uint32_t>(lane) * 16, sl);
      }
    } else if (wave == WAVES - 2) {
      if (lane == 0) {
        copy16_to_lds_uniform(reinterpret_cast<const int8_t*>(ks_base + static_cast<int64_t>(tile) * 4), 0u,
                              sl + Shape::kSeedBytes);
      }
    }
    if constexpr (MASK_DT == kKeyBias) {
      if (wave == WAVES - 3 && lane < CTA_K / 4) {
        copy16_to_lds_uniform(reinterpret_cast<const int8_t*>(bias_base + static_cast<int64_t>(tile) * CTA_K),
                              static_cast<uint32_t>(lane) * 16, lds + stage * Shape::kStageBytes + Shape::kMaskOffset);
      }
    }
  };
  // Read as a plain vector type: the compiler orders LDS reads it cannot classify
  // behind every outstanding copy into LDS, i.e. behind the next tile.
  auto tile_scales = [&](int stage, float& ks0, float& ks1) {
    typedef float v2f __attribute__((ext_vector_type(2)));
    const v2f pair = *reinterpret_cast<const v2f*>(lds + stage * Shape::kStageBytes + 2 * Shape::kTileBytes +
                                                   Shape::kSeedBytes + 8 * (grp & 1));
    ks0 = pair[0];
    ks1 = pair[1];
  };

  // --- Q operand and scales ----------------------------------------------------------
  v4i qreg[KK];
  {
    const int8_t* q_row = p.q + (bhq * p.q_len + query) * D;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      qreg[kk] = query_ok ? *reinterpret_cast<const v4i*>(q_row + kk * 64 + grp * 16) : v4i{0, 0, 0, 0};
    }
  }
  constexpr int W = D == 256 ? 16 : 32;
  const int q_groups = (p.q_len + 127) / 128 * (128 / W) * 8;
  const float q_scale = query_ok ? p.q_scale[bhq * q_groups + (query / W) * 8 + (query & 7)] : 1.0f;
  const float qs2 = p.sm2;

  float o_acc[CB][4];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int i = 0; i < 4; ++i) o_acc[cb][i] = 0.0f;
  float m_run = kRowFloor;
  float d_part = 0.0f;  // this lane's quarter of the row denominator
  float seed_value;
  asm volatile("v_mov_b32 %0, %1" : "=v"(seed_value) : "s"(kAccumulatorSeedBits));

  // capture bookkeeping (layout of the wide kernel)
  [[maybe_unused]] uint32_t* stats = nullptr;
  [[maybe_unused]] uint64_t full_words = 0;
  [[maybe_unused]] uint64_t stat_row = 0;
  if constexpr (CAPTURE) {
    const uint64_t mass_elements = static_cast<uint64_t>(p.batch) * p.q_heads * p.n_qb * p.n_kb;
    stats = reinterpret_cast<uint32_t*>(p.workspace + mass_elements);
    full_words = static_cast<uint64_t>(p.batch) * p.q_heads * p.q_len * (p.n_kb - 1) * 2;
    stat_row = static_cast<uint64_t>(bhq) * p.q_len + query;
  }
  [[maybe_unused]] const int64_t mask_row =
      TENSOR_MASK ? static_cast<int64_t>(batch) * p.mask_stride_b + static_cast<int64_t>(head) * p.mask_stride_h +
                        static_cast<int64_t>(query) * p.mask_stride_q
                  : 0;

  // Mask elements of a full tile, requested before the next tile's copies: vector memory
  // operations complete in order, so a mask load issued behind the copies could only be
  // used once they have landed.  For masks that allow one load per four keys, with 64-key
  // tiles (the tile of every query-dependent mask); other mask tensors are read inside the
  // softmax and the next tile's copies are requested after it instead.
  constexpr bool PRELOAD = TENSOR_MASK && MASK_VEC && CTA_K == 64;
  constexpr bool LATE_COPIES = TENSOR_MASK && !PRELOAD;
  constexpr int WORDS = MASK_DT == kF32 ? 4 : MASK_DT == kBool ? 1 : 2;  // 32-bit words per four keys
  [[maybe_unused]] uint32_t mask_words[PRELOAD ? KB * WORDS : 1];
  auto load_mask_words = [&](int tile) {
    if constexpr (PRELOAD) {
      constexpr int ES = MASK_DT == kF32 ? 4 : MASK_DT == kBool ? 1 : 2;
      // rows past the last query read the last row; their results are never stored
      const int64_t row = mask_row - static_cast<int64_t>(query_ok ? 0 : query - (p.q_len - 1)) * p.mask_stride_q;
      const unsigned char* base = static_cast<const unsigned char*>(p.mask) +
                                  (row + tile * CTA_K + 32 * (grp >> 1) + 4 * (grp & 1)) * ES;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const unsigned char* at = base + ((kb >> 2) * 64 + (kb & 3) * 8) * ES;
        uint32_t* words = mask_words + kb * WORDS;
        if constexpr (WORDS == 1) {
          words[0] = *reinterpret_cast<const uint32_t*>(at);
        } else if constexpr (WORDS == 2) {
          typedef uint32_t v2u __attribute__((ext_vector_type(2)));
          const v2u w = *reinterpret_cast<const v2u*>(at);
          words[0] = w[0], words[1] = w[1];
        } else {
          typedef uint32_t v4u __attribute__((ext_vector_type(4)));
          const v4u w = *reinterpret_cast<const v4u*>(at);
          words[0] = w[0], words[1] = w[1], words[2] = w[2], words[3] = w[3];
        }
      }
    }
  };

  // ---- S^T = K · Q^T ------------------------------------------------------------------
  const int key_row = 32 * (ql >> 3) + (ql & 7);  // row of this lane inside block (s, b): + 64*s + 8*b
  auto load_k_fragments = [&](const unsigned char* kl, int kk, v4i (&frag)[KB]) {
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int row = (kb >> 2) * 64 + (kb & 3) * 8 + key_row;
      frag[kb] = *reinterpret_cast<const v4i*>(
          kl + row * D + (((kk * 4 + grp) ^ narrow_key_swizzle<D>(row)) << 4));
    }
  };
  auto score_tile = [&](int stage, v4i (&first)[KB], v4i (&s)[KB]) {
    const unsigned char* kl = lds + stage * Shape::kStageBytes;
    v4i frag[2][KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) frag[0][kb] = first[kb];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) load_k_fragments(kl, kk + 1, frag[(kk + 1) & 1]);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        if (kk == 0) {
          // seeded like the wide kernel's scores (kScoreSeedBits)
          const v4i seed = {kScoreSeedBits, kScoreSeedBits, kScoreSeedBits, kScoreSeedBits};
          s[kb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(frag[kk & 1][kb], qreg[kk], seed, 0, 0, 0);
        } else {
          s[kb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(frag[kk & 1][kb], qreg[kk], s[kb], 0, 0, 0);
        }
      }
    }
  };

  // ---- scores -> U8 probabilities (as signed bytes) and the online-softmax state ------
  // Element (kb, i) is key tile*CTA_K + (kb/4)*64 + 32*(grp/2) + (kb%4)*8 + 4*(grp%2) + i,
  // K scale group (key % 8) / 2 = 2*(grp%2) + i/2.
  constexpr float kRescaleSlack = 8.0f;
  auto softmax_tile = [&](auto last_tag, int it, int tile, float ks0, float ks1, v4i (&s)[KB], v4i (&pk)[SB]) -> float {
    constexpr bool LAST = decltype(last_tag)::value;
    const float sc0 = qs2 * (q_scale * ks0);
    const float sc1 = qs2 * (q_scale * ks1);
    float tile_m;
    uint32_t row_sum = 0;
    if constexpr (GENERAL) {
      // Pre-scaled scores with masks: the decisions and the arithmetic per score of the wide
      // kernel.  Whether a tile needs any masking is uniform over the wavefront.
      const float neg_inf = -__builtin_inff();
      const int first_query = bx * QUERIES + wave * 16;
      const bool on_diagonal = p.causal && tile * CTA_K + CTA_K - 1 > first_query;
      const bool partial = LAST && (tile + 1) * CTA_K > p.k_len;
      const int key0 = tile * CTA_K + 32 * (grp >> 1) + 4 * (grp & 1);
      float mx = kRowFloor;
      // (a key-only mask whose additive row is zero over this whole tile changes nothing in it:
      // as in the wide kernel, one LDS read per wavefront and tile decides)
      [[maybe_unused]] bool zero_row = false;
      if constexpr (MASK_DT == kKeyBias) {
        if (!on_diagonal && !partial) {
          const int* whole_row = reinterpret_cast<const int*>(lds + (it & 1) * Shape::kStageBytes + Shape::kMaskOffset);
          const v4i probe = *reinterpret_cast<const v4i*>(whole_row + (lane & (CTA_K / 4 - 1)) * 4);
          const bool nonzero = (static_cast<uint32_t>(probe[0] | probe[1] | probe[2] | probe[3]) << 1) != 0;
          zero_row = __builtin_amdgcn_ballot_w64(nonzero) == 0;
        }
      }
      if ((MASK_DT < 0 || zero_row) && !on_diagonal && !partial) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float value = score_value(s[kb][i]) * ((i & 2) ? sc1 : sc0);
            s[kb][i] = __float_as_int(value);
            mx = __builtin_fmaxf(mx, value);
          }
      } else {
        auto masked_scores = [&](auto diagonal_tag) {
          constexpr bool DIAGONAL = decltype(diagonal_tag)::value;
          constexpr int ES = MASK_DT == kF32 ? 4 : MASK_DT == kBool ? 1 : 2;
          [[maybe_unused]] const unsigned char* lane_mask = nullptr;
          if constexpr (TENSOR_MASK) {
            lane_mask = static_cast<const unsigned char*>(p.mask) +
                        (mask_row + static_cast<int64_t>(key0) * p.mask_stride_k) * ES;
          }
          [[maybe_unused]] const float* bias_row = nullptr;
          if constexpr (MASK_DT == kKeyBias) {
            bias_row = reinterpret_cast<const float*>(lds + (it & 1) * Shape::kStageBytes + Shape::kMaskOffset) +
                       32 * (grp >> 1) + 4 * (grp & 1);
          }
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            const int local = (kb >> 2) * 64 + (kb & 3) * 8;  // first of this lane's four consecutive keys
            const int key = key0 + local;
            bool keep[4] = {true, true, true, true};
            float bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (MASK_DT == kKeyBias) {
              const v4f terms = *reinterpret_cast<const v4f*>(bias_row + local);
              bias[0] = terms[0], bias[1] = terms[1], bias[2] = terms[2], bias[3] = terms[3];
            } else if constexpr (PRELOAD && !LAST) {
              const uint32_t* words = mask_words + kb * WORDS;
              if constexpr (MASK_DT == kBool) {
#pragma unroll
                for (int r = 0; r < 4; ++r) keep[r] = ((words[0] >> (8 * r)) & 0xffu) != 0;
              } else if constexpr (MASK_DT == kF32) {
#pragma unroll
                for (int r = 0; r < 4; ++r) bias[r] = __uint_as_float(words[r]);
              } else {
                const uint32_t bits16[4] = {words[0] & 0xffffu, words[0] >> 16, words[1] & 0xffffu, words[1] >> 16};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                  bias[r] = MASK_DT == kF16 ? static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16[r])))
                                            : __uint_as_float(bits16[r] << 16);
                }
              }
              if constexpr (MASK_DT != kBool) {
#pragma unroll
                for (int r = 0; r < 4; ++r) keep[r] = __builtin_isfinite(bias[r]);
              }
            } else if constexpr (TENSOR_MASK) {
              if (!query_ok) {
#pragma unroll
                for (int r = 0; r < 4; ++r) keep[r] = false;
              } else if (MASK_VEC && key + 3 < p.k_len) {
                const unsigned char* at = lane_mask + local * ES;
                if constexpr (MASK_DT == kBool) {
                  const uint32_t word = *reinterpret_cast<const uint32_t*>(at);
#pragma unroll
                  for (int r = 0; r < 4; ++r) keep[r] = ((word >> (8 * r)) & 0xffu) != 0;
                } else if constexpr (MASK_DT == kF32) {
                  const v4f w = *reinterpret_cast<const v4f*>(at);
                  bias[0] = w[0], bias[1] = w[1], bias[2] = w[2], bias[3] = w[3];
                } else {
                  typedef uint32_t v2u __attribute__((ext_vector_type(2)));
                  const v2u w = *reinterpret_cast<const v2u*>(at);
                  const uint32_t bits16[4] = {w[0] & 0xffffu, w[0] >> 16, w[1] & 0xffffu, w[1] >> 16};
#pragma unroll
                  for (int r = 0; r < 4; ++r) {
                    bias[r] = MASK_DT == kF16 ? static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16[r])))
                                              : __uint_as_float(bits16[r] << 16);
                  }
                }
              } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                  keep[r] = key + r < p.k_len;
                  if (keep[r]) {
                    const unsigned char* at = lane_mask + (local + r) * p.mask_stride_k * ES;
                    if constexpr (MASK_DT == kBool) {
                      keep[r] = *at != 0;
                    } else {
                      bias[r] = load1<MASK_DT>(at, 0);
                    }
                  }
                }
              }
              if constexpr (MASK_DT != kBool) {
#pragma unroll
                for (int r = 0; r < 4; ++r) keep[r] = keep[r] && __builtin_isfinite(bias[r]);
              }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float value = score_value(s[kb][r]) * ((r & 2) ? sc1 : sc0);
              if constexpr (MASK_DT == kKeyBias) {
                value += bias[r];
              } else if constexpr (MASK_DT == kBool) {
                value = keep[r] ? value : neg_inf;
              } else if constexpr (TENSOR_MASK) {
                value = keep[r] ? value + bias[r] * kLog2e : neg_inf;
              }
              if constexpr (DIAGONAL) {
                if (key + r > query) value = neg_inf;
              }
              if constexpr (MASK_DT != kKeyBias) {
                if (LAST && key + r >= p.k_len) value = neg_inf;
              }
              s[kb][r] = __float_as_int(value);
              mx = __builtin_fmaxf(mx, value);
            }
          }
        };
        if (on_diagonal) {
          masked_scores(std::true_type{});
        } else {
          masked_scores(std::false_type{});
        }
      }
      tile_m = mx - kU8Offset;
    } else if constexpr (!LAST) {
      int mx0 = s[0][0], mx1 = s[0][2];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (i & 2)
            mx1 = max(mx1, s[kb][i]);
          else
            mx0 = max(mx0, s[kb][i]);
        }
      tile_m = __builtin_fmaxf(__builtin_fmaf(score_value(mx0), sc0, -kU8Offset),
                               __builtin_fmaf(score_value(mx1), sc1, -kU8Offset));
    } else if ((tile + 1) * CTA_K <= p.k_len) {
      // Last listed tile with all of its keys in range: the values of the formulas below from
      // the maxima of the seeded integers (the conversion is exact and monotone, the floor of
      // -50000 becomes a clamp of the converted maximum).
      int mx0 = s[0][0], mx1 = s[0][2];
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (i & 2)
            mx1 = max(mx1, s[kb][i]);
          else
            mx0 = max(mx0, s[kb][i]);
          s[kb][i] = __float_as_int(score_value(s[kb][i]));
        }
      tile_m = __builtin_fmaxf(__builtin_fmaf(__builtin_fmaxf(kRowFloor, score_value(mx0)), sc0, -kU8Offset),
                               __builtin_fmaf(__builtin_fmaxf(kRowFloor, score_value(mx1)), sc1, -kU8Offset));
    } else {
      // Last tile: out-of-range keys become -1e30 and every scale group's maximum
      // starts from -50000 before scaling.
      const int key0 = tile * CTA_K + 32 * (grp >> 1) + 4 * (grp & 1);
      float mx0 = kRowFloor, mx1 = kRowFloor;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = key0 + (kb >> 2) * 64 + (kb & 3) * 8 + i;
          const float raw = key < p.k_len ? score_value(s[kb][i]) : -1.0e30f;
          s[kb][i] = __float_as_int(raw);
          if (i & 2)
            mx1 = __builtin_fmaxf(mx1, raw);
          else
            mx0 = __builtin_fmaxf(mx0, raw);
        }
      tile_m = __builtin_fmaxf(__builtin_fmaf(mx0, sc0, -kU8Offset), __builtin_fmaf(mx1, sc1, -kU8Offset));
    }
    tile_m = max_across_halves(max_across_row_pairs(tile_m));
    const float neg_m = -tile_m;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      uint32_t packed = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float x;
        if constexpr (GENERAL) {
          x = __int_as_float(s[kb][i]) - tile_m;
        } else {
          const float raw = LAST ? __int_as_float(s[kb][i]) : score_value(s[kb][i]);
          x = __builtin_fmaf(raw, (i & 2) ? sc1 : sc0, neg_m);
        }
        packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_exp2f(x), i, packed);
      }
      row_sum = __builtin_amdgcn_udot4(packed, 0x01010101u, row_sum, false);
      pk[kb >> 2][kb & 3] = static_cast<int>(packed ^ 0x80808080u);
    }

    // The running reference only moves when a tile maximum exceeds it by more than
    // kRescaleSlack (the same deferred rescaling as the wide kernel).
    const bool raise = tile_m > m_run + kRescaleSlack;
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float o_scale = raise ? __builtin_amdgcn_exp2f(m_run - tile_m) : 1.0f;
      m_run = raise ? tile_m : m_run;
      d_part *= o_scale;
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) o_acc[cb][i] *= o_scale;
    }
    const float t_scale = __builtin_amdgcn_exp2f(tile_m - m_run);
    d_part = __builtin_fmaf(static_cast<float>(row_sum), t_scale, d_part);
    if constexpr (CAPTURE) {
      const uint32_t numerator = sum_across_halves(sum_across_row_pairs(row_sum));
      if (grp == 0 && query_ok) {
        if constexpr (!LAST) {
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

  // ---- O^T += t_scale * (128*sum(V) + V^T · P_s8^T) -------------------------------------
  // Channel blocks go through in groups of four independent accumulator chains; the
  // seeds and V fragments of the next group are requested before this group's MFMAs.
  constexpr int GROUP = 4;
  constexpr int NG = CB / GROUP;
  constexpr int SETS = NG > 2 ? 3 : 2;
  auto load_group = [&](int stage, int g, v4i (&acc)[GROUP], v4i (&frag)[GROUP][SB]) {
    const unsigned char* vl = lds + stage * Shape::kStageBytes + Shape::kTileBytes;
    const int* sl = reinterpret_cast<const int*>(lds + stage * Shape::kStageBytes + 2 * Shape::kTileBytes);
#pragma unroll
    for (int j = 0; j < GROUP; ++j) {
      const int cb = g * GROUP + j;
      acc[j] = *reinterpret_cast<const v4i*>(sl + cb * 16 + grp * 4);
#pragma unroll
      for (int sb = 0; sb < SB; ++sb)
        frag[j][sb] = *reinterpret_cast<const v4i*>(vl + swizzled<CTA_K>(cb * 16 + ql, sb * 4 + grp));
    }
  };
  auto unseed = [&](int bits) { return __int_as_float(bits) - seed_value; };
  auto fold_group = [&](int g, const v4i (&acc)[GROUP], float t_scale) {
#pragma unroll
    for (int j = 0; j < GROUP; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o_acc[g * GROUP + j][i] = __builtin_fmaf(unseed(acc[j][i]), t_scale, o_acc[g * GROUP + j][i]);
  };
  auto value_tile = [&](int stage, const v4i (&pk)[SB], v4i (&acc0)[GROUP], v4i (&frag0)[GROUP][SB], float t_scale) {
    v4i acc[SETS][GROUP];
    v4i frag[2][GROUP][SB];
#pragma unroll
    for (int j = 0; j < GROUP; ++j) {
      acc[0][j] = acc0[j];
#pragma unroll
      for (int sb = 0; sb < SB; ++sb) frag[0][j][sb] = frag0[j][sb];
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (g + 1 < NG) load_group(stage, g + 1, acc[(g + 1) % SETS], frag[(g + 1) & 1]);
#pragma unroll
      for (int sb = 0; sb < SB; ++sb)
#pragma unroll
        for (int j = 0; j < GROUP; ++j)
          acc[g % SETS][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(frag[g & 1][j][sb], pk[sb], acc[g % SETS][j], 0, 0, 0);
      if (g > 0) fold_group(g - 1, acc[(g - 1) % SETS], t_scale);
    }
    fold_group(NG - 1, acc[(NG - 1) % SETS], t_scale);
  };

  // --- main loop: one barrier per tile ---------------------------------------------------
  // At the barrier of iteration t every wave has finished tile t-1 (so stage (t+1)&1
  // may be overwritten) and has seen its own share of tile t land.  A deeper pipeline
  // (four stages, counted waits) was measured and gains nothing: the tile time is set
  // by the dependent chain barrier -> LDS -> MFMA -> row maximum -> exp2 -> MFMA.
  if (n_it > 0) {
    v4i s[KB];
    v4i pk[SB];
    v4i k_first[KB];
    v4i acc_first[GROUP];
    v4i v_first[GROUP][SB];
    float ks0, ks1;
    int tile = tile_at(0);
    issue_tile(tile, 0);
    // Listed tiles: the entry after the next one is requested a whole tile before it is
    // needed, ahead of the copies (its round trip would otherwise be waited for in every tile).
    [[maybe_unused]] int listed_next = INDEXED && n_it > 1 ? tile_at(1) : 0;
    for (int step = 0; step < n_it - 1; ++step) {
      const int stage = step & 1;
      const int next_tile = INDEXED ? listed_next : tile_at(step + 1);
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      [[maybe_unused]] int listed_after_next = 0;
      if constexpr (INDEXED) listed_after_next = indices[min(step + 2, n_it - 1)];
      load_k_fragments(lds + stage * Shape::kStageBytes, 0, k_first);
      tile_scales(stage, ks0, ks1);
      if constexpr (PRELOAD) {
        load_mask_words(tile);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (!LATE_COPIES) issue_tile(next_tile, stage ^ 1);
      __builtin_amdgcn_s_setprio(0);  // vector phases before matrix phases, as in the wide kernel
      score_tile(stage, k_first, s);
      load_group(stage, 0, acc_first, v_first);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(2);
      const float t_scale = softmax_tile(std::false_type{}, step, tile, ks0, ks1, s, pk);
      __builtin_amdgcn_s_setprio(1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (LATE_COPIES) {
        issue_tile(next_tile, stage ^ 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      value_tile(stage, pk, acc_first, v_first, t_scale);
      tile = next_tile;
      if constexpr (INDEXED) listed_next = __builtin_amdgcn_readfirstlane(listed_after_next);
    }
    const int stage = (n_it - 1) & 1;
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    load_k_fragments(lds + stage * Shape::kStageBytes, 0, k_first);
    tile_scales(stage, ks0, ks1);
    score_tile(stage, k_first, s);
    // Only the last tile of the sequence takes the last-tile formulas.
    float t_scale;
    if (KSPLIT == 1 || part == KSPLIT - 1) {
      t_scale = softmax_tile(std::true_type{}, n_it - 1, tile, ks0, ks1, s, pk);
    } else {
      t_scale = softmax_tile(std::false_type{}, n_it - 1, tile, ks0, ks1, s, pk);
    }
    load_group(stage, 0, acc_first, v_first);
    value_tile(stage, pk, acc_first, v_first, t_scale);
  }

  if constexpr (KSPLIT == 2) {
    // Both parts share the workgroup's barrier: with an odd tile count the second part has
    // walked one tile less and takes the barrier of the tile it does not have.
    if (part == 1 && (p.n_kb & 1)) __syncthreads();
  }

  // ---- merge of the two key halves ----------------------------------------------------------
  // Part 1 leaves (O, m, d) of every lane in LDS, value-major so that lanes are
  // contiguous; the wavefront of part 0 with the same queries folds them in.
  if constexpr (KSPLIT == 2) {
    constexpr int VALUES = CB * 4 + 2;
    __syncthreads();  // every wavefront is done with its stages
    float* exchange = reinterpret_cast<float*>(lds_all) + wave * (VALUES * 64) + lane;
    if (part == 1) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) exchange[(cb * 4 + i) * 64] = o_acc[cb][i];
      exchange[(CB * 4) * 64] = m_run;
      exchange[(CB * 4 + 1) * 64] = d_part;
    }
    __syncthreads();
    if (part == 1) return;
    const float other_m = exchange[(CB * 4) * 64];
    const float other_d = exchange[(CB * 4 + 1) * 64];
    const float merged_m = __builtin_fmaxf(m_run, other_m);
    const float mine = __builtin_amdgcn_exp2f(m_run - merged_m);
    const float theirs = __builtin_amdgcn_exp2f(other_m - merged_m);
    d_part = __builtin_fmaf(other_d, theirs, d_part * mine);
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o_acc[cb][i] = __builtin_fmaf(exchange[(cb * 4 + i) * 64], theirs, o_acc[cb][i] * mine);
    m_run = merged_m;
  }

  // ---- epilogue ---------------------------------------------------------------------------
  float d_total = d_part + __shfl_xor(d_part, 16);
  d_total += __shfl_xor(d_total, 32);
  if constexpr (CAPTURE) {
    if (grp == 0 && query_ok) {
      const uint64_t query_rows = static_cast<uint64_t>(p.batch) * p.q_heads * p.q_len;
      float* state = reinterpret_cast<float*>(stats + full_words + query_rows * 2);
      state[stat_row * 2] = m_run;
      state[stat_row * 2 + 1] = d_total;
    }
  }
  const float inv_d = 1.0f / d_total;
  // rows without any visible key (masks, causal): zeros
  const bool zero_row = GENERAL && (MASK_DT >= 0 || p.causal) && !(d_total > 0.0f);
  // A lane owns one query and four channels per 16-channel block: stored from there, an
  // instruction would write 32 bytes into each of 16 rows.  Two blocks are exchanged between
  // neighbouring rows of lanes first (v_permlane16_swap: the odd rows of one register for the
  // even rows of the other), after which a lane holds eight consecutive channels and an
  // instruction writes 64 contiguous bytes of each row.  (The four lanes of a query are
  // active or inactive together, so the exchange stays inside the branch.)
  if (query_ok) {
    const float* vs = p.v_scale + bhk * D;
    const float* vc = p.v_center + bhk * D;
    unsigned char* out_row = static_cast<unsigned char*>(p.out) +
                             2 * (batch * p.out_stride_b + head * p.out_stride_h +
                                  static_cast<int64_t>(query) * p.out_stride_n);
#pragma unroll
    for (int cb = 0; cb < CB; cb += 2) {
      uint32_t word[2][2];  // [block of the pair][channel pair]
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int c = (cb + j) * 16 + grp * 4;
        const v4f scale4 = *reinterpret_cast<const v4f*>(vs + c);
        const v4f center4 = *reinterpret_cast<const v4f*>(vc + c);
        float value[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          value[r] = __builtin_fmaf(o_acc[cb + j][r] * inv_d, scale4[r], center4[r]);
          value[r] = zero_row ? 0.0f : value[r];
        }
        word[j][0] = to_output_pair(value[0], value[1], p.out_dtype);
        word[j][1] = to_output_pair(value[2], value[3], p.out_dtype);
      }
      // even rows of lanes end with channels 8*(grp/2) .. +7 of the first block, odd rows
      // with the same channels of the second block
      const auto low = __builtin_amdgcn_permlane16_swap(word[0][0], word[1][0], false, false);
      const auto high = __builtin_amdgcn_permlane16_swap(word[0][1], word[1][1], false, false);
      const v4i piece = {static_cast<int>(low[0]), static_cast<int>(high[0]), static_cast<int>(low[1]),
                         static_cast<int>(high[1])};
      *reinterpret_cast<v4i*>(out_row + (cb + (grp & 1)) * 32 + (grp >> 1) * 16) = piece;
    }
    if (p.lse != nullptr && grp == 0) {
      p.lse[bhq * p.q_len + query] =
          d_total > 0.0f ? (__builtin_amdgcn_logf(d_total) + m_run) / kLog2e : -__builtin_inff();
    }
  }
}

// Launch of one variant: grid of ceil(q_len / (16 * WAVES)) * heads * batch workgroups.
template <int D, int CTA_K, int WAVES, int KSPLIT, bool INDEXED = false, bool GENERAL = false,
          bool CAPTURE = false, int MASK_DT = -1, bool MASK_VEC = false>
int launch_narrow_block(const KernelParams& p, hipStream_t stream) {
  using Shape = NarrowTileShape<D, CTA_K, MASK_DT>;
  constexpr int kLdsBytes = Shape::kLdsBytes * KSPLIT;
  auto kernel = attention_narrow_kernel<D, CTA_K, WAVES, KSPLIT, INDEXED, GENERAL, CAPTURE, MASK_DT, MASK_VEC>;
  static thread_local int configured_device = -1;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return fail("risa_attention: hipGetDevice failed");
  if (device != configured_device) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess) {
      return fail("risa_attention: cannot reserve " + std::to_string(kLdsBytes) + " bytes of LDS");
    }
    configured_device = device;
  }
  constexpr int QUERIES = 16 * WAVES;
  const unsigned query_blocks = static_cast<unsigned>((p.q_len + QUERIES - 1) / QUERIES);
  const dim3 grid(query_blocks * p.q_heads * p.batch);
  kernel<<<grid, 64 * WAVES * KSPLIT, kLdsBytes, stream>>>(p);
  return 0;
}

}  // namespace risa
