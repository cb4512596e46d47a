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
//     The result is the exact integer the unsigned product would give.
#pragma once

#include "common.hpp"
#include "launchers.hpp"

#include <type_traits>

namespace risa {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kU8Offset = 7.9943534f;
constexpr float kRowFloor = -50000.0f;
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
  const int32_t* v_tile_sum;  // 128 * sum of V codes per (kv head, key tile, channel)
  const void* mask;
  int64_t mask_stride_b, mask_stride_h, mask_stride_q, mask_stride_k;
  int mask_dtype;  // -1: no mask
  int q_len, k_len, q_heads, kv_heads, padded, n_kb, n_qb, batch;
  int64_t out_stride_b, out_stride_n, out_stride_h;
  float sm2;  // sm_scale * log2(e)
  int out_dtype;
  const int32_t* row_offsets;   // sparse CSR (index_mode 1)
  const int32_t* tile_indices;  // sparse block indices (1) or key-mask tiles (2)
  int index_mode;
  float* workspace;  // capture
  float* lse;
  int causal;
};

// Byte offset of 16-byte chunk `chunk` of row `row` in a swizzled LDS tile.
template <int ROWBYTES> __device__ __forceinline__ int swizzled(int row, int chunk) {
  constexpr int CH = ROWBYTES / 16;
  constexpr int ROWS_PER_256 = 256 / ROWBYTES;
  return row * ROWBYTES + ((chunk ^ ((row / ROWS_PER_256) & (CH - 1))) << 4);
}

__device__ __forceinline__ uint16_t to_bf16_bits(float x) {
  uint32_t bits = __float_as_uint(x);
  const uint32_t rounded = bits + 0x7fffu + ((bits >> 16) & 1u);
  return static_cast<uint16_t>((x != x ? (bits | 0x400000u) : rounded) >> 16);
}
__device__ __forceinline__ uint16_t to_f16_bits(float x) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
}

// Copies 16 bytes per lane from global memory to LDS without touching VGPRs:
// lane l of the wavefront writes LDS bytes [lds_wave_base + 16*l, +16).
__device__ __forceinline__ void copy16_to_lds(const void* src, unsigned char* lds_wave_base) {
  typedef const __attribute__((address_space(1))) void* GlobalPointer;
  typedef __attribute__((address_space(3))) void* LdsPointer;
  __builtin_amdgcn_global_load_lds((GlobalPointer)src, (LdsPointer)lds_wave_base, 16, 0, 0);
}

template <int D, int CTA_K> struct TileShape {
  static constexpr int kTileBytes = CTA_K * D;
  static constexpr int kCopiesPerWave = kTileBytes / 16 / 256;  // 1 KB copy instructions per wave
  static constexpr int kStageBytes = 2 * kTileBytes + D * 4;     // K, V, zero-point terms
  static constexpr int kLdsBytes = 2 * kStageBytes;
};

template <int D, int CTA_K, bool FAST, bool INDEXED, bool CAPTURE>
__global__ __launch_bounds__(256, (D == 256 ? 1 : 2)) void attention_kernel(const KernelParams p) {
  using Shape = TileShape<D, CTA_K>;
  constexpr int RB = CTA_K / 32;  // 32-key blocks per tile
  constexpr int CB = D / 32;      // 32-channel blocks
  constexpr int KK = D / 32;      // k-steps of the score product
  constexpr int NC = Shape::kCopiesPerWave;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, half = lane >> 5;

  int block = blockIdx.x;
  const int bx = block % p.n_qb;
  block /= p.n_qb;
  const int head = block % p.q_heads;
  const int batch = block / p.q_heads;
  const int kv_head = head / (p.q_heads / p.kv_heads);
  const int64_t bhk = static_cast<int64_t>(batch) * p.kv_heads + kv_head;
  const int64_t bhq = static_cast<int64_t>(batch) * p.q_heads + head;

  const int8_t* k_base = p.k + bhk * p.k_len * D;
  const int8_t* v_base = p.v + bhk * D * p.padded;
  const int32_t* sum_base = p.v_tile_sum + bhk * p.n_kb * D;
  const float* ks_base = p.k_scale + bhk * p.n_kb * 4;

  const int query = bx * kQueryBlock + wave * 32 + l32;
  const bool query_ok = query < p.q_len;

  // --- tile list -----------------------------------------------------------
  int n_it;
  const int32_t* indices = nullptr;
  if constexpr (INDEXED) {
    if (p.index_mode == 1) {
      const int64_t row = bhq * p.n_qb + bx;
      const int start = p.row_offsets[row];
      n_it = p.row_offsets[row + 1] - start;
      indices = p.tile_indices + start;
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
  auto tile_at = [&](int it) -> int {
    if constexpr (INDEXED) return __builtin_amdgcn_readfirstlane(indices[it]);
    return it;
  };

  // --- per-lane copy descriptors (constant over tiles) -----------------------
  // Copy instruction i of this wave fills LDS bytes [(wave*NC+i)*1024, +1024) of
  // a tile; this lane supplies chunk `lane` of that kilobyte.
  int k_src_offset[NC];          // byte offset of the source chunk inside a K tile
  int k_row[NC];                 // key row inside the tile (for the tail predicate)
  const int8_t* v_src_row[NC];   // source pointer of the chunk for tile 0
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int slot = (wave * NC + i) * 64 + lane;
    {
      constexpr int CH = D / 16;
      const int row = slot / CH, phys = slot % CH;
      const int chunk = phys ^ ((row / (256 / D)) & (CH - 1));
      k_src_offset[i] = row * D + chunk * 16;
      k_row[i] = row;
    }
    {
      constexpr int CH = CTA_K / 16;
      const int row = slot / CH, phys = slot % CH;
      const int chunk = phys ^ ((row / (256 / CTA_K)) & (CH - 1));
      v_src_row[i] = v_base + static_cast<int64_t>(row) * p.padded + chunk * 16;
    }
  }
  auto issue_tile = [&](int tile, int stage) {
    unsigned char* kl = lds + stage * Shape::kStageBytes;
    unsigned char* vl = kl + Shape::kTileBytes;
    unsigned char* sl = vl + Shape::kTileBytes;
    const int8_t* k_tile = k_base + static_cast<int64_t>(tile) * CTA_K * D;
    const int rows_left = p.k_len - tile * CTA_K;  // >= CTA_K except for the tail tile
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      if (k_row[i] < rows_left) copy16_to_lds(k_tile + k_src_offset[i], kl + (wave * NC + i) * 1024);
    }
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      copy16_to_lds(v_src_row[i] + static_cast<int64_t>(tile) * CTA_K, vl + (wave * NC + i) * 1024);
    }
    if (wave == 0 && lane < D / 4) {
      copy16_to_lds(sum_base + static_cast<int64_t>(tile) * D + lane * 4, sl);
    }
  };

  // --- Q operand and scales ------------------------------------------------
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

  float o_acc[CB][16];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[cb][i] = 0.0f;
  float m_run = kRowFloor;
  float d_part = 0.0f;  // this lane's half of the row denominator

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
      (!FAST && p.mask_dtype >= 0)
          ? static_cast<int64_t>(batch) * p.mask_stride_b + static_cast<int64_t>(head) * p.mask_stride_h +
                static_cast<int64_t>(query) * p.mask_stride_q
          : 0;

  // One key tile.  LAST selects the formulas of the last listed tile.
  auto process_tile = [&](auto last_tag, int it, int tile, int stage, float ks0, float ks1) {
    constexpr bool LAST = decltype(last_tag)::value;
    const unsigned char* kl = lds + stage * Shape::kStageBytes;
    const unsigned char* vl = kl + Shape::kTileBytes;
    const int* sl = reinterpret_cast<const int*>(vl + Shape::kTileBytes);

    // ---- S^T = K · Q^T ----------------------------------------------------
    v16i s[RB];
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const v4i a = *reinterpret_cast<const v4i*>(kl + swizzled<D>(rb * 32 + l32, kk * 2 + half));
        if (kk == 0) {
          const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          s[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qreg[kk], zero, 0, 0, 0);
        } else {
          s[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, qreg[kk], s[rb], 0, 0, 0);
        }
      }
    }

    // K scale groups of this lane: keys 8b+4*half+r, group (key % 8) / 2 = 2*half + r/2.
    const float sc0 = qs2 * (q_scale * ks0);
    const float sc1 = qs2 * (q_scale * ks1);
    const int key0 = tile * CTA_K + half * 4;  // element (rb, i) is key key0 + rb*32 + (i>>2)*8 + (i&3)

    float tile_m;
    v4i pk[RB];
    uint32_t row_sum = 0;

    if constexpr (FAST && !LAST) {
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
      tile_m = __builtin_fmaxf(__builtin_fmaf(static_cast<float>(mx0), sc0, -kU8Offset),
                               __builtin_fmaf(static_cast<float>(mx1), sc1, -kU8Offset));
      tile_m = __builtin_fmaxf(tile_m, __shfl_xor(tile_m, 32));
      const float neg_m = -tile_m;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          uint32_t packed = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x = __builtin_fmaf(static_cast<float>(s[rb][b4 * 4 + r]), (r & 2) ? sc1 : sc0, neg_m);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_exp2f(x), r, packed);
          }
          row_sum = __builtin_amdgcn_udot4(packed, 0x01010101u, row_sum, false);
          pk[rb][b4] = static_cast<int>(packed ^ 0x80808080u);
        }
    } else if constexpr (FAST) {
      // Last listed tile of the raw-score path: out-of-range keys become -1e30
      // and every scale group's maximum starts from -50000 before scaling.
      float mx0 = kRowFloor, mx1 = kRowFloor;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + rb * 32 + (i >> 2) * 8 + (i & 3);
          const float raw = key < p.k_len ? static_cast<float>(s[rb][i]) : -1.0e30f;
          s[rb][i] = __float_as_int(raw);
          if (i & 2)
            mx1 = __builtin_fmaxf(mx1, raw);
          else
            mx0 = __builtin_fmaxf(mx0, raw);
        }
      tile_m = __builtin_fmaxf(__builtin_fmaf(mx0, sc0, -kU8Offset), __builtin_fmaf(mx1, sc1, -kU8Offset));
      tile_m = __builtin_fmaxf(tile_m, __shfl_xor(tile_m, 32));
      const float neg_m = -tile_m;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int b4 = 0; b4 < 4; ++b4) {
          uint32_t packed = 0;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float x = __builtin_fmaf(__int_as_float(s[rb][b4 * 4 + r]), (r & 2) ? sc1 : sc0, neg_m);
            packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_exp2f(x), r, packed);
          }
          row_sum = __builtin_amdgcn_udot4(packed, 0x01010101u, row_sum, false);
          pk[rb][b4] = static_cast<int>(packed ^ 0x80808080u);
        }
    } else {
      // Pre-scaled scores with masks.
      const float neg_inf = -__builtin_inff();
      float mx = kRowFloor;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + rb * 32 + (i >> 2) * 8 + (i & 3);
          float value = static_cast<float>(s[rb][i]) * ((i & 2) ? sc1 : sc0);
          if (p.mask_dtype >= 0) {
            bool keep = query_ok && key < p.k_len;
            float bias = 0.0f;
            if (keep) {
              const int64_t offset = mask_row + static_cast<int64_t>(key) * p.mask_stride_k;
              if (p.mask_dtype == kBool) {
                keep = static_cast<const uint8_t*>(p.mask)[offset] != 0;
              } else {
                bias = p.mask_dtype == kF32   ? load1<kF32>(p.mask, offset)
                       : p.mask_dtype == kF16 ? load1<kF16>(p.mask, offset)
                                              : load1<kBF16>(p.mask, offset);
                keep = __builtin_isfinite(bias);
              }
            }
            value = keep ? value + bias * kLog2e : neg_inf;
          }
          if (p.causal && key > query) value = neg_inf;
          if (LAST && key >= p.k_len) value = neg_inf;
          s[rb][i] = __float_as_int(value);
          mx = __builtin_fmaxf(mx, value);
        }
      tile_m = mx - kU8Offset;
      tile_m = __builtin_fmaxf(tile_m, __shfl_xor(tile_m, 32));
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
    const float alpha = __builtin_amdgcn_exp2f(-__builtin_fabsf(m_run - tile_m));
    const float o_scale = m_run < tile_m ? alpha : 1.0f;
    const float t_scale = tile_m < m_run ? alpha : 1.0f;
    m_run = __builtin_fmaxf(m_run, tile_m);
    d_part = d_part * o_scale + static_cast<float>(row_sum) * t_scale;

    if constexpr (CAPTURE) {
      const uint32_t numerator = row_sum + __shfl_xor(row_sum, 32);
      if (half == 0 && query_ok) {
        if constexpr (!LAST) {
          const uint64_t offset = (stat_row * (p.n_kb - 1) + it) * 2;
          stats[offset] = numerator;
          stats[offset + 1] = __float_as_uint(tile_m);
        } else {
          const uint64_t offset = full_words + stat_row * 2;
          stats[offset] = __float_as_uint(static_cast<float>(numerator));
          stats[offset + 1] = __float_as_uint(tile_m);
        }
      }
    }

    // Rescaling the output accumulators is the identity unless some row of this
    // wavefront raised its running maximum.
    if (__builtin_amdgcn_ballot_w64(o_scale != 1.0f) != 0) {
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[cb][i] *= o_scale;
    }

    // ---- O^T += V^T · P^T: two channel blocks in flight per step ------------
    auto load_init = [&](int cb) {
      v16i acc;
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const v4i init = *reinterpret_cast<const v4i*>(sl + cb * 32 + b4 * 8 + half * 4);
        acc[b4 * 4 + 0] = init[0];
        acc[b4 * 4 + 1] = init[1];
        acc[b4 * 4 + 2] = init[2];
        acc[b4 * 4 + 3] = init[3];
      }
      return acc;
    };
#pragma unroll
    for (int cb = 0; cb < CB; cb += 2) {
      v16i acc0 = load_init(cb);
      v16i acc1 = load_init(cb + 1);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const v4i a0 = *reinterpret_cast<const v4i*>(vl + swizzled<CTA_K>(cb * 32 + l32, rb * 2 + half));
        const v4i a1 = *reinterpret_cast<const v4i*>(vl + swizzled<CTA_K>(cb * 32 + 32 + l32, rb * 2 + half));
        acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, pk[rb], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, pk[rb], acc1, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        o_acc[cb][i] = __builtin_fmaf(static_cast<float>(acc0[i]), t_scale, o_acc[cb][i]);
        o_acc[cb + 1][i] = __builtin_fmaf(static_cast<float>(acc1[i]), t_scale, o_acc[cb + 1][i]);
      }
    }
  };

  // --- main loop --------------------------------------------------------------
  if (n_it > 0) {
    issue_tile(tile_at(0), 0);
    int tile = tile_at(0);
    float ks0 = ks_base[tile * 4 + 2 * half];
    float ks1 = ks_base[tile * 4 + 2 * half + 1];
    for (int it = 0; it < n_it - 1; ++it) {
      const int stage = it & 1;
      const int next_tile = tile_at(it + 1);
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of the tile has landed
      __syncthreads();
      issue_tile(next_tile, stage ^ 1);
      const float next_ks0 = ks_base[next_tile * 4 + 2 * half];
      const float next_ks1 = ks_base[next_tile * 4 + 2 * half + 1];
      process_tile(std::false_type{}, it, tile, stage, ks0, ks1);
      tile = next_tile;
      ks0 = next_ks0;
      ks1 = next_ks1;
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    process_tile(std::true_type{}, n_it - 1, tile, (n_it - 1) & 1, ks0, ks1);
  }

  // ---- epilogue --------------------------------------------------------------
  const float d_total = d_part + __shfl_xor(d_part, 32);
  if constexpr (CAPTURE) {
    if (half == 0 && query_ok) {
      const uint64_t query_rows = static_cast<uint64_t>(p.batch) * p.q_heads * p.q_len;
      float* state = reinterpret_cast<float*>(stats + full_words + query_rows * 2);
      state[stat_row * 2] = m_run;
      state[stat_row * 2 + 1] = d_total;
    }
  }
  const bool guard_empty = !FAST && (p.mask_dtype >= 0 || p.causal);
  const bool row_valid = d_total > 0.0f;
  const float inv_d = 1.0f / d_total;
  if (query_ok) {
    const float* vs = p.v_scale + bhk * D;
    const float* vc = p.v_center + bhk * D;
    unsigned char* out_row = static_cast<unsigned char*>(p.out) +
                             2 * (batch * p.out_stride_b + head * p.out_stride_h +
                                  static_cast<int64_t>(query) * p.out_stride_n);
    const bool zero_row = guard_empty && !row_valid;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int b4 = 0; b4 < 4; ++b4) {
        const int c = cb * 32 + b4 * 8 + half * 4;
        const float4 scale4 = *reinterpret_cast<const float4*>(vs + c);
        const float4 center4 = *reinterpret_cast<const float4*>(vc + c);
        float value[4];
        value[0] = __builtin_fmaf(o_acc[cb][b4 * 4 + 0] * inv_d, scale4.x, center4.x);
        value[1] = __builtin_fmaf(o_acc[cb][b4 * 4 + 1] * inv_d, scale4.y, center4.y);
        value[2] = __builtin_fmaf(o_acc[cb][b4 * 4 + 2] * inv_d, scale4.z, center4.z);
        value[3] = __builtin_fmaf(o_acc[cb][b4 * 4 + 3] * inv_d, scale4.w, center4.w);
        uint32_t bits[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float x = zero_row ? 0.0f : value[r];
          bits[r] = p.out_dtype == kF16 ? to_f16_bits(x) : to_bf16_bits(x);
        }
        uint2 word;
        word.x = bits[0] | (bits[1] << 16);
        word.y = bits[2] | (bits[3] << 16);
        *reinterpret_cast<uint2*>(out_row + 2 * c) = word;
      }
    if (p.lse != nullptr && half == 0) {
      p.lse[bhq * p.q_len + query] =
          row_valid ? (__builtin_amdgcn_logf(d_total) + m_run) / kLog2e : -__builtin_inff();
    }
  }
}

}  // namespace risa
