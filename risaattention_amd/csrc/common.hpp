// Shared device/host helpers for the gfx950 kernels of the quantized attention path.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>

namespace risa {

// ---------------------------------------------------------------------------
// Error reporting across the C boundary: entry points return 0 on success and
// a non-zero code otherwise; the message is kept per host thread.
// ---------------------------------------------------------------------------
inline std::string& last_error_storage() {
  static thread_local std::string message;
  return message;
}

inline int fail(const std::string& message) {
  last_error_storage() = message;
  return 1;
}

inline int check_launch(const char* what) {
  const hipError_t error = hipGetLastError();
  if (error != hipSuccess) {
    return fail(std::string(what) + " launch failed: " + hipGetErrorString(error));
  }
  return 0;
}

// dtype codes shared with the Python side: 0 = float32, 1 = float16,
// 2 = bfloat16, 3 = bool/uint8 (masks only).
constexpr int kF32 = 0;
constexpr int kF16 = 1;
constexpr int kBF16 = 2;
constexpr int kBool = 3;
// Kernel-internal mask kind: a key-only mask staged per tile as an FP32 bias row.
constexpr int kKeyBias = 4;

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Typed loads that widen to binary32 exactly.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits16) {
  const _Float16 value = __builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16));
  return static_cast<float>(value);
}

template <int DT> struct Element;
template <> struct Element<kF32> {
  using type = float;
  static constexpr int bytes = 4;
};
template <> struct Element<kF16> {
  using type = uint16_t;
  static constexpr int bytes = 2;
};
template <> struct Element<kBF16> {
  using type = uint16_t;
  static constexpr int bytes = 2;
};

// Four consecutive elements starting at element offset `offset` (which the
// callers keep a multiple of four elements and 4-element aligned in memory).
template <int DT>
__device__ __forceinline__ void load4(const void* base, int64_t offset, float out[4]) {
  if constexpr (DT == kF32) {
    const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + offset);
    out[0] = raw.x;
    out[1] = raw.y;
    out[2] = raw.z;
    out[3] = raw.w;
  } else {
    const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + offset);
    if constexpr (DT == kBF16) {
      out[0] = bf16_bits_to_float(raw.x & 0xffffu);
      out[1] = bf16_bits_to_float(raw.x >> 16);
      out[2] = bf16_bits_to_float(raw.y & 0xffffu);
      out[3] = bf16_bits_to_float(raw.y >> 16);
    } else {
      out[0] = f16_bits_to_float(raw.x & 0xffffu);
      out[1] = f16_bits_to_float(raw.x >> 16);
      out[2] = f16_bits_to_float(raw.y & 0xffffu);
      out[3] = f16_bits_to_float(raw.y >> 16);
    }
  }
}

// Eight consecutive elements (16-byte aligned for 16-bit types, 32 for fp32).
template <int DT>
__device__ __forceinline__ void load8(const void* base, int64_t offset, float out[8]) {
  if constexpr (DT == kF32) {
    load4<DT>(base, offset, out);
    load4<DT>(base, offset + 4, out + 4);
  } else {
    const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + offset);
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (DT == kBF16) {
        out[2 * i] = bf16_bits_to_float(words[i] & 0xffffu);
        out[2 * i + 1] = bf16_bits_to_float(words[i] >> 16);
      } else {
        out[2 * i] = f16_bits_to_float(words[i] & 0xffffu);
        out[2 * i + 1] = f16_bits_to_float(words[i] >> 16);
      }
    }
  }
}

template <int DT>
__device__ __forceinline__ float load1(const void* base, int64_t offset) {
  if constexpr (DT == kF32) {
    return static_cast<const float*>(base)[offset];
  } else if constexpr (DT == kBF16) {
    return bf16_bits_to_float(static_cast<const uint16_t*>(base)[offset]);
  } else {
    return f16_bits_to_float(static_cast<const uint16_t*>(base)[offset]);
  }
}

// Round to nearest even, saturate to the signed 8-bit range, NaN -> 0.
// Round-to-nearest-even conversion of a code in [-127.5, 127.5] by adding 1.5 * 2^23: the sum's
// integer part is rint(value) (the sum has an ulp of 1 and 1.5 * 2^23 is even, so ties go to the
// even code), and the low byte of its bit pattern is the two's-complement INT8 code.  One add
// replaces round, NaN test, clamp and convert; the scales of this library keep |value| below
// 127.5 for finite inputs (scale > max / 127), so the reference's clamp never binds, and a NaN
// (0 * inf from a row with an infinity) has a zero low byte like the reference's saturating
// convert.  Not covered: a NaN in the *input* whose payload has a non-zero low byte travels
// through the additions and leaves that byte as the code where the reference stores 0; the
// scale of such a group is NaN-derived in both and the row's output meaningless either way.
constexpr float kRoundMagic = 12582912.0f;
__device__ __forceinline__ float round_to_code(float value) { return value + kRoundMagic; }
__device__ __forceinline__ float code_value(float magic_sum) { return magic_sum - kRoundMagic; }
// Byte k of the result is the code of the k-th argument.
__device__ __forceinline__ uint32_t pack_codes(float a, float b, float c, float d) {
  const uint32_t low = __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x0c0c0400u);
  const uint32_t high = __builtin_amdgcn_perm(__float_as_uint(d), __float_as_uint(c), 0x0c0c0400u);
  return low | (high << 16);
}
// Sum of the four signed bytes of a word.
__device__ __forceinline__ int sum_of_codes(uint32_t packed) {
  return __builtin_amdgcn_sdot4(static_cast<int>(packed), 0x01010101, 0, false);
}

// Maximum over lanes l and l ^ 32 (max_across_halves) or l and l ^ 16
// (max_across_row_pairs), in both lanes, with the gfx950 lane-swap instructions: one
// vector instruction instead of a round trip through the LDS crossbar.  With both
// operands equal, v_permlane32_swap leaves the lower half's value in both halves of the
// first result and the upper half's in both halves of the second; v_permlane16_swap
// does the same for the even and odd 16-lane rows of each pair.
__device__ __forceinline__ float max_across_halves(float x) {
  const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __builtin_fmaxf(__uint_as_float(both[0]), __uint_as_float(both[1]));
}
__device__ __forceinline__ float max_across_row_pairs(float x) {
  const auto both = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __builtin_fmaxf(__uint_as_float(both[0]), __uint_as_float(both[1]));
}

// Integer sum over lanes l and l ^ 32, in both lanes (exact, so the order is free).
__device__ __forceinline__ uint32_t sum_across_halves(uint32_t x) {
  const auto both = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  return both[0] + both[1];
}

// Accumulator seed of the P·V product.  The matrix cores add integers to whatever
// 32-bit pattern they start from; starting from the bits of 1.5 * 2^23 (plus the
// zero-point term) leaves the bits of the float 12582912 + n for every result
// |n| < 2^22, and 255 * 128 * 128 keys stays below that.  One exact float
// subtraction then replaces the slower integer-to-float conversion.
constexpr int32_t kAccumulatorSeedBits = 0x4B400000;
constexpr float kAccumulatorSeed = 12582912.0f;

// Position of token `t` (0..31) inside its 32-token group of the packed V
// matrix.  Byte p = 16*h + 4*b + r holds token 8*b + 4*h + r, so the sixteen
// bytes a lane of half h feeds to the 32x32x32 INT8 MFMA are the sixteen keys
// the same lane holds in the accumulator of the transposed score tile.
__host__ __device__ __forceinline__ int packed_value_position(int t) {
  return ((t >> 2) & 1) * 16 + (t >> 3) * 4 + (t & 3);
}

}  // namespace risa
