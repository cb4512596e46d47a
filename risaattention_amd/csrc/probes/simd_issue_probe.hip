// Stand-alone probe of the instruction issue rates the attention kernel is bound by on
// gfx950: (1) nanoseconds per wave64 instruction and SIMD for the vector instructions of
// the softmax and for the INT8 matrix instructions, at 1 to 8 resident wavefronts per
// SIMD; (2) whether vector and matrix instructions of one SIMD overlap.  Every loop has a
// fixed trip count; timing is HIP events around the second of two launches.
//
//   make -C risaattention_amd/csrc probes && risaattention_amd/csrc/probes/simd_issue_probe
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define CHECK(call)                                                                     \
  do {                                                                                  \
    const hipError_t status = (call);                                                   \
    if (status != hipSuccess) {                                                         \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(status));        \
      std::exit(1);                                                                     \
    }                                                                                   \
  } while (0)

constexpr int kChains = 16;     // independent dependency chains per lane
constexpr int kPerIteration = 64;

enum Op { kFma, kFmaScalarOperand, kFmac, kMul, kSub, kAddU32, kXor, kCvtF32I32, kCvtPkU8, kMax3I32, kMaxF32,
          kDot4, kExp, kExpAndTwoFma, kPermlane32Swap };

template <int OP> __global__ __launch_bounds__(256) void valu_kernel(int iterations, float* sink) {
  float f[kChains];
  for (int i = 0; i < kChains; ++i) f[i] = threadIdx.x * 0.001f + i;
  float m = 1.0001f, c = 0.0001f;
  asm volatile("" : "+v"(m), "+v"(c));
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int j = 0; j < kPerIteration; ++j) {
      float& x = f[j % kChains];
      if (OP == kFma) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(m), "v"(c));
      if (OP == kFmaScalarOperand) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(m), "s"(0x38d1b717));
      if (OP == kFmac) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(x) : "v"(m), "v"(c));
      if (OP == kMul) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x) : "v"(m));
      if (OP == kSub) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(x) : "v"(c));
      if (OP == kAddU32) asm volatile("v_add_u32 %0, %0, %1" : "+v"(x) : "v"(m));
      if (OP == kXor) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(x) : "v"(m));
      if (OP == kCvtF32I32) asm volatile("v_cvt_f32_i32 %0, %0" : "+v"(x));
      if (OP == kCvtPkU8) asm volatile("v_cvt_pk_u8_f32 %0, %1, 1, %0" : "+v"(x) : "v"(m));
      if (OP == kMax3I32) asm volatile("v_max3_i32 %0, %0, %1, %2" : "+v"(x) : "v"(m), "v"(c));
      if (OP == kMaxF32) asm volatile("v_max_f32 %0, %0, %1" : "+v"(x) : "v"(m));
      if (OP == kDot4) asm volatile("v_dot4_u32_u8 %0, %1, %2, %0" : "+v"(x) : "v"(m), "v"(c));
      if (OP == kExp) asm volatile("v_exp_f32 %0, %0" : "+v"(x));
      if (OP == kExpAndTwoFma) {
        if (j % 3 == 0) asm volatile("v_exp_f32 %0, %0" : "+v"(x));
        else asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x) : "v"(m), "v"(c));
      }
      if (OP == kPermlane32Swap) asm volatile("v_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(f[(j + 1) % kChains]));
    }
  }
  float total = 0;
  for (int i = 0; i < kChains; ++i) total += f[i];
  if (total == 12345.678f) sink[0] = total;  // keeps the chains alive
}

// MODE 0: matrix instructions only, 1: vector only, 2: MATRIX matrix then VECTOR vector
// instructions per iteration, 3: the same instructions interleaved.
template <int MODE, int MATRIX, int VECTOR, bool LARGE>
__global__ __launch_bounds__(256) void overlap_kernel(int iterations, float* sink) {
  v4i a = {static_cast<int>(threadIdx.x), 1, 2, 3}, b = {4, 5, 6, static_cast<int>(threadIdx.x)};
  v4i small[4] = {};
  v16i large[2] = {};
  float f[8];
  for (int i = 0; i < 8; ++i) f[i] = threadIdx.x * 0.001f + i;
  float m = 1.0001f, c = 0.0001f;
  asm volatile("" : "+v"(m), "+v"(c));
  auto matrix = [&](int j) {
    if (LARGE) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(large[j % 2]) : "v"(a), "v"(b));
    else asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(small[j % 4]) : "v"(a), "v"(b));
  };
  auto vector = [&](int j) { asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[j % 8]) : "v"(m), "v"(c)); };
  for (int it = 0; it < iterations; ++it) {
    if (MODE == 0 || MODE == 2) {
#pragma unroll
      for (int j = 0; j < MATRIX; ++j) matrix(j);
    }
    if (MODE == 1 || MODE == 2) {
#pragma unroll
      for (int j = 0; j < VECTOR; ++j) vector(j);
    }
    if (MODE == 3) {
#pragma unroll
      for (int j = 0; j < MATRIX; ++j) {
        matrix(j);
#pragma unroll
        for (int k = 0; k < VECTOR / MATRIX; ++k) vector(j * (VECTOR / MATRIX) + k);
      }
    }
  }
  float total = 0;
  for (int i = 0; i < 8; ++i) total += f[i];
  int integer = 0;
  for (int i = 0; i < 4; ++i) integer += small[i][0] + small[i][3];
  for (int i = 0; i < 2; ++i) integer += large[i][0] + large[i][15];
  if (total == 12345.678f || integer == 0x7fffffff) sink[0] = total + integer;
}

// The instructions of one wavefront and one 128-key tile of the dense attention kernel at
// head dim 128 (32 queries), register resident, in the kernel's order: 16 score MFMAs; per
// score a subtraction, an FMA, an exp2 and a pack, plus the maxima, the row sum and the sign
// flip; 16 value MFMAs with the 64 output updates (subtract + FMA) between them.  No memory,
// no barrier, no dependency on the matrix results: the issue-rate floor of the tile loop.
template <bool MATRIX, bool VECTOR, bool SPREAD = false>
__global__ __launch_bounds__(256) void tile_mix_kernel(int iterations, float* sink) {
  v4i a = {static_cast<int>(threadIdx.x), 1, 2, 3}, b = {4, 5, 6, static_cast<int>(threadIdx.x)};
  v16i scores[4] = {}, values[4] = {};
  float x[16], out[16];
  int top[4];
  uint32_t packed[4], sum = 0;
  for (int i = 0; i < 16; ++i) x[i] = threadIdx.x * 0.001f + i, out[i] = i;
  for (int i = 0; i < 4; ++i) top[i] = threadIdx.x + i, packed[i] = i;
  float m = 1.0001f, c = 0.0001f, seed = 12582912.0f;
  uint32_t flip = 0x80808080u, ones = 0x01010101u;
  asm volatile("" : "+v"(m), "+v"(c), "+v"(seed), "+v"(flip), "+v"(ones));
  for (int it = 0; it < iterations; ++it) {
    if (MATRIX && !SPREAD) {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(scores[j % 4]) : "v"(a), "v"(b));
    }
    if (VECTOR) {
#pragma unroll
      for (int j = 0; j < 32; ++j)
        asm volatile("v_max3_i32 %0, %0, %1, %2" : "+v"(top[j % 4]) : "v"(packed[j % 4]), "v"(flip));
#pragma unroll
      for (int j = 0; j < 64; ++j) {
        if (MATRIX && SPREAD && j % 4 == 0)
          asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(scores[(j / 4) % 4]) : "v"(a), "v"(b));
        asm volatile("v_sub_f32 %0, %0, %1" : "+v"(x[j % 16]) : "v"(seed));
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[j % 16]) : "v"(m), "v"(c));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[j % 16]));
        asm volatile("v_cvt_pk_u8_f32 %0, %1, 1, %0" : "+v"(packed[j % 4]) : "v"(x[j % 16]));
        if (j % 4 == 3) {
          asm volatile("v_dot4_u32_u8 %0, %1, %2, %0" : "+v"(sum) : "v"(packed[(j / 4) % 4]), "v"(ones));
          asm volatile("v_xor_b32 %0, %0, %1" : "+v"(packed[(j / 4) % 4]) : "v"(flip));
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (MATRIX) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(values[j % 4]) : "v"(a), "v"(b));
      if (VECTOR) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float t = x[(j * 4 + k) % 16];
          asm volatile("v_sub_f32 %0, %1, %2" : "=v"(t) : "v"(t), "v"(seed));
          asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(out[(j * 4 + k) % 16]) : "v"(t), "v"(m));
        }
      }
    }
  }
  float total = sum;
  for (int i = 0; i < 16; ++i) total += x[i] + out[i];
  int integer = 0;
  for (int i = 0; i < 4; ++i) integer += scores[i][0] + values[i][15] + top[i] + packed[i];
  if (total == 12345.678f || integer == 0x7fffffff) sink[0] = total + integer;
}

// The same instructions in a software-pipelined order: the score MFMAs of a tile run under
// the output updates of the previous tile, and the value MFMAs of each 32-key block under
// the exp2/pack chain of the next block; only the maxima have no matrix work beside them.
template <bool UPDATES_UNDER_SCORES>
__global__ __launch_bounds__(256) void tile_pipeline_kernel(int iterations, float* sink) {
  v4i a = {static_cast<int>(threadIdx.x), 1, 2, 3}, b = {4, 5, 6, static_cast<int>(threadIdx.x)};
  v16i scores[4] = {}, values[4] = {};
  float x[16], out[16];
  int top[4];
  uint32_t packed[4], sum = 0;
  for (int i = 0; i < 16; ++i) x[i] = threadIdx.x * 0.001f + i, out[i] = i;
  for (int i = 0; i < 4; ++i) top[i] = threadIdx.x + i, packed[i] = i;
  float m = 1.0001f, c = 0.0001f, seed = 12582912.0f;
  uint32_t flip = 0x80808080u, ones = 0x01010101u;
  asm volatile("" : "+v"(m), "+v"(c), "+v"(seed), "+v"(flip), "+v"(ones));
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(scores[j % 4]) : "v"(a), "v"(b));
      if (UPDATES_UNDER_SCORES) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float t = x[(j * 4 + k) % 16];
          asm volatile("v_sub_f32 %0, %1, %2" : "=v"(t) : "v"(t), "v"(seed));
          asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(out[(j * 4 + k) % 16]) : "v"(t), "v"(m));
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 32; ++j)
      asm volatile("v_max3_i32 %0, %0, %1, %2" : "+v"(top[j % 4]) : "v"(packed[j % 4]), "v"(flip));
#pragma unroll
    for (int block = 0; block < 5; ++block) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if (block > 0 && j % 4 == 0)
          asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(values[j / 4]) : "v"(a), "v"(b));
        if (block < 4) {
          asm volatile("v_sub_f32 %0, %0, %1" : "+v"(x[j]) : "v"(seed));
          asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[j]) : "v"(m), "v"(c));
          asm volatile("v_exp_f32 %0, %0" : "+v"(x[j]));
          asm volatile("v_cvt_pk_u8_f32 %0, %1, 1, %0" : "+v"(packed[j % 4]) : "v"(x[j]));
          if (j % 4 == 3) {
            asm volatile("v_dot4_u32_u8 %0, %1, %2, %0" : "+v"(sum) : "v"(packed[j / 4]), "v"(ones));
            asm volatile("v_xor_b32 %0, %0, %1" : "+v"(packed[j / 4]) : "v"(flip));
          }
        }
      }
    }
    if (!UPDATES_UNDER_SCORES) {
#pragma unroll
      for (int j = 0; j < 64; ++j) {
        float t = x[j % 16];
        asm volatile("v_sub_f32 %0, %1, %2" : "=v"(t) : "v"(t), "v"(seed));
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(out[j % 16]) : "v"(t), "v"(m));
      }
    }
  }
  float total = sum;
  for (int i = 0; i < 16; ++i) total += x[i] + out[i];
  int integer = 0;
  for (int i = 0; i < 4; ++i) integer += scores[i][0] + values[i][15] + top[i] + packed[i];
  if (total == 12345.678f || integer == 0x7fffffff) sink[0] = total + integer;
}

// Milliseconds of `iterations` loop iterations with `waves` wavefronts resident per SIMD
// on every compute unit: the dynamic LDS request limits the workgroups per compute unit.
template <typename Kernel> float time_kernel(Kernel kernel, int compute_units, int waves, int iterations, float* sink) {
  const int lds_bytes = 160 * 1024 / waves - 1024;
  CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes));
  hipEvent_t begin, end;
  CHECK(hipEventCreate(&begin));
  CHECK(hipEventCreate(&end));
  kernel<<<compute_units * waves, 256, lds_bytes>>>(iterations / 10, sink);
  CHECK(hipEventRecord(begin));
  kernel<<<compute_units * waves, 256, lds_bytes>>>(iterations, sink);
  CHECK(hipEventRecord(end));
  CHECK(hipEventSynchronize(end));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, begin, end));
  CHECK(hipEventDestroy(begin));
  CHECK(hipEventDestroy(end));
  return ms;
}

template <int OP> void valu_row(const char* name, int compute_units, float* sink) {
  const int iterations = 10000;
  std::printf("%-28s", name);
  for (int waves = 1; waves <= 8; waves *= 2) {
    const float ms = time_kernel(valu_kernel<OP>, compute_units, waves, iterations, sink);
    std::printf("  %d w/SIMD %6.2f ns", waves, ms * 1e6 / (double(iterations) * kPerIteration * waves));
  }
  std::printf("\n");
  std::fflush(stdout);
}

template <int MATRIX, int VECTOR, bool LARGE> void overlap_rows(const char* name, int compute_units, float* sink) {
  const int iterations = 20000;
  for (int waves = 1; waves <= 4; waves *= 2) {
    const float matrix = time_kernel(overlap_kernel<0, MATRIX, VECTOR, LARGE>, compute_units, waves, iterations, sink);
    const float vector = time_kernel(overlap_kernel<1, MATRIX, VECTOR, LARGE>, compute_units, waves, iterations, sink);
    const float blocked = time_kernel(overlap_kernel<2, MATRIX, VECTOR, LARGE>, compute_units, waves, iterations, sink);
    const float mixed = time_kernel(overlap_kernel<3, MATRIX, VECTOR, LARGE>, compute_units, waves, iterations, sink);
    std::printf("%s x%d + v_fma_f32 x%d, %d w/SIMD: matrix %.2f ms (%.1f ns each), vector %.2f ms, blocked %.2f ms, "
                "interleaved %.2f ms; sum %.2f, max %.2f\n",
                name, MATRIX, VECTOR, waves, matrix, matrix * 1e6 / (double(iterations) * MATRIX * waves), vector,
                blocked, mixed, matrix + vector, matrix > vector ? matrix : vector);
    std::fflush(stdout);
  }
}

int main() {
  int compute_units = 0;
  CHECK(hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, 0));
  float* sink = nullptr;
  CHECK(hipMalloc(&sink, sizeof(float)));
  std::printf("compute units: %d; ns per wave64 instruction and SIMD\n", compute_units);
  valu_row<kAddU32>("v_add_u32", compute_units, sink);
  valu_row<kXor>("v_xor_b32", compute_units, sink);
  valu_row<kMul>("v_mul_f32", compute_units, sink);
  valu_row<kSub>("v_sub_f32", compute_units, sink);
  valu_row<kFmac>("v_fmac_f32", compute_units, sink);
  valu_row<kFma>("v_fma_f32", compute_units, sink);
  valu_row<kFmaScalarOperand>("v_fma_f32 (scalar operand)", compute_units, sink);
  valu_row<kCvtF32I32>("v_cvt_f32_i32", compute_units, sink);
  valu_row<kCvtPkU8>("v_cvt_pk_u8_f32", compute_units, sink);
  valu_row<kMax3I32>("v_max3_i32", compute_units, sink);
  valu_row<kMaxF32>("v_max_f32", compute_units, sink);
  valu_row<kDot4>("v_dot4_u32_u8", compute_units, sink);
  valu_row<kExp>("v_exp_f32", compute_units, sink);
  valu_row<kExpAndTwoFma>("v_exp_f32 + 2 v_fma_f32 (avg)", compute_units, sink);
  valu_row<kPermlane32Swap>("v_permlane32_swap_b32", compute_units, sink);
  std::printf("\nmatrix and vector instructions on one SIMD (blocked: one after the other in a wavefront)\n");
  overlap_rows<8, 64, false>("v_mfma_i32_16x16x64_i8", compute_units, sink);
  overlap_rows<8, 128, true>("v_mfma_i32_32x32x32_i8", compute_units, sink);
  std::printf("\none wavefront x one 128-key tile of the dense attention kernel (head dim 128), register resident\n");
  for (int waves = 1; waves <= 2; ++waves) {
    const int iterations = 5000;
    const double scale = 1e6 / (double(iterations) * waves);
    const float matrix = time_kernel(tile_mix_kernel<true, false>, compute_units, waves, iterations, sink);
    const float vector = time_kernel(tile_mix_kernel<false, true>, compute_units, waves, iterations, sink);
    const float both = time_kernel(tile_mix_kernel<true, true>, compute_units, waves, iterations, sink);
    const float spread = time_kernel(tile_mix_kernel<true, true, true>, compute_units, waves, iterations, sink);
    const float pipelined = time_kernel(tile_pipeline_kernel<true>, compute_units, waves, iterations, sink);
    const float half_pipelined = time_kernel(tile_pipeline_kernel<false>, compute_units, waves, iterations, sink);
    std::printf("%d w/SIMD: 32 MFMAs %.0f ns, vector instructions %.0f ns, both %.0f ns per wavefront and tile "
                "(%.0f ns with the score MFMAs spread through the softmax instructions, %.0f ns software pipelined, %.0f ns with only the value MFMAs pipelined)\n",
                waves, matrix * scale, vector * scale, both * scale, spread * scale, pipelined * scale, half_pipelined * scale);
    std::fflush(stdout);
  }
  CHECK(hipFree(sink));
  return 0;
}
