// Launcher of the sixteen-queries-per-wavefront attention kernel used for launches that
// leave compute units with at most one workgroup.
#include "attention_narrow_kernel.hpp"

namespace risa {

int narrow_attention_limit();

namespace {

template <int D, int CTA_K, int WAVES, int KSPLIT, bool INDEXED = false, bool GENERAL = false,
          bool CAPTURE = false, int MASK_DT = -1, bool MASK_VEC = false>
int launch_block(const KernelParams& p, hipStream_t stream) {
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

// Queries per workgroup: 128, or 64 / 32 when that still leaves compute units without
// a workgroup (every SIMD then runs one wavefront with a quarter of the usual work).
// Those smaller workgroups also split four or more key tiles over two sets of wavefronts:
// the launch is short of work, not of hardware.
template <int D, int CTA_K> int launch_narrow(const KernelParams& p, hipStream_t stream) {
  const int64_t workgroups = static_cast<int64_t>(p.n_qb) * p.q_heads * p.batch;
  const int compute_units = narrow_attention_limit();
  // two sets of stages must fit the 160 KB of LDS of a compute unit
  constexpr bool kSplitFits = 2 * TileShape<D, CTA_K>::kLdsBytes <= 160 * 1024;
  const bool split = kSplitFits && p.n_kb >= 4;
  if (p.index_mode == 1) {
    // sparse reuse: the tile lists stay whole
    if (workgroups * 4 <= compute_units) return launch_block<D, CTA_K, 2, 1, true>(p, stream);
    if (workgroups * 2 <= compute_units) return launch_block<D, CTA_K, 4, 1, true>(p, stream);
    return launch_block<D, CTA_K, 8, 1, true>(p, stream);
  }
  if (workgroups * 4 <= compute_units) {
    if constexpr (kSplitFits) {
      if (split) return launch_block<D, CTA_K, 2, 2>(p, stream);
    }
    return launch_block<D, CTA_K, 2, 1>(p, stream);
  }
  if (workgroups * 2 <= compute_units) {
    if constexpr (kSplitFits) {
      if (split) return launch_block<D, CTA_K, 4, 2>(p, stream);
    }
    return launch_block<D, CTA_K, 4, 1>(p, stream);
  }
  return launch_block<D, CTA_K, 8, 1>(p, stream);
}

// Head dim 256 beyond the plain dense and reuse launches: tile lists of key-only masks,
// capture, and the pre-scaled path (masks, causal, scale <= 0), all with 128-query workgroups.
template <int CTA_K, bool GENERAL, int MASK_DT, bool MASK_VEC>
int launch_wide_head_variant(const KernelParams& p, bool indexed, bool capture, hipStream_t stream) {
  if (capture) return launch_block<256, CTA_K, 8, 1, false, GENERAL, true, MASK_DT, MASK_VEC>(p, stream);
  if (indexed) return launch_block<256, CTA_K, 8, 1, true, GENERAL, false, MASK_DT, MASK_VEC>(p, stream);
  return launch_block<256, CTA_K, 8, 1, false, GENERAL, false, MASK_DT, MASK_VEC>(p, stream);
}

template <int CTA_K, int MASK_DT>
int launch_wide_head_mask(const KernelParams& p, bool vector_loads, bool indexed, bool capture, hipStream_t stream) {
  if (vector_loads) return launch_wide_head_variant<CTA_K, true, MASK_DT, true>(p, indexed, capture, stream);
  return launch_wide_head_variant<CTA_K, true, MASK_DT, false>(p, indexed, capture, stream);
}

template <int CTA_K>
int launch_wide_head(const KernelParams& p, bool fast, bool indexed, bool capture, int mask_mode, hipStream_t stream) {
  if (fast) return launch_wide_head_variant<CTA_K, false, -1, false>(p, indexed, capture, stream);
  const bool vector_loads = mask_mode != kMaskScalar;
  switch (p.mask_dtype) {
    case kBool: return launch_wide_head_mask<CTA_K, kBool>(p, vector_loads, indexed, capture, stream);
    case kF32: return launch_wide_head_mask<CTA_K, kF32>(p, vector_loads, indexed, capture, stream);
    case kF16: return launch_wide_head_mask<CTA_K, kF16>(p, vector_loads, indexed, capture, stream);
    case kBF16: return launch_wide_head_mask<CTA_K, kBF16>(p, vector_loads, indexed, capture, stream);
    case kKeyBias: return launch_wide_head_variant<CTA_K, true, kKeyBias, false>(p, indexed, capture, stream);
    default: return launch_wide_head_variant<CTA_K, true, -1, false>(p, indexed, capture, stream);
  }
}

}  // namespace

int launch_attention_wide_head(const KernelParams& p, int cta_k, bool fast, bool indexed, bool capture,
                               int mask_mode, hipStream_t stream) {
  if (mask_mode == kMaskLanes) return fail("risa_attention: lane words are not read with head dim 256");
  if (cta_k == 128) return launch_wide_head<128>(p, fast, indexed, capture, mask_mode, stream);
  return launch_wide_head<64>(p, fast, indexed, capture, mask_mode, stream);
}

// Number of workgroups up to which the narrow kernel is the faster one: the number of
// compute units, below which the wide kernel runs one wavefront per SIMD.
int narrow_attention_limit() {
  static thread_local int cached_device = -1;
  static thread_local int compute_units = 0;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  if (device != cached_device) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    compute_units = count;
    cached_device = device;
  }
  return compute_units;
}

int launch_attention_narrow(const KernelParams& p, int head_dim, int cta_k, hipStream_t stream) {
  if (head_dim == 64) return launch_narrow<64, 64>(p, stream);
  if (head_dim == 128) return cta_k == 128 ? launch_narrow<128, 128>(p, stream) : launch_narrow<128, 64>(p, stream);
  if (head_dim == 256) return cta_k == 128 ? launch_narrow<256, 128>(p, stream) : launch_narrow<256, 64>(p, stream);
  return fail("risa_attention: unsupported head_dim");
}

}  // namespace risa
