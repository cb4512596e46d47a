// Per-head-dim instantiation of the attention kernel (one translation unit per
// head dim so the variants compile in parallel).
#pragma once

#include "attention_kernel.hpp"

namespace risa {

template <int D> int launch_attention_variant(const KernelParams& p, int cta_k, bool fast, bool indexed,
                                              bool capture, int mask_mode, hipStream_t stream);

template <int D, int CTA_K, bool FAST, bool INDEXED, bool CAPTURE, int MASK_DT, int MASK_MODE = kMaskScalar>
int launch_one(const KernelParams& p, hipStream_t stream) {
  using Shape = AttentionTileShape<D, CTA_K, MASK_DT, MASK_MODE>;
  auto kernel = attention_kernel<D, CTA_K, FAST, INDEXED, CAPTURE, MASK_DT, MASK_MODE>;
  // The dynamic LDS limit is a per-device property of the function; setting it
  // again is cheap and keeps the launcher free of host-side caches.
  static thread_local int configured_device = -1;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return fail("risa_attention: hipGetDevice failed");
  if (device != configured_device) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            Shape::kLdsBytes) != hipSuccess) {
      return fail("risa_attention: cannot reserve " + std::to_string(Shape::kLdsBytes) +
                  " bytes of LDS");
    }
    configured_device = device;
  }
  const dim3 grid(static_cast<unsigned>(p.n_qb) * p.q_heads * p.batch);
  kernel<<<grid, 256, Shape::kLdsBytes, stream>>>(p);
  return 0;
}

template <int D, int CTA_K, int MASK_DT, int MASK_MODE = kMaskScalar>
int launch_general(const KernelParams& p, bool indexed, bool capture, hipStream_t stream) {
  if (capture) return launch_one<D, CTA_K, false, false, true, MASK_DT, MASK_MODE>(p, stream);
  if (indexed) return launch_one<D, CTA_K, false, true, false, MASK_DT, MASK_MODE>(p, stream);
  return launch_one<D, CTA_K, false, false, false, MASK_DT, MASK_MODE>(p, stream);
}

// Mask tensors read per score, by the best mode the tensor allows (`mask_mode`, decided
// on the host).  Vector and staged reads exist for 64-key tiles only, the tile every
// query-dependent mask runs with (a key-only mask given without its bias row still
// works, element by element).
template <int D, int CTA_K, int MASK_DT>
int launch_masked(const KernelParams& p, int mask_mode, bool indexed, bool capture, hipStream_t stream) {
  if constexpr (CTA_K == 64) {
    if constexpr (MASK_DT == kBool) {
      if (mask_mode == kMaskLanes) return launch_general<D, CTA_K, MASK_DT, kMaskLanes>(p, indexed, capture, stream);
    }
    if (mask_mode == kMaskStaged) return launch_general<D, CTA_K, MASK_DT, kMaskStaged>(p, indexed, capture, stream);
    if (mask_mode != kMaskScalar) return launch_general<D, CTA_K, MASK_DT, kMaskVector>(p, indexed, capture, stream);
  }
  return launch_general<D, CTA_K, MASK_DT, kMaskScalar>(p, indexed, capture, stream);
}

template <int D, int CTA_K>
int launch_tile(const KernelParams& p, bool fast, bool indexed, bool capture, int mask_mode,
                hipStream_t stream) {
  if (fast) {
    if (capture) return launch_one<D, CTA_K, true, false, true, -1>(p, stream);
    if (indexed) return launch_one<D, CTA_K, true, true, false, -1>(p, stream);
    return launch_one<D, CTA_K, true, false, false, -1>(p, stream);
  }
  switch (p.mask_dtype) {
    case kBool: return launch_masked<D, CTA_K, kBool>(p, mask_mode, indexed, capture, stream);
    case kF32: return launch_masked<D, CTA_K, kF32>(p, mask_mode, indexed, capture, stream);
    case kF16: return launch_masked<D, CTA_K, kF16>(p, mask_mode, indexed, capture, stream);
    case kBF16: return launch_masked<D, CTA_K, kBF16>(p, mask_mode, indexed, capture, stream);
    case kKeyBias: return launch_general<D, CTA_K, kKeyBias>(p, indexed, capture, stream);
    default: return launch_general<D, CTA_K, -1>(p, indexed, capture, stream);
  }
}

#define RISA_DEFINE_ATTENTION_VARIANT(DIM)                                                        \
  template <>                                                                                     \
  int launch_attention_variant<DIM>(const KernelParams& p, int cta_k, bool fast, bool indexed,    \
                                    bool capture, int mask_mode, hipStream_t stream) {            \
    if constexpr (DIM != 64) {                                                                    \
      if (cta_k == 128)                                                                           \
        return launch_tile<DIM, 128>(p, fast, indexed, capture, mask_mode, stream);               \
    }                                                                                             \
    return launch_tile<DIM, 64>(p, fast, indexed, capture, mask_mode, stream);                    \
  }

}  // namespace risa
