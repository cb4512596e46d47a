// The sixteen-queries-per-wavefront kernel beyond the plain dense and reuse launches: tile
// lists of key-only masks, capture, and the pre-scaled path (masks, causal, scale <= 0), all
// with 128-query workgroups.  Every such launch with head dim 256 comes here, and those of
// the other head dims that leave compute units with at most one workgroup.
#include "attention_narrow_kernel.hpp"

namespace risa {
namespace {

template <int D, int CTA_K, bool GENERAL, int MASK_DT, bool MASK_VEC>
int launch_variant(const KernelParams& p, bool indexed, bool capture, hipStream_t stream) {
  if (capture) return launch_narrow_block<D, CTA_K, 8, 1, false, GENERAL, true, MASK_DT, MASK_VEC>(p, stream);
  if (indexed) return launch_narrow_block<D, CTA_K, 8, 1, true, GENERAL, false, MASK_DT, MASK_VEC>(p, stream);
  return launch_narrow_block<D, CTA_K, 8, 1, false, GENERAL, false, MASK_DT, MASK_VEC>(p, stream);
}

template <int D, int CTA_K, int MASK_DT>
int launch_mask(const KernelParams& p, bool vector_loads, bool indexed, bool capture, hipStream_t stream) {
  if (vector_loads) return launch_variant<D, CTA_K, true, MASK_DT, true>(p, indexed, capture, stream);
  return launch_variant<D, CTA_K, true, MASK_DT, false>(p, indexed, capture, stream);
}

template <int D, int CTA_K>
int launch_tile(const KernelParams& p, bool fast, bool indexed, bool capture, int mask_mode, hipStream_t stream) {
  if (fast) return launch_variant<D, CTA_K, false, -1, false>(p, indexed, capture, stream);
  const bool vector_loads = mask_mode != kMaskScalar;
  switch (p.mask_dtype) {
    case kBool: return launch_mask<D, CTA_K, kBool>(p, vector_loads, indexed, capture, stream);
    case kF32: return launch_mask<D, CTA_K, kF32>(p, vector_loads, indexed, capture, stream);
    case kF16: return launch_mask<D, CTA_K, kF16>(p, vector_loads, indexed, capture, stream);
    case kBF16: return launch_mask<D, CTA_K, kBF16>(p, vector_loads, indexed, capture, stream);
    case kKeyBias: return launch_variant<D, CTA_K, true, kKeyBias, false>(p, indexed, capture, stream);
    default: return launch_variant<D, CTA_K, true, -1, false>(p, indexed, capture, stream);
  }
}

}  // namespace

int launch_attention_narrow_general(const KernelParams& p, int head_dim, int cta_k, bool fast, bool indexed,
                                    bool capture, int mask_mode, hipStream_t stream) {
  if (mask_mode == kMaskLanes) return fail("risa_attention: lane words are not read by the sixteen-query kernel");
  if (head_dim == 64) return launch_tile<64, 64>(p, fast, indexed, capture, mask_mode, stream);
  if (head_dim == 128) {
    if (cta_k == 128) return launch_tile<128, 128>(p, fast, indexed, capture, mask_mode, stream);
    return launch_tile<128, 64>(p, fast, indexed, capture, mask_mode, stream);
  }
  if (head_dim == 256) {
    if (cta_k == 128) return launch_tile<256, 128>(p, fast, indexed, capture, mask_mode, stream);
    return launch_tile<256, 64>(p, fast, indexed, capture, mask_mode, stream);
  }
  return fail("risa_attention: unsupported head_dim");
}

}  // namespace risa
