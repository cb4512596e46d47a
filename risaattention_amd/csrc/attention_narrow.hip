// Launcher of the sixteen-queries-per-wavefront attention kernel used for launches that
// leave compute units with at most one workgroup.
#include "attention_narrow_kernel.hpp"

namespace risa {


namespace {

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
    if (workgroups * 4 <= compute_units) return launch_narrow_block<D, CTA_K, 2, 1, true>(p, stream);
    if (workgroups * 2 <= compute_units) return launch_narrow_block<D, CTA_K, 4, 1, true>(p, stream);
    return launch_narrow_block<D, CTA_K, 8, 1, true>(p, stream);
  }
  if (workgroups * 4 <= compute_units) {
    if constexpr (kSplitFits) {
      if (split) return launch_narrow_block<D, CTA_K, 2, 2>(p, stream);
    }
    return launch_narrow_block<D, CTA_K, 2, 1>(p, stream);
  }
  if (workgroups * 2 <= compute_units) {
    if constexpr (kSplitFits) {
      if (split) return launch_narrow_block<D, CTA_K, 4, 2>(p, stream);
    }
    return launch_narrow_block<D, CTA_K, 4, 1>(p, stream);
  }
  return launch_narrow_block<D, CTA_K, 8, 1>(p, stream);
}

}  // namespace

// Number of workgroups up to which the narrow kernel is the faster one: the number of
// compute units, below which the wide kernel runs one wavefront per SIMD.  Where no device can
// be queried (size queries made on a host without a GPU) it is the MI355X's 256.
int narrow_attention_limit() {
  constexpr int kMi355xComputeUnits = 256;
  static thread_local int cached_device = -1;
  static thread_local int compute_units = 0;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return kMi355xComputeUnits;
  if (device != cached_device) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
      return kMi355xComputeUnits;
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
