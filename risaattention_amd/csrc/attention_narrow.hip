// Launcher of the sixteen-queries-per-wavefront attention kernel used for launches that
// leave compute units with at most one workgroup.
#include "attention_narrow_kernel.hpp"

namespace risa {

namespace {

template <int D, int CTA_K> int launch_narrow(const KernelParams& p, hipStream_t stream) {
  using Shape = TileShape<D, CTA_K>;
  auto kernel = attention_narrow_kernel<D, CTA_K>;
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
  kernel<<<grid, kNarrowThreads, Shape::kLdsBytes, stream>>>(p);
  return 0;
}

}  // namespace

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
