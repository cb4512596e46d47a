// Launchers of the Q/K preparation kernels (prep_qk_kernels.hpp) and the LSE anchor
// correction.

#include "prep_qk_kernels.hpp"

namespace risa {
namespace {

template <int DT, int DK, int ROT>
void launch_q(const QkArgs& a, hipStream_t stream) {
  constexpr int W = DK == 256 ? 16 : 32;
  const int slices = (a.q_len + 127) / 128 * (128 / W);
  dim3 grid(slices, a.q_heads, a.batch);
  quantize_q_kernel<DT, DK, ROT><<<grid, 256, 0, stream>>>(
      a.q, a.q_codes, a.q_scale, a.q_len, a.q_heads, slices * 8, a.q_stride_b, a.q_stride_h,
      a.q_stride_n, rows_are_16_byte_aligned(a.q, a.q_stride_b, a.q_stride_h, a.q_stride_n, a.dtype));
}

template <int DT, int DK, int CTA_K, int ROT>
void launch_k(const QkArgs& a, hipStream_t stream) {
  const int tiles = (a.k_len + CTA_K - 1) / CTA_K;
  dim3 grid(2 * tiles, a.kv_heads, a.batch);  // half a tile (two scale groups) per workgroup
  quantize_k_kernel<DT, DK, CTA_K, ROT><<<grid, 256, 0, stream>>>(
      a.k, a.k_codes, a.k_scale, a.anchors, a.k_len, a.kv_heads, tiles * 4, a.k_stride_b,
      a.k_stride_h, a.k_stride_n,
      rows_are_16_byte_aligned(a.k, a.k_stride_b, a.k_stride_h, a.k_stride_n, a.dtype), a.permutation);
}

template <int DT, int DK, int ROT>
void launch_qk_rot(const QkArgs& a, hipStream_t stream) {
  launch_q<DT, DK, ROT>(a, stream);
  if constexpr (DK == 64) {
    launch_k<DT, DK, 64, ROT>(a, stream);
  } else {
    if (a.cta_k == 128)
      launch_k<DT, DK, 128, ROT>(a, stream);
    else
      launch_k<DT, DK, 64, ROT>(a, stream);
  }
}

template <int DT> void launch_qk_dtype(const QkArgs& a, hipStream_t stream) {
  dim3 grid(a.kv_heads, a.batch);
  detect_anchor_kernel<DT><<<grid, 128, 0, stream>>>(a.k, a.anchors, a.k_len, a.head_dim,
                                                     a.kv_heads, a.k_stride_b, a.k_stride_h,
                                                     a.k_stride_n, a.permutation);
  const bool short_keys = a.k_len <= 256;
  if (a.head_dim == 64) {
    if (short_keys)
      launch_qk_rot<DT, 64, kRot4>(a, stream);
    else
      launch_qk_rot<DT, 64, kRot64>(a, stream);
  } else if (a.head_dim == 128) {
    if (short_keys)
      launch_qk_rot<DT, 128, kRot4>(a, stream);
    else
      launch_qk_rot<DT, 128, kRot128Signed>(a, stream);
  } else {
    if (short_keys)
      launch_qk_rot<DT, 256, kRot4>(a, stream);
    else
      launch_qk_rot<DT, 256, kRot128Plain>(a, stream);
  }
}

}  // namespace

int launch_quantize_qk(const QkArgs& a, hipStream_t stream) {
  if (a.dtype == kF32)
    launch_qk_dtype<kF32>(a, stream);
  else if (a.dtype == kF16)
    launch_qk_dtype<kF16>(a, stream);
  else
    launch_qk_dtype<kBF16>(a, stream);
  return check_launch("risa_quantize_qk");
}

// ---------------------------------------------------------------------------
// LSE anchor correction: out[b,h,i] = scale * <q[b,h,i], k[b,h/G,anchor]>,
// products and sums kept separate, lanes stride 32 over channels, shuffle-down
// tree (reference csrc/kernels/lse_correction.cu:4-28).
// grid (ceil(Lq/8), Hq, B), 256 threads: one 32-lane half per query row.
// ---------------------------------------------------------------------------
namespace {
template <int DT>
__global__ __launch_bounds__(256) void lse_shift_kernel(const void* __restrict__ q,
                                                        const void* __restrict__ k,
                                                        const int* __restrict__ anchors,
                                                        float* __restrict__ out, int q_heads,
                                                        int kv_heads, int q_len, int dim,
                                                        int64_t qb, int64_t qh, int64_t qn,
                                                        int64_t kb, int64_t kh, int64_t kn,
                                                        float scale) {
  const int sub = threadIdx.x & 31;
  const int row = blockIdx.x * 8 + (threadIdx.x >> 5);
  const int head = blockIdx.y, batch = blockIdx.z;
  if (row >= q_len) return;
  const int kv_head = head / (q_heads / kv_heads);
  const int anchor = anchors[batch * kv_heads + kv_head];
  float sum = 0.0f;
  if (anchor >= 0) {
    const int64_t q_base = batch * qb + head * qh + static_cast<int64_t>(row) * qn;
    const int64_t k_base = batch * kb + kv_head * kh + static_cast<int64_t>(anchor) * kn;
    for (int d = sub; d < dim; d += 32) {
      const float product = load1<DT>(q, q_base + d) * load1<DT>(k, k_base + d);
      sum = sum + product;
    }
    sum = segment_down_sum(sum);
  }
  if (sub == 0) out[(static_cast<int64_t>(batch) * q_heads + head) * q_len + row] = sum * scale;
}
}  // namespace

int launch_lse_shift(const LseShiftArgs& a, hipStream_t stream) {
  dim3 grid((a.q_len + 7) / 8, a.q_heads, a.batch);
#define RISA_LSE(DTV)                                                                             \
  lse_shift_kernel<DTV><<<grid, 256, 0, stream>>>(a.q, a.k, a.anchors, a.out, a.q_heads,           \
                                                  a.kv_heads, a.q_len, a.head_dim, a.q_stride_b,   \
                                                  a.q_stride_h, a.q_stride_n, a.k_stride_b,        \
                                                  a.k_stride_h, a.k_stride_n, a.scale)
  if (a.dtype == kF32)
    RISA_LSE(kF32);
  else if (a.dtype == kF16)
    RISA_LSE(kF16);
  else
    RISA_LSE(kBF16);
#undef RISA_LSE
  return check_launch("risa_lse_shift");
}

}  // namespace risa
