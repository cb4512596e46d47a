// Retained-mass tile selection and broadcast key-mask tile metadata for gfx950.
//
// Contract: reference csrc/kernels/sparse_selection.cu:9-159 (FP64 total and
// prefix over masses already sorted in descending order, shortest prefix whose
// mass reaches theta * total, CSR compaction in ascending tile order, summary)
// and csrc/kernels/key_mask_tiles.cu:10-43.

#include "common.hpp"
#include "launchers.hpp"

namespace risa {
namespace {

// One 32-lane half of a wavefront per row, so that lane-strided sums and the
// 32-wide inclusive scans associate exactly as in the contract.
__global__ __launch_bounds__(64) void select_rows_kernel(const float* __restrict__ sorted_mass,
                                                         const int64_t* __restrict__ order,
                                                         int32_t* __restrict__ counts,
                                                         uint8_t* __restrict__ support,
                                                         double* __restrict__ row_totals, int rows,
                                                         int tiles, double theta) {
  const int sub = threadIdx.x & 31;
  const int row = blockIdx.x * 2 + (threadIdx.x >> 5);
  if (row >= rows) return;
  const int64_t base = static_cast<int64_t>(row) * tiles;
  double lane_total = 0.0;
  for (int rank = sub; rank < tiles; rank += 32) {
    lane_total += static_cast<double>(sorted_mass[base + rank]);
    support[base + rank] = 0;
  }
  double total = lane_total;
#pragma unroll
  for (int offset = 16; offset > 0; offset >>= 1) total += __shfl_down(total, offset, 32);
  total = __shfl(total, 0, 32);

  const double target = theta * total;
  double cumulative = 0.0;
  double selected = total;
  int count = tiles;
  for (int chunk = 0; chunk < tiles; chunk += 32) {
    const int rank = chunk + sub;
    double prefix = rank < tiles ? static_cast<double>(sorted_mass[base + rank]) : 0.0;
#pragma unroll
    for (int offset = 1; offset < 32; offset <<= 1) {
      const double previous = __shfl_up(prefix, offset, 32);
      if (sub >= offset) prefix += previous;
    }
    const bool reaches = rank < tiles && cumulative + prefix >= target;
    const uint64_t ballot = __ballot(reaches);
    const uint32_t votes = static_cast<uint32_t>(ballot >> (threadIdx.x & 32));
    if (votes != 0) {
      const int first = __builtin_ctz(votes);
      count = chunk + first + 1;
      selected = cumulative + __shfl(prefix, first, 32);
      break;
    }
    cumulative += __shfl(prefix, 31, 32);
  }
  // The support bytes of this row were cleared by these same 32 lanes above.
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  for (int rank = sub; rank < count; rank += 32) {
    support[base + static_cast<int>(order[base + rank])] = 1;
  }
  if (sub == 0) {
    counts[row] = count;
    row_totals[row * 2] = selected;
    row_totals[row * 2 + 1] = total;
  }
}

// Descending order of every row's masses with ties by ascending tile id (what a stable
// descending sort gives; the contract sorts with torch.sort in Python, reference
// src/risa_attention/sparse.py:24, and documents ties as free): one workgroup per row, a bitonic
// network over the row padded to a power of two in LDS.  Padding entries (-inf, ids past the row)
// end up last and are not written.
// THREADS: 64 for rows of up to 1024 entries (a single wavefront's barriers cost next to nothing
// and sixteen such workgroups share a compute unit), 256 beyond.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void sort_rows_kernel(const float* __restrict__ masses,
                                                            float* __restrict__ sorted_mass,
                                                            int64_t* __restrict__ order, int tiles, int padded) {
  extern __shared__ unsigned char sort_lds[];
  float* key = reinterpret_cast<float*>(sort_lds);
  int* id = reinterpret_cast<int*>(key + padded);
  const int tid = threadIdx.x;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * tiles;
  for (int i = tid; i < padded; i += THREADS) {
    key[i] = i < tiles ? masses[base + i] : -__builtin_inff();
    id[i] = i;
  }
  __syncthreads();
  for (int k = 2; k <= padded; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < padded / 2; t += THREADS) {
        const int low = (t / j) * 2 * j + (t % j), high = low + j;
        const float a = key[low], b = key[high];
        const int ia = id[low], ib = id[high];
        const bool b_first = b > a || (b == a && ib < ia);  // b belongs in front of a
        const bool a_first = a > b || (a == b && ia < ib);
        // the first half of every 2k block ends up in order, the second half reversed
        if (((low & k) == 0) ? b_first : a_first) {
          key[low] = b, key[high] = a;
          id[low] = ib, id[high] = ia;
        }
      }
      __syncthreads();
    }
  }
  for (int i = tid; i < tiles; i += THREADS) {
    sorted_mass[base + i] = key[i];
    order[base + i] = id[i];
  }
}

// Single workgroup: exclusive scan of the per-row counts and the FP64 summary
// (pairwise tree over 256 partial sums, as in the contract).
__global__ __launch_bounds__(256) void offsets_summary_kernel(const int32_t* __restrict__ counts,
                                                              const double* __restrict__ row_totals,
                                                              int32_t* __restrict__ row_offsets,
                                                              double* __restrict__ summary, int rows) {
  __shared__ double selected_sums[256];
  __shared__ double total_sums[256];
  __shared__ int scan[256];
  __shared__ int carry;
  const int tid = threadIdx.x;
  double selected = 0.0, total = 0.0;
  for (int row = tid; row < rows; row += 256) {
    selected += row_totals[row * 2];
    total += row_totals[row * 2 + 1];
  }
  selected_sums[tid] = selected;
  total_sums[tid] = total;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int stride = 128; stride > 0; stride >>= 1) {
    if (tid < stride) {
      selected_sums[tid] += selected_sums[tid + stride];
      total_sums[tid] += total_sums[tid + stride];
    }
    __syncthreads();
  }
  // Exclusive scan of the counts: every thread owns a run of consecutive rows, the 256 run
  // totals are scanned through LDS once, and every thread then writes its run (integer sums:
  // any order gives the same offsets).
  const int run = (rows + 255) / 256;
  const int first = tid * run, last = min(first + run, rows);
  int mine = 0;
  for (int row = first; row < last; ++row) mine += counts[row];
  scan[tid] = mine;
  __syncthreads();
  for (int offset = 1; offset < 256; offset <<= 1) {
    const int add = tid >= offset ? scan[tid - offset] : 0;
    __syncthreads();
    scan[tid] += add;
    __syncthreads();
  }
  int running = scan[tid] - mine;
  for (int row = first; row < last; ++row) {
    row_offsets[row] = running;
    running += counts[row];
  }
  if (tid == 255) carry = scan[255];
  __syncthreads();
  if (tid == 0) {
    row_offsets[rows] = carry;
    summary[0] = selected_sums[0];
    summary[1] = total_sums[0];
    summary[2] = static_cast<double>(carry);
  }
}

// One wavefront per row: ordered compaction of the support bytes.
__global__ __launch_bounds__(256) void compact_rows_kernel(const uint8_t* __restrict__ support,
                                                           const int32_t* __restrict__ row_offsets,
                                                           int32_t* __restrict__ block_indices,
                                                           int rows, int tiles) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t base = static_cast<int64_t>(row) * tiles;
  int written = row_offsets[row];
  for (int chunk = 0; chunk < tiles; chunk += 64) {
    const int tile = chunk + lane;
    const bool keep = tile < tiles && support[base + tile] != 0;
    const uint64_t votes = __ballot(keep);
    if (keep) {
      const uint64_t lower = lane == 0 ? 0ull : (votes & ((1ull << lane) - 1ull));
      block_indices[written + __builtin_popcountll(lower)] = tile;
    }
    written += __builtin_popcountll(votes);
  }
}

__device__ __forceinline__ bool key_visible(const void* mask, int64_t index, int dtype) {
  if (dtype == kBool) return static_cast<const uint8_t*>(mask)[index] != 0;
  const float bias = dtype == kF32   ? load1<kF32>(mask, index)
                     : dtype == kF16 ? load1<kF16>(mask, index)
                                     : load1<kBF16>(mask, index);
  return __builtin_isfinite(bias);
}

// One workgroup per (batch, head): flag tiles with any visible key, then one
// wavefront compacts the active tile ids in ascending order and appends the count.
__global__ __launch_bounds__(256) void key_mask_tiles_kernel(const void* __restrict__ mask,
                                                             int32_t* __restrict__ output, int heads,
                                                             int length, int tile_size,
                                                             int64_t stride_b, int64_t stride_h,
                                                             int64_t stride_k, int dtype) {
  const int tiles = (length + tile_size - 1) / tile_size;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * heads + blockIdx.y;
  const int64_t mask_row = blockIdx.x * stride_b + blockIdx.y * stride_h;
  int32_t* out = output + row * (tiles + 1);
  extern __shared__ int active_flags[];
  for (int tile = wave; tile < tiles; tile += 4) {
    bool visible = false;
    for (int offset = lane; offset < tile_size; offset += 64) {
      const int key = tile * tile_size + offset;
      if (key < length) visible |= key_visible(mask, mask_row + key * stride_k, dtype);
    }
    const bool any = __ballot(visible) != 0;
    if (lane == 0) active_flags[tile] = any ? 1 : 0;
  }
  __syncthreads();
  if (wave == 0) {
    int count = 0;
    for (int base = 0; base < tiles; base += 64) {
      const int tile = base + lane;
      const bool active = tile < tiles && active_flags[tile] != 0;
      const uint64_t votes = __ballot(active);
      if (active) {
        const uint64_t lower = lane == 0 ? 0ull : (votes & ((1ull << lane) - 1ull));
        out[count + __builtin_popcountll(lower)] = tile;
      }
      count += __builtin_popcountll(votes);
    }
    // Slots behind the active ids are never read by the attention kernel.
    for (int slot = count + lane; slot < tiles; slot += 64) out[slot] = -1;
    if (lane == 0) out[tiles] = count;
  }
}

// grid (ceil(padded/256), heads, batch), 256 threads: one key each.  The product
// bias * log2(e) is the FP32 product the attention kernel would form per score.
__global__ __launch_bounds__(256) void key_bias_kernel(const void* __restrict__ mask,
                                                       float* __restrict__ bias, int length,
                                                       int padded, int64_t stride_b, int64_t stride_h,
                                                       int64_t stride_k, int dtype) {
  const int key = blockIdx.x * 256 + threadIdx.x;
  if (key >= padded) return;
  float value = -__builtin_inff();
  if (key < length) {
    const int64_t index = blockIdx.z * stride_b + blockIdx.y * stride_h + key * stride_k;
    if (dtype == kBool) {
      if (static_cast<const uint8_t*>(mask)[index] != 0) value = 0.0f;
    } else {
      const float raw = dtype == kF32   ? load1<kF32>(mask, index)
                        : dtype == kF16 ? load1<kF16>(mask, index)
                                        : load1<kBF16>(mask, index);
      if (__builtin_isfinite(raw)) value = raw * 1.44269504088896340736f;
    }
  }
  bias[(static_cast<int64_t>(blockIdx.z) * gridDim.y + blockIdx.y) * padded + key] = value;
}


// Lane words of a boolean mask (the form kMaskLanes of the attention kernel reads): for
// every block of 32 queries and 64-key tile, 32 words; bit l of word 16*rb + i is the mask
// element of query 32*block + l % 32 and key 64*tile + 32*rb + 8*(i / 4) + 4*(l / 32) + i % 4,
// which is score (rb, i) of lane l in the attention kernel.  Rows past the last query and
// keys past the last key have no bit set.
//
// grid (groups of 16 tiles, blocks of 32 queries, batch*heads of the mask), 256 threads: a
// wavefront takes four consecutive key tiles of one query block (256 mask bytes per row, all
// requested before the first is used).  Lane (row, half) reads, per tile and 32-key block,
// the sixteen elements at keys 16*half .. 16*half+15 of the block (one 16-byte load when
// ALIGNED): the eight-key groups b4 = 2*half and 2*half+1, both four-key halves of each.
// A vote over element (b', h', r) of every lane therefore holds, in its low 32 bits, the
// rows' decisions for group b' and, in its high 32 bits, those for group 2+b', four-key
// half h' each; a lane word wants the two halves h' of one group side by side, which is a
// regrouping of 32-bit scalar registers.  Lane s keeps word s, so the 32 words of a tile
// leave in one 256-byte store.
constexpr int kLaneTilesPerWave = 4;
// A wave-uniform 32-bit value written into one lane of a vector register.
__device__ __forceinline__ void write_lane(uint32_t& target, uint32_t uniform_value, int lane_index) {
  asm("v_writelane_b32 %0, %1, %2" : "+v"(target) : "s"(uniform_value), "n"(lane_index));
}
template <bool ALIGNED>
__global__ __launch_bounds__(256) void mask_lanes_kernel(const uint8_t* __restrict__ mask,
                                                         uint64_t* __restrict__ lanes,
                                                         int32_t* __restrict__ classes, int heads,
                                                         int q_len, int k_len, int key_tiles,
                                                         int query_waves, int64_t stride_b,
                                                         int64_t stride_h, int64_t stride_q) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int query_wave = blockIdx.y, plane = blockIdx.z;
  const int row = query_wave * 32 + (lane & 31), half = lane >> 5;
  const bool row_ok = row < q_len;
  const uint8_t* row_mask = mask + (plane / heads) * stride_b + (plane % heads) * stride_h +
                            static_cast<int64_t>(row_ok ? row : q_len - 1) * stride_q;
  uint64_t* out = lanes + (static_cast<int64_t>(plane) * query_waves + query_wave) * key_tiles * 32;
  const int first_tile = (blockIdx.x * 4 + wave) * kLaneTilesPerWave;
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  v4u chunk[kLaneTilesPerWave][2];
#pragma unroll
  for (int t = 0; t < kLaneTilesPerWave; ++t) {
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      const int key = (first_tile + t) * 64 + rb * 32 + half * 16;
      v4u words = {0u, 0u, 0u, 0u};
      if (ALIGNED && key + 15 < k_len) {
        words = *reinterpret_cast<const v4u*>(row_mask + key);
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          if (key + j < k_len && row_mask[key + j] != 0) words[j >> 2] |= 1u << (8 * (j & 3));
        }
      }
      if (!row_ok) words = v4u{0u, 0u, 0u, 0u};
      chunk[t][rb] = words;
    }
  }
#pragma unroll
  for (int t = 0; t < kLaneTilesPerWave; ++t) {
    if (first_tile + t >= key_tiles) break;  // wave-uniform
    // word s of the tile goes to lane s, 32 bits at a time, straight from the scalar registers
    uint32_t mine_low = 0, mine_high = 0;
    uint64_t every = ~uint64_t{0}, any = 0;  // what all words of the tile / at least one of them hold
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
      for (int group = 0; group < 2; ++group) {  // b'
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint64_t first = __ballot(((chunk[t][rb][group * 2] >> (8 * r)) & 0xffu) != 0);
          const uint64_t second = __ballot(((chunk[t][rb][group * 2 + 1] >> (8 * r)) & 0xffu) != 0);
          every &= first & second;
          any |= first | second;
          const int low_slot = rb * 16 + group * 4 + r;        // b4 = b'
          const int high_slot = rb * 16 + (2 + group) * 4 + r;  // b4 = 2 + b'
          write_lane(mine_low, static_cast<uint32_t>(first), low_slot);
          write_lane(mine_high, static_cast<uint32_t>(second), low_slot);
          write_lane(mine_low, static_cast<uint32_t>(first >> 32), high_slot);
          write_lane(mine_high, static_cast<uint32_t>(second >> 32), high_slot);
        }
      }
    }
    const uint64_t mine = mine_low | (static_cast<uint64_t>(mine_high) << 32);
    if (lane < 32) out[static_cast<int64_t>(first_tile + t) * 32 + lane] = mine;
    if (lane == 0) {
      classes[(static_cast<int64_t>(plane) * query_waves + query_wave) * key_tiles + first_tile + t] =
          every == ~uint64_t{0} ? kLaneTileVisible : any == 0 ? kLaneTileHidden : kLaneTileMixed;
    }
  }
}

}  // namespace

// Tile lists of the mask: grid (query blocks, planes), one wavefront.  A tile is listed for a
// block of 128 queries unless all four of its 32-query classes say "no visible key"; entry
// [tiles] of a list holds its length (the layout the attention kernel reads for key-mask
// tiles).  A block that sees nothing keeps an empty list: its rows come out as zeros.
__global__ __launch_bounds__(64) void mask_tile_lists_kernel(const int32_t* __restrict__ classes,
                                                            int32_t* __restrict__ lists, int key_tiles,
                                                            int query_blocks) {
  const int lane = threadIdx.x;
  const int block = blockIdx.x, plane = blockIdx.y;
  const int32_t* wave_classes = classes + (static_cast<int64_t>(plane) * query_blocks + block) * 4 * key_tiles;
  int32_t* list = lists + (static_cast<int64_t>(plane) * query_blocks + block) * (key_tiles + 1);
  int count = 0;
  for (int first = 0; first < key_tiles; first += 64) {
    const int tile = first + lane;
    bool listed = false;
    if (tile < key_tiles) {
#pragma unroll
      for (int w = 0; w < 4; ++w) listed = listed || wave_classes[w * key_tiles + tile] != kLaneTileHidden;
    }
    const uint64_t ballot = __ballot(listed);
    if (listed) list[count + __popcll(ballot & ((uint64_t{1} << lane) - 1))] = tile;
    count += __popcll(ballot);
  }
  if (lane == 0) list[key_tiles] = count;
}

size_t mask_lane_words(int batch, int heads, int q_len, int k_len) {
  const size_t query_waves = (static_cast<size_t>(q_len) + 127) / 128 * 4;
  const size_t key_tiles = (static_cast<size_t>(k_len) + 63) / 64;
  return static_cast<size_t>(batch) * heads * query_waves * key_tiles * 32;
}

// The buffer of one mask: the lane words, then one 32-bit class per 32 words (kLaneTile...),
// then per mask plane and block of 128 queries the list of tiles with a visible key.
size_t mask_lane_class_offset(int batch, int heads, int q_len, int k_len) {
  return mask_lane_words(batch, heads, q_len, k_len) * sizeof(uint64_t);
}
size_t mask_tile_list_offset(int batch, int heads, int q_len, int k_len) {
  const size_t classes = mask_lane_words(batch, heads, q_len, k_len) / 32;
  return mask_lane_class_offset(batch, heads, q_len, k_len) + (classes * sizeof(int32_t) + 7) / 8 * 8;
}
size_t mask_lane_bytes(int batch, int heads, int q_len, int k_len) {
  const size_t query_blocks = (static_cast<size_t>(q_len) + 127) / 128;
  const size_t key_tiles = (static_cast<size_t>(k_len) + 63) / 64;
  const size_t lists = static_cast<size_t>(batch) * heads * query_blocks * (key_tiles + 1);
  return mask_tile_list_offset(batch, heads, q_len, k_len) + (lists * sizeof(int32_t) + 7) / 8 * 8;
}

int launch_mask_lanes(const void* mask, uint64_t* lanes, int batch, int heads, int q_len, int k_len,
                      int64_t stride_b, int64_t stride_h, int64_t stride_q, hipStream_t stream) {
  const int query_waves = (q_len + 127) / 128 * 4;
  const int key_tiles = (k_len + 63) / 64;
  if (query_waves > 65535 || static_cast<int64_t>(batch) * heads > 65535)
    return fail("risa_prepare_mask_lanes: more query blocks or mask planes than one launch covers");
  const dim3 grid((key_tiles + 4 * kLaneTilesPerWave - 1) / (4 * kLaneTilesPerWave), query_waves, batch * heads);
  const bool aligned = reinterpret_cast<uintptr_t>(mask) % 16 == 0 && ((stride_b | stride_h | stride_q) & 15) == 0;
  auto kernel = aligned ? mask_lanes_kernel<true> : mask_lanes_kernel<false>;
  unsigned char* bytes = reinterpret_cast<unsigned char*>(lanes);
  int32_t* classes = reinterpret_cast<int32_t*>(bytes + mask_lane_class_offset(batch, heads, q_len, k_len));
  int32_t* lists = reinterpret_cast<int32_t*>(bytes + mask_tile_list_offset(batch, heads, q_len, k_len));
  kernel<<<grid, 256, 0, stream>>>(static_cast<const uint8_t*>(mask), lanes, classes, heads, q_len, k_len,
                                   key_tiles, query_waves, stride_b, stride_h, stride_q);
  mask_tile_lists_kernel<<<dim3(query_waves / 4, batch * heads), 64, 0, stream>>>(classes, lists, key_tiles,
                                                                              query_waves / 4);
  return check_launch("risa_prepare_mask_lanes");
}

int launch_key_bias(const void* mask, float* bias, int batch, int heads, int length, int padded,
                    int64_t stride_b, int64_t stride_h, int64_t stride_k, int dtype,
                    hipStream_t stream) {
  const dim3 grid((padded + 255) / 256, heads, batch);
  key_bias_kernel<<<grid, 256, 0, stream>>>(mask, bias, length, padded, stride_b, stride_h, stride_k,
                                            dtype);
  return check_launch("risa_prepare_key_bias");
}

int launch_sort_rows(const float* masses, float* sorted_mass, int64_t* order, int rows, int tiles,
                     hipStream_t stream) {
  int padded = 2;
  while (padded < tiles) padded <<= 1;
  if (padded > kSortableTiles) return fail("risa_sort_select_retained_mass: more key tiles than one workgroup sorts");
  if (padded <= 1024) {
    sort_rows_kernel<64><<<rows, 64, static_cast<size_t>(padded) * 8, stream>>>(masses, sorted_mass, order, tiles, padded);
  } else {
    sort_rows_kernel<256><<<rows, 256, static_cast<size_t>(padded) * 8, stream>>>(masses, sorted_mass, order, tiles, padded);
  }
  return check_launch("risa_sort_select_retained_mass");
}

int launch_select_retained_mass(const SelectArgs& a, hipStream_t stream) {
  select_rows_kernel<<<(a.rows + 1) / 2, 64, 0, stream>>>(a.sorted_mass, a.descending_indices,
                                                          a.counts, a.support, a.row_totals, a.rows,
                                                          a.tiles, a.theta);
  offsets_summary_kernel<<<1, 256, 0, stream>>>(a.counts, a.row_totals, a.row_offsets, a.summary,
                                                a.rows);
  compact_rows_kernel<<<(a.rows + 3) / 4, 256, 0, stream>>>(a.support, a.row_offsets,
                                                            a.block_indices, a.rows, a.tiles);
  return check_launch("risa_select_retained_mass");
}

int launch_key_mask_tiles(const void* mask, int32_t* tiles, int batch, int heads, int length,
                          int tile_size, int64_t stride_b, int64_t stride_h, int64_t stride_k,
                          int dtype, hipStream_t stream) {
  const int count = (length + tile_size - 1) / tile_size;
  const dim3 grid(batch, heads);
  key_mask_tiles_kernel<<<grid, 256, count * sizeof(int), stream>>>(
      mask, tiles, heads, length, tile_size, stride_b, stride_h, stride_k, dtype);
  return check_launch("risa_prepare_key_mask_tiles");
}

}  // namespace risa
