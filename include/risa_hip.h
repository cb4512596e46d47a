/*
 * C ABI of the gfx950 (MI355X) implementation of RISA's quantized attention path.
 *
 * This header replaces the nanobind module `risa_attention._C`
 * (reference csrc/bindings.cpp:642-673) and the launcher interface behind it
 * (reference csrc/launchers.h:8-64).  Conventions shared by every entry point:
 *
 *   - All pointers are device pointers on the current HIP device unless stated
 *     otherwise.  The caller allocates and owns every buffer; the library
 *     borrows them for the duration of the asynchronous launch, never
 *     allocates, never synchronises and keeps no pointer after returning.
 *   - `stream` is a hipStream_t passed as void* (PyTorch-ROCm:
 *     torch.cuda.current_stream().cuda_stream).  Work is enqueued on it only.
 *   - Strides are in elements, as int64_t.
 *   - dtype codes: 0 = float32, 1 = float16, 2 = bfloat16, 3 = bool/uint8
 *     (masks only).  Output dtype codes: 1 or 2.
 *   - Return value 0 means success.  Any other value means the call was
 *     rejected or a launch failed; risa_last_error() returns the message for
 *     the calling host thread (the reference throws std::runtime_error with
 *     the same wording).
 */
#ifndef RISA_HIP_H
#define RISA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Message of the last failed call on this host thread ("" if none). */
const char* risa_last_error(void);

/* Library/ABI version, bumped when a signature or a packed layout changes. */
int risa_abi_version(void);

/*
 * Q/K preparation: anchor detection, rotation, per-group INT8 codes and scales.
 * Replaces launch_quantize_qk (reference csrc/launchers.h:13-19, implemented in
 * csrc/kernels/quantize_qk_impl.cuh:660-826) as called from risa_sdpa_quantize
 * (csrc/bindings.cpp:254-258).
 *   q [B,Hq,Lq,D], k [B,Hkv,Lk,D] with the given batch/head/token strides, last
 *   dim contiguous, D in {64,128,256}, base and strides 4-element aligned.
 *   q_int8 [B,Hq,Lq,D], k_int8 [B,Hkv,Lk,D] contiguous.
 *   q_scale [B,Hq,ceil(Lq/128)*(D==256?64:32)], k_scale [B,Hkv,ceil(Lk/cta_k)*4].
 *   anchor_indices int32 [B,Hkv]: receives the anchor row or -1.
 *   kv_permutation (nullable) int32 [B,Hkv,Lk]: key n is read from source token
 *   kv_permutation[b,h,n] (the reference's fused gather, csrc/kernels/
 *   quantize_gather.cu, bindings.cpp:195-272 permutation_ptr); anchors, codes
 *   and scales are those of the gathered K.  Every [b,h] row must be a bijection of
 *   0..Lk-1: the library does not check it, and the V range pass reads the rows in
 *   storage order (exact for a permutation only; a subset or a list with duplicates
 *   would give other V scales than a materialised gather).
 */
int risa_quantize_qk(const void* q, void* q_int8, float* q_scale, const void* k, void* k_int8,
                     float* k_scale, int batch, int q_heads, int q_len, int kv_heads, int k_len,
                     int head_dim, int cta_k, int64_t q_stride_b, int64_t q_stride_h,
                     int64_t q_stride_n, int64_t k_stride_b, int64_t k_stride_h,
                     int64_t k_stride_n, int input_dtype, int32_t* anchor_indices,
                     const int32_t* kv_permutation, void* stream);

/*
 * V preparation.  Replaces launch_quantize_v (reference csrc/launchers.h:30-34,
 * csrc/kernels/quantize_v_impl.cuh:314-409).
 *   v [B,Hkv,L,D] strided (16-byte aligned rows), out int8 [B*Hkv*D, padded] in
 *   the packed order documented at risa_unpack_order, scale/center [B*Hkv*D],
 *   tile_sum int32 [B*Hkv, padded/cta_k, D]: the accumulator seeds of the P*V
 *   product, 128 x the sum of the codes of each key tile (the zero-point term
 *   of the signed product) + 0x4B400000 (the bits of 1.5 * 2^23, which make the
 *   finished integer accumulator readable as a float); no reference counterpart,
 *   workspace of risa_quantize_v_workspace_bytes(...) bytes.
 *   kv_permutation (nullable) int32 [B,Hkv,L] as for risa_quantize_qk (a bijection per row).
 */
size_t risa_quantize_v_workspace_bytes(int batch, int heads, int length, int head_dim,
                                       int midpoint_affine);
int risa_quantize_v(const void* v, void* out, float* scale, float* center, int32_t* tile_sum,
                    void* workspace, size_t workspace_bytes, int batch, int heads, int length,
                    int head_dim, int padded_length, int cta_k, int64_t stride_b,
                    int64_t stride_h, int64_t stride_n, int input_dtype, int midpoint_affine,
                    const int32_t* kv_permutation, void* stream);

/*
 * V preparation for callers that cannot allocate: same arguments, kernels and results as
 * risa_quantize_v without the workspace, which is an array of
 * RISA_QUANTIZE_V_NOALLOC_MAX_BYTES (16 MiB) built into the library.  No counterpart in the reference: it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  The
 * call allocates nothing; the first call on each device resolves the array's address
 * (hipGetSymbolAddress), so make that call outside a capture.  Problems whose workspace
 * (risa_quantize_v_workspace_bytes) exceeds the array are rejected with an error.  All calls
 * on one GPU share the array: calls that overlap in time on the same GPU race (serialise
 * them on one stream); nothing in it has to be cleared between calls, every kernel writes
 * what it later reads.
 */
#define RISA_QUANTIZE_V_NOALLOC_MAX_BYTES (16u << 20)
int risa_quantize_v_noalloc(const void* v, void* out, float* scale, float* center, int32_t* tile_sum,
                            int batch, int heads, int length, int head_dim, int padded_length,
                            int cta_k, int64_t stride_b, int64_t stride_h, int64_t stride_n,
                            int input_dtype, int midpoint_affine, const int32_t* kv_permutation,
                            void* stream);

/*
 * Q, K and V preparation in one call.  Replaces risa_sdpa_quantize (reference
 * csrc/bindings.cpp:195-272), which also prepares all three operands at once.
 * Arguments as for risa_quantize_qk and risa_quantize_v (padded length =
 * ceil(k_len / cta_k) * cta_k; the workspace is the V workspace).  Same results as
 * the two separate calls, in two launches (three beyond 4096 tokens) instead of
 * five to seven.
 */
int risa_sdpa_quantize(const void* q, void* q_int8, float* q_scale, const void* k, void* k_int8,
                       float* k_scale, const void* v, void* v_int8, float* v_scale, float* v_center,
                       int32_t* v_tile_sum, void* v_workspace, size_t v_workspace_bytes, int batch,
                       int q_heads, int q_len, int kv_heads, int k_len, int head_dim, int cta_k,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b,
                       int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_b, int64_t v_stride_h,
                       int64_t v_stride_n, int input_dtype, int midpoint_affine,
                       int32_t* anchor_indices, const int32_t* kv_permutation, void* stream);

/*
 * Zero-point terms (128 x tile sums) of an already packed V matrix (for callers that build packed V
 * themselves, as reference tests/cuda/test_large_offsets.py:35-36 does).
 */
int risa_value_tile_sums(const void* v_int8, int32_t* tile_sum, int batch_heads, int head_dim,
                         int padded_length, int cta_k, void* stream);

/*
 * Writes into order[0..31] the token (0..31) stored at each byte position of a
 * 32-token group of packed V: order[16*h + 4*b + r] = 8*b + 4*h + r.  Host
 * call.  The reference's 16-token order (csrc/kernels/quantize_v_impl.cuh:47-52)
 * follows the NVIDIA mma fragment; this one follows the 32x32x32 INT8 MFMA.
 */
void risa_unpack_order(int32_t* order);

/*
 * Fused attention over prepared tensors: dense, sparse-support, block-mass
 * capture, custom / key-only masks, causal, optional LSE.  Replaces
 * launch_attention (reference csrc/launchers.h:44-55,
 * csrc/kernels/attention_dispatch.cu:113-296) as called from
 * risa_sdpa_prequantized (csrc/bindings.cpp:277-461).
 *   q_int8/k_int8 contiguous [B,H,L,D]; v_int8 [B*Hkv*D, padded];
 *   out [B,Hq,Lq,D] fp16/bf16 with the given batch/token/head strides (last
 *   dim contiguous; base 16-byte aligned, strides multiples of 8 elements: rows
 *   are written 16 bytes per lane); mask (nullable) expanded to [B,Hq,Lq,Lk] with its strides,
 *   query stride 0 selecting the key-only path; sparse_row_offsets int32
 *   [B*Hq*ceil(Lq/128)+1] and sparse_block_indices int32 (both or neither; the tile
 *   ids of every row ascending, without repeats and below the number of key tiles, as
 *   risa_select_retained_mass writes them: a row that lists every tile is walked as
 *   0, 1, 2, ... without being read, and only the last listed tile is treated as the
 *   one that may be partial);
 *   block_mass (nullable) float32 workspace laid out as mass
 *   [B*Hq*ceil(Lq/128), tiles] ++ full-tile stats [B*Hq, tiles-1, Lq, 2]
 *   (u32 sum of U8 probabilities, f32 tile maximum; tile-major so that the
 *   stores of neighbouring queries coalesce) ++ last-tile stats [rows, 2]
 *   (f32, f32) ++ state [rows, 2] (m, d), rows = B*Hq*Lq (same contents and
 *   total size as reference attention_int8.cuh:51-143, 871-898, whose full-tile
 *   stats are row-major); lse (nullable) float32
 *   [B,Hq,Lq]; key_mask_tiles (nullable) int32 [B,Hq,tiles+1] from
 *   risa_prepare_key_mask_tiles (ascending ids, count in the last entry; same
 *   ordering contract as the sparse lists); key_bias (nullable) float32 [Bm,Hm,padded keys]
 *   from risa_prepare_key_bias with its batch and head strides in elements (0
 *   for a broadcast extent): given together with a key-only mask (mask_stride_q
 *   0), the kernel stages this row per key tile instead of reading mask elements;
 *   mask_lanes (nullable) the lane words of a query-dependent boolean mask from
 *   risa_prepare_mask_lanes with their batch and head strides in 64-bit words (0
 *   for a broadcast extent): given together with that mask (unit key stride) and 64-key
 *   tiles, the kernel applies the words instead of reading mask elements.  The two strides
 *   also fix the layout of the buffer: a non-zero stride means the buffer was made for
 *   `batch` (resp. `q_heads`) planes, zero for one, and the classes and tile lists are
 *   looked up behind the words of that many planes, for this q_len and k_len; pass the
 *   buffer exactly as risa_prepare_mask_lanes filled it.
 */
int risa_attention(const void* q_int8, const void* k_int8, const void* v_int8, void* out,
                   const float* q_scale, const float* k_scale, const float* v_scale,
                   const float* v_center, const int32_t* v_tile_sum, const void* mask,
                   int64_t mask_stride_b, int64_t mask_stride_h, int64_t mask_stride_q,
                   int64_t mask_stride_k, int mask_dtype, int cta_k, int batch, int q_len,
                   int k_len, int q_heads, int kv_heads, int head_dim, int64_t out_stride_b,
                   int64_t out_stride_n, int64_t out_stride_h, float sm_scale, int out_dtype,
                   const int32_t* sparse_row_offsets, const int32_t* sparse_block_indices,
                   float* block_mass, int is_causal, float* lse, const int32_t* key_mask_tiles,
                   const float* key_bias, int64_t key_bias_stride_b, int64_t key_bias_stride_h,
                   const uint64_t* mask_lanes, int64_t mask_lanes_stride_b,
                   int64_t mask_lanes_stride_h, void* stream);

/*
 * Quantise and attend in one call.  Replaces risa_sdpa (reference
 * csrc/bindings.cpp:497-616): the calls above back to back on one stream, with
 * every intermediate buffer (codes, scales, accumulator seeds, anchors, the V
 * workspace, the key bias row and key tile list of a key-only mask) carved from
 * one caller-provided workspace of risa_sdpa_workspace_bytes(...) bytes (256-byte
 * aligned).  q/k/v are [B,H,L,D] with element strides, head_dim 64, 128 or 256;
 * out and the mask as for risa_attention; mask_batch / mask_heads are the mask's
 * own extents (1 where it broadcasts).  The size query takes the description of the
 * mask that will be passed (mask_dtype -1 for none): a key-only mask needs room for its
 * bias row and tile list, a boolean mask shared by several heads for its lane words.
 * sparse_row_offsets /
 * sparse_block_indices (both or neither, as for risa_attention) restrict the
 * attention to a retained-mass pattern: the reuse call of the sparse path
 * (reference src/risa_attention/sparse.py:150-191) in one call as well.
 */
size_t risa_sdpa_workspace_bytes(int batch, int q_heads, int q_len, int kv_heads, int k_len,
                                 int head_dim, int cta_k, int midpoint_affine, int mask_dtype,
                                 int64_t mask_stride_q, int64_t mask_stride_k, int mask_batch,
                                 int mask_heads);
int risa_sdpa(const void* q, const void* k, const void* v, void* out, void* workspace,
              size_t workspace_bytes, int batch, int q_heads, int q_len, int kv_heads, int k_len,
              int head_dim, int cta_k, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_n,
              int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_b,
              int64_t v_stride_h, int64_t v_stride_n, int64_t out_stride_b, int64_t out_stride_n,
              int64_t out_stride_h, float sm_scale, int input_dtype, int output_dtype,
              int midpoint_affine, const void* mask, int64_t mask_stride_b, int64_t mask_stride_h,
              int64_t mask_stride_q, int64_t mask_stride_k, int mask_dtype, int mask_batch,
              int mask_heads, int is_causal, const int32_t* sparse_row_offsets,
              const int32_t* sparse_block_indices, void* stream);

/*
 * Retained-mass selection over masses already sorted in descending order.
 * Replaces launch_select_retained_mass and retained_mass_selector_workspace_size
 * (reference csrc/launchers.h:56-63, csrc/kernels/sparse_selection.cu:129-159).
 * The scan needs no workspace here; the size query is kept for callers that
 * allocate one and always returns 0.
 */
size_t risa_selector_workspace_size(int row_count);
int risa_select_retained_mass(const float* sorted_mass, const int64_t* descending_indices,
                              int32_t* counts, uint8_t* support, double* row_totals,
                              int32_t* row_offsets, int32_t* block_indices, double* summary,
                              int row_count, int key_blocks, double theta, void* stream);

/*
 * The same selection over unsorted masses: sorts every row in the library first
 * (descending, ties by ascending tile id, i.e. the order of a stable descending sort; the
 * reference sorts with torch.sort in Python, src/risa_attention/sparse.py:24, and leaves ties
 * open), then selects as risa_select_retained_mass does.  sorted_mass float32 and
 * descending_indices int64, both [row_count, key_blocks], are outputs the caller provides.
 * Rows of up to risa_sortable_key_blocks() tiles; longer rows are rejected (sort outside and
 * call risa_select_retained_mass).
 */
int risa_sortable_key_blocks(void);
int risa_sort_select_retained_mass(const float* masses, float* sorted_mass, int64_t* descending_indices,
                                   int32_t* counts, uint8_t* support, double* row_totals,
                                   int32_t* row_offsets, int32_t* block_indices, double* summary,
                                   int row_count, int key_blocks, double theta, void* stream);

/*
 * Active key tiles of a broadcast key mask.  Replaces
 * launch_prepare_key_mask_tiles (reference csrc/launchers.h:39-43,
 * csrc/kernels/key_mask_tiles.cu:45-61).
 */
int risa_prepare_key_mask_tiles(const void* mask, int32_t* tiles, int batch, int q_heads,
                                int key_length, int tile_size, int64_t stride_b, int64_t stride_h,
                                int64_t stride_k, int mask_dtype, void* stream);

/*
 * Additive form of a key-only mask, in the exp2 domain: bias[b,h,key] =
 * mask * log2(e) for finite float entries, 0 for true, -inf for false, non-finite
 * and padded keys (key_length <= key < padded_length).  batch and heads are the
 * mask's own extents (1 where it broadcasts); bias is [batch,heads,padded_length]
 * float32.  No counterpart in the reference, whose kernel reads the mask per
 * score (csrc/kernels/attention_masks.cuh); the values are the ones it adds.
 */
int risa_prepare_key_bias(const void* mask, float* bias, int batch, int heads, int key_length,
                          int padded_length, int64_t stride_b, int64_t stride_h, int64_t stride_k,
                          int mask_dtype, void* stream);

/*
 * Lane words of a query-dependent boolean mask with unit key stride, for 64-key tiles:
 * lanes[b,h,w,t,16*rb+i] (64-bit words; b, h over the mask's own extents, w over
 * 4*ceil(q_len/128) blocks of 32 queries, t over ceil(k_len/64) key tiles) has bit l set
 * when query 32*w + l%32 may attend to key 64*t + 32*rb + 8*(i/4) + 4*(l/32) + i%4; no bit
 * is set past the last query or key.  The attention kernel applies one word per score
 * from scalar registers.  Behind the words of all planes the buffer holds one int32 class
 * per (b, h, w, t) (1: every bit of the 32 words set, 2: none, 0: neither) and, per
 * (b, h, block of 128 queries), the ascending list of the key tiles in which the block sees
 * at least one key, int32 [tiles + 1] with the length in the last entry: the attention
 * kernel (no causal flag, no sparse pattern, no capture) walks these lists, so tiles that
 * a block-structured mask hides from a whole query block cost nothing (they would add
 * zeros).  risa_mask_lanes_bytes returns the size of the whole buffer, or 0
 * when the form does not apply or does not pay: the mask is not boolean, the tiles are
 * not 64 keys, the head dim is 256 (that kernel holds its scores in another layout), the
 * key stride is not 1, the query stride is 0, the launch has no more workgroups of 128
 * queries than the device has compute units (it runs the sixteen-query kernel), or fewer than eight
 * (batch, head) pairs share each mask plane (the conversion reads the mask once, the
 * attention kernel would read it once per pair).  No counterpart in the reference, whose
 * kernel reads the mask per score (csrc/kernels/attention_masks.cuh:27-164); the
 * decisions are the ones it takes.
 */
size_t risa_mask_lanes_bytes(int mask_dtype, int head_dim, int cta_k, int64_t mask_stride_q,
                             int64_t mask_stride_k, int batch, int q_heads, int mask_batch,
                             int mask_heads, int q_len, int k_len);
int risa_prepare_mask_lanes(const void* mask, uint64_t* lanes, int mask_batch, int mask_heads,
                            int q_len, int k_len, int64_t stride_b, int64_t stride_h,
                            int64_t stride_q, void* stream);

/*
 * LSE anchor correction out[b,h,i] = scale * <q[b,h,i], k[b,h/G,anchor[b,h/G]]>.
 * Replaces launch_correct_lse (reference csrc/launchers.h:9-12,
 * csrc/kernels/lse_correction.cu:30-44).
 */
int risa_lse_shift(const void* q, const void* k, const int32_t* anchors, float* out, int batch,
                   int q_heads, int kv_heads, int q_len, int head_dim, int64_t q_stride_b,
                   int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_b, int64_t k_stride_h,
                   int64_t k_stride_n, float scale, int dtype, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* RISA_HIP_H */
