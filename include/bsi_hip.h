/*
 * bsi_hip.h -- C ABI of libbsi_hip.so, the MI355X (gfx950) implementation of the bsi_ops
 * fixed-bit tensor-dot path: BSI builder, EWAH codec, weighted-popcount dot.
 *
 * Plain pointers and sizes only.  Every pointer named "device" must be memory of the current HIP
 * device; `stream` is a hipStream_t passed as void* (NULL = the default stream).  All work is
 * enqueued on `stream` and returns without synchronising unless stated.  Every function returns
 * BSI_OK or an error code; bsi_hip_last_error() gives the message of the calling thread's last
 * failure.  The caller owns every buffer.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference
 * tree, bsi_ops/csrc/cuda/).  The reference declares these as `extern "C" void launch_*`
 * (bsi_vector_cuda.cpp:91-242, bsi_cuda.cpp:29-57); the argument meaning is kept, `cudaStream_t`
 * becomes `void*`, and an error code is returned instead of nothing.
 *
 * Canonical bit-plane layout ("words"): uint64 [rows, slices, W64], W64 = ceil(d / 64); bit b of
 * word w of slice s is bit s of the two's-complement quantised value of element 64*w + b; bits
 * past d are zero.  A "chunk" is 256 elements = 4 words; chunk scales are float [rows, chunks].
 */
#ifndef BSI_HIP_H
#define BSI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BSI_OK 0
#define BSI_ERR_INVALID 1     /* bad argument (null pointer, negative size, unsupported combination) */
#define BSI_ERR_HIP 2         /* a HIP runtime call or kernel launch failed */
#define BSI_ERR_UNSUPPORTED 3 /* valid request that this build has no kernel for */

/* Input element types; same codes as the reference's `input_dtype` (bsi_vector_cuda.cpp:346-351). */
#define BSI_DTYPE_F32 0
#define BSI_DTYPE_F16 1
#define BSI_DTYPE_BF16 2

/* Arithmetic core of the dot. */
#define BSI_CORE_AUTO 0 /* MFMA when it applies, else VALU */
#define BSI_CORE_VALU 1 /* v_and_b32 + v_bcnt_u32_b32 on bit-planes staged in LDS */
#define BSI_CORE_MFMA 2 /* planes recombined to int8 in registers, v_mfma_i32_16x16x64_i8 */

/* Layout of the key planes handed to the dot. */
#define BSI_LAYOUT_CANONICAL 0 /* [R, Sb, W64] */
#define BSI_LAYOUT_TILED16 1   /* [ceil(R/16), chunks, Sb, 64, 1] words: see bsi_hip_tile_key_planes */
#define BSI_LAYOUT_INT8 2      /* int8 [R, chunks*256]: the recombined image bsi_hip_planes_to_int8 writes */
#define BSI_LAYOUT_INT8_TILED 3 /* the same bytes tiled by 64 rows and half-chunks: bsi_hip_planes_to_int8_tiled */

const char* bsi_hip_version(void);
const char* bsi_hip_last_error(void);
/* Name of the device architecture (e.g. "gfx950"), CU count and LDS bytes per workgroup. */
int bsi_hip_device_info(char* arch, int arch_len, int* cu_count, int* lds_bytes);

/* The identifier of the graph capture `stream` is recording into (hipStreamGetCaptureInfo), 0 when it is not
 * capturing.  Host-side callers that reuse work across launches (a query build shared by layers fed the same tensor)
 * key that reuse by it: what one capture recorded is not part of another capture's graph.  No counterpart in the
 * reference, which never records its launches. */
int bsi_hip_stream_capture_id(void* stream, unsigned long long* id);

/* ---------------------------------------------------------------- builder */

/* out[i] = round_half_away((double)(float)x[i] * dec_scale).
 * Replaces launch_quantize_round_to_int64_batch (bsi_cuda_kernels_quant.cuh:638-668). */
int bsi_hip_quantize_round_to_int64(const void* x_device, int dtype, int64_t total, double dec_scale,
                                    int64_t* out_device, void* stream);

/* out[i] = (int64)(float(x[i]) * factor): the product rounded to float, the conversion towards zero.  The value rule
 * of the reference's scalar entry points dot_product / vector_dot_product (bsiFunctions.cpp:265-271, :165-170:
 * static_cast<long>(m_a[i] * precision_factor_long)). */
int bsi_hip_quantize_trunc_to_int64(const void* x_device, int dtype, int64_t total, float factor, int64_t* out,
                                    void* stream);

/* Per-row / per-(row, 256-element chunk) shift and power-of-two scale from already rounded ints.
 * Replace launch_compute_row_shift_scale / launch_compute_chunk_shift_scale
 * (bsi_cuda_kernels_quant.cuh:670-700). shifts/scales are [Q] or [Q, chunks]. */
int bsi_hip_compute_row_shift_scale(const int64_t* ints_device, int64_t Q, int64_t d, int fixed_bits, float clip_k,
                                    int32_t* shifts_device, float* scales_device, void* stream);
int bsi_hip_compute_chunk_shift_scale(const int64_t* ints_device, int64_t Q, int64_t d, int chunks, int fixed_bits,
                                      float clip_k, int32_t* shifts_device, float* scales_device, void* stream);

/* In-place rounded right shift and clamp to fixed_bits.
 * Replace launch_apply_row_shift_clamp / launch_apply_chunk_shift_clamp (quant.cuh:702-734). */
int bsi_hip_apply_row_shift_clamp(int64_t* ints_device, int64_t Q, int64_t d, const int32_t* shifts_device,
                                  int fixed_bits, void* stream);
int bsi_hip_apply_chunk_shift_clamp(int64_t* ints_device, int64_t Q, int64_t d, int chunks,
                                    const int32_t* shifts_device, int fixed_bits, void* stream);

/* Same shift/scale rule computed straight from the float input (no int64 staging).
 * Replace launch_compute_row_shift_scale_from_input / launch_compute_chunk_shift_scale_from_input
 * (quant.cuh:490-557). */
int bsi_hip_compute_row_shift_scale_from_input(const void* x_device, int dtype, int64_t Q, int64_t d, double dec_scale,
                                               int fixed_bits, float clip_k, int32_t* shifts_device,
                                               float* scales_device, void* stream);
int bsi_hip_compute_chunk_shift_scale_from_input(const void* x_device, int dtype, int64_t Q, int64_t d, int chunks,
                                                 double dec_scale, int fixed_bits, float clip_k,
                                                 int32_t* shifts_device, float* scales_device, void* stream);

/* Round, shift, clamp and pack into canonical words [Q, slices, words_per_slice] in one pass.
 * Replace launch_quantize_shift_pack_row_batch / launch_quantize_shift_pack_chunk_batch
 * (quant.cuh:559-636). */
int bsi_hip_quantize_shift_pack_row_batch(const void* x_device, int dtype, int64_t Q, int64_t d, int slices,
                                          int words_per_slice, double dec_scale, int fixed_bits,
                                          const int32_t* shifts_device, uint64_t* words_device, void* stream);
int bsi_hip_quantize_shift_pack_chunk_batch(const void* x_device, int dtype, int64_t Q, int64_t d, int chunks,
                                            int slices, int words_per_slice, double dec_scale, int fixed_bits,
                                            const int32_t* shifts_device, uint64_t* words_device, void* stream);

/* Decimal mode (no fixed bits; the slice count follows the data).  From the rounded ints [Q, d]:
 * *max_abs_device = largest |value| of the batch (0 when all are zero) and row_negative_device[q] = 1
 * when row q holds a negative value.  The caller reads max_abs back, takes
 * S = min(64, bit_width(max_abs) + 2) (2 when all zero), packs with bsi_hip_pack_bits_batch and gives
 * rows with a negative value the two's-complement slice weights, the others the unsigned ones.
 * Replaces the ATen reductions of the non-fixed batch builder (bsi_vector_cuda.cpp:1088-1100, 1146-1152;
 * slice-count rule :746-754) and of the 1-D builder (:788-797). */
int bsi_hip_decimal_stats(const int64_t* ints_device, int64_t Q, int64_t d, uint64_t* max_abs_device,
                          int32_t* row_negative_device, void* stream);

/* int64 [Q, d] -> canonical words [Q, slices, words_per_slice] (low `slices` bits of each value).
 * Replaces launch_pack_bits_all_ballot_batch / launch_pack_bits_all_ballot (Q = 1)
 * (bsi_cuda_kernels_pack.cuh:176-230). */
int bsi_hip_pack_bits_batch(const int64_t* ints_device, int64_t Q, int64_t d, int slices, int words_per_slice,
                            uint64_t* words_device, void* stream);

/* The whole fixed-bit build of a [Q, d] batch in one call: shift/scale pass + quantise/pack pass
 * (one fused kernel when chunk_scale != 0).  chunk_scale != 0 gives shifts/scales [Q, ceil(d/256)],
 * else [Q].  Optional extra output `ints8_device` (may be NULL): the quantised values as int8
 * [Q, chunks*256] in the MFMA core's in-chunk element order (bsi_hip_planes_to_int8 gives the same).
 * Replaces the host orchestration bsi_cuda_build_fixed_query_words_fused
 * (bsi_vector_cuda.cpp:401-557) and, with chunk_scale = 0 and fixed_bits = 6, the key quantiser
 * + packer (bsi_vector_cuda.cpp:559-744, 1125-1141). */
int bsi_hip_build_fixed(const void* x_device, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits,
                        int chunk_scale, float clip_k, uint64_t* words_device, int32_t* shifts_device,
                        float* scales_device, int8_t* ints8_device, void* stream);

/* ---------------------------------------------------------------- EWAH */

/* counts[s] = popcount of slice s.  Replaces launch_slice_popcount_sum (ewah.cuh:71-81). */
int bsi_hip_slice_popcount_sum(const uint64_t* words_device, int S, int W, uint64_t* counts_device, void* stream);
/* flags[s] = (1 - (1-p)^128 - p^128 <= threshold), p = counts[s] / (64 W).
 * Replaces launch_compress_flags_from_density (ewah.cuh:104-115). */
int bsi_hip_compress_flags_from_density(const uint64_t* counts_device, int S, int W, double threshold,
                                        int32_t* flags_device, void* stream);
/* sizes[s] = number of u64 the encoder emits for slice s.  Replaces launch_ewah_size (ewah.cuh:164-175). */
int bsi_hip_ewah_size(const uint64_t* words_device, int S, int W, const int32_t* flags_device,
                      uint64_t* sizes_device, void* stream);
/* Emit marker + literal words of every slice at off[s]; out_len[s] = words written.
 * Marker = run_bit | run_len << 1 | literal_count << 33.  Replaces launch_ewah_emit (ewah.cuh:234-247). */
int bsi_hip_ewah_emit(const uint64_t* words_device, int S, int W, const int32_t* flags_device,
                      const uint64_t* off_device, uint64_t* out_device, int32_t* out_len_device, void* stream);
/* One stream -> W literal words.  Replaces launch_ewah_decompress (ewah.cuh:35-42). */
int bsi_hip_ewah_decompress(const uint64_t* in_device, int in_len, int W, uint64_t* out_device, void* stream);
/* S streams (stream s at comp + off[s], len[s] words) -> canonical [S, W]; the batched form the
 * hybrid query builder needs (the reference loops launch_ewah_decompress on the host,
 * bsi_cuda.cpp:402-414). */
int bsi_hip_ewah_decompress_batch(const uint64_t* comp_device, const int64_t* off_device, const int32_t* len_device,
                                  int S, int W, uint64_t* out_device, void* stream);

/* ---------------------------------------------------------------- dot */

/* Permute canonical key words [R, Sb, W64] into the streaming layout of the MFMA core:
 * word (r, j, 4c+g) goes to ((((r/16) * chunks + c) * Sb + j) * 64 + g*16 + r%16); rows past R and
 * words past W64 are zero.  out must hold ceil(R/16)*16 * Sb * chunks*4 words.
 * No counterpart in the reference (its kernels read the canonical layout through cp.async/TMA). */
int bsi_hip_tile_key_planes(const uint64_t* words_device, int64_t R, int Sb, int W64, uint64_t* out_device,
                            void* stream);

/* Canonical planes [rows, S, W64] -> int8 [rows, chunks*256]: value << (8 - S), bytes of a chunk in
 * the MFMA core's element order (element 32w + 8m + t of the chunk at byte 32w + 4t + m).
 * No counterpart in the reference. */
int bsi_hip_planes_to_int8(const uint64_t* words_device, int64_t rows, int S, int W64, int8_t* out_device,
                           void* stream);

/* The same bytes in the tiled key image [ceil(rows / 64)][2 chunks half-chunks][64 rows][128 bytes] (layout
 * BSI_LAYOUT_INT8_TILED, bsi_hip_int8_tiled_bytes bytes; rows padding the last tile are zero): the key rows a
 * workgroup reads for one half-chunk are contiguous, so a keyset that is not cache-resident (every layer of a
 * model but the last few) streams from HBM in whole pages instead of 128-byte pieces of 64 rows.
 * No counterpart in the reference. */
size_t bsi_hip_int8_tiled_bytes(int64_t rows, int W64);
int bsi_hip_planes_to_int8_tiled(const uint64_t* words_device, int64_t rows, int S, int W64, int8_t* out_device,
                                 void* stream);

/* Tuning knobs (process-wide, not thread-safe; set before launching).  No counterpart in the reference,
 * whose kernel selection is read from environment variables on every call (bsi_cuda_kernels_dot.cuh:2642). */
#define BSI_OPT_I8_TILE 1 /* tile of the int8-image kernel: 128 (128 keys x 128 queries), 12864 (128 x 64), 64 (64 x 64),
                             6432 (64 x 32) or 1284 (128 x 128 on four MFMA waves of 64 x 64 with one accumulator set);
                             0 (default) = chosen per call from the grid each tile would give on the 256 CUs */
#define BSI_OPT_DIGITS_ROUTE 2 /* bsi_hip_dot_digits: 1 = stacked digits and a combine pass, 2 = digits recombined in the
                                  accumulator where the int32 bound allows; 0 (default) = the cheaper by a cost estimate */
#define BSI_OPT_BUILD_ITEMS 3 /* (row, chunk) items per wave of the fused chunk-scale builder: 1, 2, 4 or 8; 0 (default)
                                 = chosen per call from the number of items */
#define BSI_OPT_OUTPUT_STORES 4 /* how the int8-image kernels store whole output tiles: 1 = plain stores (the output stays
                                   in the caches for the next kernel), 2 = nontemporal stores (it leaves them as it is
                                   written); 0 (default) = plain from the linear-layer entry points (bsi_hip_dot_bias,
                                   bsi_hip_dot_bias_warm, bsi_hip_linear), nontemporal from the other dot entry points */
#define BSI_OPT_I8_SPLIT 5 /* D-split of the int8-image dot (see bsi_hip_dot_attach_split_scratch): 1 = never, n >= 2 = n
                              segments (on the tile BSI_OPT_I8_TILE forces, 128 or 12864; 128 otherwise) whenever the
                              attached scratch holds them; 0 (default) = chosen per call by a cost model */
int bsi_hip_set_option(int option, int value);

/* Bytes of device workspace bsi_hip_dot needs for this shape and core (0 when none). */
size_t bsi_hip_dot_workspace_bytes(int64_t Q, int W64, int core);

/*
 * The fixed-bit weighted-popcount dot, out[q, r] = scale_inv * chain_c fmaf((float)I[q,r,c],
 * qscale[q,c] * Bw[r*Sb], acc), I[q,r,c] = sum_{i,j} +-(popc(A_i & B_j over chunk c) << (i+j)),
 * negative iff (i == Sa-1) xor (j == Sb-1).
 * Replaces launch_popcount_weighted_keys_literal_fused_multiq (bsi_cuda_kernels_dot.cuh:2616-3090)
 * and through it the fixed76 chunk-scale kernels (:1285-2307).
 *   A              canonical query words [Q, Sa, W64]
 *   A_ints8        optional int8 [Q, chunks*256] from bsi_hip_build_fixed (NULL: derived from A
 *                  into `workspace` when the MFMA core runs)
 *   A_chunk_scales float [Q, A_scale_stride]; A_scale_stride == chunks for per-chunk scales,
 *                  1 for one scale per row (broadcast over chunks)
 *   B              key words in `b_layout`; Bw float [R, Sb] slice weights (only Bw[r*Sb] is read, and its magnitude used: the row scale 2^shift_r)
 *   out            float [Q, R_total] (row stride R_total >= R); every element [q, r<R] is written
 *   chunk_ints     optional int32 [Q, R, chunks]: the integer accumulators I (parity checks)
 * Sa, Sb in [2, 8] for the MFMA core and [1, 63] for the VALU core (canonical or tiled16 key planes); the MFMA core
 * takes rows of up to 32768 chunks (2^23 elements: its 32-bit operand offsets), BSI_CORE_AUTO falls back to the VALU
 * core beyond that.
 */
int bsi_hip_dot(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride, int Sa,
                int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core, void* workspace,
                size_t workspace_bytes, void* stream);

/*
 * D-split of the int8-image dot.  A call of a few hundred query rows against a few thousand keys has fewer output
 * tiles of 128 x 128 than the GPU has CUs; smaller tiles fill the GPU but move twice the operand bytes per
 * multiply-add into the CUs.  With a scratch region attached, such a call runs the large tile with several
 * workgroups per output tile, each over its own run of chunks, and the tile's last workgroup adds the partial sums.
 * The result is the one sequential chunk chain of bsi_cuda_kernels_dot.cuh:1516-1540 bit for bit, not within a
 * tolerance: every operand of the chain is an integer times one power of two, so a chain whose values all stay below
 * 2^24 units never rounds and equals the exact sum in any order of addition; every workgroup measures the largest
 * magnitude its chain values take, and a tile whose segments do not all stay below 2^24 / segments units is computed
 * again by its last workgroup over all chunks in order.  No counterpart in the reference, whose grid is one workgroup
 * per 32 x 32 output tile (bsi_cuda_kernels_dot.cuh:2780-2993).
 *
 * bsi_hip_dot_attach_split_scratch names the region the CALLING THREAD's later dots (every entry point that reaches
 * the int8-image kernel: bsi_hip_dot, _bias, _bias_warm, _timed, bsi_hip_linear, bsi_hip_dot_ewah_batch) may use on
 * the current device; NULL / 0 detaches.  The region is `bytes` of device memory, 256-byte aligned, whose first
 * BSI_SPLIT_COUNTER_BYTES are ZERO when it is attached for the first time (hipMemset once after hipMalloc); every
 * launch that completes leaves them zero.  bsi_hip_dot_split_scratch_bytes() is the size that serves every shape the
 * choice can make.  Launches that use one region must not overlap on the GPU (one region per stream).
 */
#define BSI_SPLIT_COUNTER_BYTES 4096
/* Layout of those bytes, as uint32 words: one counter per output tile (a split launch has at most BSI_SPLIT_MAX_TILES
 * tiles), then two running totals that the kernels only ever add to: output tiles whose partial sums were added, and
 * output tiles that were computed again in chunk order (a caller may read or clear the totals between launches). */
#define BSI_SPLIT_MAX_TILES 1008
#define BSI_SPLIT_STAT_COMBINED 1008
#define BSI_SPLIT_STAT_RECOMPUTED 1009
size_t bsi_hip_dot_split_scratch_bytes(void);
int bsi_hip_dot_attach_split_scratch(void* scratch_device, size_t bytes);
/* What a chain-mode int8-image dot of this shape would do on the calling thread right now: *tile = 128 or 12864 and
 * *segments >= 2 for a D-split launch, *tile = the unsplit tile and *segments = 1 otherwise.  Host only. */
int bsi_hip_dot_split_plan(int64_t R, int64_t Q, int W64, int* tile, int* segments);

/* bsi_hip_dot on the matrix cores for callers that cannot allocate device memory or hold a workspace of their own
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The int8 query operands are derived from the planes A into a BSI_STATIC_SCRATCH_BYTES array inside the
 * library's device image (one per GPU, held until the process ends) instead of a caller's workspace; the call makes no
 * hipMalloc / hipFree and no other allocating call.  Q * ceil(W64 / 4) * 256 must not exceed BSI_STATIC_SCRATCH_BYTES
 * (BSI_ERR_INVALID otherwise; bsi_hip_dot with a workspace has no such limit).  Every call on a GPU writes the same
 * array: calls that overlap on one GPU (two streams, two threads) race, calls on one stream do not.  Nothing in the
 * array has to start at zero: each call overwrites the part it reads.  The FIRST call on a device (it looks the
 * array's address up) and the first call of each kernel it selects (the kernel's one-time LDS opt-in and code
 * load) do host-side set-up that a stream capture must not see: make one call of the same shape class (same key
 * layout, Q above or up to 32) outside the capture before recording it.  Arguments and results as bsi_hip_dot. */
#define BSI_STATIC_SCRATCH_BYTES (8u << 20)
int bsi_hip_dot_static_scratch(const uint64_t* A, const float* A_chunk_scales, int A_scale_stride, int Sa, int W64,
                               const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                               float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, void* stream);

/* bsi_hip_dot followed by out[q, r] += bias[r] (bias: float [R], may be NULL), the two steps of a BSI-linear
 * forward (scores = dot(...); scores + bias, verify_accuracy_bsi.py:185-209) in one call.  The sum is rounded as
 * the separate addition would round it; the matrix-core kernels add the bias in their epilogue, the others
 * are followed by a small addition kernel. */
int bsi_hip_dot_bias(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride, int Sa,
                     int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                     float scale_inv, int64_t R_total, const float* bias, float* out, int core, void* workspace,
                     size_t workspace_bytes, void* stream);

/* out[q, r] += bias[r] for q < Q, r < R on out float [Q, R_total]: the bias step of a BSI-linear forward
 * (scores + bias, verify_accuracy_bsi.py:193-195, a PyTorch addition in the reference) for the dots that do not
 * take a bias argument (bsi_hip_dot with chunk_ints, bsi_hip_dot_weighted). */
int bsi_hip_add_bias(float* out, const float* bias, int64_t Q, int64_t R, int64_t R_total, void* stream);

/* bsi_hip_dot_bias that also warms the memory-side cache for the NEXT dot: `warm` .. `warm + warm_bytes` (device
 * memory, typically the key operand of the layer that runs next) is read once, one access per 128-byte line, by
 * the int8-image kernel's loader waves after they have issued their last stage.  A keyset that is not cache-resident
 * costs that kernel about 15 to 35 % more than a resident one (its loads wait on HBM latency), and in a model
 * every keyset is cold by the time its layer comes round again; the hint turns those reads into cache hits.
 * Results are those of bsi_hip_dot_bias; kernels other than the int8-image one ignore the hint.
 * No counterpart in the reference. */
int bsi_hip_dot_bias_warm(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                          int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                          float scale_inv, int64_t R_total, const float* bias, float* out, int core, void* workspace,
                          size_t workspace_bytes, const void* warm, size_t warm_bytes, void* stream);

/* A whole BSI-linear layer for at most 4 activation rows (a decode step) in ONE launch: the chunk-scale query
 * build of bsi_hip_build_fixed (x [Q, d] of dtype, decimal_places, fixed_bits in [2, 8], no clipping) is done
 * inside the few-rows dot kernel -- every workgroup quantises the rows into LDS while its first key planes are
 * on their way -- and the result is that of bsi_hip_build_fixed followed by bsi_hip_dot_bias on the tiled planes,
 * bit for bit.  d must give a multiple of 4 words per slice (chunk scales), Sb must be 6, and the rows' int8
 * image and scales (260 bytes per row and 256 elements) must fit 96 KiB of LDS.  Replaces, for such calls, the sequence
 * build_bsi_queries_cuda_batch_packed + batch_dot_product_multiquery_cuda_batch_caps of a layer forward
 * (verify_accuracy_bsi.py:143-178). */
int bsi_hip_linear_few_rows(const void* x_device, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits,
                            const uint64_t* B_tiled, const float* Bw, int Sb, int64_t R, float scale_inv, int64_t R_total,
                            const float* bias, float* out, void* stream);

/* A BSI-linear layer in one call for any number of rows: bsi_hip_build_fixed (chunk scales, no clipping) into
 * `workspace`, then bsi_hip_dot_bias_warm on what it built -- the two launches a layer forward makes
 * (verify_accuracy_bsi.py:143-178: build_bsi_queries_cuda_batch_packed, then
 * batch_dot_product_multiquery_cuda_batch_caps), with one trip through the host binding instead of two and no
 * per-call operand allocations.  rebuild = 0 skips the build and reuses the workspace's contents (layers that
 * read the same activations).  workspace: bsi_hip_linear_workspace_bytes(Q, d, fixed_bits) bytes, 256-aligned,
 * owned by the caller; B / b_layout as for bsi_hip_dot (int8 image or planes); warm as for bsi_hip_dot_bias_warm. */
size_t bsi_hip_linear_workspace_bytes(int64_t Q, int64_t d, int fixed_bits);
int bsi_hip_linear(const void* x_device, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits, int rebuild,
                   void* workspace, size_t workspace_bytes, const uint64_t* B, int b_layout, const float* Bw, int Sb,
                   int64_t R, float scale_inv, int64_t R_total, const float* bias, float* out, int core, const void* warm,
                   size_t warm_bytes, void* stream);

/* 1 when bsi_hip_linear_few_rows, for this shape, issues the loads of the whole query build before its first key
 * loads (the case in which the launch costs the GPU no more than the dot alone), 0 when some of the build waits
 * behind the key traffic (then the one launch still saves host time, but build + dot is the faster pair on the
 * GPU).  A host-side query: no GPU work.  No counterpart in the reference. */
int bsi_hip_linear_few_rows_upfront(int64_t Q, int64_t d, int64_t R);

/* The same dot for ONE query whose slices are EWAH streams (the hybrid query form of
 * build_bsi_query_cuda_hybrid, bsi_cuda.cpp:386-431): stream s at comp_words + comp_off[s], comp_len[s]
 * words, decoded to W64 words per slice inside the kernel's load stage with the semantics of
 * ewah_decompress_kernel (bsi_cuda_kernels_ewah.cuh:5-33).  The reference decodes on the host side of the
 * dot (one <<<1,1>>> launch per slice, bsi_cuda.cpp:402-414) and feeds verbatim words to the kernel; this
 * entry point removes that pass.  Keys: tiled16 planes with Sb = 6.  out: float [R]; chunk_ints: optional
 * int32 [R, chunks]. */
int bsi_hip_dot_ewah_query(const uint64_t* comp_words, const int64_t* comp_off, const int32_t* comp_len, int Sa,
                           int W64, const float* A_chunk_scales, int A_scale_stride, const uint64_t* B_tiled,
                           const float* Bw, int Sb, int64_t R, float scale_inv, float* out, int32_t* chunk_ints,
                           void* stream);

/* The same dot for a BATCH of queries kept as EWAH streams (no counterpart in the reference, which compresses the
 * single hybrid query only and feeds verbatim words to its kernels, bsi_cuda.cpp:386-431): stream q * Sa + s, at
 * comp_words + comp_off[q * Sa + s] with comp_len[q * Sa + s] words, is slice s of query q, encoded as
 * bsi_hip_ewah_emit writes it and decoded with the semantics of ewah_decompress_kernel
 * (bsi_cuda_kernels_ewah.cuh:5-33).  The result is that of bsi_hip_dot_bias on the decoded planes, bit for bit.
 * Verbatim planes are never written; where the decode runs depends on the number of rows:
 *   - at most 32 rows on tiled16 6-plane keys (the bandwidth-bound regime): inside the dot kernel's load stage --
 *     every workgroup expands its 16 queries' streams into LDS planes, then streams the key planes once;
 *   - otherwise: a separate launch, ahead of the dot, decodes the streams into the int8 query image in `workspace`
 *     (bsi_hip_dot_ewah_batch_workspace_bytes: 1 byte per element, more than the 7/8 byte of verbatim planes), and
 *     the int8-image kernel contracts it.  (Every key-tile workgroup of the compute-bound kernel reads the whole
 *     query tile; decoding there would repeat the work once per key tile.)
 * Slices whose stream is the encoder's all-zero form are skipped, not expanded.
 * What it costs: streams are a STORAGE format here, not a faster route.  With chunk scales only the sign plane of
 * ReLU'd activations and the top planes of outlier chunks compress (Q512 x D8192 after ReLU: 3.28 MB stored against
 * 3.74 MB verbatim), and the decode launch adds to the dot: Q512 x R2048 x D8192 25 us from streams against 16.3 us
 * on the int8 image the fused builder writes (bsi_hip_build_fixed) and 23.7 us from verbatim planes without that
 * image; 16 rows x R4096 x D4096 9.7 us against 5.7 us.  A caller that has the activations should build the image.
 * B / b_layout / Bw / out / chunk_ints / bias as for bsi_hip_dot and bsi_hip_dot_bias; Sa, Sb in [2, 8]. */
size_t bsi_hip_dot_ewah_batch_workspace_bytes(int64_t Q, int W64);
int bsi_hip_dot_ewah_batch(const uint64_t* comp_words, const int64_t* comp_off, const int32_t* comp_len, int Sa, int W64,
                           const float* A_chunk_scales, int A_scale_stride, const uint64_t* B, int b_layout,
                           const float* Bw, int Sb, int64_t R, int64_t Q, float scale_inv, int64_t R_total,
                           const float* bias, float* out, int32_t* chunk_ints, void* workspace, size_t workspace_bytes,
                           void* stream);

/* Weighted-slice dot for operands with arbitrary per-slice float weights (decimal-mode operands, whose
 * slice count follows the data, or fixed-bit operands without chunk scales):
 *   out[q, idx[r]] = float(sum_{i,j,w} popcount(A[q,i,w] & B[r,j,w]) * double(Aw[q,i] * Bw[r,j])) * scale_inv
 * A [Q, Sa, W64], Aw [Q, Sa], B [R, Sb, W64] (canonical or tiled16), Bw [R, Sb], Sa, Sb in [1, 64];
 * key_indices (may be NULL = identity) maps row r of B to its output column, as the reference's keys grouped
 * by slice count need (bsi_cuda.cpp:956-1000).  The sum is exact in float64 while it stays below 2^53 and is
 * rounded once, where the reference adds the same terms in fp32 in an order set by its launch shape (the two agree
 * bit for bit while every fp32 partial sum stays below 2^24, and to the reference order's own rounding error beyond).
 * Replaces launch_popcount_weighted_keys_literal_fused_multiq without chunk scales
 * (bsi_cuda_kernels_dot.cuh:58-190 fallback kernel, :211-1283 tensor-core kernel, dispatch :2575-3090). */
int bsi_hip_dot_weighted(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B, int b_layout,
                         const float* Bw, int Sb, int64_t R, int64_t Q, const int64_t* key_indices, float scale_inv,
                         int64_t R_total, float* out, void* stream);

/* The same weighted sum, unscaled and unrounded, as float64: out[q, idx[r]] = sum of popcount * (Aw * Bw), exact
 * while its magnitude stays below 2^53.  The double results of the reference's scalar entry points divide this
 * integer by 10^(decimals) on the host (bsiFunctions.cpp:368-373, :455-459: raw = vec->dot(other);
 * score = raw / scale). */
int bsi_hip_dot_weighted_f64(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B, int b_layout,
                             const float* Bw, int Sb, int64_t R, int64_t Q, const int64_t* key_indices, int64_t R_total,
                             double* out, void* stream);

/* Decimal-mode operands on the matrix cores.  bsi_hip_planes_to_int8_digits splits the two's-complement values
 * of S planes [rows, S, W64] into ceil(S / 7) int8 digit images out[digit][row][chunks * 256] (value =
 * sum_j digit_j * 128^j: unsigned 7-bit groups of planes, the top group sign-extended; in-chunk element order as
 * bsi_hip_planes_to_int8, no pre-shift).  bsi_hip_dot_digits multiplies the stacked digit images with one int8
 * GEMM into int32 (workspace: nq * Q * nk * R * 4 bytes, see bsi_hip_dot_digits_workspace_bytes) and puts the
 * digit products back together exactly in float64:
 *   out[q, idx[r]] = float(sum_{i,j} I_ij[q, r] * 2^(7 (i + j) - preshift) * Aw[q, 0] * Bw[r, 0]) * scale_inv (+ bias[r])
 * which is the weighted-slice dot of bsi_hip_dot_weighted whenever the slice weights are the builders' own
 * (w_s = 2^s times a per-row power of two, top slice negative for two's-complement rows).  A fixed-bit key image
 * from bsi_hip_planes_to_int8 is one digit pre-shifted by 8 - S bits; preshift is the sum of both operands'
 * pre-shifts (0 for digit images).  k_tiled != 0: K_digits is one digit in the tiled layout of
 * bsi_hip_planes_to_int8_tiled.  Rows of at most 2^17 elements.
 * No counterpart in the reference, whose decimal-mode dot is the popcount kernel cited at bsi_hip_dot_weighted. */
int bsi_hip_planes_to_int8_digits(const uint64_t* words_device, int64_t rows, int S, int W64, int8_t* out_device,
                                  void* stream);
size_t bsi_hip_dot_digits_workspace_bytes(int64_t Q, int nq, int64_t R, int nk);
int bsi_hip_dot_digits(const int8_t* A_digits, int nq, const float* Aw, int Sa, const int8_t* K_digits, int nk,
                       int preshift, const float* Bw, int Sb, int W64, int64_t R, int64_t Q,
                       const int64_t* key_indices, float scale_inv, int64_t R_total, const float* bias, float* out,
                       void* workspace, size_t workspace_bytes, int k_tiled, void* stream);

/* Runs fn-independent timing of `iters` back-to-back bsi_hip_dot launches between two HIP events
 * recorded on `stream`, synchronises, and returns the mean launch duration in microseconds.
 * Mirrors the reference's BSI_PROFILE event pair (bsi_cuda.cpp:713-722,798-806). */
int bsi_hip_dot_timed(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                      int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                      float scale_inv, int64_t R_total, float* out, int core, void* workspace, size_t workspace_bytes,
                      int iters, float* mean_us, void* stream);

/* Peak probes used by the benchmark to print measured next to published peaks: a pure
 * v_and/v_bcnt loop (returns lane-ops per second), a pure v_mfma_i32_16x16x64_i8 loop (int8
 * ops per second) and a streaming read (bytes per second).  Each synchronises. */
int bsi_hip_probe_valu_popcount(double* lane_ops_per_s, void* stream);
int bsi_hip_probe_mfma_i8(double* ops_per_s, void* stream);
/* The same MFMA loop on chosen operand data: random_operands = 0, the near-constant registers of
 * bsi_hip_probe_mfma_i8 (the chip's ceiling); 1, pseudo-random bytes shaped like the dot's int8 images.  The shader
 * clock follows the switching activity of the data, so the second is what real operands can sustain.  No counterpart
 * in the reference: a measuring aid. */
int bsi_hip_probe_mfma_i8_operands(int random_operands, double* ops_per_s, void* stream);
int bsi_hip_probe_stream_read(const void* buf_device, size_t bytes, double* bytes_per_s, void* stream);
/* Timeline build only (make -C bsipytorch_amd/csrc TIMELINE=1 -> libbsi_hip_timeline.so; the ordinary library returns
 * BSI_ERR_INVALID): copies out the wall-clock stamps (100 MHz ticks) that the last int8-image chunk-scale dot left,
 * 8 per workgroup for the first `workgroups` workgroups of its grid, in the order: MFMA wave entered, first stage in
 * LDS, chunk loop done, outputs stored, loader wave entered, loader wave done, first stage load issued, three stages
 * issued; a workgroup that has not run since the last read gives zeros (the read clears the stamps).  Synchronises the
 * device.  No counterpart in the reference: a measuring aid. */
int bsi_hip_timeline_read(unsigned long long* stamps_host, int workgroups);
/* The shader-clock counter (clock64: cycles of the clock the waves run on) read at the same points by the same launch,
 * same layout; not cleared (bsi_hip_timeline_read clears the wall-clock stamps, which tell which workgroups ran).  The
 * ratio of a cycle difference to a wall-clock difference is the clock the GPU held between two points.  Same builds,
 * same error from the ordinary one. */
int bsi_hip_timeline_read_cycles(unsigned long long* cycles_host, int workgroups);
/* What the int8-image kernel's operand path delivers: every CU streams an L2-resident part of buf_device (at least
 * 2 MiB are read) into LDS with LDS-direct 16-byte buffer loads, 96 KiB in flight per CU, all CUs at once; the result
 * is the aggregate rate over all CUs in bytes per second.  loader_pattern = 0: eight issuing waves per CU, contiguous
 * 1 KiB pieces (the path's best); 1: four issuing waves and pieces of 8 rows x 128 bytes out of 2 KiB rows, as the
 * loader waves fetch a row-major operand; 2: four issuing waves, contiguous pieces; 3: eight issuing waves, row
 * pieces.  Synchronises. */
int bsi_hip_probe_l2_to_lds(const void* buf_device, size_t bytes, int loader_pattern, double* bytes_per_s, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BSI_HIP_H */
