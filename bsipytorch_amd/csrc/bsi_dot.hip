// Fixed-bit weighted-popcount dot for gfx950:  out[q,r] = scale_inv * sum_c  I[q,r,c] * qscale[q,c] * bscale[r]
// with I[q,r,c] = sum_{i,j} +-(popc(A_i & B_j over chunk c) << (i+j)) -- which is exactly the integer
// dot product of the two's-complement values the planes encode.  Two cores compute I:
//
//   VALU  v_and_b32 + v_bcnt_u32_b32 on bit-planes.  A 64x64 output tile per workgroup, key and
//         query plane tiles of one 256-element chunk staged in LDS, 4x4 outputs per lane, the key
//         planes of a half chunk held in VGPRs while the query planes stream through.
//   MFMA  planes are recombined to int8 (value << (8 - S), so the two's-complement sign bit lands on
//         the int8 sign bit) by an 8x8 bit-matrix transpose in registers, then
//         v_mfma_i32_16x16x64_i8 accumulates 2^(16-Sa-Sb) * I per chunk.  Keys are the M operand,
//         queries the N operand, so a lane owns one query column: its chunk scale is one value.
//
//         Kernels of this core, chosen by bsi_hip_dot from the key layout and the number of query rows:
//           dot_mfma_i8_kernel       compute-bound calls on the cached int8 image of the keys
//           dot_mfma_stream_kernel   a few query rows: streams the packed planes once (bandwidth-bound)
//           dot_mfma_stream_ewah_kernel   the same for one query handed over as EWAH streams
//           dot_mfma_ws_kernel       many rows on tiled planes (producer waves recombine the planes)
//           dot_mfma_kernel          canonical planes or slice counts other than 6
//
// Operands whose slice count follows the data (decimal mode) carry float slice weights instead of scales:
//   dot_weighted_kernel      popcounts per slice pair, summed exactly in float64 (any Sa, Sb <= 64)
//   dot_mfma_i8_kernel in its int32-sum mode on int8 digit images (planes_to_digits_kernel), the digits put back
//   together in the accumulator or by digits_combine_kernel: the same sum on the matrix cores
//
// Both feed the same fp32 epilogue, in chunk order:  acc = fmaf((float)I, qscale[q,c], acc), then
// out = (acc * bscale[r]) * scale_inv.  bscale is a power of two, so hoisting it out of the chain is
// exact and the result is bit-identical to fmaf((float)I, qscale*bscale, acc) of the reference
// kernel (bsi_ops/csrc/cuda/bsi_cuda_kernels_dot.cuh:1447-1540).
//
// This file: validation, kernel selection and the entry points of the fixed-bit dot.  The kernels live by family in
// bsi_dot_i8.hip (int8 image of the keys), bsi_dot_few_rows.hip (a few query rows, planes streamed once),
// bsi_dot_planes.hip (many rows on planes), bsi_dot_valu.hip (popcount cores, weighted slices, bias) and
// bsi_dot_layouts.hip (operand layouts); bsi_dot_device.h holds the device helpers they share.
#include "bsi_dot_internal.h"

using namespace bsi;

extern "C" int bsi_hip_set_option(int option, int value) {
    switch (option) {
        case BSI_OPT_DIGITS_ROUTE:
            BSI_REQUIRE(value >= 0 && value <= 2, "route must be 0, 1 or 2");
            g_digits_route = value;
            return BSI_OK;
        case BSI_OPT_I8_TILE:
            BSI_REQUIRE(value == 0 || value == 128 || value == 1284 || value == 12864 || value == 64 || value == 6432,
                        "tile must be 0, 128, 1284, 12864, 64 or 6432");
            g_i8_tile = value;
            return BSI_OK;
        case BSI_OPT_OUTPUT_STORES:
            BSI_REQUIRE(value >= 0 && value <= 2, "output stores must be 0 (by entry point), 1 (plain) or 2 (nontemporal)");
            g_output_stores = value;
            return BSI_OK;
        case BSI_OPT_I8_SPLIT:
            BSI_REQUIRE(value >= 0 && value <= 64, "split must be 0 (by cost), 1 (never) or a number of segments up to 64");
            g_i8_split = value;
            return BSI_OK;
        case BSI_OPT_BUILD_ITEMS:
            BSI_REQUIRE(value == 0 || value == 1 || value == 2 || value == 4 || value == 8, "items must be 0, 1, 2, 4 or 8");
            g_build_items = value;
            return BSI_OK;
        default:
            return fail(BSI_ERR_INVALID, "unknown option %d", option);
    }
}

extern "C" size_t bsi_hip_dot_workspace_bytes(int64_t Q, int W64, int core) {
    if (core == BSI_CORE_VALU || Q <= 0 || W64 <= 0) return 0;
    return static_cast<size_t>(Q) * static_cast<size_t>((W64 + 3) / 4) * 256;
}

extern "C" size_t bsi_hip_dot_split_scratch_bytes(void) {
    // one round of 256 workgroups, each with the partial sums of a 128 x 128 tile
    return kSplitCounterBytes + static_cast<size_t>(256) * 128 * 128 * sizeof(float);
}

extern "C" int bsi_hip_dot_attach_split_scratch(void* scratch_device, size_t bytes) {
    if (scratch_device == nullptr || bytes == 0) {
        t_split_scratch = nullptr;
        t_split_bytes = 0;
        t_split_device = -1;
        return BSI_OK;
    }
    BSI_REQUIRE((reinterpret_cast<uintptr_t>(scratch_device) & 255) == 0, "the split scratch must be 256-byte aligned");
    BSI_REQUIRE(bytes > kSplitCounterBytes, "a split scratch holds %zu bytes of counters and then the partial sums (got %zu bytes)",
                kSplitCounterBytes, bytes);
    int dev = -1;
    BSI_HIP_CHECK(hipGetDevice(&dev));
    t_split_scratch = static_cast<unsigned char*>(scratch_device);
    t_split_bytes = bytes;
    t_split_device = dev;
    return BSI_OK;
}

extern "C" int bsi_hip_dot_split_plan(int64_t R, int64_t Q, int W64, int* tile, int* segments) {
    BSI_REQUIRE(tile && segments && R >= 1 && Q >= 1 && W64 >= 1, "bad arguments");
    const int split_tile = choose_i8_split(R, Q, (W64 + 3) / 4, segments);
    *tile = split_tile != 0 ? split_tile : choose_i8_tile(R, Q);
    return BSI_OK;
}

// Validation, kernel selection and launch.  `bias` (optional) is added to every output; *bias_fused tells
// the caller whether the selected kernel did that in its own epilogue.
static int dot_launch(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                      int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                      float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core, void* workspace,
                      size_t workspace_bytes, void* stream, const float* bias, bool* bias_fused) {
    *bias_fused = false;
    BSI_REQUIRE(Q >= 0 && R >= 0, "negative Q or R");
    BSI_REQUIRE(W64 >= 1, "W64 must be >= 1");
    BSI_REQUIRE(Sa >= 1 && Sa <= 63 && Sb >= 1 && Sb <= 63, "Sa and Sb must be in [1, 63]");
    BSI_REQUIRE(R_total >= R, "R_total must be >= R");
    // per-row operands (slice weights, bias, chunk scales) are fetched with 32-bit byte offsets
    BSI_REQUIRE(R <= (1 << 25) && Q <= (1 << 25), "at most 2^25 key rows and query rows per call (got R = %lld, Q = %lld)",
                static_cast<long long>(R), static_cast<long long>(Q));
    // query tiles (32 rows in the smallest kernel tile) ride on the launch grid's second dimension, which holds 65535
    BSI_REQUIRE((Q + 31) / 32 <= 65535, "at most 65535 x 32 query rows per call (got Q = %lld); split the batch",
                static_cast<long long>(Q));
    BSI_REQUIRE(b_layout == BSI_LAYOUT_CANONICAL || b_layout == BSI_LAYOUT_TILED16 || b_layout == BSI_LAYOUT_INT8 ||
                    b_layout == BSI_LAYOUT_INT8_TILED,
                "unknown key layout %d", b_layout);
    if (Q == 0 || R == 0) return BSI_OK;
    const int chunks = (W64 + 3) / 4;
    BSI_REQUIRE(A_chunk_scales != nullptr, "A_chunk_scales is required (pass a [Q,1] array of row scales if there are no chunk scales)");
    BSI_REQUIRE(A_scale_stride == chunks || A_scale_stride == 1,
                "chunk scale stride mismatch: got %d expected %d (or 1 for row scales)", A_scale_stride, chunks);
    BSI_REQUIRE(B && Bw && out, "null pointer");
    BSI_REQUIRE(A || A_ints8, "neither query planes nor int8 queries given");
    hipStream_t st = as_stream(stream);

    // The matrix-core kernels address a tile's operand rows with 32-bit buffer offsets inside a descriptor of at most
    // 2 GiB: 128 rows of chunks * 256 bytes must stay below that.
    constexpr int kMfmaMaxChunks = 32768;
    const bool mfma_ok = (Sa >= 2 && Sa <= 8 && Sb >= 2 && Sb <= 8);
    if (core == BSI_CORE_AUTO) core = (mfma_ok && chunks <= kMfmaMaxChunks) ? BSI_CORE_MFMA : BSI_CORE_VALU;

    if (core == BSI_CORE_MFMA) {
        if (!mfma_ok) return fail(BSI_ERR_UNSUPPORTED, "MFMA core needs Sa, Sb in [2, 8] (got %d, %d)", Sa, Sb);
        if (chunks > kMfmaMaxChunks)
            return fail(BSI_ERR_UNSUPPORTED, "MFMA core takes rows of up to %d chunks of 256 elements (got %d)", kMfmaMaxChunks, chunks);
        const int8_t* A8 = A_ints8;
        BSI_REQUIRE((reinterpret_cast<uintptr_t>(A8) & 15) == 0 && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0,
                    "int8 queries / workspace must be 16-byte aligned");
        if (A8 == nullptr) {
            const size_t need = bsi_hip_dot_workspace_bytes(Q, W64, core);
            BSI_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                        "MFMA core without int8 queries needs %zu bytes of workspace (got %zu)", need, workspace_bytes);
            if (int rc = launch_planes_to_int8(A, Q, Sa, W64, static_cast<int8_t*>(workspace), st)) return rc;
            A8 = static_cast<const int8_t*>(workspace);
        }
        const int down_shift = 16 - Sa - Sb;
        if (b_layout == BSI_LAYOUT_INT8 || b_layout == BSI_LAYOUT_INT8_TILED) {
            BSI_REQUIRE((reinterpret_cast<uintptr_t>(B) & 15) == 0, "int8 key image must be 16-byte aligned");
            launch_mfma_i8(A8, A_chunk_scales, A_scale_stride, reinterpret_cast<const int8_t*>(B), Bw, Sb, chunks, R, Q,
                           down_shift, scale_inv, R_total, out, chunk_ints, bias, st,
                           b_layout == BSI_LAYOUT_INT8_TILED ? 1 : 0);
            BSI_LAUNCH_CHECK("dot_mfma_i8_kernel");
            *bias_fused = true;
            return BSI_OK;
        }
        const bool tiled = (b_layout == BSI_LAYOUT_TILED16);
        if (Sb == 6 && tiled && Q <= kStreamMaxQ) {
            launch_mfma_stream_by_shape(A8, A_chunk_scales, A_scale_stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total,
                                        out, chunk_ints, bias, st);
            BSI_LAUNCH_CHECK("dot_mfma_stream_kernel");
            *bias_fused = true;
            return BSI_OK;
        }
        const char* kernel = launch_mfma_planes(tiled, A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q,
                                                down_shift, scale_inv, R_total, out, chunk_ints, st);
        BSI_LAUNCH_CHECK(kernel);
        return BSI_OK;
    }

    if (core != BSI_CORE_VALU) return fail(BSI_ERR_INVALID, "unknown core %d", core);
    if (b_layout == BSI_LAYOUT_INT8 || b_layout == BSI_LAYOUT_INT8_TILED)
        return fail(BSI_ERR_UNSUPPORTED, "the popcount core reads key planes, not the int8 image");
    BSI_REQUIRE(A != nullptr, "VALU core needs the query planes");
    if (Sa == 7 && Sb == 6) {
        launch_valu76(b_layout == BSI_LAYOUT_TILED16, A, A_chunk_scales, A_scale_stride, B, Bw, W64, chunks, R, Q, scale_inv,
                      R_total, out, chunk_ints, st);
        BSI_LAUNCH_CHECK("dot_valu_kernel");
        return BSI_OK;
    }
    const int64_t total = Q * R;
    BSI_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, "too many outputs for one launch of the any-width kernel");
    launch_valu_generic(A, A_chunk_scales, A_scale_stride, Sa, B, Bw, Sb, W64, chunks, R, Q, scale_inv, R_total, out,
                        chunk_ints, b_layout == BSI_LAYOUT_TILED16 ? 1 : 0, st);
    BSI_LAUNCH_CHECK("dot_valu_generic_kernel");
    return BSI_OK;
}

namespace bsi {

int dot_with_bias(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                         int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                         float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core, void* workspace,
                         size_t workspace_bytes, void* stream, const float* bias) {
    bool fused = false;
    const int rc = dot_launch(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                              R_total, out, chunk_ints, core, workspace, workspace_bytes, stream, bias, &fused);
    if (rc != BSI_OK || bias == nullptr || fused || Q == 0 || R == 0) return rc;
    launch_add_bias(out, bias, Q, R, R_total, as_stream(stream));
    BSI_LAUNCH_CHECK("add_bias_kernel");
    return BSI_OK;
}

}  // namespace bsi

extern "C" int bsi_hip_dot(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                           int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R,
                           int64_t Q, float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core,
                           void* workspace, size_t workspace_bytes, void* stream) {
    return dot_with_bias(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                         R_total, out, chunk_ints, core, workspace, workspace_bytes, stream, nullptr);
}

extern "C" int bsi_hip_dot_bias(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales,
                                int A_scale_stride, int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw,
                                int Sb, int64_t R, int64_t Q, float scale_inv, int64_t R_total, const float* bias,
                                float* out, int core, void* workspace, size_t workspace_bytes, void* stream) {
    t_layer_output = 1;
    const int rc = dot_with_bias(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                                 R_total, out, nullptr, core, workspace, workspace_bytes, stream, bias);
    t_layer_output = 0;
    return rc;
}

extern "C" int bsi_hip_dot_bias_warm(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales,
                                     int A_scale_stride, int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw,
                                     int Sb, int64_t R, int64_t Q, float scale_inv, int64_t R_total, const float* bias,
                                     float* out, int core, void* workspace, size_t workspace_bytes, const void* warm,
                                     size_t warm_bytes, void* stream) {
    BSI_REQUIRE(warm != nullptr || warm_bytes == 0, "null warm-up region");
    g_warm_ptr = warm;
    g_warm_bytes = warm_bytes;
    t_layer_output = 1;
    const int rc = dot_with_bias(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                                 R_total, out, nullptr, core, workspace, workspace_bytes, stream, bias);
    g_warm_ptr = nullptr;
    g_warm_bytes = 0;
    t_layer_output = 0;
    return rc;
}

// ------------------------------------------------------------------ the dot without any allocation
// The int8 query operands that bsi_hip_dot derives into a caller's workspace go, here, into an array that is part
// of the library's device image: one copy per GPU, there from the moment the code object is loaded until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the device address it
// returns (one per device) is what the kernels get.
constexpr size_t kStaticScratchBytes = BSI_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::atomic<void*> g_scratch_ptr[64];  // per device: the array's address there, once looked up

static int static_scratch(void** out) {
    int dev = 0;
    BSI_HIP_CHECK(hipGetDevice(&dev));
    BSI_REQUIRE(dev >= 0 && dev < 64, "device index %d is beyond the 64 this entry point keeps addresses for", dev);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        BSI_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        BSI_REQUIRE(p != nullptr, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return BSI_OK;
}

extern "C" int bsi_hip_dot_static_scratch(const uint64_t* A, const float* A_chunk_scales, int A_scale_stride, int Sa,
                                          int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R,
                                          int64_t Q, float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints,
                                          void* stream) {
    BSI_REQUIRE(A != nullptr, "the query planes are required (the int8 operands are derived from them)");
    BSI_REQUIRE(Sa >= 2 && Sa <= 8 && Sb >= 2 && Sb <= 8, "the matrix-core dot needs Sa, Sb in [2, 8] (got %d, %d)", Sa, Sb);
    BSI_REQUIRE(Q >= 0 && W64 >= 1, "bad shape");
    const size_t need = bsi_hip_dot_workspace_bytes(Q, W64, BSI_CORE_MFMA);
    BSI_REQUIRE(need <= kStaticScratchBytes,
                "Q x padded D = %zu bytes of int8 query operands exceed the %zu-byte static scratch; use bsi_hip_dot "
                "with a workspace", need, kStaticScratchBytes);
    void* ws = nullptr;
    if (int rc = static_scratch(&ws)) return rc;
    return dot_with_bias(A, nullptr, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv, R_total,
                         out, chunk_ints, BSI_CORE_MFMA, ws, kStaticScratchBytes, stream, nullptr);
}

// Workspace of bsi_hip_linear: the query operands of one build (planes, shifts, scales, int8 image), each 256-aligned.
struct LinearWorkspace {
    size_t words, shifts, scales, ints8, total;
};
static LinearWorkspace linear_workspace(int64_t Q, int64_t d, int fixed_bits) {
    const size_t W = static_cast<size_t>((d + 63) / 64), chunks = static_cast<size_t>((d + 255) / 256);
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    LinearWorkspace w;
    w.words = 0;
    w.shifts = up(static_cast<size_t>(Q) * fixed_bits * W * 8);
    w.scales = w.shifts + up(static_cast<size_t>(Q) * chunks * 4);
    w.ints8 = w.scales + up(static_cast<size_t>(Q) * chunks * 4);
    w.total = w.ints8 + up(static_cast<size_t>(Q) * chunks * 256);
    return w;
}

extern "C" size_t bsi_hip_linear_workspace_bytes(int64_t Q, int64_t d, int fixed_bits) {
    if (Q <= 0 || d <= 0 || fixed_bits < 2 || fixed_bits > 8) return 0;
    return linear_workspace(Q, d, fixed_bits).total;
}

extern "C" int bsi_hip_linear(const void* x, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits, int rebuild,
                              void* workspace, size_t workspace_bytes, const uint64_t* B, int b_layout, const float* Bw,
                              int Sb, int64_t R, float scale_inv, int64_t R_total, const float* bias, float* out, int core,
                              const void* warm, size_t warm_bytes, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0 && d >= 1, "bad shape");
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 8, "fixed_bits must be in [2, 8] (got %d)", fixed_bits);
    const int W64 = static_cast<int>((d + 63) / 64);
    if (W64 % 4 != 0)
        return fail(BSI_ERR_UNSUPPORTED, "chunk scales need a multiple of 4 words per slice (d = %lld)", static_cast<long long>(d));
    if (Q == 0 || R == 0) return BSI_OK;
    const LinearWorkspace w = linear_workspace(Q, d, fixed_bits);
    BSI_REQUIRE(workspace != nullptr && workspace_bytes >= w.total, "workspace of %zu bytes needed, %zu given", w.total,
                workspace_bytes);
    BSI_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "workspace must be 256-byte aligned");
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    uint64_t* words = reinterpret_cast<uint64_t*>(ws + w.words);
    int32_t* shifts = reinterpret_cast<int32_t*>(ws + w.shifts);
    float* scales = reinterpret_cast<float*>(ws + w.scales);
    int8_t* ints8 = reinterpret_cast<int8_t*>(ws + w.ints8);
    if (rebuild) {
        const int rc = bsi_hip_build_fixed(x, dtype, Q, d, decimal_places, fixed_bits, 1, 0.0f, words, shifts, scales, ints8, stream);
        if (rc != BSI_OK) return rc;
    }
    return bsi_hip_dot_bias_warm(words, ints8, scales, W64 / 4, fixed_bits, W64, B, b_layout, Bw, Sb, R, Q, scale_inv, R_total,
                                 bias, out, core, nullptr, 0, warm, warm_bytes, stream);
}

extern "C" int bsi_hip_dot_timed(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales,
                                 int A_scale_stride, int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw,
                                 int Sb, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out, int core,
                                 void* workspace, size_t workspace_bytes, int iters, float* mean_us, void* stream) {
    BSI_REQUIRE(iters >= 1 && mean_us, "iters must be >= 1 and mean_us non-null");
    hipStream_t st = as_stream(stream);
    hipEvent_t e0, e1;
    BSI_HIP_CHECK(hipEventCreate(&e0));
    if (hipError_t ec = hipEventCreate(&e1); ec != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BSI_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(ec));
    }
    int rc = BSI_OK;
    hipError_t se = hipEventRecord(e0, st);
    for (int i = 0; i < iters && rc == BSI_OK; ++i)
        rc = bsi_hip_dot(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                         R_total, out, nullptr, core, workspace, workspace_bytes, stream);
    if (se == hipSuccess) se = hipEventRecord(e1, st);
    if (se == hipSuccess) se = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (se == hipSuccess) se = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != BSI_OK) return rc;
    if (se != hipSuccess) return fail(BSI_ERR_HIP, "event timing failed: %s", hipGetErrorString(se));
    *mean_us = ms * 1000.0f / static_cast<float>(iters);
    return BSI_OK;
}
