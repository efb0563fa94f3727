// libbsi_reference_launchers.so -- the reference's own `extern "C" launch_*` symbols, served by libbsi_hip.so.
//
// The reference's C++ sources (bsi_ops/csrc/cuda/bsi_cuda.cpp:29-57, bsi_vector_cuda.cpp:91-242) call these
// launchers, which it compiles from CUDA sources that cannot build for AMD GPUs.  A ROCm build of the reference
// extension links this library in place of bsi_cuda_kernels.cu: every function below has the reference's exact
// name and argument list (cudaStream_t is hipStream_t under ROCm's torch headers) and forwards to the C ABI of
// include/bsi_hip.h.  Plain host code: no torch, no kernels.
//
// One stream per device at a time, as the reference uses them: the dot's int8 query operands go to the library's
// per-device static scratch (or a per-device buffer of this module), and the query image remembered for registered
// keysets is per device too, so launchers running on two streams of one device at the same time would race on them.
//
// The launchers return void, as in the reference, so a failure is kept for the caller to ask about:
// bsi_launchers_last_status() / bsi_launchers_last_error() report the calling thread's last failing launcher
// (BSI_OK / "" when none failed since the last bsi_launchers_clear_status()), and the first failure of a process
// is also printed to stderr.
#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <atomic>
#include <cstdio>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/bsi_hip.h"

namespace {

thread_local int t_status = BSI_OK;
thread_local std::string t_error;
std::atomic<bool> g_reported{false};

void note(const char* launcher, int rc) {
    if (rc == BSI_OK) return;
    t_status = rc;
    t_error = std::string(launcher) + ": " + bsi_hip_last_error();
    if (!g_reported.exchange(true)) fprintf(stderr, "[bsi_hip] %s (code %d)\n", t_error.c_str(), rc);
}

void note_msg(const char* launcher, int rc, const char* msg) {
    t_status = rc;
    t_error = std::string(launcher) + ": " + msg;
    if (!g_reported.exchange(true)) fprintf(stderr, "[bsi_hip] %s (code %d)\n", t_error.c_str(), rc);
}

// The reference packers keep `value & value_mask`; its callers always pass the low `slices` bits
// (bsi_vector_cuda.cpp:1118-1124), which is what the library's packers keep.
bool mask_is_low_bits(unsigned long long value_mask, int slices) {
    const unsigned long long want = slices >= 64 ? ~0ULL : ((1ULL << slices) - 1ULL);
    return value_mask == want;
}

// Device workspace for the int8 query operands of a dot whose caller hands over planes only: the library's own
// static scratch when the operands fit it, else a buffer of this module that grows on demand and is kept (one per
// device; launches on one device are serialised by the reference's own single-stream use).
struct Workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool recorded = false;  // a launch recorded into a graph holds this address: the buffer is never freed
};
std::mutex g_ws_mutex;
Workspace g_ws[64];

// A buffer of this module that has to grow: the old one is freed once the device is idle (launches in flight may
// still read it) -- unless a graph has recorded a launch on it, which may be replayed at any later time: that buffer
// is left allocated for the rest of the process.
bool release_for_growth(void* ptr, bool recorded) {
    if (ptr == nullptr || recorded) return true;
    if (hipDeviceSynchronize() != hipSuccess) return false;
    (void)hipFree(ptr);
    return true;
}

// Growing the buffer synchronises the device and allocates memory, which a stream that is being captured into a
// graph must not see: while `stream` is capturing, a need beyond the present buffer is refused (run the call once
// eagerly first, and the buffer is there).
int workspace_for(size_t need, hipStream_t stream, void** ptr, size_t* bytes) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return BSI_ERR_HIP;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) return BSI_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace& w = g_ws[dev];
    if (w.bytes < need) {
        if (capturing != hipStreamCaptureStatusNone) return BSI_ERR_UNSUPPORTED;
        if (!release_for_growth(w.ptr, w.recorded)) return BSI_ERR_HIP;
        w = Workspace{};
        const size_t size = (need + (size_t{1} << 20) - 1) & ~((size_t{1} << 20) - 1);
        if (hipMalloc(&w.ptr, size) != hipSuccess) {
            w = Workspace{};
            return BSI_ERR_HIP;
        }
        w.bytes = size;
    }
    if (capturing != hipStreamCaptureStatusNone) w.recorded = true;
    *ptr = w.ptr;
    *bytes = w.bytes;
    return BSI_OK;
}

// ---- keysets registered for the fast dot
//
// The reference hands the dot launcher canonical key planes (bsi_cuda.cpp:724-746), which the library can only run on
// its plane-reading kernel.  A ROCm build of the reference registers a keyset once, after building it
// (build_bsi_keys_cuda, bsi_cuda.cpp:863-910): the int8 image of the same integers is derived into memory this module
// owns, and every later dot on those planes contracts the image instead -- the library's compute-bound kernel, the
// planes and the results unchanged.  The query side is remembered the same way: launch_quantize_shift_pack_chunk_batch
// also derives the int8 image of the planes it has just packed (one more launch in the build, none in the dot), and the
// dot finds it by the planes' address.
struct RegisteredKeys {
    const void* planes;
    int R, Sb, W, device;
    int8_t* image;
};
std::mutex g_keys_mutex;
std::vector<RegisteredKeys> g_keys;

struct QueryImage {  // per device: the int8 image of the query planes packed last
    const void* planes = nullptr;
    int64_t Q = 0;
    int Sa = 0, W = 0;
    int8_t* image = nullptr;
    size_t bytes = 0;
    bool recorded = false;  // as for Workspace
};
QueryImage g_query_image[64];

// Every other launcher that writes plane words: whatever image is remembered may describe planes that are being
// replaced at the same address.
void forget_query_image() {
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) g_query_image[dev].planes = nullptr;
}

const int8_t* registered_key_image(const void* planes, int R, int Sb, int W) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lock(g_keys_mutex);
    for (const RegisteredKeys& k : g_keys)
        if (k.planes == planes && k.R == R && k.Sb == Sb && k.W == W && k.device == dev) return k.image;
    return nullptr;
}

}  // namespace

extern "C" {

int bsi_launchers_forget_keys(const unsigned long long* B);

int bsi_launchers_register_keys(const unsigned long long* B, int R, int Sb, int W, hipStream_t stream) {
    static const char* kName = "bsi_launchers_register_keys";
    if (B == nullptr || R <= 0 || W <= 0 || Sb < 2 || Sb > 8) {
        note_msg(kName, BSI_ERR_INVALID, "needs key planes [R, Sb, W] with 2 <= Sb <= 8");
        return BSI_ERR_INVALID;
    }
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return BSI_ERR_HIP;
    (void)bsi_launchers_forget_keys(B);  // planes built anew at an address registered before
    int8_t* image = nullptr;
    const size_t bytes = static_cast<size_t>(R) * static_cast<size_t>((W + 3) / 4) * 256;
    if (hipMalloc(reinterpret_cast<void**>(&image), bytes) != hipSuccess) {
        note_msg(kName, BSI_ERR_HIP, "could not allocate the int8 key image");
        return BSI_ERR_HIP;
    }
    const int rc = bsi_hip_planes_to_int8(reinterpret_cast<const uint64_t*>(B), R, Sb, W, image, stream);
    if (rc != BSI_OK) {
        (void)hipFree(image);
        note(kName, rc);
        return rc;
    }
    std::lock_guard<std::mutex> lock(g_keys_mutex);
    g_keys.push_back(RegisteredKeys{B, R, Sb, W, dev, image});
    return BSI_OK;
}

// Forgets the keyset registered for these planes (when the reference's keyset capsule is destroyed).  The image is
// freed, which waits for work in flight on the device, so: not while a stream is being captured, and not while a
// graph that has recorded a dot against this keyset may still be replayed (as for the keyset's own tensors).
int bsi_launchers_forget_keys(const unsigned long long* B) {
    int8_t* image = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_keys_mutex);
        for (size_t i = 0; i < g_keys.size(); ++i)
            if (g_keys[i].planes == B) {
                image = g_keys[i].image;
                g_keys.erase(g_keys.begin() + static_cast<long>(i));
                break;
            }
    }
    if (image == nullptr) return BSI_OK;
    return hipFree(image) == hipSuccess ? BSI_OK : BSI_ERR_HIP;
}

int bsi_launchers_last_status(void) { return t_status; }
const char* bsi_launchers_last_error(void) { return t_error.c_str(); }
void bsi_launchers_clear_status(void) {
    t_status = BSI_OK;
    t_error.clear();
}

// ---- bsi_cuda.cpp:29-57

void launch_ewah_decompress(const unsigned long long* in, int in_len, int W, unsigned long long* out, hipStream_t stream) {
    forget_query_image();
    note("launch_ewah_decompress", bsi_hip_ewah_decompress(reinterpret_cast<const uint64_t*>(in), in_len, W,
                                                           reinterpret_cast<uint64_t*>(out), stream));
}

// The dot (bsi_cuda_kernels_dot.cuh:2616-3090).  With chunk scales the operands are fixed-bit (the reference only
// builds chunk scales for them, bsi_vector_cuda.cpp:980-994): Aw holds the two's-complement powers of two and
// Bw[r, j] = +-2^j * 2^shift_r, and the library's chunk-scale dot reads Bw[r, 0] as the key factor exactly as the
// reference's fixed76 kernels do (:1497).  Without chunk scales every slice pair is weighted by Aw[q, i] * Bw[r, j]
// (:58-190), which is bsi_hip_dot_weighted.  q_tile / r_tile are tuning hints of the CUDA kernels and are not used.
void launch_popcount_weighted_keys_literal_fused_multiq(const unsigned long long* A, const float* Aw,
                                                        const float* A_chunk_scales, int A_scale_stride, int Sa, int W,
                                                        const unsigned long long* B, const float* Bw, int Sb, int R,
                                                        int Q, int q_tile, int r_tile, const long long* indices_r,
                                                        const long long* indices_q, float scale_inv, int R_total,
                                                        float* out_global, hipStream_t stream) {
    static const char* kName = "launch_popcount_weighted_keys_literal_fused_multiq";
    (void)q_tile;
    (void)r_tile;
    if (indices_q != nullptr) {
        // the reference's callers pass the identity (nullptr) here (bsi_cuda.cpp:726)
        note_msg(kName, BSI_ERR_UNSUPPORTED, "a query index array is not supported (packed batches use the identity order)");
        return;
    }
    const bool chunk_scales = A_chunk_scales != nullptr && A_scale_stride > 0;
    if (!chunk_scales) {
        note(kName, bsi_hip_dot_weighted(reinterpret_cast<const uint64_t*>(A), Aw, Sa, W, reinterpret_cast<const uint64_t*>(B),
                                         BSI_LAYOUT_CANONICAL, Bw, Sb, R, Q, reinterpret_cast<const int64_t*>(indices_r),
                                         scale_inv, R_total, out_global, stream));
        return;
    }
    if (indices_r != nullptr) {
        note_msg(kName, BSI_ERR_UNSUPPORTED, "key index indirection with chunk scales (the reference's fixed-bit keysets are one group in identity order)");
        return;
    }
    const int core = (Sa >= 2 && Sa <= 8 && Sb >= 2 && Sb <= 8) ? BSI_CORE_MFMA : BSI_CORE_VALU;
    if (core == BSI_CORE_MFMA && Q > 32) {  // up to 32 rows the library streams the planes, which is the faster read there
        if (const int8_t* image = registered_key_image(B, R, Sb, W)) {
            int dev = 0;
            const int8_t* a8 = nullptr;
            if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) {
                const QueryImage& qi = g_query_image[dev];
                if (qi.planes == A && qi.Q == Q && qi.Sa == Sa && qi.W == W) a8 = qi.image;
            }
            if (a8 != nullptr) {
                note(kName, bsi_hip_dot(reinterpret_cast<const uint64_t*>(A), a8, A_chunk_scales, A_scale_stride, Sa, W,
                                        reinterpret_cast<const uint64_t*>(image), BSI_LAYOUT_INT8, Bw, Sb, R, Q, scale_inv,
                                        R_total, out_global, nullptr, core, nullptr, 0, stream));
                return;
            }
            const size_t qneed = bsi_hip_dot_workspace_bytes(Q, W, core);
            if (qneed <= BSI_STATIC_SCRATCH_BYTES) {
                note(kName, bsi_hip_dot_static_scratch(reinterpret_cast<const uint64_t*>(A), A_chunk_scales, A_scale_stride,
                                                       Sa, W, reinterpret_cast<const uint64_t*>(image), BSI_LAYOUT_INT8, Bw,
                                                       Sb, R, Q, scale_inv, R_total, out_global, nullptr, stream));
                return;
            }
        }
    }
    const size_t need = bsi_hip_dot_workspace_bytes(Q, W, core);
    if (need <= BSI_STATIC_SCRATCH_BYTES && core == BSI_CORE_MFMA) {
        note(kName, bsi_hip_dot_static_scratch(reinterpret_cast<const uint64_t*>(A), A_chunk_scales, A_scale_stride, Sa, W,
                                               reinterpret_cast<const uint64_t*>(B), BSI_LAYOUT_CANONICAL, Bw, Sb, R, Q,
                                               scale_inv, R_total, out_global, nullptr, stream));
        return;
    }
    void* ws = nullptr;
    size_t ws_bytes = 0;
    if (need > 0) {
        const int rc = workspace_for(need, stream, &ws, &ws_bytes);
        if (rc != BSI_OK) {
            note_msg(kName, rc, rc == BSI_ERR_UNSUPPORTED
                                    ? "the int8 query workspace would have to grow while the stream is being captured; run "
                                      "this call once outside the capture first"
                                    : "could not allocate the int8 query workspace");
            return;
        }
    }
    note(kName, bsi_hip_dot(reinterpret_cast<const uint64_t*>(A), nullptr, A_chunk_scales, A_scale_stride, Sa, W,
                            reinterpret_cast<const uint64_t*>(B), BSI_LAYOUT_CANONICAL, Bw, Sb, R, Q, scale_inv, R_total,
                            out_global, nullptr, core, ws, ws_bytes, stream));
}

// ---- bsi_vector_cuda.cpp:91-242

void launch_pack_bits_all_ballot(const long long* values, long long n, int slices, int words_per_slice,
                                 unsigned long long value_mask, unsigned long long* out, hipStream_t stream) {
    forget_query_image();
    if (!mask_is_low_bits(value_mask, slices)) {
        note_msg("launch_pack_bits_all_ballot", BSI_ERR_UNSUPPORTED, "value_mask must be the low `slices` bits");
        return;
    }
    note("launch_pack_bits_all_ballot", bsi_hip_pack_bits_batch(reinterpret_cast<const int64_t*>(values), 1, n, slices,
                                                                words_per_slice, reinterpret_cast<uint64_t*>(out), stream));
}

void launch_pack_bits_all_ballot_batch(const long long* values, int Q, long long n, int slices, int words_per_slice,
                                       unsigned long long value_mask, unsigned long long* out, hipStream_t stream) {
    forget_query_image();
    if (!mask_is_low_bits(value_mask, slices)) {
        note_msg("launch_pack_bits_all_ballot_batch", BSI_ERR_UNSUPPORTED, "value_mask must be the low `slices` bits");
        return;
    }
    note("launch_pack_bits_all_ballot_batch", bsi_hip_pack_bits_batch(reinterpret_cast<const int64_t*>(values), Q, n, slices,
                                                                      words_per_slice, reinterpret_cast<uint64_t*>(out), stream));
}

void launch_quantize_round_to_int64_batch(const void* input, int input_dtype, int64_t Q, int64_t d, double dec_scale,
                                          long long* out_ints, hipStream_t stream) {
    note("launch_quantize_round_to_int64_batch",
         bsi_hip_quantize_round_to_int64(input, input_dtype, Q * d, dec_scale, reinterpret_cast<int64_t*>(out_ints), stream));
}

void launch_compute_row_shift_scale(const long long* ints, int64_t Q, int64_t d, int fixed_bits, float clip_k, int* shifts,
                                    float* scales, hipStream_t stream) {
    note("launch_compute_row_shift_scale", bsi_hip_compute_row_shift_scale(reinterpret_cast<const int64_t*>(ints), Q, d, fixed_bits,
                                                                           clip_k, shifts, scales, stream));
}

void launch_compute_chunk_shift_scale(const long long* ints, int64_t Q, int64_t d, int chunks, int fixed_bits, float clip_k,
                                      int* shifts, float* scales, hipStream_t stream) {
    note("launch_compute_chunk_shift_scale", bsi_hip_compute_chunk_shift_scale(reinterpret_cast<const int64_t*>(ints), Q, d, chunks,
                                                                               fixed_bits, clip_k, shifts, scales, stream));
}

void launch_apply_row_shift_clamp(long long* ints, int64_t Q, int64_t d, const int* shifts, int fixed_bits, hipStream_t stream) {
    note("launch_apply_row_shift_clamp",
         bsi_hip_apply_row_shift_clamp(reinterpret_cast<int64_t*>(ints), Q, d, shifts, fixed_bits, stream));
}

void launch_apply_chunk_shift_clamp(long long* ints, int64_t Q, int64_t d, int chunks, const int* shifts, int fixed_bits,
                                    hipStream_t stream) {
    note("launch_apply_chunk_shift_clamp",
         bsi_hip_apply_chunk_shift_clamp(reinterpret_cast<int64_t*>(ints), Q, d, chunks, shifts, fixed_bits, stream));
}

void launch_compute_row_shift_scale_from_input(const void* input, int input_dtype, int64_t Q, int64_t d, double dec_scale,
                                               int fixed_bits, float clip_k, int* shifts, float* scales, hipStream_t stream) {
    note("launch_compute_row_shift_scale_from_input",
         bsi_hip_compute_row_shift_scale_from_input(input, input_dtype, Q, d, dec_scale, fixed_bits, clip_k, shifts, scales, stream));
}

void launch_compute_chunk_shift_scale_from_input(const void* input, int input_dtype, int64_t Q, int64_t d, int chunks,
                                                 double dec_scale, int fixed_bits, float clip_k, int* shifts, float* scales,
                                                 hipStream_t stream) {
    note("launch_compute_chunk_shift_scale_from_input",
         bsi_hip_compute_chunk_shift_scale_from_input(input, input_dtype, Q, d, chunks, dec_scale, fixed_bits, clip_k, shifts,
                                                      scales, stream));
}

void launch_quantize_shift_pack_row_batch(const void* input, int input_dtype, int64_t Q, int64_t d, int slices,
                                          int words_per_slice, unsigned long long value_mask, double dec_scale, int fixed_bits,
                                          const int* shifts, unsigned long long* out, hipStream_t stream) {
    forget_query_image();
    if (!mask_is_low_bits(value_mask, slices)) {
        note_msg("launch_quantize_shift_pack_row_batch", BSI_ERR_UNSUPPORTED, "value_mask must be the low `slices` bits");
        return;
    }
    note("launch_quantize_shift_pack_row_batch",
         bsi_hip_quantize_shift_pack_row_batch(input, input_dtype, Q, d, slices, words_per_slice, dec_scale, fixed_bits, shifts,
                                               reinterpret_cast<uint64_t*>(out), stream));
}

void launch_quantize_shift_pack_chunk_batch(const void* input, int input_dtype, int64_t Q, int64_t d, int chunks, int slices,
                                            int words_per_slice, unsigned long long value_mask, double dec_scale,
                                            int fixed_bits, const int* shifts, unsigned long long* out, hipStream_t stream) {
    forget_query_image();
    if (!mask_is_low_bits(value_mask, slices)) {
        note_msg("launch_quantize_shift_pack_chunk_batch", BSI_ERR_UNSUPPORTED, "value_mask must be the low `slices` bits");
        return;
    }
    const int rc = bsi_hip_quantize_shift_pack_chunk_batch(input, input_dtype, Q, d, chunks, slices, words_per_slice, dec_scale,
                                                           fixed_bits, shifts, reinterpret_cast<uint64_t*>(out), stream);
    note("launch_quantize_shift_pack_chunk_batch", rc);
    // The int8 image of these planes, for a dot against a registered keyset: kept per device, for the planes packed
    // last.  Its buffer grows outside stream captures only; without it the dot derives the image itself.
    int dev = 0;
    if (rc != BSI_OK || slices < 2 || slices > 8 || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
    QueryImage& qi = g_query_image[dev];
    qi.planes = nullptr;
    bool any_keys;
    {
        std::lock_guard<std::mutex> lock(g_keys_mutex);
        any_keys = !g_keys.empty();
    }
    if (!any_keys || Q <= 32) return;
    const size_t bytes = static_cast<size_t>(Q) * static_cast<size_t>((words_per_slice + 3) / 4) * 256;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) return;
    if (qi.bytes < bytes) {
        if (capturing != hipStreamCaptureStatusNone) return;
        const bool released = release_for_growth(qi.image, qi.recorded);
        qi.image = nullptr;
        qi.bytes = 0;
        qi.recorded = false;
        if (!released) return;
        const size_t size = (bytes + (size_t{1} << 20) - 1) & ~((size_t{1} << 20) - 1);
        if (hipMalloc(reinterpret_cast<void**>(&qi.image), size) != hipSuccess) {
            qi.image = nullptr;
            return;
        }
        qi.bytes = size;
    }
    if (capturing != hipStreamCaptureStatusNone) qi.recorded = true;
    if (bsi_hip_planes_to_int8(reinterpret_cast<const uint64_t*>(out), Q, slices, words_per_slice, qi.image, stream) != BSI_OK) return;
    qi.planes = out;
    qi.Q = Q;
    qi.Sa = slices;
    qi.W = words_per_slice;
}

void launch_slice_popcount_sum(const unsigned long long* words, int S, int W, unsigned long long* out_counts, hipStream_t stream) {
    note("launch_slice_popcount_sum", bsi_hip_slice_popcount_sum(reinterpret_cast<const uint64_t*>(words), S, W,
                                                                 reinterpret_cast<uint64_t*>(out_counts), stream));
}

void launch_compress_flags_from_density(const unsigned long long* counts, int S, int W, double threshold, int* out_flags,
                                        hipStream_t stream) {
    note("launch_compress_flags_from_density",
         bsi_hip_compress_flags_from_density(reinterpret_cast<const uint64_t*>(counts), S, W, threshold, out_flags, stream));
}

void launch_ewah_size(const unsigned long long* words, int S, int W, const int* flags, unsigned long long* sizes,
                      hipStream_t stream) {
    note("launch_ewah_size", bsi_hip_ewah_size(reinterpret_cast<const uint64_t*>(words), S, W, flags,
                                               reinterpret_cast<uint64_t*>(sizes), stream));
}

void launch_ewah_emit(const unsigned long long* words, int S, int W, const int* flags, const unsigned long long* off,
                      unsigned long long* out, int* out_len, hipStream_t stream) {
    note("launch_ewah_emit", bsi_hip_ewah_emit(reinterpret_cast<const uint64_t*>(words), S, W, flags,
                                               reinterpret_cast<const uint64_t*>(off), reinterpret_cast<uint64_t*>(out), out_len,
                                               stream));
}

}  // extern "C"
