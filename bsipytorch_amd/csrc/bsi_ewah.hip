// EWAH run/literal codec for bit-plane slices (gfx950).
//
// Stream format (one per slice), as in the reference (bsi_ops/csrc/cuda/bsi_cuda_kernels_ewah.cuh:5-33,
// 178-232; bsi_vector_utils.h:74): a sequence of [marker][literal words...], marker =
// run_bit | run_len << 1 | literal_count << 33 (32-bit run length, 31-bit literal count).  A slice
// whose compress flag is 0 is one marker with literal_count = W followed by its W words.
//
// Encoding is two passes (size, emit) with a single walker per slice, as the stream is inherently
// sequential; parallelism comes from the number of slices (rows x planes), one lane per slice.
// The density pass uses one wave per slice.
#include "bsi_common.h"

namespace bsi {

constexpr int kEwahBlock = 256;

// one wave per slice
__global__ void slice_popcount_kernel(const unsigned long long* __restrict__ words, int S, int W,
                                      unsigned long long* __restrict__ counts) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t s = static_cast<int64_t>(blockIdx.x) * (kEwahBlock / BSI_WAVE) + (threadIdx.x >> 6);
    if (s >= S) return;
    const unsigned long long* base = words + static_cast<size_t>(s) * W;
    unsigned long long local = 0ULL;
    for (int w = lane; w < W; w += BSI_WAVE) local += static_cast<unsigned long long>(__popcll(base[w]));
    local = wave_sum_u64(local);
    if (lane == 0) counts[s] = local;
}

__global__ void compress_flags_kernel(const unsigned long long* __restrict__ counts, int S, int W, double threshold,
                                      int* __restrict__ flags) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= S) return;
    const double total_bits = static_cast<double>(W) * 64.0;
    double p = (total_bits > 0.0) ? (static_cast<double>(counts[s]) / total_bits) : 0.0;
    if (p < 0.0) p = 0.0;
    if (p > 1.0) p = 1.0;
    const double a = pow(1.0 - p, 128.0);
    const double b = pow(p, 128.0);
    const double M = 1.0 - a - b;
    flags[s] = (M <= threshold) ? 1 : 0;
}

// Walk one slice: (optional run of equal clean words)(literals up to the next clean word) ...
// out == nullptr: size pass.
__device__ __forceinline__ unsigned long long ewah_walk(const unsigned long long* __restrict__ base, int W,
                                                        int compress, unsigned long long* __restrict__ out) {
    unsigned long long o = 0ULL;
    int idx = 0;
    while (idx < W) {
        int run_len = 0, run_bit = 0;
        if (compress) {
            const unsigned long long v = base[idx];
            if (v == 0ULL || v == ~0ULL) {
                run_bit = (v == ~0ULL) ? 1 : 0;
                int k = idx;
                while (k < W && base[k] == v) ++k;
                run_len = k - idx;
                idx = k;
            }
        }
        int lit = 0;
        const int lit_start = idx;
        while (idx < W) {
            const unsigned long long v = base[idx];
            if (compress && (v == 0ULL || v == ~0ULL)) break;
            ++lit;
            ++idx;
        }
        if (out != nullptr) {
            out[o] = static_cast<unsigned long long>(run_bit) |
                     ((static_cast<unsigned long long>(run_len) & 0xFFFFFFFFULL) << 1) |
                     (static_cast<unsigned long long>(lit) << 33);
            for (int k = 0; k < lit; ++k) out[o + 1 + k] = base[lit_start + k];
        }
        o += 1ULL + static_cast<unsigned long long>(lit);
    }
    return o;
}

__global__ void ewah_size_kernel(const unsigned long long* __restrict__ words, int S, int W,
                                 const int* __restrict__ flags, unsigned long long* __restrict__ sizes) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= S) return;
    sizes[s] = ewah_walk(words + static_cast<size_t>(s) * W, W, flags[s], nullptr);
}

__global__ void ewah_emit_kernel(const unsigned long long* __restrict__ words, int S, int W,
                                 const int* __restrict__ flags, const unsigned long long* __restrict__ off,
                                 unsigned long long* __restrict__ out, int* __restrict__ out_len) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= S) return;
    out_len[s] = static_cast<int>(ewah_walk(words + static_cast<size_t>(s) * W, W, flags[s], out + off[s]));
}

__device__ __forceinline__ void ewah_decode(const unsigned long long* __restrict__ in, int in_len, int W,
                                            unsigned long long* __restrict__ out) {
    int idx = 0, o = 0;
    while (idx < in_len && o < W) {
        const unsigned long long rlw = in[idx++];
        const unsigned long long run_val = (rlw & 1ULL) ? ~0ULL : 0ULL;
        const unsigned int run_len = static_cast<unsigned int>((rlw >> 1) & 0xFFFFFFFFULL);
        const unsigned int lit = static_cast<unsigned int>(rlw >> 33);
        for (unsigned int k = 0; k < run_len && o < W; ++k) out[o++] = run_val;
        for (unsigned int k = 0; k < lit && o < W && idx < in_len; ++k) out[o++] = in[idx++];
    }
    while (o < W) out[o++] = 0ULL;
}

__global__ void ewah_decompress_batch_kernel(const unsigned long long* __restrict__ comp,
                                             const long long* __restrict__ off, const int* __restrict__ len, int S,
                                             int W, unsigned long long* __restrict__ out) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= S) return;
    const long long o = off ? off[s] : 0;
    ewah_decode(comp + o, len[s], W, out + static_cast<size_t>(s) * W);
}

__global__ void ewah_decompress_one_kernel(const unsigned long long* __restrict__ in, int in_len, int W,
                                           unsigned long long* __restrict__ out) {
    if (blockIdx.x == 0 && threadIdx.x == 0) ewah_decode(in, in_len, W, out);
}

}  // namespace bsi

using namespace bsi;

extern "C" int bsi_hip_slice_popcount_sum(const uint64_t* words, int S, int W, uint64_t* counts, void* stream) {
    BSI_REQUIRE(S >= 0 && W >= 0, "negative size");
    if (S == 0) return BSI_OK;
    BSI_REQUIRE(words && counts, "null pointer");
    const unsigned grid = static_cast<unsigned>((S + 3) / 4);
    hipLaunchKernelGGL(slice_popcount_kernel, dim3(grid), dim3(kEwahBlock), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(words), S, W,
                       reinterpret_cast<unsigned long long*>(counts));
    BSI_LAUNCH_CHECK("slice_popcount_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_compress_flags_from_density(const uint64_t* counts, int S, int W, double threshold,
                                                   int32_t* flags, void* stream) {
    BSI_REQUIRE(S >= 0 && W >= 0, "negative size");
    if (S == 0) return BSI_OK;
    BSI_REQUIRE(counts && flags, "null pointer");
    hipLaunchKernelGGL(compress_flags_kernel, dim3((S + 127) / 128), dim3(128), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(counts), S, W, threshold, flags);
    BSI_LAUNCH_CHECK("compress_flags_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_ewah_size(const uint64_t* words, int S, int W, const int32_t* flags, uint64_t* sizes,
                                 void* stream) {
    BSI_REQUIRE(S >= 0 && W >= 0, "negative size");
    if (S == 0) return BSI_OK;
    BSI_REQUIRE(words && flags && sizes, "null pointer");
    hipLaunchKernelGGL(ewah_size_kernel, dim3((S + 63) / 64), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(words), S, W, flags,
                       reinterpret_cast<unsigned long long*>(sizes));
    BSI_LAUNCH_CHECK("ewah_size_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_ewah_emit(const uint64_t* words, int S, int W, const int32_t* flags, const uint64_t* off,
                                 uint64_t* out, int32_t* out_len, void* stream) {
    BSI_REQUIRE(S >= 0 && W >= 0, "negative size");
    if (S == 0) return BSI_OK;
    BSI_REQUIRE(words && flags && off && out && out_len, "null pointer");
    hipLaunchKernelGGL(ewah_emit_kernel, dim3((S + 63) / 64), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(words), S, W, flags,
                       reinterpret_cast<const unsigned long long*>(off), reinterpret_cast<unsigned long long*>(out),
                       out_len);
    BSI_LAUNCH_CHECK("ewah_emit_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_ewah_decompress(const uint64_t* in, int in_len, int W, uint64_t* out, void* stream) {
    BSI_REQUIRE(in_len >= 0 && W >= 0, "negative size");
    if (W == 0) return BSI_OK;
    BSI_REQUIRE(out && (in || in_len == 0), "null pointer");
    hipLaunchKernelGGL(ewah_decompress_one_kernel, dim3(1), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(in), in_len, W,
                       reinterpret_cast<unsigned long long*>(out));
    BSI_LAUNCH_CHECK("ewah_decompress_one_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_ewah_decompress_batch(const uint64_t* comp, const int64_t* off, const int32_t* len, int S,
                                             int W, uint64_t* out, void* stream) {
    BSI_REQUIRE(S >= 0 && W >= 0, "negative size");
    if (S == 0 || W == 0) return BSI_OK;
    BSI_REQUIRE(comp && off && len && out, "null pointer");
    hipLaunchKernelGGL(ewah_decompress_batch_kernel, dim3((S + 63) / 64), dim3(64), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(comp), reinterpret_cast<const long long*>(off), len,
                       S, W, reinterpret_cast<unsigned long long*>(out));
    BSI_LAUNCH_CHECK("ewah_decompress_batch_kernel");
    return BSI_OK;
}
