// EWAH run/literal codec for bit-plane slices (gfx950).
//
// Stream format (one per slice), as in the reference (bsi_ops/csrc/cuda/bsi_cuda_kernels_ewah.cuh:5-33,
// 178-232; bsi_vector_utils.h:74): a sequence of [marker][literal words...], marker =
// run_bit | run_len << 1 | literal_count << 33 (32-bit run length, 31-bit literal count).  A slice
// whose compress flag is 0 is one marker with literal_count = W followed by its W words.
//
// Every kernel here gives one wave to one slice.  Encoding (size pass, emit pass): the wave classifies 64 words at
// a time (literal, zero fill, one fill); a marker starts at word 0 and at every clean word whose predecessor is a
// literal or a clean word of the other kind, so ballots of the three classes give, by population counts, every
// word's place in the stream and every marker's two counts -- no lane walks the slice.  Decoding: the markers of a
// stream form a chain (each one tells where the next sits), which the wave follows through a 64-word window of the
// stream held one word per lane (a lane broadcast per marker instead of a dependent memory load); runs are written
// and literal blocks copied by all lanes together.
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

// One wave encodes one slice of W words (out == nullptr: size pass only).  Returns the stream length in every lane.
// The stream is the reference's greedy one (bsi_cuda_kernels_ewah.cuh:118-232): [marker: run of equal clean words,
// only when the slice is flagged][literals up to the next clean word] ..., an unflagged slice being one marker with
// W literals.
__device__ __forceinline__ unsigned long long ewah_encode_wave(const unsigned long long* __restrict__ base, int W,
                                                               int compress, unsigned long long* __restrict__ out,
                                                               int lane) {
    const unsigned long long lt = (1ULL << lane) - 1ULL;  // lanes below this one
    unsigned long long n_starts = 0, n_lits = 0;          // markers / literal words before the current block
    // the segment that is open when a block begins: where it started, literals before it, its marker's place
    long long open_at = -1;
    unsigned long long open_lits = 0, open_pos = 0, open_bit = 0;
    unsigned long long prev_word = 0;
    bool prev_clean = false;
    for (int b = 0; b < W; b += BSI_WAVE) {
        const int i = b + lane;
        const bool valid = i < W;
        const unsigned long long v = valid ? base[i] : 0ULL;
        const bool clean = compress && valid && (v == 0ULL || v == ~0ULL);
        unsigned long long pv = __shfl_up(v, 1, BSI_WAVE);
        bool pc = __shfl_up(static_cast<int>(clean), 1, BSI_WAVE) != 0;
        if (lane == 0) {
            pv = prev_word;
            pc = prev_clean;
        }
        const bool start = valid && (i == 0 || (clean && (!pc || pv != v)));
        const bool lit = valid && !clean;
        const unsigned long long smask = __ballot(start), lmask = __ballot(lit), omask = __ballot(clean && v == ~0ULL);
        const unsigned long long starts_before = n_starts + __popcll(smask & lt);
        const unsigned long long lits_before = n_lits + __popcll(lmask & lt);
        if (out != nullptr) {
            if (lit) out[starts_before + (start ? 1ULL : 0ULL) + lits_before] = v;
            if (start && i > 0) {
                // this lane closes the segment before it: the nearest start below it in this block, else the open one
                const unsigned long long below = smask & lt;
                long long at;
                unsigned long long at_lits, at_pos, at_bit;
                if (below != 0ULL) {
                    const int L = 63 - __clzll(below);
                    const unsigned long long ltL = (1ULL << L) - 1ULL;
                    at = b + L;
                    at_lits = n_lits + __popcll(lmask & ltL);
                    at_pos = n_starts + __popcll(smask & ltL) + at_lits;
                    at_bit = (omask >> L) & 1ULL;
                } else {
                    at = open_at, at_lits = open_lits, at_pos = open_pos, at_bit = open_bit;
                }
                const unsigned long long seg_lits = lits_before - at_lits;
                const unsigned long long run_len = static_cast<unsigned long long>(i - at) - seg_lits;
                out[at_pos] = (run_len ? at_bit : 0ULL) | ((run_len & 0xFFFFFFFFULL) << 1) | (seg_lits << 33);
            }
        }
        if (smask != 0ULL) {  // the last start of this block is the open segment of the next one
            const int L = 63 - __clzll(smask);
            const unsigned long long ltL = (1ULL << L) - 1ULL;
            open_at = b + L;
            open_lits = n_lits + __popcll(lmask & ltL);
            open_pos = n_starts + __popcll(smask & ltL) + open_lits;
            open_bit = (omask >> L) & 1ULL;
        }
        n_starts += __popcll(smask);
        n_lits += __popcll(lmask);
        prev_word = __shfl(v, BSI_WAVE - 1, BSI_WAVE);
        prev_clean = __shfl(static_cast<int>(clean), BSI_WAVE - 1, BSI_WAVE) != 0;
    }
    if (out != nullptr && open_at >= 0 && lane == 0) {  // the last segment ends with the slice
        const unsigned long long seg_lits = n_lits - open_lits;
        const unsigned long long run_len = static_cast<unsigned long long>(W - open_at) - seg_lits;
        out[open_pos] = (run_len ? open_bit : 0ULL) | ((run_len & 0xFFFFFFFFULL) << 1) | (seg_lits << 33);
    }
    return n_starts + n_lits;
}

__global__ void ewah_size_kernel(const unsigned long long* __restrict__ words, int S, int W,
                                 const int* __restrict__ flags, unsigned long long* __restrict__ sizes) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t s = static_cast<int64_t>(blockIdx.x) * (kEwahBlock / BSI_WAVE) + (threadIdx.x >> 6);
    if (s >= S) return;
    const unsigned long long n = ewah_encode_wave(words + static_cast<size_t>(s) * W, W, flags[s], nullptr, lane);
    if (lane == 0) sizes[s] = n;
}

__global__ void ewah_emit_kernel(const unsigned long long* __restrict__ words, int S, int W,
                                 const int* __restrict__ flags, const unsigned long long* __restrict__ off,
                                 unsigned long long* __restrict__ out, int* __restrict__ out_len) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t s = static_cast<int64_t>(blockIdx.x) * (kEwahBlock / BSI_WAVE) + (threadIdx.x >> 6);
    if (s >= S) return;
    const unsigned long long n = ewah_encode_wave(words + static_cast<size_t>(s) * W, W, flags[s], out + off[s], lane);
    if (lane == 0) out_len[s] = static_cast<int>(n);
}

// one wave per stream
__global__ void ewah_decompress_batch_kernel(const unsigned long long* __restrict__ comp,
                                             const long long* __restrict__ off, const int* __restrict__ len, int S,
                                             int W, unsigned long long* __restrict__ out) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t s = static_cast<int64_t>(blockIdx.x) * (kEwahBlock / BSI_WAVE) + (threadIdx.x >> 6);
    if (s >= S) return;
    const long long o = off ? off[s] : 0;
    ewah_expand_wave(comp + o, len[s], W, out + static_cast<size_t>(s) * W, W, lane);
}

__global__ void ewah_decompress_one_kernel(const unsigned long long* __restrict__ in, int in_len, int W,
                                           unsigned long long* __restrict__ out) {
    ewah_expand_wave(in, in_len, W, out, W, static_cast<int>(threadIdx.x));
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
    hipLaunchKernelGGL(ewah_size_kernel, dim3((S + 3) / 4), dim3(kEwahBlock), 0, as_stream(stream),
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
    hipLaunchKernelGGL(ewah_emit_kernel, dim3((S + 3) / 4), dim3(kEwahBlock), 0, as_stream(stream),
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
    // one stream = a batch of one: `len` is read from a kernel argument instead of an array
    hipLaunchKernelGGL(ewah_decompress_one_kernel, dim3(1), dim3(BSI_WAVE), 0, as_stream(stream),
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
    hipLaunchKernelGGL(ewah_decompress_batch_kernel, dim3((S + 3) / 4), dim3(kEwahBlock), 0, as_stream(stream),
                       reinterpret_cast<const unsigned long long*>(comp), reinterpret_cast<const long long*>(off), len,
                       S, W, reinterpret_cast<unsigned long long*>(out));
    BSI_LAUNCH_CHECK("ewah_decompress_batch_kernel");
    return BSI_OK;
}
