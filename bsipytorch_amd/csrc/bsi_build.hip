// BSI builder for gfx950: float -> rounded decimal ints -> block-floating shift -> fixed-bit
// two's-complement values -> bit-planes in canonical [rows, slices, W64] words.
//
// wave64 mapping: one wavefront owns one 256-element chunk of one row.  A lane loads elements
// lane, lane+64, lane+128, lane+192 of the chunk (four fully coalesced 256-byte wave loads), the
// chunk maximum is a butterfly reduction across the wave, and one 64-bit `__ballot` per slice per
// load IS the packed plane word (no lo/hi merge, no LDS, no block barrier).  The chunk-scale
// build is therefore a single pass over the activations.
//
// Arithmetic follows the reference's quantiser kernels (bsi_ops/csrc/cuda/bsi_cuda_kernels_quant.cuh:
// rounding :24-29, shift :82-108, rounded shift + clamp :205-226) and packer
// (bsi_cuda_kernels_pack.cuh:129-174).
#include "bsi_common.h"

namespace bsi {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / BSI_WAVE;

// ---------------------------------------------------------------- elementwise

template <typename T>
__global__ void round_to_int64_kernel(const T* __restrict__ x, int64_t total, double dec_scale,
                                      long long* __restrict__ out) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride)
        out[i] = round_scaled(load_as_float<T>(x, i), dec_scale);
}

// (long long)(x * factor) with the product rounded to float first and the conversion towards zero: the scalar
// entry points' value rule (bsiFunctions.cpp:265-271)
template <typename T>
__global__ void trunc_to_int64_kernel(const T* __restrict__ x, int64_t total, float factor, long long* __restrict__ out) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride)
        out[i] = static_cast<long long>(__fmul_rn(load_as_float<T>(x, i), factor));
}

__global__ void apply_shift_clamp_kernel(long long* __restrict__ ints, int64_t total, int64_t d, int chunks,
                                         const int* __restrict__ shifts, long long qmin, long long qmax) {
    // chunks == 0: one shift per row; else one per (row, col >> 8)
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t row = i / d;
        int shift;
        if (chunks > 0) {
            int c = static_cast<int>((i - row * d) >> 8);
            if (c >= chunks) c = chunks - 1;
            shift = shifts[row * chunks + c];
        } else {
            shift = shifts[row];
        }
        ints[i] = shift_clamp(ints[i], shift, qmin, qmax);
    }
}

// ---------------------------------------------------------------- shift / scale passes

// Source of rounded ints: either the float input (rounded on the fly) or staged int64.
template <typename T>
struct RoundedFromInput {
    const T* x;
    double dec_scale;
    __device__ __forceinline__ long long operator()(int64_t i) const { return round_scaled(load_as_float<T>(x, i), dec_scale); }
};
struct RoundedFromInts {
    const long long* v;
    __device__ __forceinline__ long long operator()(int64_t i) const { return v[i]; }
};

// One wave per (row, chunk).
template <typename Src>
__global__ void chunk_shift_scale_kernel(Src src, int64_t Q, int64_t d, int chunks, int fixed_bits, float clip_k,
                                         int* __restrict__ shifts, float* __restrict__ scales) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    if (wave >= Q * chunks) return;
    const int64_t row = wave / chunks;
    const int c = static_cast<int>(wave - row * chunks);
    const int64_t start = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS;
    int64_t valid = d - start;
    if (valid > BSI_CHUNK_ELEMS) valid = BSI_CHUNK_ELEMS;
    if (valid < 0) valid = 0;
    unsigned long long mx = 0ULL;
    double sum = 0.0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = k * BSI_WAVE + lane;
        if (e < valid) {
            const unsigned long long av = uabs_ll(src(row * d + start + e));
            if (av > mx) mx = av;
            sum += static_cast<double>(av);
        }
    }
    mx = wave_max_u64(mx);
    sum = wave_sum_f64(sum);
    if (lane == 0) {
        const int shift = (valid > 0) ? compute_shift(mx, sum, static_cast<int>(valid), fixed_bits, clip_k) : 0;
        shifts[wave] = shift;
        scales[wave] = static_cast<float>(1ULL << shift);
    }
}

// One block per row.
template <typename Src>
__global__ void row_shift_scale_kernel(Src src, int64_t Q, int64_t d, int fixed_bits, float clip_k,
                                       int* __restrict__ shifts, float* __restrict__ scales) {
    __shared__ unsigned long long smax[kWavesPerBlock];
    __shared__ double ssum[kWavesPerBlock];
    const int64_t row = blockIdx.x;
    if (row >= Q) return;
    unsigned long long mx = 0ULL;
    double sum = 0.0;
    for (int64_t e = threadIdx.x; e < d; e += kBlock) {
        const unsigned long long av = uabs_ll(src(row * d + e));
        if (av > mx) mx = av;
        sum += static_cast<double>(av);
    }
    mx = wave_max_u64(mx);
    sum = wave_sum_f64(sum);
    if ((threadIdx.x & (BSI_WAVE - 1)) == 0) {
        smax[threadIdx.x >> 6] = mx;
        ssum[threadIdx.x >> 6] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kWavesPerBlock; ++w) {
            if (smax[w] > mx) mx = smax[w];
            sum += ssum[w];
        }
        const int shift = compute_shift(mx, sum, static_cast<int>(d), fixed_bits, clip_k);
        shifts[row] = shift;
        scales[row] = static_cast<float>(1ULL << shift);
    }
}

// ---------------------------------------------------------------- pack

// Ballot-pack the four 64-element groups of one chunk held as v[0..3] (low `slices` bits valid) and
// store words 4c..4c+3 of every slice.  Lane s keeps slice s, so each active lane issues one
// contiguous run of stores.
__device__ __forceinline__ void ballot_pack_store(const unsigned long long v[4], int slices, int lane, int c,
                                                  int words_per_slice, unsigned long long* __restrict__ out_row) {
    unsigned long long keep[4] = {0ULL, 0ULL, 0ULL, 0ULL};
    for (int s = 0; s < slices; ++s) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const unsigned long long word = __ballot(((v[k] >> s) & 1ULL) != 0ULL);
            if (lane == (s & (BSI_WAVE - 1))) keep[k] = word;
        }
        if (lane == (s & (BSI_WAVE - 1))) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int w = c * BSI_CHUNK_WORDS + k;
                if (w < words_per_slice) out_row[static_cast<size_t>(s) * words_per_slice + w] = keep[k];
            }
        }
    }
}

// Quantise (given shifts) + pack.  chunks > 0: shift per (row, chunk); chunks == 0: shift per row.
// One wave per (row, group of 4 words).
template <typename Src, bool kQuantise>
__global__ void shift_pack_kernel(Src src, int64_t Q, int64_t d, int chunks, int slices, int words_per_slice,
                                  int fixed_bits, const int* __restrict__ shifts, unsigned long long* __restrict__ out) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int groups = (words_per_slice + BSI_CHUNK_WORDS - 1) / BSI_CHUNK_WORDS;
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    if (wave >= Q * groups) return;
    const int64_t row = wave / groups;
    const int c = static_cast<int>(wave - row * groups);
    const unsigned long long mask = (slices >= 64) ? ~0ULL : ((1ULL << slices) - 1ULL);
    int shift = 0;
    long long qmin = 0, qmax = 0;
    if (kQuantise) {
        int sc = c;
        if (chunks > 0 && sc >= chunks) sc = chunks - 1;
        shift = (chunks > 0) ? shifts[row * chunks + sc] : shifts[row];
        qmax = (1LL << (fixed_bits - 1)) - 1LL;
        qmin = -(1LL << (fixed_bits - 1));
    }
    unsigned long long v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t e = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS + k * BSI_WAVE + lane;
        v[k] = 0ULL;
        if (e < d) {
            long long r = src(row * d + e);
            if (kQuantise) r = shift_clamp(r, shift, qmin, qmax);
            v[k] = static_cast<unsigned long long>(r) & mask;
        }
    }
    ballot_pack_store(v, slices, lane, c, words_per_slice,
                      out + static_cast<size_t>(row) * slices * words_per_slice);
}

// ---------------------------------------------------------------- fused builds

// Chunk-scale build of one (row, chunk) item by one wave: round, reduce, shift, clamp, pack (64-bit
// arithmetic throughout: any magnitude, any slice count, optional clipping).
template <typename T>
__device__ __forceinline__ void build_chunk_item(const T* __restrict__ x, int64_t item, int64_t d, int chunks, int slices,
                                                 int words_per_slice, double dec_scale, float clip_k,
                                                 unsigned long long* __restrict__ words, int* __restrict__ shifts,
                                                 float* __restrict__ scales, int8_t* __restrict__ ints8, int lane) {
    const int64_t row = item / chunks;
    const int c = static_cast<int>(item - row * chunks);
    const int64_t start = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS;
    int64_t valid = d - start;
    if (valid > BSI_CHUNK_ELEMS) valid = BSI_CHUNK_ELEMS;
    if (valid < 0) valid = 0;

    long long r[4];
    unsigned long long mx = 0ULL;
    double sum = 0.0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = k * BSI_WAVE + lane;
        r[k] = 0;
        if (e < valid) {
            r[k] = round_scaled(load_as_float<T>(x, row * d + start + e), dec_scale);
            const unsigned long long av = uabs_ll(r[k]);
            if (av > mx) mx = av;
            sum += static_cast<double>(av);
        }
    }
    mx = wave_max_u64(mx);
    if (clip_k > 0.0f) sum = wave_sum_f64(sum);
    const int shift = (valid > 0) ? compute_shift(mx, sum, static_cast<int>(valid), slices, clip_k) : 0;
    if (lane == 0) {
        shifts[item] = shift;
        scales[item] = static_cast<float>(1ULL << shift);
    }
    const long long qmax = (1LL << (slices - 1)) - 1LL;
    const long long qmin = -(1LL << (slices - 1));
    const unsigned long long mask = (1ULL << slices) - 1ULL;
    unsigned long long v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = k * BSI_WAVE + lane;
        const long long q = (e < valid) ? shift_clamp(r[k], shift, qmin, qmax) : 0;
        v[k] = static_cast<unsigned long long>(q) & mask;
        if (ints8 != nullptr)
            ints8[static_cast<size_t>(item) * BSI_CHUNK_ELEMS + mfma_byte_pos(e)] =
                static_cast<int8_t>(static_cast<int>(q) << (8 - slices));
    }
    ballot_pack_store(v, slices, lane, c, words_per_slice,
                      words + static_cast<size_t>(row) * slices * words_per_slice);
}

template <typename T>
__global__ void build_fixed_chunk_kernel(const T* __restrict__ x, int64_t Q, int64_t d, int chunks, int slices,
                                         int words_per_slice, double dec_scale, float clip_k,
                                         unsigned long long* __restrict__ words, int* __restrict__ shifts,
                                         float* __restrict__ scales, int8_t* __restrict__ ints8) {
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    if (wave >= Q * chunks) return;
    build_chunk_item<T>(x, wave, d, chunks, slices, words_per_slice, dec_scale, clip_k, words, shifts, scales, ints8, lane);
}

// The same build for the common case (at most 8 slices, no clipping, whole chunks of words), about
// seven times fewer instructions per element.  One wave takes 8 consecutive (row, chunk) items:
//   * round-half-away(v * 10^dec) comes from the float's mantissa in 32-bit integer arithmetic when 10^dec is
//     an integer of at most 127 (the same integer as the exact float64 product + 0.5 and floor, checked on every
//     float), else from that float64 sequence; everything after it is 32-bit integer work; an item holding a
//     magnitude the 32-bit route does not cover (2^31 or more after scaling, a NaN) is handed to the 64-bit
//     routine above, so results never differ;
//   * the quantised values go to LDS as the int8 image (value << (8 - slices), the MFMA core's
//     in-chunk order); the image is the bit-transpose of the planes, 32 elements at a time, so
//     lane (item j, unit w) reads its 8 dwords, transposes the 8x8 bit blocks in registers and
//     has one 32-bit half-word of every slice: no ballots, and all 64 lanes busy.
// kFastItems = items per wave (1, 2, 4 or 8): fewer for small inputs, where the length of one wave's
// instruction stream, not the throughput, sets the kernel's duration.
template <typename T, int kFastItems>
__global__ __launch_bounds__(kBlock) void build_fixed_chunk_fast_kernel(
    const T* __restrict__ x, int64_t Q, int64_t d, int chunks, int slices, int words_per_slice, double dec_scale,
    unsigned scale_int, unsigned long long* __restrict__ words, int* __restrict__ shifts, float* __restrict__ scales,
    int8_t* __restrict__ ints8) {
    __shared__ uint32_t image[kWavesPerBlock][kFastItems][BSI_CHUNK_ELEMS / 4];
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int wib = threadIdx.x >> 6;
    const int64_t total = Q * chunks;
    const int64_t item0 = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wib) * kFastItems;
    // (row, chunk) of item0 + j without a 64-bit division per item
    const int64_t row0 = item0 / chunks;
    const unsigned c0 = static_cast<unsigned>(item0 - row0 * chunks);
#define BSI_ITEM_ROW_CHUNK(j, row, c)                                  \
    const unsigned cj_##row = c0 + static_cast<unsigned>(j);          \
    const unsigned dr_##row = cj_##row / static_cast<unsigned>(chunks); \
    const int64_t row = row0 + dr_##row;                               \
    const int c = static_cast<int>(cj_##row - dr_##row * static_cast<unsigned>(chunks));
    const int qmax = (1 << (slices - 1)) - 1, qmin = -(1 << (slices - 1));
    unsigned slow = 0u;  // items that took the 64-bit routine (their outputs are already written)
    // all loads of the wave's 8 items first: one memory latency, not eight
    float raw[kFastItems][4];
#pragma unroll
    for (int j = 0; j < kFastItems; ++j) {
        const int64_t item = item0 + j;
        BSI_ITEM_ROW_CHUNK(j, row, c)
        const int64_t start = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t e = start + k * BSI_WAVE + lane;
            raw[j][k] = (item < total && e < d) ? load_as_float<T>(x, row * d + e) : 0.0f;
        }
    }
#pragma unroll
    for (int j = 0; j < kFastItems; ++j) {
        const int64_t item = item0 + j;
        if (item < total) {
            BSI_ITEM_ROW_CHUNK(j, row, c)
            (void)row;
            const int64_t start = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS;
            const int valid = static_cast<int>((d - start) < BSI_CHUNK_ELEMS ? (d - start) : BSI_CHUNK_ELEMS);
            // magnitudes of round-half-away(x * 10^dec): from the float's mantissa when 10^dec is a small integer
            // (scaled_magnitude_u32), else in float64; elements past the end were loaded as 0
            unsigned mag[4];
            bool big = false;
            if (scale_int != 0u) {
#pragma unroll
                for (int k = 0; k < 4; ++k) mag[k] = scaled_magnitude_u32(raw[j][k], scale_int, big);
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const double xs = __dmul_rn(static_cast<double>(raw[j][k]), dec_scale);
                    const bool b = !(fabs(xs) < 2147483000.0);
                    big = big || b;
                    mag[k] = b ? 0u : static_cast<unsigned>(static_cast<int>(floor(__dadd_rn(fabs(xs), 0.5))));
                }
            }
            if (__any(big)) {
                slow |= 1u << j;  // done below by the 64-bit routine
            } else {
                unsigned mx = 0u;
#pragma unroll
                for (int k = 0; k < 4; ++k) mx = mag[k] > mx ? mag[k] : mx;
                mx = wave_max_u32(mx);
                const int shift = compute_shift(static_cast<unsigned long long>(mx), 0.0, valid, slices, 0.0f);
                if (lane == 0) {
                    shifts[item] = shift;
                    scales[item] = static_cast<float>(1ULL << shift);
                }
                const unsigned round_add = (shift > 0) ? (1u << (shift - 1)) : 0u;
                unsigned char* img = reinterpret_cast<unsigned char*>(image[wib][j]);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int qa = static_cast<int>((mag[k] + round_add) >> shift);
                    int q = (raw[j][k] < 0.0f) ? -qa : qa;
                    q = q < qmin ? qmin : (q > qmax ? qmax : q);
                    img[mfma_byte_pos(k * BSI_WAVE + lane)] = static_cast<unsigned char>(q << (8 - slices));
                }
            }
        }
    }
    if (slow != 0u) {
#pragma unroll 1
        for (int j = 0; j < kFastItems; ++j)
            if (slow & (1u << j))
                build_chunk_item<T>(x, item0 + j, d, chunks, slices, words_per_slice, dec_scale, 0.0f, words, shifts,
                                    scales, ints8, lane);
    }
    __syncthreads();
    // the int8 image: 256 bytes per item, one dword per lane
    if (ints8 != nullptr) {
#pragma unroll 1
        for (int j = 0; j < kFastItems; ++j) {
            const int64_t item = item0 + j;
            if (item >= total) break;
            if (slow & (1u << j)) continue;
            reinterpret_cast<uint32_t*>(ints8)[static_cast<size_t>(item) * (BSI_CHUNK_ELEMS / 4) + lane] = image[wib][j][lane];
        }
    }
    // the planes: lane = (item j, 32-element unit w)
    {
        const int j = lane >> 3, w = lane & 7;
        const int64_t item = item0 + j;
        if (j < kFastItems && item < total && !(slow & (1u << j))) {
            uint32_t y[8];
            const uint4 lo = *reinterpret_cast<const uint4*>(&image[wib][j][w * 8]);
            const uint4 hi = *reinterpret_cast<const uint4*>(&image[wib][j][w * 8 + 4]);
            y[0] = lo.x; y[1] = lo.y; y[2] = lo.z; y[3] = lo.w;
            y[4] = hi.x; y[5] = hi.y; y[6] = hi.z; y[7] = hi.w;
            // bit b of image byte (element 8m + t) <-> bit (8m + t) of plane b's half-word: an 8x8 bit transpose
            uint32_t a[8];
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) {
                const uint32_t l = y[s2], h = y[s2 + 4];
                a[s2] = (l & 0x0F0F0F0Fu) | ((h << 4) & 0xF0F0F0F0u);
                a[s2 + 4] = ((l >> 4) & 0x0F0F0F0Fu) | (h & 0xF0F0F0F0u);
            }
#pragma unroll
            for (int b = 0; b < 8; b += 4)
#pragma unroll
                for (int s2 = b; s2 < b + 2; ++s2) {
                    const uint32_t l = a[s2], h = a[s2 + 2];
                    y[s2] = (l & 0x33333333u) | ((h << 2) & 0xCCCCCCCCu);
                    y[s2 + 2] = ((l >> 2) & 0x33333333u) | (h & 0xCCCCCCCCu);
                }
#pragma unroll
            for (int s2 = 0; s2 < 8; s2 += 2) {
                const uint32_t l = y[s2], h = y[s2 + 1];
                a[s2] = (l & 0x55555555u) | ((h << 1) & 0xAAAAAAAAu);
                a[s2 + 1] = ((l >> 1) & 0x55555555u) | (h & 0xAAAAAAAAu);
            }
            BSI_ITEM_ROW_CHUNK(j, row, c)
            uint32_t* out32 = reinterpret_cast<uint32_t*>(words) +
                              (static_cast<size_t>(row) * slices * words_per_slice + static_cast<size_t>(c) * 4) * 2 + w;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int sl = t - (8 - slices);  // image bit t is slice t - (8 - slices)
                if (sl >= 0) out32[static_cast<size_t>(sl) * words_per_slice * 2] = a[t];
            }
        }
    }
}
#undef BSI_ITEM_ROW_CHUNK

// Row-scale build: one block per row; pass 1 reduces the row maximum, pass 2 (row now in cache)
// quantises and packs, one wave per group of 4 words.
template <typename T>
__global__ void build_fixed_row_kernel(const T* __restrict__ x, int64_t Q, int64_t d, int slices,
                                       int words_per_slice, double dec_scale, float clip_k,
                                       unsigned long long* __restrict__ words, int* __restrict__ shifts,
                                       float* __restrict__ scales, int8_t* __restrict__ ints8) {
    __shared__ unsigned long long smax[kWavesPerBlock];
    __shared__ double ssum[kWavesPerBlock];
    __shared__ int sshift;
    const int64_t row = blockIdx.x;
    if (row >= Q) return;
    const int lane = threadIdx.x & (BSI_WAVE - 1);
    const int wid = threadIdx.x >> 6;
    unsigned long long mx = 0ULL;
    double sum = 0.0;
    for (int64_t e = threadIdx.x; e < d; e += kBlock) {
        const unsigned long long av = uabs_ll(round_scaled(load_as_float<T>(x, row * d + e), dec_scale));
        if (av > mx) mx = av;
        sum += static_cast<double>(av);
    }
    mx = wave_max_u64(mx);
    sum = wave_sum_f64(sum);
    if (lane == 0) {
        smax[wid] = mx;
        ssum[wid] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kWavesPerBlock; ++w) {
            if (smax[w] > mx) mx = smax[w];
            sum += ssum[w];
        }
        const int shift = compute_shift(mx, sum, static_cast<int>(d), slices, clip_k);
        sshift = shift;
        shifts[row] = shift;
        scales[row] = static_cast<float>(1ULL << shift);
    }
    __syncthreads();
    const int shift = sshift;
    const long long qmax = (1LL << (slices - 1)) - 1LL;
    const long long qmin = -(1LL << (slices - 1));
    const unsigned long long mask = (1ULL << slices) - 1ULL;
    const int groups = (words_per_slice + BSI_CHUNK_WORDS - 1) / BSI_CHUNK_WORDS;
    for (int c = wid; c < groups; c += kWavesPerBlock) {
        unsigned long long v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int el = k * BSI_WAVE + lane;
            const int64_t e = static_cast<int64_t>(c) * BSI_CHUNK_ELEMS + el;
            long long q = 0;
            if (e < d) q = shift_clamp(round_scaled(load_as_float<T>(x, row * d + e), dec_scale), shift, qmin, qmax);
            v[k] = static_cast<unsigned long long>(q) & mask;
            if (ints8 != nullptr)
                ints8[(static_cast<size_t>(row) * groups + c) * BSI_CHUNK_ELEMS + mfma_byte_pos(el)] =
                    static_cast<int8_t>(static_cast<int>(q) << (8 - slices));
        }
        ballot_pack_store(v, slices, lane, c, words_per_slice,
                          words + static_cast<size_t>(row) * slices * words_per_slice);
    }
}

static inline unsigned grid_for(int64_t waves) {
    return static_cast<unsigned>((waves + kWavesPerBlock - 1) / kWavesPerBlock);
}
static inline unsigned grid_elementwise(int64_t total) {
    int64_t b = (total + kBlock - 1) / kBlock;
    if (b > 65535 * 16) b = 65535 * 16;
    if (b < 1) b = 1;
    return static_cast<unsigned>(b);
}

}  // namespace bsi

using namespace bsi;

#define BSI_DISPATCH_DTYPE(dtype, ...)                                                   \
    switch (dtype) {                                                                     \
        case BSI_DTYPE_F32: { using T = float; __VA_ARGS__; break; }                     \
        case BSI_DTYPE_F16: { using T = __half; __VA_ARGS__; break; }                    \
        case BSI_DTYPE_BF16: { using T = __hip_bfloat16; __VA_ARGS__; break; }           \
        default: return fail(BSI_ERR_INVALID, "unknown dtype code %d", dtype);           \
    }

extern "C" int bsi_hip_quantize_round_to_int64(const void* x, int dtype, int64_t total, double dec_scale,
                                               int64_t* out, void* stream) {
    BSI_REQUIRE(total >= 0, "total must be >= 0");
    if (total == 0) return BSI_OK;
    BSI_REQUIRE(x && out, "null pointer");
    BSI_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(round_to_int64_kernel<T>, dim3(grid_elementwise(total)), dim3(kBlock),
                                                 0, as_stream(stream), static_cast<const T*>(x), total, dec_scale,
                                                 reinterpret_cast<long long*>(out)));
    BSI_LAUNCH_CHECK("round_to_int64_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_quantize_trunc_to_int64(const void* x, int dtype, int64_t total, float factor, int64_t* out,
                                               void* stream) {
    BSI_REQUIRE(total >= 0, "total must be >= 0");
    if (total == 0) return BSI_OK;
    BSI_REQUIRE(x && out, "null pointer");
    BSI_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(trunc_to_int64_kernel<T>, dim3(grid_elementwise(total)), dim3(kBlock),
                                                 0, as_stream(stream), static_cast<const T*>(x), total, factor,
                                                 reinterpret_cast<long long*>(out)));
    BSI_LAUNCH_CHECK("trunc_to_int64_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_compute_row_shift_scale(const int64_t* ints, int64_t Q, int64_t d, int fixed_bits, float clip_k,
                                               int32_t* shifts, float* scales, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(ints && shifts && scales, "null pointer");
    RoundedFromInts src{reinterpret_cast<const long long*>(ints)};
    hipLaunchKernelGGL(row_shift_scale_kernel<RoundedFromInts>, dim3(static_cast<unsigned>(Q)), dim3(kBlock), 0,
                       as_stream(stream), src, Q, d, fixed_bits, clip_k, shifts, scales);
    BSI_LAUNCH_CHECK("row_shift_scale_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_compute_chunk_shift_scale(const int64_t* ints, int64_t Q, int64_t d, int chunks, int fixed_bits,
                                                 float clip_k, int32_t* shifts, float* scales, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0 && chunks >= 0, "negative size");
    if (Q == 0 || chunks == 0) return BSI_OK;
    BSI_REQUIRE(ints && shifts && scales, "null pointer");
    RoundedFromInts src{reinterpret_cast<const long long*>(ints)};
    hipLaunchKernelGGL(chunk_shift_scale_kernel<RoundedFromInts>, dim3(grid_for(Q * chunks)), dim3(kBlock), 0,
                       as_stream(stream), src, Q, d, chunks, fixed_bits, clip_k, shifts, scales);
    BSI_LAUNCH_CHECK("chunk_shift_scale_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_apply_row_shift_clamp(int64_t* ints, int64_t Q, int64_t d, const int32_t* shifts, int fixed_bits,
                                             void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 63, "fixed_bits must be in [2, 63]");
    if (Q == 0 || d == 0) return BSI_OK;
    BSI_REQUIRE(ints && shifts, "null pointer");
    hipLaunchKernelGGL(apply_shift_clamp_kernel, dim3(grid_elementwise(Q * d)), dim3(kBlock), 0, as_stream(stream),
                       reinterpret_cast<long long*>(ints), Q * d, d, 0, shifts, -(1LL << (fixed_bits - 1)),
                       (1LL << (fixed_bits - 1)) - 1LL);
    BSI_LAUNCH_CHECK("apply_shift_clamp_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_apply_chunk_shift_clamp(int64_t* ints, int64_t Q, int64_t d, int chunks, const int32_t* shifts,
                                               int fixed_bits, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0 && chunks > 0, "bad size");
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 63, "fixed_bits must be in [2, 63]");
    if (Q == 0 || d == 0) return BSI_OK;
    BSI_REQUIRE(ints && shifts, "null pointer");
    hipLaunchKernelGGL(apply_shift_clamp_kernel, dim3(grid_elementwise(Q * d)), dim3(kBlock), 0, as_stream(stream),
                       reinterpret_cast<long long*>(ints), Q * d, d, chunks, shifts, -(1LL << (fixed_bits - 1)),
                       (1LL << (fixed_bits - 1)) - 1LL);
    BSI_LAUNCH_CHECK("apply_shift_clamp_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_compute_row_shift_scale_from_input(const void* x, int dtype, int64_t Q, int64_t d,
                                                          double dec_scale, int fixed_bits, float clip_k,
                                                          int32_t* shifts, float* scales, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(x && shifts && scales, "null pointer");
    BSI_DISPATCH_DTYPE(dtype, {
        RoundedFromInput<T> src{static_cast<const T*>(x), dec_scale};
        hipLaunchKernelGGL(row_shift_scale_kernel<RoundedFromInput<T>>, dim3(static_cast<unsigned>(Q)), dim3(kBlock),
                           0, as_stream(stream), src, Q, d, fixed_bits, clip_k, shifts, scales);
    });
    BSI_LAUNCH_CHECK("row_shift_scale_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_compute_chunk_shift_scale_from_input(const void* x, int dtype, int64_t Q, int64_t d, int chunks,
                                                            double dec_scale, int fixed_bits, float clip_k,
                                                            int32_t* shifts, float* scales, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0 && chunks >= 0, "negative size");
    if (Q == 0 || chunks == 0) return BSI_OK;
    BSI_REQUIRE(x && shifts && scales, "null pointer");
    BSI_DISPATCH_DTYPE(dtype, {
        RoundedFromInput<T> src{static_cast<const T*>(x), dec_scale};
        hipLaunchKernelGGL(chunk_shift_scale_kernel<RoundedFromInput<T>>, dim3(grid_for(Q * chunks)), dim3(kBlock), 0,
                           as_stream(stream), src, Q, d, chunks, fixed_bits, clip_k, shifts, scales);
    });
    BSI_LAUNCH_CHECK("chunk_shift_scale_kernel");
    return BSI_OK;
}

static int check_pack_args(int64_t Q, int64_t d, int slices, int words_per_slice) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    BSI_REQUIRE(slices >= 1 && slices <= 64, "slices must be in [1, 64]");
    BSI_REQUIRE(words_per_slice >= 1 && static_cast<int64_t>(words_per_slice) * 64 >= d,
                "words_per_slice * 64 must cover d");
    return BSI_OK;
}

extern "C" int bsi_hip_quantize_shift_pack_row_batch(const void* x, int dtype, int64_t Q, int64_t d, int slices,
                                                     int words_per_slice, double dec_scale, int fixed_bits,
                                                     const int32_t* shifts, uint64_t* words, void* stream) {
    if (int rc = check_pack_args(Q, d, slices, words_per_slice)) return rc;
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 63, "fixed_bits must be in [2, 63]");
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(x && shifts && words, "null pointer");
    const int groups = (words_per_slice + 3) / 4;
    BSI_DISPATCH_DTYPE(dtype, {
        RoundedFromInput<T> src{static_cast<const T*>(x), dec_scale};
        hipLaunchKernelGGL((shift_pack_kernel<RoundedFromInput<T>, true>), dim3(grid_for(Q * groups)), dim3(kBlock), 0,
                           as_stream(stream), src, Q, d, 0, slices, words_per_slice, fixed_bits, shifts,
                           reinterpret_cast<unsigned long long*>(words));
    });
    BSI_LAUNCH_CHECK("shift_pack_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_quantize_shift_pack_chunk_batch(const void* x, int dtype, int64_t Q, int64_t d, int chunks,
                                                       int slices, int words_per_slice, double dec_scale,
                                                       int fixed_bits, const int32_t* shifts, uint64_t* words,
                                                       void* stream) {
    if (int rc = check_pack_args(Q, d, slices, words_per_slice)) return rc;
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 63, "fixed_bits must be in [2, 63]");
    BSI_REQUIRE(chunks > 0, "chunks must be > 0");
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(x && shifts && words, "null pointer");
    const int groups = (words_per_slice + 3) / 4;
    BSI_DISPATCH_DTYPE(dtype, {
        RoundedFromInput<T> src{static_cast<const T*>(x), dec_scale};
        hipLaunchKernelGGL((shift_pack_kernel<RoundedFromInput<T>, true>), dim3(grid_for(Q * groups)), dim3(kBlock), 0,
                           as_stream(stream), src, Q, d, chunks, slices, words_per_slice, fixed_bits, shifts,
                           reinterpret_cast<unsigned long long*>(words));
    });
    BSI_LAUNCH_CHECK("shift_pack_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_pack_bits_batch(const int64_t* ints, int64_t Q, int64_t d, int slices, int words_per_slice,
                                       uint64_t* words, void* stream) {
    if (int rc = check_pack_args(Q, d, slices, words_per_slice)) return rc;
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(ints && words, "null pointer");
    const int groups = (words_per_slice + 3) / 4;
    RoundedFromInts src{reinterpret_cast<const long long*>(ints)};
    hipLaunchKernelGGL((shift_pack_kernel<RoundedFromInts, false>), dim3(grid_for(Q * groups)), dim3(kBlock), 0,
                       as_stream(stream), src, Q, d, 0, slices, words_per_slice, 0, nullptr,
                       reinterpret_cast<unsigned long long*>(words));
    BSI_LAUNCH_CHECK("shift_pack_kernel");
    return BSI_OK;
}

// ---- decimal mode (no fixed bits): the slice count follows the data ----

// One workgroup per row: largest |value| of the whole batch (atomic max into *max_abs, cleared by the
// launcher) and, per row, whether any value is negative.
__global__ __launch_bounds__(kBlock) void decimal_stats_kernel(const long long* __restrict__ ints, int64_t d,
                                                               unsigned long long* __restrict__ max_abs,
                                                               int* __restrict__ row_negative) {
    __shared__ unsigned long long smax[kBlock / BSI_WAVE];
    __shared__ int sneg[kBlock / BSI_WAVE];
    const int64_t q = blockIdx.x;
    const long long* row = ints + q * d;
    unsigned long long m = 0;
    int neg = 0;
    for (int64_t e = threadIdx.x; e < d; e += kBlock) {
        const long long v = row[e];
        const unsigned long long a = v < 0 ? 0ULL - static_cast<unsigned long long>(v) : static_cast<unsigned long long>(v);
        m = a > m ? a : m;
        neg |= v < 0;
    }
#pragma unroll
    for (int off = BSI_WAVE / 2; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(m, off, BSI_WAVE);
        m = o > m ? o : m;
        neg |= __shfl_xor(neg, off, BSI_WAVE);
    }
    const int wave = threadIdx.x / BSI_WAVE;
    if ((threadIdx.x & (BSI_WAVE - 1)) == 0) {
        smax[wave] = m;
        sneg[wave] = neg;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / BSI_WAVE; ++w) {
            m = smax[w] > m ? smax[w] : m;
            neg |= sneg[w];
        }
        row_negative[q] = neg;
        if (m != 0) atomicMax(max_abs, m);
    }
}

__global__ void clear_u64_kernel(unsigned long long* p) { *p = 0ULL; }

extern "C" int bsi_hip_decimal_stats(const int64_t* ints, int64_t Q, int64_t d, uint64_t* max_abs,
                                     int32_t* row_negative, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    BSI_REQUIRE(max_abs != nullptr, "null pointer");
    BSI_REQUIRE(Q <= 0x7fffffffLL, "too many rows for one launch");
    hipLaunchKernelGGL(clear_u64_kernel, dim3(1), dim3(1), 0, as_stream(stream),
                       reinterpret_cast<unsigned long long*>(max_abs));
    BSI_LAUNCH_CHECK("clear_u64_kernel");
    if (Q == 0) return BSI_OK;
    BSI_REQUIRE(row_negative != nullptr && (ints != nullptr || d == 0), "null pointer");
    hipLaunchKernelGGL(decimal_stats_kernel, dim3(static_cast<unsigned>(Q)), dim3(kBlock), 0, as_stream(stream),
                       reinterpret_cast<const long long*>(ints), d, reinterpret_cast<unsigned long long*>(max_abs),
                       row_negative);
    BSI_LAUNCH_CHECK("decimal_stats_kernel");
    return BSI_OK;
}

std::atomic<int> bsi::g_build_items{0};

extern "C" int bsi_hip_build_fixed(const void* x, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits,
                                   int chunk_scale, float clip_k, uint64_t* words, int32_t* shifts, float* scales,
                                   int8_t* ints8, void* stream) {
    BSI_REQUIRE(Q >= 0 && d >= 0, "negative size");
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 63, "fixed_bits must be in [2, 63]");
    BSI_REQUIRE(ints8 == nullptr || fixed_bits <= 8, "int8 output needs fixed_bits <= 8");
    if (Q == 0 || d == 0) return BSI_OK;
    BSI_REQUIRE(x && words && shifts && scales, "null pointer");
    const int W = static_cast<int>((d + 63) / 64);
    const int chunks = static_cast<int>((d + 255) / 256);
    const double dec_scale = pow(10.0, static_cast<double>(decimal_places));
    if (chunk_scale && fixed_bits <= 8 && !(clip_k > 0.0f) && W % 4 == 0) {
        const int64_t items = Q * chunks;
#define BSI_LAUNCH_FAST(N)                                                                                          \
    {                                                                                                               \
        const int64_t waves = (items + (N) - 1) / (N);                                                              \
        BSI_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((build_fixed_chunk_fast_kernel<T, N>), dim3(grid_for(waves)),   \
                                                     dim3(kBlock), 0, as_stream(stream), static_cast<const T*>(x), Q, \
                                                     d, chunks, fixed_bits, W, dec_scale,                            \
                                                     integer_decimal_scale(dec_scale),                               \
                                                     reinterpret_cast<unsigned long long*>(words), shifts, scales,   \
                                                     ints8));                                                        \
    }
        // a wave gets more items only once there are about 8 waves per SIMD (8192 in all); measured on
        // 4096 ... 131072 items, every other choice is within a few percent or slower
        int per_wave = g_build_items.load(std::memory_order_relaxed);
        if (per_wave == 0) per_wave = items > 8 * 16384 ? 8 : (items >= 16384 ? 4 : (items >= 8192 ? 2 : 1));
        if (per_wave == 8) BSI_LAUNCH_FAST(8)
        else if (per_wave == 4) BSI_LAUNCH_FAST(4)
        else if (per_wave == 2) BSI_LAUNCH_FAST(2)
        else BSI_LAUNCH_FAST(1)
#undef BSI_LAUNCH_FAST
        BSI_LAUNCH_CHECK("build_fixed_chunk_fast_kernel");
    } else if (chunk_scale) {
        BSI_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(build_fixed_chunk_kernel<T>, dim3(grid_for(Q * chunks)),
                                                     dim3(kBlock), 0, as_stream(stream), static_cast<const T*>(x), Q,
                                                     d, chunks, fixed_bits, W, dec_scale, clip_k,
                                                     reinterpret_cast<unsigned long long*>(words), shifts, scales,
                                                     ints8));
        BSI_LAUNCH_CHECK("build_fixed_chunk_kernel");
    } else {
        BSI_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(build_fixed_row_kernel<T>, dim3(static_cast<unsigned>(Q)),
                                                     dim3(kBlock), 0, as_stream(stream), static_cast<const T*>(x), Q,
                                                     d, fixed_bits, W, dec_scale, clip_k,
                                                     reinterpret_cast<unsigned long long*>(words), shifts, scales,
                                                     ints8));
        BSI_LAUNCH_CHECK("build_fixed_row_kernel");
    }
    return BSI_OK;
}
