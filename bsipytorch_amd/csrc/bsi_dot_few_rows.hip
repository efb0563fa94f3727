// The dot for a few query rows (decode steps): kernels that stream the packed key planes once -- on a built int8
// query image, with the query build inside, or with queries handed over as EWAH streams -- and the stream -> int8
// image pass for larger batches of EWAH queries.
#include "bsi_dot_device.h"
#include "bsi_dot_internal.h"

namespace bsi {

// ------------------------------------------------------------------ MFMA core, few query rows
//
// Decode-like shapes (a handful of query rows against a large key matrix) are bound by reading the
// packed key planes once.  One workgroup owns one 16-key tile of the tiled layout over all chunks
// and up to 16 * NT query rows; its waves take the chunks round-robin.  A lane loads the six plane
// words of (key row lane % 16, 64-bit word lane / 16), transposes them in registers into the four
// 16-byte MFMA operands of that row (no LDS staging: with a k permutation shared by both operands
// any assignment of chunk elements to MFMA k-slots gives the same integer), loads the matching 64
// int8 query bytes from L2, and issues 4 MFMAs per query tile.  The int32 results go to LDS
// indexed by chunk; after a workgroup barrier 256 * NT lanes run the fp32 chain of their (query,
// key) pair over the chunks in order, so the result is bit-identical to a sequential pass
// whatever the number of waves.  Problems with more chunks than LDS slots run in several passes.

constexpr int kStreamLdsInts = 16384;  // at most 64 KiB of chunk accumulators per pass

template <int NT, int KT, bool kInts>
__global__ __launch_bounds__(1024) void dot_mfma_stream_kernel(
    const int8_t* __restrict__ A8, const float* __restrict__ qscale, int qscale_stride,
    const unsigned long long* __restrict__ B64,  // tiled key planes, Sb = 6
    const float* __restrict__ Bw, int chunks, int pass_chunks, int64_t R, int64_t Q, int down_shift, float scale_inv,
    int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints, const float* __restrict__ bias) {
    extern __shared__ __attribute__((aligned(16))) int ints[];  // [pass_chunks][KT][NT][16 queries][16 keys]
    constexpr int kSlot = KT * NT * 256;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = static_cast<int>(blockDim.x >> 6);
    const int ln = lane & 15, lg = lane >> 4;
    const int64_t ntiles = (R + 15) / 16;
    const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * KT;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * (16 * NT);
    const size_t ktile = static_cast<size_t>(chunks) * (6 * 64);  // words per key tile
    const unsigned long long* ksrc[KT];
#pragma unroll
    for (int k = 0; k < KT; ++k) {
        const int64_t t = (tile0 + k < ntiles) ? tile0 + k : ntiles - 1;  // clamped: its outputs are never stored
        ksrc[k] = B64 + static_cast<size_t>(t) * ktile + lane;
    }
    const size_t arow = static_cast<size_t>(chunks) * 256;

    // the chain lanes: tid <-> (key tile, query tile, query, key), keys fastest so output stores are contiguous
    float accf = 0.0f;
    const bool chain = tid < kSlot;
    const int ck = tid / (NT * 256), ct = (tid >> 8) % NT, cn = (tid >> 4) & 15, ckey = tid & 15;
    const int64_t cq = q0 + ct * 16 + cn, cr = (tile0 + ck) * 16 + ckey;
    const bool cvalid = chain && cq < Q && cr < R;
    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
    const float* csrc = qscale + (cvalid ? cq : 0) * qscale_stride;
    const int sstep = (qscale_stride == 1) ? 0 : 1;
    const EpilogueOperands eo = load_epilogue_operands(Bw, bias, R, cvalid, cr);

    for (int p0 = 0; p0 < chunks; p0 += pass_chunks) {
        const int pend = (p0 + pass_chunks < chunks) ? p0 + pass_chunks : chunks;
        int c = p0 + wave;
        uint2 kc[KT][6];
        if (c < pend) {
#pragma unroll
            for (int k = 0; k < KT; ++k)
#pragma unroll
                for (int j = 0; j < 6; ++j) {
                    const unsigned long long w = ksrc[k][(static_cast<size_t>(c) * 6 + j) * 64];
                    kc[k][j] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
                }
        }
        for (; c < pend; c += nwaves) {
            // query operands of this chunk (L2 resident), then the key planes of the wave's next chunk
            v4i qb[NT][4];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int64_t q = q0 + t * 16 + ln;
                if (q < Q) {
                    const v4i* src = reinterpret_cast<const v4i*>(A8 + static_cast<size_t>(q) * arow + c * 256 + lg * 64);
#pragma unroll
                    for (int m = 0; m < 4; ++m) qb[t][m] = src[m];
                } else {
#pragma unroll
                    for (int m = 0; m < 4; ++m) qb[t][m] = (v4i){0, 0, 0, 0};
                }
            }
            uint2 kn[KT][6];
            const int cnext = c + nwaves;
            if (cnext < pend) {
#pragma unroll
                for (int k = 0; k < KT; ++k)
#pragma unroll
                    for (int j = 0; j < 6; ++j) {
                        const unsigned long long w = ksrc[k][(static_cast<size_t>(cnext) * 6 + j) * 64];
                        kn[k][j] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
                    }
            }
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                uint32_t lo[8], hi[8];
                transpose_6planes(kc[k][0].x, kc[k][1].x, kc[k][2].x, kc[k][3].x, kc[k][4].x, kc[k][5].x, lo);
                transpose_6planes(kc[k][0].y, kc[k][1].y, kc[k][2].y, kc[k][3].y, kc[k][4].y, kc[k][5].y, hi);
                v4i ka[4];
                ka[0] = (v4i){static_cast<int>(lo[0]), static_cast<int>(lo[1]), static_cast<int>(lo[2]), static_cast<int>(lo[3])};
                ka[1] = (v4i){static_cast<int>(lo[4]), static_cast<int>(lo[5]), static_cast<int>(lo[6]), static_cast<int>(lo[7])};
                ka[2] = (v4i){static_cast<int>(hi[0]), static_cast<int>(hi[1]), static_cast<int>(hi[2]), static_cast<int>(hi[3])};
                ka[3] = (v4i){static_cast<int>(hi[4]), static_cast<int>(hi[5]), static_cast<int>(hi[6]), static_cast<int>(hi[7])};
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    v4i acc = {0, 0, 0, 0};
#pragma unroll
                    for (int m = 0; m < 4; ++m) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[m], qb[t][m], acc, 0, 0, 0);
                    // the lane holds keys 4*lg .. 4*lg+3 of query ln
                    *reinterpret_cast<v4i*>(&ints[(c - p0) * kSlot + (k * NT + t) * 256 + ln * 16 + lg * 4]) = acc;
                }
            }
            if (cnext < pend) {
#pragma unroll
                for (int k = 0; k < KT; ++k)
#pragma unroll
                    for (int j = 0; j < 6; ++j) kc[k][j] = kn[k][j];
            }
        }
        __syncthreads();
        if (cvalid) {
            accf = chain_chunks(accf, p0, pend, down, [&](int cc) { return ints[(cc - p0) * kSlot + tid]; },
                                [&](int cc) { return csrc[cc * sstep]; });
            if (kInts)
                for (int cc = p0; cc < pend; ++cc)
                    chunk_ints[(cq * R + cr) * chunks + cc] = ints[(cc - p0) * kSlot + tid] >> down_shift;
        }
        if (pend < chunks) __syncthreads();
    }
    if (cvalid) {
        float v = (accf * eo.bw) * scale_inv;
        if (bias != nullptr) v = v + eo.bias;
        out[static_cast<size_t>(cq) * R_total + cr] = v;
    }
}

// The few-rows kernel with the query build inside (at most kFusedMaxQ rows: a decode step).  Every workgroup first
// issues the loads of its first key planes, then quantises the activations itself while those are in flight: the
// (chunk, row) items go round-robin over the waves, each one the builder's per-chunk routine -- round half away of
// x * 10^dec, the chunk's shift from its largest magnitude, rounded shift and clamp -- and leave the int8 MFMA
// operand and the chunk scale in LDS.  After a barrier the kernel is the few-rows kernel above with its query
// operand in LDS.  Every workgroup repeats that small amount of arithmetic (a few hundred VALU cycles per wave
// against microseconds of key traffic), and a BSI-linear layer becomes ONE launch instead of a build and a dot.
// Same integers, scales and fp32 chain as bsi_hip_build_fixed + bsi_hip_dot, so the same bits.
constexpr int kFusedMaxQ = 4;
constexpr size_t kFusedQueryLdsBytes = 96 * 1024;  // int8 image + chunk scales of all rows: chunks * Q * 260 bytes

// Element i of a buffer of T as float; 0 past the descriptor's range.
template <typename T>
__device__ __forceinline__ float buffer_load_as_float(bsi_rsrc r, int i);
template <>
__device__ __forceinline__ float buffer_load_as_float<float>(bsi_rsrc r, int i) {
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, i * 4, 0, 0));
}
template <>
__device__ __forceinline__ float buffer_load_as_float<__half>(bsi_rsrc r, int i) {
    const unsigned short h = static_cast<unsigned short>(__builtin_amdgcn_raw_buffer_load_b16(r, i * 2, 0, 0));
    return __half2float(__ushort_as_half(h));
}
template <>
__device__ __forceinline__ float buffer_load_as_float<__hip_bfloat16>(bsi_rsrc r, int i) {
    const unsigned short h = static_cast<unsigned short>(__builtin_amdgcn_raw_buffer_load_b16(r, i * 2, 0, 0));
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// One (chunk, row) item: the wave's 256 activations xv[k] = element k * 64 + lane (0 past the row's end) become 256
// image bytes at img and one scale.  scale_int is 10^dec when that is at most 127 (else 0: float64 arithmetic).
// Magnitudes below 2^31 (all but pathological inputs) go through 32-bit integer arithmetic; an item with a larger
// one is left untouched and reported (true, for the whole wave) for fused_quantize_item_wide -- the same two routes,
// with the same results, as the builder's fast kernel.
__device__ __forceinline__ bool fused_quantize_item(const float (&xv)[4], double dec_scale, unsigned scale_int, int slices,
                                                    int valid, int lane, unsigned char* img, float* scale_out) {
    unsigned mag[4];
    bool big = false;
    if (scale_int != 0u) {
#pragma unroll
        for (int k = 0; k < 4; ++k) mag[k] = scaled_magnitude_u32(xv[k], scale_int, big);
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const double xs = __dmul_rn(static_cast<double>(xv[k]), dec_scale);
            const bool b = !(fabs(xs) < 2147483000.0);
            big = big || b;
            mag[k] = b ? 0u : static_cast<unsigned>(static_cast<int>(floor(__dadd_rn(fabs(xs), 0.5))));
        }
    }
    if (__any(big)) return true;
    unsigned mx = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) mx = mag[k] > mx ? mag[k] : mx;
    mx = wave_max_u32(mx);
    // compute_shift without clipping: the bits of the largest magnitude beyond the slices' magnitude bits
    int shift = (32 - __clz(static_cast<int>(mx))) - (slices - 1);  // mx < 2^31; __clz(0) = 32
    shift = (shift < 0 || valid <= 0) ? 0 : shift;
    if (lane == 0) *scale_out = static_cast<float>(1ULL << shift);
    const unsigned round_add = (shift > 0) ? (1u << (shift - 1)) : 0u;
    const int qmax32 = (1 << (slices - 1)) - 1, qmin32 = -(1 << (slices - 1));
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int qa = static_cast<int>((mag[k] + round_add) >> shift);
        int v = (xv[k] < 0.0f) ? -qa : qa;
        v = v < qmin32 ? qmin32 : (v > qmax32 ? qmax32 : v);
        img[mfma_byte_pos(k * BSI_WAVE + lane)] = static_cast<unsigned char>(v << (8 - slices));
    }
    return false;
}

// The rare item (a magnitude of 2^31 or more, an infinity, a NaN): the builder's 64-bit routine, reading the chunk
// from memory (xsrc = its first element) in rolled loops, so that it costs the kernel no registers.
template <typename T>
__device__ __forceinline__ void fused_quantize_item_wide(const T* xsrc, double dec_scale, int slices, int valid, int lane,
                                                         unsigned char* img, float* scale_out) {
    const long long qmax = (1LL << (slices - 1)) - 1LL, qmin = -(1LL << (slices - 1));
    unsigned long long mx = 0ULL;
#pragma unroll 1
    for (int k = 0; k < 4; ++k) {
        const int e = k * BSI_WAVE + lane;
        if (e < valid) {
            const unsigned long long av = uabs_ll(round_scaled(load_as_float<T>(xsrc, e), dec_scale));
            if (av > mx) mx = av;
        }
    }
    mx = wave_max_u64(mx);
    const int shift = (valid > 0) ? compute_shift(mx, 0.0, valid, slices, 0.0f) : 0;
    if (lane == 0) *scale_out = static_cast<float>(1ULL << shift);
#pragma unroll 1
    for (int k = 0; k < 4; ++k) {
        const int e = k * BSI_WAVE + lane;
        const long long v = (e < valid) ? shift_clamp(round_scaled(load_as_float<T>(xsrc, e), dec_scale), shift, qmin, qmax) : 0;
        img[mfma_byte_pos(e)] = static_cast<unsigned char>(static_cast<int>(v) << (8 - slices));
    }
}

template <typename T, int KT, int NI>
__global__ __launch_bounds__(1024) void dot_mfma_stream_fused_kernel(
    const T* __restrict__ x, int64_t d, double dec_scale, unsigned scale_int, int slices,
    const unsigned long long* __restrict__ B64,  // tiled key planes, Sb = 6
    const float* __restrict__ Bw, int chunks, int pass_chunks, int64_t R, int Q, float scale_inv, int64_t R_total,
    float* __restrict__ out, const float* __restrict__ bias) {
    // [pass_chunks][KT][16 queries][16 keys] ints | [chunks][Q][256] image bytes | [chunks][Q] scales
    extern __shared__ __attribute__((aligned(16))) int ints[];
    constexpr int kSlot = KT * 256;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = static_cast<int>(blockDim.x >> 6);
    const int ln = lane & 15, lg = lane >> 4;
    unsigned char* const qimg = reinterpret_cast<unsigned char*>(ints + static_cast<size_t>(pass_chunks) * kSlot);
    float* const qsc = reinterpret_cast<float*>(qimg + static_cast<size_t>(chunks) * Q * 256);
    const int64_t ntiles = (R + 15) / 16;
    const int64_t tile0 = static_cast<int64_t>(blockIdx.x) * KT;
    const size_t ktile = static_cast<size_t>(chunks) * (6 * 64);  // words per key tile
    const unsigned long long* ksrc[KT];
#pragma unroll
    for (int k = 0; k < KT; ++k) {
        const int64_t t = (tile0 + k < ntiles) ? tile0 + k : ntiles - 1;  // clamped: its outputs are never stored
        ksrc[k] = B64 + static_cast<size_t>(t) * ktile + lane;
    }
    const int down_shift = 16 - slices - 6;

    // the chain lanes: tid <-> (key tile, query, key), keys fastest so output stores are contiguous
    float accf = 0.0f;
    const int ck = tid >> 8, cn = (tid >> 4) & 15, ckey = tid & 15;
    const int64_t cr = (tile0 + ck) * 16 + ckey;
    const bool cvalid = tid < kSlot && cn < Q && cr < R;
    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);

    // The wave's share of the query build: (chunk, row) items wave, wave + nwaves, ...  The loads of a CU return in
    // order, so the activations are requested BEFORE the first key planes (they would otherwise wait behind that
    // traffic, one round trip per item) and all at once: up to kFusedItems items per wave sit in registers while
    // the key loads are issued, then they are quantised under the latency of those.
    constexpr int kFusedItems = NI;  // 1, 2 or (one key tile only) 4: what the registers hold beside the key planes
    const int items = chunks * Q;
    // Buffer loads, one descriptor per row: past the row's end they return 0 without a branch (with loads in
    // conditional blocks the compiler waits for every outstanding load, the key planes included, before a use).
    auto load_item = [&](int item, float (&dst)[4]) {
        const int ic = item / Q, iq = item - ic * Q;
        const bsi_rsrc row = make_rsrc(x + static_cast<int64_t>(iq) * d, static_cast<size_t>(d) * sizeof(T));
        const int e0 = ic * BSI_CHUNK_ELEMS + lane;
#pragma unroll
        for (int k = 0; k < 4; ++k) dst[k] = buffer_load_as_float<T>(row, e0 + k * BSI_WAVE);
    };
    auto quantize = [&](int item, const float (&xv)[4]) -> bool {
        const int ic = item / Q;
        const int64_t left = d - static_cast<int64_t>(ic) * BSI_CHUNK_ELEMS;
        const int valid = static_cast<int>(left < BSI_CHUNK_ELEMS ? left : BSI_CHUNK_ELEMS);
        return fused_quantize_item(xv, dec_scale, scale_int, slices, valid, lane, qimg + static_cast<size_t>(item) * 256,
                                   qsc + item);
    };
    auto quantize_wide = [&](int item) {
        const int ic = item / Q, iq = item - ic * Q;
        const int64_t s0 = static_cast<int64_t>(ic) * BSI_CHUNK_ELEMS, left = d - s0;
        const int valid = static_cast<int>(left < BSI_CHUNK_ELEMS ? left : BSI_CHUNK_ELEMS);
        fused_quantize_item_wide<T>(x + static_cast<int64_t>(iq) * d + s0, dec_scale, slices, valid, lane,
                                    qimg + static_cast<size_t>(item) * 256, qsc + item);
    };
    float xr[kFusedItems][4];
#pragma unroll
    for (int i = 0; i < kFusedItems; ++i) {
        const int item = wave + i * nwaves;
        load_item(item < items ? item : items - 1, xr[i]);
    }

    uint2 kc[KT][6];
    auto load_keys = [&](int chunk, uint2 (&dst)[KT][6]) {
#pragma unroll
        for (int k = 0; k < KT; ++k)
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                const unsigned long long w = ksrc[k][(static_cast<size_t>(chunk) * 6 + j) * 64];
                dst[k][j] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
            }
    };
    // the first pass's first chunk; a wave without one loads the last chunk's planes for nothing, because a branch
    // here would make the compiler's load counting assume the worst and wait for these loads in the query build
    load_keys(wave < pass_chunks ? wave : pass_chunks - 1, kc);
    const EpilogueOperands eo = load_epilogue_operands(Bw, bias, R, cvalid, cr);
    __builtin_amdgcn_sched_barrier(0);
    {
        unsigned wide = 0u;  // items left to the 64-bit routine
#pragma unroll
        for (int i = 0; i < kFusedItems; ++i) {
            // no branch here either (the compiler would sink the item's loads into it, behind the key loads): a wave
            // with fewer items repeats the last one, and writes the bytes its owner writes
            const int item = wave + i * nwaves;
            const bool w = quantize(item < items ? item : items - 1, xr[i]);
            wide |= (w && item < items) ? 1u << i : 0u;
            __builtin_amdgcn_sched_barrier(0);  // one item at a time: interleaving them costs registers, gains nothing
        }
        // longer rows: the rest one item at a time (each waits for its own loads)
#pragma unroll 1
        for (int item = wave + kFusedItems * nwaves; item < items; item += nwaves) {
            float xa[4];
            load_item(item, xa);
            if (quantize(item, xa)) wide |= 1u << 31;
        }
#pragma unroll 1
        for (int i = 0; wide != 0u && i < kFusedItems; ++i)
            if (wide & (1u << i)) quantize_wide(wave + i * nwaves);
        if (wide >> 31) {  // some item past the first ones: find it again (rare twice over)
#pragma unroll 1
            for (int item = wave + kFusedItems * nwaves; item < items; item += nwaves) {
                float xa[4];
                load_item(item, xa);
                bool big = false;
#pragma unroll
                for (int k = 0; k < 4; ++k) big = big || !(fabs(__dmul_rn(static_cast<double>(xa[k]), dec_scale)) < 2147483000.0);
                if (__any(big)) quantize_wide(item);
            }
        }
        __syncthreads();
    }

    for (int p0 = 0; p0 < chunks; p0 += pass_chunks) {
        const int pend = (p0 + pass_chunks < chunks) ? p0 + pass_chunks : chunks;
        int c = p0 + wave;
        if (p0 > 0 && c < pend) load_keys(c, kc);
        for (; c < pend; c += nwaves) {
            // query operand of this chunk from LDS, then the key planes of the wave's next chunk
            v4i qb[4];
            if (ln < Q) {
                const v4i* src = reinterpret_cast<const v4i*>(qimg + (static_cast<size_t>(c) * Q + ln) * 256 + lg * 64);
#pragma unroll
                for (int m = 0; m < 4; ++m) qb[m] = src[m];
            } else {
#pragma unroll
                for (int m = 0; m < 4; ++m) qb[m] = (v4i){0, 0, 0, 0};
            }
            uint2 kn[KT][6];
            const int cnext = c + nwaves;
            if (cnext < pend) {
#pragma unroll
                for (int k = 0; k < KT; ++k)
#pragma unroll
                    for (int j = 0; j < 6; ++j) {
                        const unsigned long long w = ksrc[k][(static_cast<size_t>(cnext) * 6 + j) * 64];
                        kn[k][j] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
                    }
            }
#pragma unroll
            for (int k = 0; k < KT; ++k) {
                uint32_t lo[8], hi[8];
                transpose_6planes(kc[k][0].x, kc[k][1].x, kc[k][2].x, kc[k][3].x, kc[k][4].x, kc[k][5].x, lo);
                transpose_6planes(kc[k][0].y, kc[k][1].y, kc[k][2].y, kc[k][3].y, kc[k][4].y, kc[k][5].y, hi);
                v4i ka[4];
                ka[0] = (v4i){static_cast<int>(lo[0]), static_cast<int>(lo[1]), static_cast<int>(lo[2]), static_cast<int>(lo[3])};
                ka[1] = (v4i){static_cast<int>(lo[4]), static_cast<int>(lo[5]), static_cast<int>(lo[6]), static_cast<int>(lo[7])};
                ka[2] = (v4i){static_cast<int>(hi[0]), static_cast<int>(hi[1]), static_cast<int>(hi[2]), static_cast<int>(hi[3])};
                ka[3] = (v4i){static_cast<int>(hi[4]), static_cast<int>(hi[5]), static_cast<int>(hi[6]), static_cast<int>(hi[7])};
                v4i acc = {0, 0, 0, 0};
#pragma unroll
                for (int m = 0; m < 4; ++m) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[m], qb[m], acc, 0, 0, 0);
                // the lane holds keys 4*lg .. 4*lg+3 of query ln
                *reinterpret_cast<v4i*>(&ints[(c - p0) * kSlot + k * 256 + ln * 16 + lg * 4]) = acc;
            }
            if (cnext < pend) {
#pragma unroll
                for (int k = 0; k < KT; ++k)
#pragma unroll
                    for (int j = 0; j < 6; ++j) kc[k][j] = kn[k][j];
            }
        }
        __syncthreads();
        if (cvalid) {
            accf = chain_chunks(accf, p0, pend, down, [&](int cc) { return ints[(cc - p0) * kSlot + tid]; },
                                [&](int cc) { return qsc[cc * Q + cn]; });
        }
        if (pend < chunks) __syncthreads();
    }
    if (cvalid) {
        float v = (accf * eo.bw) * scale_inv;
        if (bias != nullptr) v = v + eo.bias;
        out[static_cast<size_t>(cn) * R_total + cr] = v;
    }
}

// ------------------------------------------------------------------ EWAH-compressed queries, decode inline
//
// The hybrid query form keeps each of a query's Sa slices as an EWAH stream ([marker][literals...],
// marker = run_bit | run_len << 1 | literal_count << 33; bsi_cuda_kernels_ewah.cuh:5-33 is the
// decoder this follows, including its bounds: output clipped at W words, input at the stream's
// length, the rest zero).  This kernel is the few-rows kernel for up to 16 such queries per workgroup
// (stream q * Sa + s is slice s of query q) with the decode folded into its load stage: every workgroup
// first expands the streams into bit planes in LDS (a wave per stream: ewah_expand_wave), then
// recombines the planes of each chunk into the int8 MFMA operand in registers, exactly as it does for
// the key planes it streams from HBM.  A slice whose stream says "all zero" (one marker, a zero run
// over the whole slice: the sign plane of ReLU'd activations, the high planes of small values) is not
// expanded at all: its plane reads as zero without touching LDS.
constexpr int kEwahQueriesPerGroup = 16;
__host__ __device__ inline int ewah_stream_stride(int wpad) { return wpad + 1; }  // odd stride: queries spread over the banks
// bytes of the plane region of `group` queries (a multiple of 16: the accumulators behind it are stored 16 bytes at a time)
__host__ __device__ inline size_t ewah_plane_region(int group, int Sa, int wpad) {
    return (static_cast<size_t>(group) * Sa * ewah_stream_stride(wpad) * 8 + 15) & ~static_cast<size_t>(15);
}

// Whether the stream is the encoder's form of an all-zero slice of W words (every lane gets the answer).
__device__ __forceinline__ bool ewah_stream_is_zero(const unsigned long long* __restrict__ in, int in_len, int W) {
    if (in_len == 0) return true;
    if (in_len != 1) return false;
    const unsigned long long m = in[0];
    return (m & 1ULL) == 0ULL && ((m >> 1) & 0xFFFFFFFFULL) >= static_cast<unsigned long long>(W);
}

template <bool kInts>
__global__ __launch_bounds__(1024) void dot_mfma_stream_ewah_kernel(
    const unsigned long long* __restrict__ comp, const long long* __restrict__ comp_off,
    const int* __restrict__ comp_len, int Sa, int W64, const float* __restrict__ qscale, int qscale_stride,
    const unsigned long long* __restrict__ B64,  // tiled key planes, Sb = 6
    const float* __restrict__ Bw, int chunks, int pass_chunks, int64_t R, int64_t Q, int group, int down_shift,
    float scale_inv, int64_t R_total, const float* __restrict__ bias, float* __restrict__ out,
    int* __restrict__ chunk_ints) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // group = queries per workgroup (min(Q, 16)); LDS: [group][Sa] streams of ewah_stream_stride(4 * chunks) plane
    // words, one presence byte per stream (128 bytes), then the chunk accumulators
    const int wpad = chunks * 4, sstride = ewah_stream_stride(wpad);
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * kEwahQueriesPerGroup;
    const int nq = static_cast<int>((Q - q0) < kEwahQueriesPerGroup ? (Q - q0) : kEwahQueriesPerGroup);
    const int nstreams = nq * Sa;
    unsigned long long* planes = reinterpret_cast<unsigned long long*>(smem);
    unsigned char* present = smem + ewah_plane_region(group, Sa, wpad);
    int* ints = reinterpret_cast<int*>(present + 128);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nwaves = static_cast<int>(blockDim.x >> 6);
    const int ln = lane & 15, lg = lane >> 4;
    const int64_t tile = blockIdx.x;
    const unsigned long long* ksrc = B64 + static_cast<size_t>(tile) * chunks * (6 * 64) + lane;

    // ---- inline EWAH decode: the group's streams round-robin over the waves.  Three kinds of stream: all zero
    // (nothing to do), verbatim (one marker followed by the W64 words of the slice: the words are read where they
    // lie, straight from the stream, when their chunk comes up), anything else (expanded into LDS planes now).
    for (int s = wave; s < nstreams; s += nwaves) {
        const unsigned long long* in = comp + comp_off[q0 * Sa + s];
        const int in_len = comp_len[q0 * Sa + s];
        const bool zero = ewah_stream_is_zero(in, in_len, W64);
        const bool verbatim = !zero && in_len == W64 + 1 && in[0] == (static_cast<unsigned long long>(W64) << 33);
        if (lane == 0) present[s] = zero ? 0 : (verbatim ? 2 : 1);
        if (!zero && !verbatim) ewah_expand_wave(in, in_len, W64, planes + static_cast<size_t>(s) * sstride, wpad, lane);
    }
    __syncthreads();

    const bool chain = tid < 256;
    const int ckey = tid & 15, cn = (tid >> 4) & 15;
    const int64_t cr = tile * 16 + ckey;
    const bool cvalid = chain && cn < nq && cr < R;
    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
    const int sstep = (qscale_stride == 1) ? 0 : 1;
    const float* myscale = qscale + (q0 + (cn < nq ? cn : 0)) * qscale_stride;
    float accf = 0.0f;
    // the planes of the lane's query (row t of the 8 x 8 transposes): expanded in LDS (have), verbatim in the stream (verb)
    unsigned have = 0, verb = 0;
    const unsigned long long* vptr[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int j = t - (8 - Sa);
        vptr[t] = comp;
        if (ln < nq && j >= 0) {
            const int cls = present[ln * Sa + j];
            if (cls == 1) have |= 1u << t;
            if (cls == 2) {
                verb |= 1u << t;
                vptr[t] = comp + comp_off[(q0 + ln) * Sa + j] + 1;  // past the marker
            }
        }
    }
    const unsigned long long* myplanes = planes + static_cast<size_t>(ln < nq ? ln : 0) * Sa * sstride;

    for (int p0 = 0; p0 < chunks; p0 += pass_chunks) {
        const int pend = (p0 + pass_chunks < chunks) ? p0 + pass_chunks : chunks;
        for (int c = p0 + wave; c < pend; c += nwaves) {
            uint2 kc[6];
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                const unsigned long long w = ksrc[(static_cast<size_t>(c) * 6 + j) * 64];
                kc[j] = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
            }
            // the query operand of this chunk from the decoded planes: MFMA column ln is query q0 + ln
            uint32_t qlo[8], qhi[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int j = t - (8 - Sa);
                unsigned long long w = 0ULL;
                if ((verb >> t) & 1u) w = (c * 4 + lg < W64) ? vptr[t][c * 4 + lg] : 0ULL;
                else if ((have >> t) & 1u) w = myplanes[static_cast<size_t>(j) * sstride + c * 4 + lg];
                qlo[t] = static_cast<uint32_t>(w);
                qhi[t] = static_cast<uint32_t>(w >> 32);
            }
            transpose8x8(qlo);
            transpose8x8(qhi);
            v4i qb[4];
            qb[0] = (v4i){static_cast<int>(qlo[0]), static_cast<int>(qlo[1]), static_cast<int>(qlo[2]), static_cast<int>(qlo[3])};
            qb[1] = (v4i){static_cast<int>(qlo[4]), static_cast<int>(qlo[5]), static_cast<int>(qlo[6]), static_cast<int>(qlo[7])};
            qb[2] = (v4i){static_cast<int>(qhi[0]), static_cast<int>(qhi[1]), static_cast<int>(qhi[2]), static_cast<int>(qhi[3])};
            qb[3] = (v4i){static_cast<int>(qhi[4]), static_cast<int>(qhi[5]), static_cast<int>(qhi[6]), static_cast<int>(qhi[7])};
            uint32_t lo[8], hi[8];
            transpose_6planes(kc[0].x, kc[1].x, kc[2].x, kc[3].x, kc[4].x, kc[5].x, lo);
            transpose_6planes(kc[0].y, kc[1].y, kc[2].y, kc[3].y, kc[4].y, kc[5].y, hi);
            v4i ka[4];
            ka[0] = (v4i){static_cast<int>(lo[0]), static_cast<int>(lo[1]), static_cast<int>(lo[2]), static_cast<int>(lo[3])};
            ka[1] = (v4i){static_cast<int>(lo[4]), static_cast<int>(lo[5]), static_cast<int>(lo[6]), static_cast<int>(lo[7])};
            ka[2] = (v4i){static_cast<int>(hi[0]), static_cast<int>(hi[1]), static_cast<int>(hi[2]), static_cast<int>(hi[3])};
            ka[3] = (v4i){static_cast<int>(hi[4]), static_cast<int>(hi[5]), static_cast<int>(hi[6]), static_cast<int>(hi[7])};
            v4i acc = {0, 0, 0, 0};
#pragma unroll
            for (int m = 0; m < 4; ++m) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[m], qb[m], acc, 0, 0, 0);
            *reinterpret_cast<v4i*>(&ints[(c - p0) * 256 + ln * 16 + lg * 4]) = acc;
        }
        __syncthreads();
        if (cvalid) {
            accf = chain_chunks(accf, p0, pend, down, [&](int cc) { return ints[(cc - p0) * 256 + cn * 16 + ckey]; },
                                [&](int cc) { return myscale[cc * sstep]; });
            if (kInts)
                for (int cc = p0; cc < pend; ++cc)
                    chunk_ints[((q0 + cn) * R + cr) * chunks + cc] = ints[(cc - p0) * 256 + cn * 16 + ckey] >> down_shift;
        }
        if (pend < chunks) __syncthreads();
    }
    if (cvalid) {
        float v = (accf * Bw[cr * 6]) * scale_inv;
        if (bias != nullptr) v = v + bias[cr];
        out[(q0 + cn) * R_total + cr] = v;
    }
}

// EWAH streams of a whole query batch -> the int8 query image the compute-bound dot contracts (value << (8 - Sa),
// in-chunk byte order of planes_to_int8_kernel): one workgroup per query row expands the row's Sa streams into LDS
// (a wave per stream, all-zero slices skipped) and recombines them 32 elements per thread.  The verbatim planes
// never exist in memory.
constexpr int kEwahToInt8Block = 512;  // 8 waves: the (at most 8) streams of a row decode side by side
__global__ __launch_bounds__(kEwahToInt8Block) void ewah_streams_to_int8_kernel(const unsigned long long* __restrict__ comp,
                                                                    const long long* __restrict__ comp_off,
                                                                    const int* __restrict__ comp_len, int Sa, int W64,
                                                                    int chunks, uint32_t* __restrict__ out32) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int wpad = chunks * 4;
    unsigned long long* planes = reinterpret_cast<unsigned long long*>(smem);  // [Sa][wpad]
    unsigned char* present = smem + static_cast<size_t>(Sa) * wpad * 8;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t row = blockIdx.x;
    for (int s = wave; s < Sa; s += kEwahToInt8Block / BSI_WAVE) {
        const unsigned long long* in = comp + comp_off[row * Sa + s];
        const int in_len = comp_len[row * Sa + s];
        const bool zero = ewah_stream_is_zero(in, in_len, W64);
        if (lane == 0) present[s] = zero ? 0 : 1;
        if (!zero) ewah_expand_wave(in, in_len, W64, planes + static_cast<size_t>(s) * wpad, wpad, lane);
    }
    __syncthreads();
    const uint32_t* planes32 = reinterpret_cast<const uint32_t*>(planes);
    const int cols = chunks * 8;
    for (int col = tid; col < cols; col += kEwahToInt8Block) {
        uint32_t y[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int j = t - (8 - Sa);
            y[t] = (j >= 0 && present[j]) ? planes32[static_cast<size_t>(j) * wpad * 2 + col] : 0u;
        }
        transpose8x8(y);
        uint4* dst = reinterpret_cast<uint4*>(out32 + (static_cast<size_t>(row) * cols + col) * 8);
        dst[0] = make_uint4(y[0], y[1], y[2], y[3]);
        dst[1] = make_uint4(y[4], y[5], y[6], y[7]);
    }
}

template <int NT, int KT>
static void launch_mfma_stream(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                               int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                               float* out, int32_t* chunk_ints, const float* bias, hipStream_t st) {
    constexpr int kSlot = KT * NT * 256;
    const int64_t ntiles = (R + 15) / 16;
    const dim3 grid(static_cast<unsigned>((ntiles + KT - 1) / KT), static_cast<unsigned>((Q + 16 * NT - 1) / (16 * NT)));
    // one workgroup per CU at most: more waves each streaming their own chunks; else 8 and several workgroups
    int waves = (grid.x * grid.y <= 256) ? 16 : 8;
    if (waves > chunks) waves = chunks;             // one chunk per wave and pass at least
    if (waves < kSlot / 64) waves = kSlot / 64;     // the chain needs one lane per output
    if (waves > 16) waves = 16;
    int pass_chunks = kStreamLdsInts / kSlot;
    if (pass_chunks > chunks) pass_chunks = chunks;
    const size_t lds = static_cast<size_t>(pass_chunks) * kSlot * sizeof(int);
    if (chunk_ints)
        hipLaunchKernelGGL((dot_mfma_stream_kernel<NT, KT, true>), grid, dim3(waves * 64), lds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, pass_chunks, R, Q, down_shift,
                           scale_inv, R_total, out, chunk_ints, bias);
    else
        hipLaunchKernelGGL((dot_mfma_stream_kernel<NT, KT, false>), grid, dim3(waves * 64), lds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, pass_chunks, R, Q, down_shift,
                           scale_inv, R_total, out, chunk_ints, bias);
}

void launch_mfma_stream_by_shape(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                                 int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                                 float* out, int32_t* chunk_ints, const float* bias, hipStream_t st) {
    // two key tiles per workgroup halve the query re-reads once there are enough tiles to fill the GPU
    const bool two = (R + 15) / 16 >= 1024;
#define BSI_STREAM_ARGS A8, qscale, stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, st
    if (Q <= 16) { if (two) launch_mfma_stream<1, 2>(BSI_STREAM_ARGS); else launch_mfma_stream<1, 1>(BSI_STREAM_ARGS); }
    else { if (two) launch_mfma_stream<2, 2>(BSI_STREAM_ARGS); else launch_mfma_stream<2, 1>(BSI_STREAM_ARGS); }
#undef BSI_STREAM_ARGS
}

// Launch shape of the fused few-rows kernel: key tiles per workgroup, waves, and how many (chunk, row) items of the
// query build a wave takes up front (loads issued before the key loads; the rest go one at a time, each waiting for
// its own loads).
struct FusedPlan {
    int key_tiles, waves, upfront, per_wave;
    unsigned grid;
};
static FusedPlan fused_plan(int64_t Q, int chunks, int64_t R) {
    FusedPlan p;
    const int64_t ntiles = (R + 15) / 16;
    p.key_tiles = ntiles >= 1024 ? 2 : 1;  // as bsi_hip_dot: two key tiles per workgroup once the GPU is full
    p.grid = static_cast<unsigned>((ntiles + p.key_tiles - 1) / p.key_tiles);
    p.waves = (p.grid <= 256) ? 16 : 8;  // as the few-rows kernel: one workgroup per CU gets more waves
    if (p.waves > chunks) p.waves = chunks;
    if (p.waves < p.key_tiles * 4) p.waves = p.key_tiles * 4;
    p.per_wave = static_cast<int>((static_cast<int64_t>(chunks) * Q + p.waves - 1) / p.waves);
    const int cap = p.key_tiles == 1 ? 4 : 2;
    p.upfront = p.per_wave <= 1 ? 1 : (p.per_wave <= 2 ? 2 : cap);
    return p;
}

template <typename T, int KT, int NI>
static void launch_stream_fused(const FusedPlan& plan, const T* x, int64_t d, double dec_scale, int slices, const uint64_t* B,
                                const float* Bw, int chunks, int64_t R, int Q, float scale_inv, int64_t R_total, float* out,
                                const float* bias, hipStream_t st) {
    constexpr int kSlot = KT * 256;
    // LDS: the query image and scales of all chunks, then as many chunk accumulators as fit beside them
    const size_t query_bytes = static_cast<size_t>(chunks) * Q * (256 + sizeof(float));
    int pass_chunks = kStreamLdsInts / kSlot;
    const int fit = static_cast<int>((150 * 1024 - query_bytes) / (kSlot * sizeof(int)));
    if (pass_chunks > fit) pass_chunks = fit;
    if (pass_chunks > chunks) pass_chunks = chunks;
    const size_t lds = static_cast<size_t>(pass_chunks) * kSlot * sizeof(int) + query_bytes;
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_stream_fused_kernel<T, KT, NI>), 160 * 1024);
    const unsigned scale_int = integer_decimal_scale(dec_scale);
    hipLaunchKernelGGL((dot_mfma_stream_fused_kernel<T, KT, NI>), dim3(plan.grid), dim3(plan.waves * 64), lds, st, x, d,
                       dec_scale, scale_int, slices, reinterpret_cast<const unsigned long long*>(B), Bw, chunks, pass_chunks,
                       R, Q, scale_inv, R_total, out, bias);
}

template <typename T>
static void launch_stream_fused_t(const T* x, int64_t d, double dec_scale, int slices, const uint64_t* B, const float* Bw,
                                  int chunks, int64_t R, int Q, float scale_inv, int64_t R_total, float* out,
                                  const float* bias, hipStream_t st) {
    const FusedPlan p = fused_plan(Q, chunks, R);
#define BSI_FUSED_GO(KT, NI) \
    launch_stream_fused<T, KT, NI>(p, x, d, dec_scale, slices, B, Bw, chunks, R, Q, scale_inv, R_total, out, bias, st)
    if (p.key_tiles == 2) {
        if (p.upfront == 1) BSI_FUSED_GO(2, 1);
        else BSI_FUSED_GO(2, 2);
    } else {
        if (p.upfront == 1) BSI_FUSED_GO(1, 1);
        else if (p.upfront == 2) BSI_FUSED_GO(1, 2);
        else BSI_FUSED_GO(1, 4);
    }
#undef BSI_FUSED_GO
}

}  // namespace bsi

using namespace bsi;

extern "C" int bsi_hip_linear_few_rows_upfront(int64_t Q, int64_t d, int64_t R) {
    if (Q < 1 || Q > kFusedMaxQ || d < 1 || R < 1) return 0;
    const FusedPlan p = fused_plan(Q, static_cast<int>((d + 255) / 256), R);
    return p.per_wave <= p.upfront ? 1 : 0;
}

extern "C" int bsi_hip_linear_few_rows(const void* x, int dtype, int64_t Q, int64_t d, int decimal_places, int fixed_bits,
                                       const uint64_t* B_tiled, const float* Bw, int Sb, int64_t R, float scale_inv,
                                       int64_t R_total, const float* bias, float* out, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0 && d >= 1, "bad shape");
    BSI_REQUIRE(Q <= kFusedMaxQ, "the fused few-rows kernel takes at most %d query rows (got %lld)", kFusedMaxQ,
                static_cast<long long>(Q));
    BSI_REQUIRE(fixed_bits >= 2 && fixed_bits <= 8, "fixed_bits must be in [2, 8] (got %d)", fixed_bits);
    BSI_REQUIRE(R_total >= R, "R_total must be >= R");
    if (Sb != 6) return fail(BSI_ERR_UNSUPPORTED, "the fused few-rows kernel reads 6-plane tiled keys (got Sb = %d)", Sb);
    const int W64 = static_cast<int>((d + 63) / 64);
    if (W64 % 4 != 0)
        return fail(BSI_ERR_UNSUPPORTED, "chunk scales need a multiple of 4 words per slice (d = %lld)", static_cast<long long>(d));
    if (Q == 0 || R == 0) return BSI_OK;
    BSI_REQUIRE(x && B_tiled && Bw && out, "null pointer");
    const int chunks = W64 / 4;
    if (static_cast<size_t>(chunks) * Q * (256 + sizeof(float)) > kFusedQueryLdsBytes)
        return fail(BSI_ERR_UNSUPPORTED, "%lld rows of %lld elements do not fit the kernel's LDS query buffer (%zu bytes)",
                    static_cast<long long>(Q), static_cast<long long>(d), kFusedQueryLdsBytes);
    const double dec_scale = pow(10.0, static_cast<double>(decimal_places));
    hipStream_t st = as_stream(stream);
#define BSI_FUSED(T)                                                                                                \
    launch_stream_fused_t<T>(static_cast<const T*>(x), d, dec_scale, fixed_bits, B_tiled, Bw, chunks, R, static_cast<int>(Q), \
                             scale_inv, R_total, out, bias, st);
    if (dtype == BSI_DTYPE_F32) { BSI_FUSED(float) }
    else if (dtype == BSI_DTYPE_F16) { BSI_FUSED(__half) }
    else if (dtype == BSI_DTYPE_BF16) { BSI_FUSED(__hip_bfloat16) }
    else return fail(BSI_ERR_INVALID, "unknown dtype %d", dtype);
#undef BSI_FUSED
    BSI_LAUNCH_CHECK("dot_mfma_stream_fused_kernel");
    return BSI_OK;
}

// Launch of the inline-decode kernel for Q queries (groups of 16 along grid.y), or BSI_ERR_UNSUPPORTED when the
// planes of a group do not fit LDS.
static int launch_stream_ewah(const uint64_t* comp_words, const int64_t* comp_off, const int32_t* comp_len, int Sa, int W64,
                              const float* A_chunk_scales, int A_scale_stride, const uint64_t* B_tiled, const float* Bw,
                              int64_t R, int64_t Q, float scale_inv, int64_t R_total, const float* bias, float* out,
                              int32_t* chunk_ints, hipStream_t st) {
    const int chunks = (W64 + 3) / 4;
    const int group = static_cast<int>(Q < kEwahQueriesPerGroup ? Q : kEwahQueriesPerGroup);
    const size_t plane_bytes = ewah_plane_region(group, Sa, chunks * 4) + 128;
    if (plane_bytes > 120 * 1024)
        return fail(BSI_ERR_UNSUPPORTED, "%d words per slice do not fit the LDS plane buffer of the inline-decode kernel", W64);
    int pass_chunks = static_cast<int>((kStreamLdsInts * sizeof(int) < 156 * 1024 - plane_bytes
                                            ? kStreamLdsInts * sizeof(int)
                                            : 156 * 1024 - plane_bytes) / 1024);
    if (pass_chunks > chunks) pass_chunks = chunks;
    const size_t lds = plane_bytes + static_cast<size_t>(pass_chunks) * 1024;
    int waves = chunks < 16 ? chunks : 16;
    if (waves < 4) waves = 4;
    const dim3 grid(static_cast<unsigned>((R + 15) / 16), static_cast<unsigned>((Q + kEwahQueriesPerGroup - 1) / kEwahQueriesPerGroup));
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_stream_ewah_kernel<true>), 160 * 1024);
    static LdsOptIn once1;
    lds_opt_in(once1, reinterpret_cast<const void*>(&dot_mfma_stream_ewah_kernel<false>), 160 * 1024);
    const int down_shift = 16 - Sa - 6;
#define BSI_EWAH_ARGS reinterpret_cast<const unsigned long long*>(comp_words), reinterpret_cast<const long long*>(comp_off), \
                      comp_len, Sa, W64, A_chunk_scales, A_scale_stride, reinterpret_cast<const unsigned long long*>(B_tiled), \
                      Bw, chunks, pass_chunks, R, Q, group, down_shift, scale_inv, R_total, bias, out, chunk_ints
    if (chunk_ints) hipLaunchKernelGGL((dot_mfma_stream_ewah_kernel<true>), grid, dim3(waves * 64), lds, st, BSI_EWAH_ARGS);
    else hipLaunchKernelGGL((dot_mfma_stream_ewah_kernel<false>), grid, dim3(waves * 64), lds, st, BSI_EWAH_ARGS);
#undef BSI_EWAH_ARGS
    BSI_LAUNCH_CHECK("dot_mfma_stream_ewah_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_dot_ewah_query(const uint64_t* comp_words, const int64_t* comp_off, const int32_t* comp_len,
                                      int Sa, int W64, const float* A_chunk_scales, int A_scale_stride,
                                      const uint64_t* B_tiled, const float* Bw, int Sb, int64_t R, float scale_inv,
                                      float* out, int32_t* chunk_ints, void* stream) {
    BSI_REQUIRE(R >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(Sa >= 2 && Sa <= 8, "Sa must be in [2, 8] (got %d)", Sa);
    if (Sb != 6) return fail(BSI_ERR_UNSUPPORTED, "the inline-decode kernel reads 6-plane tiled keys (got Sb = %d)", Sb);
    if (R == 0) return BSI_OK;
    BSI_REQUIRE(comp_words && comp_off && comp_len && A_chunk_scales && B_tiled && Bw && out, "null pointer");
    const int chunks = (W64 + 3) / 4;
    BSI_REQUIRE(A_scale_stride == chunks || A_scale_stride == 1,
                "chunk scale stride mismatch: got %d expected %d (or 1 for a row scale)", A_scale_stride, chunks);
    return launch_stream_ewah(comp_words, comp_off, comp_len, Sa, W64, A_chunk_scales, A_scale_stride, B_tiled, Bw, R, 1,
                              scale_inv, R, nullptr, out, chunk_ints, as_stream(stream));
}

extern "C" size_t bsi_hip_dot_ewah_batch_workspace_bytes(int64_t Q, int W64) {
    return bsi_hip_dot_workspace_bytes(Q, W64, BSI_CORE_MFMA);
}

extern "C" int bsi_hip_dot_ewah_batch(const uint64_t* comp_words, const int64_t* comp_off, const int32_t* comp_len, int Sa,
                                      int W64, const float* A_chunk_scales, int A_scale_stride, const uint64_t* B,
                                      int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q, float scale_inv,
                                      int64_t R_total, const float* bias, float* out, int32_t* chunk_ints, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0 && W64 >= 1 && R_total >= R, "bad shape");
    BSI_REQUIRE(Sa >= 2 && Sa <= 8 && Sb >= 2 && Sb <= 8, "the matrix-core dot needs Sa, Sb in [2, 8] (got %d, %d)", Sa, Sb);
    if (Q == 0 || R == 0) return BSI_OK;
    BSI_REQUIRE(comp_words && comp_off && comp_len && A_chunk_scales && B && Bw && out, "null pointer");
    const int chunks = (W64 + 3) / 4;
    BSI_REQUIRE(A_scale_stride == chunks || A_scale_stride == 1,
                "chunk scale stride mismatch: got %d expected %d (or 1 for row scales)", A_scale_stride, chunks);
    hipStream_t st = as_stream(stream);
    // A few rows against the packed planes: the call is bound by streaming the keys once, and each workgroup can
    // afford to expand the queries itself -- the decode is part of the dot kernel's load stage.
    const int64_t group = Q < kEwahQueriesPerGroup ? Q : kEwahQueriesPerGroup;
    if (Q <= kStreamMaxQ && b_layout == BSI_LAYOUT_TILED16 && Sb == 6 &&
        ewah_plane_region(static_cast<int>(group), Sa, chunks * 4) + 128 <= 120 * 1024)
        return launch_stream_ewah(comp_words, comp_off, comp_len, Sa, W64, A_chunk_scales, A_scale_stride, B, Bw, R, Q,
                                  scale_inv, R_total, bias, out, chunk_ints, st);
    // Many rows: every key-tile workgroup of the compute-bound kernel reads the whole query tile, so expanding the
    // streams there would repeat the decode and the plane -> int8 recombination once per key tile (32 times at
    // Q512 x R2048).  The call's load stage therefore runs once, as a launch of its own: streams -> int8 query
    // image in the workspace (the verbatim planes are never materialised), then the dot on that image.
    const size_t need = bsi_hip_dot_ewah_batch_workspace_bytes(Q, W64);
    BSI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "%zu bytes of workspace needed for the int8 query image (got %zu)",
                need, workspace_bytes);
    BSI_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, "workspace must be 16-byte aligned");
    const size_t lds = static_cast<size_t>(Sa) * chunks * 4 * 8 + 64;
    if (lds > 150 * 1024)
        return fail(BSI_ERR_UNSUPPORTED, "%d words per slice do not fit the LDS plane buffer of the stream decoder", W64);
    static LdsOptIn once;
    lds_opt_in(once, reinterpret_cast<const void*>(&ewah_streams_to_int8_kernel), 160 * 1024);
    hipLaunchKernelGGL(ewah_streams_to_int8_kernel, dim3(static_cast<unsigned>(Q)), dim3(kEwahToInt8Block), lds, st,
                       reinterpret_cast<const unsigned long long*>(comp_words), reinterpret_cast<const long long*>(comp_off),
                       comp_len, Sa, W64, chunks, static_cast<uint32_t*>(workspace));
    BSI_LAUNCH_CHECK("ewah_streams_to_int8_kernel");
    return dot_with_bias(nullptr, static_cast<const int8_t*>(workspace), A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout,
                         Bw, Sb, R, Q, scale_inv, R_total, out, chunk_ints, BSI_CORE_MFMA, nullptr, 0, stream, bias);
}
