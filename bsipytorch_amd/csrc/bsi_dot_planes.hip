// The matrix-core dot on key PLANES (canonical or tiled16): the workgroup recombines the planes of its key tile
// into int8 itself.  Many query rows without a cached int8 image of the keys, and slice counts other than 6.
#include "bsi_dot_device.h"
#include "bsi_dot_internal.h"

namespace bsi {

// ------------------------------------------------------------------ MFMA core

constexpr int kMfmaBlock = 256;
constexpr int kTileR = 128;            // keys per workgroup
constexpr int kTileQ = 128;            // queries per workgroup
constexpr int kRowBytes = 256 + 32;    // one chunk of int8 per row + pad: b128 reads of 16 consecutive rows hit all 64 banks once

// Fetch plane j's 32-bit column `col` (0..7 within the chunk) of key row r.
template <bool kTiled>
__device__ __forceinline__ uint32_t key_word32(const uint32_t* __restrict__ B32, int64_t r, int j, int Sb, int W64,
                                               int chunks, int c, int col) {
    if (kTiled) {
        const size_t w64 = ((((static_cast<size_t>(r >> 4) * chunks + c) * Sb + j) << 6) + ((col >> 1) << 4) + (r & 15));
        return B32[w64 * 2 + (col & 1)];
    }
    const int w = c * 4 + (col >> 1);
    return (w < W64) ? B32[((static_cast<size_t>(r) * Sb + j) * W64 + w) * 2 + (col & 1)] : 0u;
}

template <int SB, bool kTiled, bool kInts>
__global__ __launch_bounds__(kMfmaBlock) void dot_mfma_kernel(
    const int8_t* __restrict__ A8,         // [Q, chunks*256] int8, value << (8 - Sa), MFMA element order
    const float* __restrict__ qscale, int qscale_stride,
    const uint32_t* __restrict__ B32,      // key planes as 32-bit words
    const float* __restrict__ Bw, int Sb_rt, int W64, int chunks, int64_t R, int64_t Q, int down_shift,
    float scale_inv, int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // (kTileR + kTileQ) * kRowBytes
    unsigned char* K8 = lds;
    unsigned char* Q8 = lds + kTileR * kRowBytes;

    const int Sb = (SB > 0) ? SB : Sb_rt;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wr = wave & 1;   // which 64-key half of the tile
    const int wq = wave >> 1;  // which 64-query half
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kTileR;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * kTileQ;
    const int ln = lane & 15;
    const int lg = lane >> 4;
    const int64_t Rlim = kTiled ? ((R + 15) / 16) * 16 : R;  // rows that exist in the key buffer

    float accf[4][4][4];  // [key tile][query tile][reg]
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;

    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);  // 2^-down_shift

    for (int c = 0; c < chunks; ++c) {
        // ---- stage: key planes -> int8 rows in LDS (each thread: 4 (row, 32-bit column) cells)
#pragma unroll
        for (int it = 0; it < (kTileR * 8) / kMfmaBlock; ++it) {
            const int cell = tid + it * kMfmaBlock;
            const int row = cell >> 3;
            const int col = cell & 7;
            const int64_t r = r0 + row;
            uint32_t y[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                if (SB > 0) {
                    y[s] = (s >= 8 - SB && r < Rlim) ? key_word32<kTiled>(B32, r, s - (8 - SB), SB, W64, chunks, c, col) : 0u;
                } else {
                    const int j = s - (8 - Sb);
                    y[s] = (j >= 0 && r < Rlim) ? key_word32<kTiled>(B32, r, j, Sb, W64, chunks, c, col) : 0u;
                }
            }
            transpose8x8(y);
            uint4* dst = reinterpret_cast<uint4*>(K8 + row * kRowBytes + col * 32);
            dst[0] = make_uint4(y[0], y[1], y[2], y[3]);
            dst[1] = make_uint4(y[4], y[5], y[6], y[7]);
        }
        // ---- stage: int8 query rows (16 B pieces)
#pragma unroll
        for (int it = 0; it < (kTileQ * 16) / kMfmaBlock; ++it) {
            const int piece = tid + it * kMfmaBlock;
            const int row = piece >> 4;
            const int seg = piece & 15;
            const int64_t q = q0 + row;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (q < Q) v = *reinterpret_cast<const uint4*>(A8 + (static_cast<size_t>(q) * chunks + c) * 256 + seg * 16);
            *reinterpret_cast<uint4*>(Q8 + row * kRowBytes + seg * 16) = v;
        }
        __syncthreads();

        // ---- 4 k-steps of 64 over this chunk: 4x4 tiles of 16x16
        v4i acc[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[a][b] = (v4i){0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            v4i ka[4], qb[4];
#pragma unroll
            for (int a = 0; a < 4; ++a)
                ka[a] = *reinterpret_cast<const v4i*>(K8 + (wr * 64 + a * 16 + ln) * kRowBytes + ks * 64 + lg * 16);
#pragma unroll
            for (int b = 0; b < 4; ++b)
                qb[b] = *reinterpret_cast<const v4i*>(Q8 + (wq * 64 + b * 16 + ln) * kRowBytes + ks * 64 + lg * 16);
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[a], qb[b], acc[a][b], 0, 0, 0);
        }

        // ---- epilogue of the chunk: lane owns query column (b*16 + ln), key rows a*16 + lg*4 + e
        const int cs = (qscale_stride == 1) ? 0 : c;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t q = q0 + wq * 64 + b * 16 + ln;
            const float qs = (q < Q) ? qscale[q * qscale_stride + cs] * down : 0.0f;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    accf[a][b][e] = fmaf(static_cast<float>(acc[a][b][e]), qs, accf[a][b][e]);
                    if (kInts) {
                        const int64_t r = r0 + wr * 64 + a * 16 + lg * 4 + e;
                        if (q < Q && r < R) chunk_ints[(static_cast<size_t>(q) * R + r) * chunks + c] = acc[a][b][e] >> down_shift;
                    }
                }
        }
        __syncthreads();
    }

    // ---- write out: (acc * bscale) * scale_inv
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int64_t rb = r0 + wr * 64 + a * 16 + lg * 4;
        float bs[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) bs[e] = (rb + e < R) ? key_factor(Bw[(rb + e) * Sb]) : 0.0f;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t q = q0 + wq * 64 + b * 16 + ln;
            if (q >= Q) continue;
            float* dst = out + static_cast<size_t>(q) * R_total + rb;
            if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                *reinterpret_cast<float4*>(dst) =
                    make_float4((accf[a][b][0] * bs[0]) * scale_inv, (accf[a][b][1] * bs[1]) * scale_inv,
                                (accf[a][b][2] * bs[2]) * scale_inv, (accf[a][b][3] * bs[3]) * scale_inv);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (rb + e < R) dst[e] = (accf[a][b][e] * bs[e]) * scale_inv;
            }
        }
    }
}

// ------------------------------------------------------------------ MFMA core, producer/consumer form
//
// 768 threads: waves 0-7 are consumers (64 keys x 32 queries each, 32 MFMAs per chunk), waves 8-11
// are producers.  A producer wave owns 32 key rows and 32 query rows of the 128 x 128 tile: per
// chunk it reads its key planes from the tiled layout (one coalesced 512-byte wave load per plane
// and 16-key tile: lane (m, g) gets words32 2g, 2g+1 of row m), transposes them to 64 int8 per
// lane, and copies its query int8 rows and chunk scales; all go to the LDS buffer of the NEXT chunk
// while the consumers run the MFMAs of the current one out of the other buffer.  The loads for the
// chunk after that are issued before the barrier, so their latency is covered by a whole
// iteration.  Each SIMD hosts two consumer waves and one producer wave: a single wave cannot pull
// more than about 32 B/clk out of LDS, two consumers per SIMD keep the matrix pipe fed, and the
// transposes run on the VALU meanwhile.

constexpr int kWsConsumers = 8;                      // consumer waves: 64 keys x 32 queries each
constexpr int kWsBlock = (kWsConsumers + 4) * 64;    // + 4 producer waves

// LDS buffer of one chunk: int8 key rows (padded, written through registers), int8 query rows
// (unpadded, 16-byte columns XOR-swizzled by row & 15, written by direct global->LDS loads) and
// the chunk scales of the 128 queries (64 floats per producer wave, the upper 32 unused).
constexpr int kWsQOff = kTileR * kRowBytes;
constexpr int kWsScaleOff = kWsQOff + kTileQ * 256;
constexpr int kWsStage = kWsScaleOff + 4 * 64 * 4;  // bytes of one LDS buffer


// Key planes of one chunk for the producer's two 16-key tiles -> registers (words32 2g, 2g+1 of
// row m).  `src0/src1` are the wave-uniform addresses of the two tiles' first plane of this chunk.
template <int SB>
__device__ __forceinline__ void ws_load_keys(uint2 (&k)[2][SB], const unsigned long long* __restrict__ src0,
                                             const unsigned long long* __restrict__ src1, int lane) {
#pragma unroll
    for (int j = 0; j < SB; ++j) {
        const unsigned long long w0 = src0[j * 64 + lane];
        const unsigned long long w1 = src1[j * 64 + lane];
        k[0][j] = make_uint2(static_cast<uint32_t>(w0), static_cast<uint32_t>(w0 >> 32));
        k[1][j] = make_uint2(static_cast<uint32_t>(w1), static_cast<uint32_t>(w1 >> 32));
    }
}

// int8 query rows and chunk scales of one chunk straight into the LDS buffer (no registers): a
// wave instruction fills 1 KiB = 4 rows; lane L lands at row L/16, physical column L%16 and
// therefore fetches logical column (L%16) ^ (row & 15) (the per-lane byte offsets `qoff`).
// `a8c` / `qsc` are the wave-uniform bases of this chunk.
__device__ __forceinline__ void ws_load_queries_to_lds(unsigned char* __restrict__ qdst, unsigned char* __restrict__ sdst,
                                                       const int8_t* __restrict__ a8c, const uint32_t (&qoff)[8],
                                                       const float* __restrict__ qsc, uint32_t soff) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
        __builtin_amdgcn_global_load_lds(BSI_GLOBAL_PTR(a8c + qoff[i]), BSI_LDS_PTR(qdst + i * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds(BSI_GLOBAL_PTR(reinterpret_cast<const char*>(qsc) + soff), BSI_LDS_PTR(sdst), 4, 0, 0);
}

// Transpose the two key tiles to int8 and write them to the LDS buffer (`dst` = this lane's row
// and 64-byte column group of tile 0; tile 1 is 16 rows further).
template <int SB>
__device__ __forceinline__ void ws_store_keys(const uint2 (&k)[2][SB], unsigned char* __restrict__ dst) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        uint32_t lo[8], hi[8];
        if (SB == 6) {
            transpose_6planes(k[t][0].x, k[t][1].x, k[t][2].x, k[t][3].x, k[t][4].x, k[t][5].x, lo);
            transpose_6planes(k[t][0].y, k[t][1].y, k[t][2].y, k[t][3].y, k[t][4].y, k[t][5].y, hi);
        } else {
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                lo[s] = (s >= 8 - SB) ? k[t][s - (8 - SB)].x : 0u;
                hi[s] = (s >= 8 - SB) ? k[t][s - (8 - SB)].y : 0u;
            }
            transpose8x8(lo);
            transpose8x8(hi);
        }
        uint4* d = reinterpret_cast<uint4*>(dst + t * 16 * kRowBytes);
        d[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        d[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        d[2] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        d[3] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    }
}

// One producer iteration with the 21 vector-memory instructions spread between the transpose
// stages (the memory pipeline accepts a wave's loads only slowly; issued in one burst they would
// block the wave for longer than the transposes take).  Order of the loads: 8 query row groups and
// the scales straight to LDS (for the chunk being staged), then the 12 key-plane loads of the
// chunk after it into `kn` -- the final wait leaves exactly those 12 in flight.
// `kc` holds the key planes of the chunk being staged (loaded one iteration earlier).
__device__ __forceinline__ void ws_produce6(const uint2 (&kc)[2][6], uint2 (&kn)[2][6], unsigned char* __restrict__ kdst,
                                            unsigned char* __restrict__ qdst, unsigned char* __restrict__ sdst,
                                            const int8_t* __restrict__ a8c, const uint32_t (&qoff)[8],
                                            const float* __restrict__ qsc, uint32_t soff,
                                            const unsigned long long* __restrict__ kn0,
                                            const unsigned long long* __restrict__ kn1, int lane) {
#define BSI_LQ(i) __builtin_amdgcn_global_load_lds(BSI_GLOBAL_PTR(a8c + qoff[i]), BSI_LDS_PTR(qdst + (i) * 1024), 16, 0, 0)
#define BSI_LK(t, j)                                                                             \
    {                                                                                            \
        const unsigned long long w_ = ((t) ? kn1 : kn0)[(j) * 64 + lane];                        \
        kn[t][j] = make_uint2(static_cast<uint32_t>(w_), static_cast<uint32_t>(w_ >> 32));       \
    }
#define BSI_SB __builtin_amdgcn_sched_barrier(0)
    uint32_t x[8], a[8], y[8];
    uint4* d0 = reinterpret_cast<uint4*>(kdst);
    uint4* d1 = reinterpret_cast<uint4*>(kdst + 16 * kRowBytes);
    // tile 0, low words
    BSI_LQ(0); BSI_LQ(1); BSI_SB;
    t6_stage1(kc[0][0].x, kc[0][1].x, kc[0][2].x, kc[0][3].x, kc[0][4].x, kc[0][5].x, x); BSI_SB;
    BSI_LQ(2); BSI_LQ(3); BSI_SB;
    t6_stage2(x, a); BSI_SB;
    BSI_LQ(4); BSI_LQ(5); BSI_SB;
    t6_stage3(a, y);
    d0[0] = make_uint4(y[0], y[1], y[2], y[3]); d0[1] = make_uint4(y[4], y[5], y[6], y[7]); BSI_SB;
    // tile 0, high words
    BSI_LQ(6); BSI_LQ(7); BSI_SB;
    t6_stage1(kc[0][0].y, kc[0][1].y, kc[0][2].y, kc[0][3].y, kc[0][4].y, kc[0][5].y, x); BSI_SB;
    __builtin_amdgcn_global_load_lds(BSI_GLOBAL_PTR(reinterpret_cast<const char*>(qsc) + soff), BSI_LDS_PTR(sdst), 4, 0, 0);
    BSI_LK(0, 0); BSI_SB;
    t6_stage2(x, a); BSI_SB;
    BSI_LK(0, 1); BSI_LK(0, 2); BSI_SB;
    t6_stage3(a, y);
    d0[2] = make_uint4(y[0], y[1], y[2], y[3]); d0[3] = make_uint4(y[4], y[5], y[6], y[7]); BSI_SB;
    // tile 1, low words
    BSI_LK(0, 3); BSI_LK(0, 4); BSI_SB;
    t6_stage1(kc[1][0].x, kc[1][1].x, kc[1][2].x, kc[1][3].x, kc[1][4].x, kc[1][5].x, x); BSI_SB;
    BSI_LK(0, 5); BSI_LK(1, 0); BSI_SB;
    t6_stage2(x, a); BSI_SB;
    BSI_LK(1, 1); BSI_LK(1, 2); BSI_SB;
    t6_stage3(a, y);
    d1[0] = make_uint4(y[0], y[1], y[2], y[3]); d1[1] = make_uint4(y[4], y[5], y[6], y[7]); BSI_SB;
    // tile 1, high words
    BSI_LK(1, 3); BSI_SB;
    t6_stage1(kc[1][0].y, kc[1][1].y, kc[1][2].y, kc[1][3].y, kc[1][4].y, kc[1][5].y, x); BSI_SB;
    BSI_LK(1, 4); BSI_SB;
    t6_stage2(x, a); BSI_SB;
    BSI_LK(1, 5); BSI_SB;
    t6_stage3(a, y);
    d1[2] = make_uint4(y[0], y[1], y[2], y[3]); d1[3] = make_uint4(y[4], y[5], y[6], y[7]); BSI_SB;
#undef BSI_LQ
#undef BSI_LK
#undef BSI_SB
}

// One chunk of a consumer wave: 4 k-steps of 8 MFMAs.  The instruction order is fixed by hand
// (sched_barrier after every group, the compiler's scheduler would otherwise pull every LDS read
// next to its first use): each MFMA is preceded by one LDS read of the NEXT k-step's operands and
// followed by two VALU operations of the fp32 epilogue of the PREVIOUS chunk, so the LDS queue
// never fills, the matrix pipe always has the next MFMA waiting and the epilogue rides in its
// shadow.  Reads are issued in the order the next k-step consumes them.
template <bool kHasPrev, bool kInts>
__device__ __forceinline__ void ws_consume_chunk(const unsigned char* __restrict__ kbase,
                                                 const unsigned char* __restrict__ qrow, const int (&qcol)[4],
                                                 v4i (&cur)[4][2],
                                                 const v4i (&prev)[4][2], const float (&qs_prev)[2],
                                                 float (&accf)[4][2][4], int* __restrict__ ints_prev, int down_shift,
                                                 const int64_t (&int_off)[4][2], const int (&int_rows)[4], int chunks) {
    v4i ka[2][4], qb[2][2];
    ka[0][0] = *reinterpret_cast<const v4i*>(kbase);
    qb[0][0] = *reinterpret_cast<const v4i*>(qrow + qcol[0]);
    qb[0][1] = *reinterpret_cast<const v4i*>(qrow + 16 * 256 + qcol[0]);
    ka[0][1] = *reinterpret_cast<const v4i*>(kbase + 16 * kRowBytes);
    ka[0][2] = *reinterpret_cast<const v4i*>(kbase + 32 * kRowBytes);
    ka[0][3] = *reinterpret_cast<const v4i*>(kbase + 48 * kRowBytes);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int nx = (ks + 1) & 1, cu = ks & 1;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            const int a = g >> 1, b = g & 1;
            if (ks < 3) {  // one operand read of k-step ks+1, in consumption order
                const int off = (ks + 1) * 64;
                if (g == 0) ka[nx][0] = *reinterpret_cast<const v4i*>(kbase + off);
                if (g == 1) qb[nx][0] = *reinterpret_cast<const v4i*>(qrow + qcol[(ks + 1) & 3]);
                if (g == 2) qb[nx][1] = *reinterpret_cast<const v4i*>(qrow + 16 * 256 + qcol[(ks + 1) & 3]);
                if (g == 3) ka[nx][1] = *reinterpret_cast<const v4i*>(kbase + 16 * kRowBytes + off);
                if (g == 4) ka[nx][2] = *reinterpret_cast<const v4i*>(kbase + 32 * kRowBytes + off);
                if (g == 5) ka[nx][3] = *reinterpret_cast<const v4i*>(kbase + 48 * kRowBytes + off);
            }
            __builtin_amdgcn_sched_barrier(0);
            const v4i c0 = (ks == 0) ? (v4i){0, 0, 0, 0} : cur[a][b];
            cur[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[cu][a], qb[cu][b], c0, 0, 0, 0);
            if (kHasPrev) {
                // epilogue of the previous chunk: key tile ks, query tile g >> 2, element g & 3
                const int pb = g >> 2, pe = g & 3;
                accf[ks][pb][pe] = fmaf(static_cast<float>(prev[ks][pb][pe]), qs_prev[pb], accf[ks][pb][pe]);
                if (kInts && int_off[ks][pb] >= 0 && pe < int_rows[ks])
                    ints_prev[int_off[ks][pb] + static_cast<int64_t>(pe) * chunks] = prev[ks][pb][pe] >> down_shift;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <int SB, bool kInts>
__global__ __launch_bounds__(kWsBlock) void dot_mfma_ws_kernel(
    const int8_t* __restrict__ A8, const float* __restrict__ qscale, int qscale_stride,
    const unsigned long long* __restrict__ B64,  // tiled key planes
    const float* __restrict__ Bw, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
    float* __restrict__ out, int* __restrict__ chunk_ints) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 2 * kWsStage

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps addresses scalar
    const bool consumer = wave < kWsConsumers;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kTileR;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * kTileQ;
    const int64_t ntiles = (R + 15) / 16;
    const int64_t tile0 = r0 / 16;

    if (consumer) {
        const int wr = wave & 1, wq = wave >> 1;  // 64-key half, 32-query quarter
        const int ln = lane & 15, lg = lane >> 4;
        float accf[4][2][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;
        const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
        // offsets of this lane's accumulators in chunk_ints (parity builds only); -1 = outside
        int64_t int_off[4][2];
        int int_rows[4];  // how many of the lane's four key rows of tile a exist
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t r = r0 + wr * 64 + a * 16 + lg * 4;
            int_rows[a] = static_cast<int>((R - r) < 4 ? (R - r) : 4);
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int64_t q = q0 + wq * 32 + b * 16 + ln;
                int_off[a][b] = (kInts && q < Q && r < R) ? (q * R + r) * chunks : -1;
            }
        }
        const int koff = (wr * 64 + ln) * kRowBytes + lg * 16;
        const int qoff = kWsQOff + (wq * 32 + ln) * 256;  // row; the 16-byte column of k-step ks is swizzled:
        int qcol[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qcol[ks] = (((ks * 4 + lg) ^ ln) & 15) * 16;
        const int soff = kWsScaleOff + wq * 256 + ln * 4;
        v4i acc0[4][2], acc1[4][2];
        float qs0[2], qs1[2];
        lds_barrier();  // buffer 0 filled by the producers' prologue

        // software pipeline over chunk pairs: MFMAs of chunk c run with the epilogue of chunk c-1
        int c = 0;
        {
            const unsigned char* buf = lds;
            ws_consume_chunk<false, kInts>(buf + koff, buf + qoff, qcol, acc0, acc1, qs1, accf, chunk_ints, down_shift, int_off, int_rows, chunks);
#pragma unroll
            for (int b = 0; b < 2; ++b) qs0[b] = *reinterpret_cast<const float*>(buf + soff + b * 64) * down;
            lds_barrier();
            c = 1;
        }
        for (; c + 1 < chunks; c += 2) {
            const unsigned char* b1 = lds + kWsStage;  // odd chunk
            ws_consume_chunk<true, kInts>(b1 + koff, b1 + qoff, qcol, acc1, acc0, qs0, accf, chunk_ints + (c - 1), down_shift, int_off, int_rows, chunks);
#pragma unroll
            for (int b = 0; b < 2; ++b) qs1[b] = *reinterpret_cast<const float*>(b1 + soff + b * 64) * down;
            lds_barrier();
            const unsigned char* b0 = lds;             // even chunk
            ws_consume_chunk<true, kInts>(b0 + koff, b0 + qoff, qcol, acc0, acc1, qs1, accf, chunk_ints + c, down_shift, int_off, int_rows, chunks);
#pragma unroll
            for (int b = 0; b < 2; ++b) qs0[b] = *reinterpret_cast<const float*>(b0 + soff + b * 64) * down;
            lds_barrier();
        }
        if (c < chunks) {  // one odd chunk left
            const unsigned char* b1 = lds + kWsStage;
            ws_consume_chunk<true, kInts>(b1 + koff, b1 + qoff, qcol, acc1, acc0, qs0, accf, chunk_ints + (c - 1), down_shift, int_off, int_rows, chunks);
#pragma unroll
            for (int b = 0; b < 2; ++b) qs1[b] = *reinterpret_cast<const float*>(b1 + soff + b * 64) * down;
            lds_barrier();
            ++c;
        }
        // epilogue of the last chunk (c - 1): it sits in acc0 when c - 1 is even
        {
            const bool last_even = ((chunks - 1) & 1) == 0;
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = last_even ? acc0[a][b][e] : acc1[a][b][e];
                        const float qsv = last_even ? qs0[b] : qs1[b];
                        accf[a][b][e] = fmaf(static_cast<float>(v), qsv, accf[a][b][e]);
                        if (kInts && int_off[a][b] >= 0 && e < int_rows[a])
                            chunk_ints[int_off[a][b] + static_cast<int64_t>(e) * chunks + (chunks - 1)] = v >> down_shift;
                    }
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t rb = r0 + wr * 64 + a * 16 + lg * 4;
            float bs[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) bs[e] = (rb + e < R) ? key_factor(Bw[(rb + e) * SB]) : 0.0f;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int64_t q = q0 + wq * 32 + b * 16 + ln;
                if (q >= Q) continue;
                float* dst = out + static_cast<size_t>(q) * R_total + rb;
                if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                    *reinterpret_cast<float4*>(dst) =
                        make_float4((accf[a][b][0] * bs[0]) * scale_inv, (accf[a][b][1] * bs[1]) * scale_inv,
                                    (accf[a][b][2] * bs[2]) * scale_inv, (accf[a][b][3] * bs[3]) * scale_inv);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (rb + e < R) dst[e] = (accf[a][b][e] * bs[e]) * scale_inv;
                }
            }
        }
    } else {
        // Producer iteration c stages chunk c+1: (1) direct global->LDS loads of its query rows and
        // scales, (2) key-plane loads of chunk c+2 into the other register set, (3) transposes and
        // LDS stores of the key planes of chunk c+1 (loaded one iteration ago), (4) wait for (1)
        // only -- the 2*SB loads of (2) stay in flight across the barrier.
        // Rows past the end of Q or R are clamped to the last one: their outputs are never written.
        const int p = wave - kWsConsumers;
        const int m = lane & 15, g = lane >> 4;
        int64_t t0 = tile0 + p * 2, t1 = t0 + 1;
        t0 = t0 < ntiles ? t0 : ntiles - 1;
        t1 = t1 < ntiles ? t1 : ntiles - 1;
        const size_t kchunk = static_cast<size_t>(SB) * 64;  // words per (tile, chunk)
        const unsigned long long* ksrc0 = B64 + static_cast<size_t>(t0) * chunks * kchunk;
        const unsigned long long* ksrc1 = B64 + static_cast<size_t>(t1) * chunks * kchunk;
        uint32_t qoff[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = p * 32 + i * 4 + (lane >> 4);
            int64_t q = q0 + row;
            q = q < Q ? q : Q - 1;
            qoff[i] = static_cast<uint32_t>(q * chunks * 256 + (((lane & 15) ^ (row & 15)) * 16));
        }
        int64_t qsrow = q0 + p * 32 + (lane & 31);
        qsrow = qsrow < Q ? qsrow : Q - 1;
        const uint32_t soff = static_cast<uint32_t>(qsrow * qscale_stride * 4);
        const int sstep = (qscale_stride == 1) ? 0 : 1;
        unsigned char* kdst0 = lds + (p * 32 + m) * kRowBytes + g * 64;  // even buffer
        unsigned char* kdst1 = kdst0 + kWsStage;
        unsigned char* qdst0 = lds + kWsQOff + p * 32 * 256;
        unsigned char* qdst1 = qdst0 + kWsStage;
        unsigned char* sdst0 = lds + kWsScaleOff + p * 256;
        unsigned char* sdst1 = sdst0 + kWsStage;

        uint2 k0[2][SB], k1[2][SB];  // k0: even chunks, k1: odd chunks
        ws_load_queries_to_lds(qdst0, sdst0, A8, qoff, qscale, soff);
        ws_load_keys<SB>(k0, ksrc0, ksrc1, lane);
        if (chunks > 1) ws_load_keys<SB>(k1, ksrc0 + kchunk, ksrc1 + kchunk, lane);
        ws_store_keys<SB>(k0, kdst0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        int c = 0;
        for (; c + 2 < chunks; c += 2) {
            // iteration c (even): stage chunk c+1 (odd buffer), prefetch keys of c+2
            ws_produce6(k1, k0, kdst1, qdst1, sdst1, A8 + static_cast<size_t>(c + 1) * 256, qoff, qscale + (c + 1) * sstep,
                        soff, ksrc0 + (c + 2) * kchunk, ksrc1 + (c + 2) * kchunk, lane);
            asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
            lds_barrier();
            // iteration c+1 (odd): stage chunk c+2 (even buffer), prefetch keys of c+3 (clamped to the
            // last chunk when there is none: a harmless reload keeps the loop free of branches)
            const int cn = (c + 3 < chunks) ? c + 3 : chunks - 1;
            ws_produce6(k0, k1, kdst0, qdst0, sdst0, A8 + static_cast<size_t>(c + 2) * 256, qoff, qscale + (c + 2) * sstep,
                        soff, ksrc0 + cn * kchunk, ksrc1 + cn * kchunk, lane);
            asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
            lds_barrier();
        }
        // c is even and c + 2 >= chunks: chunk c is being consumed; chunk c+1 may remain to be staged
        if (c + 1 < chunks) {
            ws_load_queries_to_lds(qdst1, sdst1, A8 + static_cast<size_t>(c + 1) * 256, qoff, qscale + (c + 1) * sstep, soff);
            ws_store_keys<SB>(k1, kdst1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            lds_barrier();  // end of iteration c
            lds_barrier();  // end of iteration c+1
        } else {
            lds_barrier();  // end of iteration c
        }
    }
}

template <int SB, bool kTiled>
static void launch_mfma(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw, int Sb,
                        int W64, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                        float* out, int32_t* chunk_ints, hipStream_t st) {
    const dim3 grid(static_cast<unsigned>((R + kTileR - 1) / kTileR), static_cast<unsigned>((Q + kTileQ - 1) / kTileQ));
    constexpr int kLds = (kTileR + kTileQ) * kRowBytes;  // above the 64 KiB default: opt in once per kernel
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_kernel<SB, kTiled, true>), kLds);
    static LdsOptIn once1;
    lds_opt_in(once1, reinterpret_cast<const void*>(&dot_mfma_kernel<SB, kTiled, false>), kLds);
    if (chunk_ints)
        hipLaunchKernelGGL((dot_mfma_kernel<SB, kTiled, true>), grid, dim3(kMfmaBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const uint32_t*>(B), Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
    else
        hipLaunchKernelGGL((dot_mfma_kernel<SB, kTiled, false>), grid, dim3(kMfmaBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const uint32_t*>(B), Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
}

template <int SB>
static void launch_mfma_ws(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                           int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                           float* out, int32_t* chunk_ints, hipStream_t st) {
    const dim3 grid(static_cast<unsigned>((R + kTileR - 1) / kTileR), static_cast<unsigned>((Q + kTileQ - 1) / kTileQ));
    constexpr int kLds = 2 * kWsStage;
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_ws_kernel<SB, true>), kLds);
    static LdsOptIn once1;
    lds_opt_in(once1, reinterpret_cast<const void*>(&dot_mfma_ws_kernel<SB, false>), kLds);
    if (chunk_ints)
        hipLaunchKernelGGL((dot_mfma_ws_kernel<SB, true>), grid, dim3(kWsBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
    else
        hipLaunchKernelGGL((dot_mfma_ws_kernel<SB, false>), grid, dim3(kWsBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
}

const char* launch_mfma_planes(bool tiled, const int8_t* A8, const float* qscale, int stride, const uint64_t* B,
                               const float* Bw, int Sb, int W64, int chunks, int64_t R, int64_t Q, int down_shift,
                               float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, hipStream_t st) {
    if (Sb == 6 && tiled) {
        launch_mfma_ws<6>(A8, qscale, stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        return "dot_mfma_ws_kernel";
    }
    if (Sb == 6) {  // canonical planes (the tiled ones went to the kernel above)
        launch_mfma<6, false>(A8, qscale, stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
    } else {
        if (tiled) launch_mfma<0, true>(A8, qscale, stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        else launch_mfma<0, false>(A8, qscale, stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
    }
    return "dot_mfma_kernel";
}

}  // namespace bsi
