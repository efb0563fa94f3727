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
// Both feed the same fp32 epilogue, in chunk order:  acc = fmaf((float)I, qscale[q,c], acc), then
// out = (acc * bscale[r]) * scale_inv.  bscale is a power of two, so hoisting it out of the chain is
// exact and the result is bit-identical to fmaf((float)I, qscale*bscale, acc) of the reference
// kernel (bsi_ops/csrc/cuda/bsi_cuda_kernels_dot.cuh:1447-1540).
#include "bsi_common.h"

namespace bsi {

typedef int v4i __attribute__((ext_vector_type(4)));

// In-place transpose of the 8x8 bit matrices (row = register index, column = bit within byte) held
// in the four byte lanes of x[0..7]: afterwards bit s of byte m of x[t] is the old bit t of byte m
// of x[s].  Three butterfly stages of bitfield inserts.
__device__ __forceinline__ void transpose8x8(uint32_t x[8]) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        const uint32_t lo = x[s], hi = x[s + 4];
        x[s] = (lo & 0x0F0F0F0Fu) | ((hi << 4) & 0xF0F0F0F0u);
        x[s + 4] = ((lo >> 4) & 0x0F0F0F0Fu) | (hi & 0xF0F0F0F0u);
    }
#pragma unroll
    for (int b = 0; b < 8; b += 4) {
#pragma unroll
        for (int s = b; s < b + 2; ++s) {
            const uint32_t lo = x[s], hi = x[s + 2];
            x[s] = (lo & 0x33333333u) | ((hi << 2) & 0xCCCCCCCCu);
            x[s + 2] = ((lo >> 2) & 0x33333333u) | (hi & 0xCCCCCCCCu);
        }
    }
#pragma unroll
    for (int s = 0; s < 8; s += 2) {
        const uint32_t lo = x[s], hi = x[s + 1];
        x[s] = (lo & 0x55555555u) | ((hi << 1) & 0xAAAAAAAAu);
        x[s + 1] = ((lo >> 1) & 0x55555555u) | (hi & 0xAAAAAAAAu);
    }
}

// Recombine one 32-bit column of S planes into 32 int8 values (8 dwords): plane j goes to bit
// j + 8 - S of each byte.  Output dword t, byte m = element 8m + t of the 32.
template <int S>
__device__ __forceinline__ void planes32_to_bytes(const uint32_t p[S], uint32_t y[8]) {
#pragma unroll
    for (int s = 0; s < 8; ++s) y[s] = (s >= 8 - S) ? p[s - (8 - S)] : 0u;
    transpose8x8(y);
}

// ------------------------------------------------------------------ planes -> int8 pre-pass
// One thread per (row, 32-bit column).
__global__ void planes_to_int8_kernel(const uint32_t* __restrict__ words32, int64_t rows, int S, int W64, int chunks,
                                      uint32_t* __restrict__ out32) {
    const int cols = chunks * 8;  // 32-bit columns per row, padded to whole chunks
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= rows * cols) return;
    const int64_t row = idx / cols;
    const int col = static_cast<int>(idx - row * cols);
    uint32_t y[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int j = s - (8 - S);
        y[s] = (j >= 0 && col < 2 * W64) ? words32[(static_cast<size_t>(row) * S + j) * (2 * W64) + col] : 0u;
    }
    transpose8x8(y);
    uint4* dst = reinterpret_cast<uint4*>(out32 + (static_cast<size_t>(row) * cols + col) * 8);
    dst[0] = make_uint4(y[0], y[1], y[2], y[3]);
    dst[1] = make_uint4(y[4], y[5], y[6], y[7]);
}

// ------------------------------------------------------------------ key plane tiling
__global__ void tile_key_planes_kernel(const unsigned long long* __restrict__ in, int64_t R, int Sb, int W64,
                                       int chunks, int64_t total, unsigned long long* __restrict__ out) {
    const int64_t o = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (o >= total) return;
    // o = (((tile * chunks + c) * Sb + j) * 64 + g * 16 + rr)
    const int lane = static_cast<int>(o & 63);
    int64_t t = o >> 6;
    const int j = static_cast<int>(t % Sb);
    t /= Sb;
    const int c = static_cast<int>(t % chunks);
    const int64_t tile = t / chunks;
    const int64_t r = tile * 16 + (lane & 15);
    const int w = c * 4 + (lane >> 4);
    out[o] = (r < R && w < W64) ? in[(static_cast<size_t>(r) * Sb + j) * W64 + w] : 0ULL;
}

// ------------------------------------------------------------------ MFMA core

constexpr int kMfmaBlock = 256;
constexpr int kTileR = 128;            // keys per workgroup
constexpr int kTileQ = 128;            // queries per workgroup
constexpr int kRowBytes = 256 + 16;    // one chunk of int8 per row + pad (17 x 16 B: conflict-free b128 reads)

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
        for (int e = 0; e < 4; ++e) bs[e] = (rb + e < R) ? Bw[(rb + e) * Sb] : 0.0f;
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
// 512 threads: waves 0-3 are consumers (64 keys x 64 queries each, 64 MFMAs per chunk), waves 4-7
// are producers.  A producer wave owns 32 key rows and 32 query rows of the 128 x 128 tile: per
// chunk it reads its key planes from the tiled layout (one coalesced 512-byte wave load per plane
// and 16-key tile: lane (m, g) gets words32 2g, 2g+1 of row m), transposes them to 64 int8 per
// lane, and copies its query int8 rows; both go to the LDS buffer of the NEXT chunk while the
// consumers run the MFMAs of the current one out of the other buffer.  The loads for the chunk
// after that are issued before the barrier, so their latency is covered by a whole iteration.
// Each SIMD hosts one consumer and one producer wave: the transposes run on the VALU while the
// matrix pipe works.

constexpr int kWsBlock = 512;
constexpr int kWsStage = (kTileR + kTileQ) * kRowBytes;  // bytes of one LDS buffer

template <int SB>
struct WsRegs {
    uint2 k[2][SB];  // two 16-key tiles x SB planes: words32 (2g, 2g+1) of row m
    uint4 q[8];      // 8 x 16 B of the wave's 32 query rows
};

template <int SB>
__device__ __forceinline__ void ws_load(WsRegs<SB>& rg, const unsigned long long* __restrict__ B64,
                                        const int8_t* __restrict__ A8, int chunks, int c, int64_t tile0,
                                        int64_t ntiles, int64_t q0, int64_t Q, int p, int lane) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int64_t tile = tile0 + p * 2 + t;
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            uint2 v = make_uint2(0u, 0u);
            if (tile < ntiles) {
                const unsigned long long w = B64[((static_cast<size_t>(tile) * chunks + c) * SB + j) * 64 + lane];
                v = make_uint2(static_cast<uint32_t>(w), static_cast<uint32_t>(w >> 32));
            }
            rg.k[t][j] = v;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        // piece = i * 64 + lane of the wave's 32 rows x 16 pieces
        const int piece = i * 64 + lane;
        const int64_t q = q0 + p * 32 + (piece >> 4);
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (q < Q) v = *reinterpret_cast<const uint4*>(A8 + (static_cast<size_t>(q) * chunks + c) * 256 + (piece & 15) * 16);
        rg.q[i] = v;
    }
}

template <int SB>
__device__ __forceinline__ void ws_store(const WsRegs<SB>& rg, unsigned char* __restrict__ buf, int p, int lane) {
    unsigned char* K8 = buf;
    unsigned char* Q8 = buf + kTileR * kRowBytes;
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        uint32_t lo[8], hi[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            lo[s] = (s >= 8 - SB) ? rg.k[t][s - (8 - SB)].x : 0u;
            hi[s] = (s >= 8 - SB) ? rg.k[t][s - (8 - SB)].y : 0u;
        }
        transpose8x8(lo);
        transpose8x8(hi);
        uint4* dst = reinterpret_cast<uint4*>(K8 + (p * 32 + t * 16 + m) * kRowBytes + g * 64);
        dst[0] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        dst[1] = make_uint4(lo[4], lo[5], lo[6], lo[7]);
        dst[2] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        dst[3] = make_uint4(hi[4], hi[5], hi[6], hi[7]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int piece = i * 64 + lane;
        *reinterpret_cast<uint4*>(Q8 + (p * 32 + (piece >> 4)) * kRowBytes + (piece & 15) * 16) = rg.q[i];
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
    const int wave = tid >> 6;
    const bool consumer = wave < 4;
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kTileR;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * kTileQ;
    const int64_t ntiles = (R + 15) / 16;
    const int64_t tile0 = r0 / 16;

    if (consumer) {
        const int wr = wave & 1, wq = wave >> 1;
        const int ln = lane & 15, lg = lane >> 4;
        float accf[4][4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;
        const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
        const int qstep = (qscale_stride == 1) ? 0 : 1;
        // this lane's four query columns: their scale pointers
        const float* qsp[4];
        bool qok[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t q = q0 + wq * 64 + b * 16 + ln;
            qok[b] = q < Q;
            qsp[b] = qscale + (qok[b] ? q : 0) * qscale_stride;
        }
        __syncthreads();  // buffer 0 filled by the producers' prologue
        for (int c = 0; c < chunks; ++c) {
            const unsigned char* K8 = lds + (c & 1) * kWsStage;
            const unsigned char* Q8 = K8 + kTileR * kRowBytes;
            float qs[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) qs[b] = qok[b] ? qsp[b][c * qstep] * down : 0.0f;
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
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        accf[a][b][e] = fmaf(static_cast<float>(acc[a][b][e]), qs[b], accf[a][b][e]);
                        if (kInts) {
                            const int64_t q = q0 + wq * 64 + b * 16 + ln;
                            const int64_t r = r0 + wr * 64 + a * 16 + lg * 4 + e;
                            if (q < Q && r < R)
                                chunk_ints[(static_cast<size_t>(q) * R + r) * chunks + c] = acc[a][b][e] >> down_shift;
                        }
                    }
            __syncthreads();
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t rb = r0 + wr * 64 + a * 16 + lg * 4;
            float bs[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) bs[e] = (rb + e < R) ? Bw[(rb + e) * SB] : 0.0f;
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
    } else {
        const int p = wave - 4;
        WsRegs<SB> rg;
        ws_load<SB>(rg, B64, A8, chunks, 0, tile0, ntiles, q0, Q, p, lane);
        ws_store<SB>(rg, lds, p, lane);
        if (chunks > 1) ws_load<SB>(rg, B64, A8, chunks, 1, tile0, ntiles, q0, Q, p, lane);
        __syncthreads();
        for (int c = 0; c < chunks; ++c) {
            if (c + 1 < chunks) {
                ws_store<SB>(rg, lds + ((c + 1) & 1) * kWsStage, p, lane);
                if (c + 2 < chunks) ws_load<SB>(rg, B64, A8, chunks, c + 2, tile0, ntiles, q0, Q, p, lane);
            }
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------ VALU popcount core (Sa = 7, Sb = 6 shape templated)

constexpr int kValuBlock = 256;
constexpr int kValuTile = 64;  // 64 x 64 outputs per workgroup, 4 x 4 per lane

template <int SA, int SB, bool kTiled, bool kInts>
__global__ __launch_bounds__(kValuBlock) void dot_valu_kernel(
    const uint32_t* __restrict__ A32, const float* __restrict__ qscale, int qscale_stride,
    const uint32_t* __restrict__ B32, const float* __restrict__ Bw, int W64, int chunks, int64_t R, int64_t Q,
    float scale_inv, int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints) {
    // row = SA (or SB) planes x 32 B + 16 B pad: an odd number of 16-byte groups, so 16 consecutive
    // rows hit 16 different bank groups on b128 reads
    constexpr int kARow = SA * 32 + 16;
    constexpr int kBRow = SB * 32 + 16;
    __shared__ __attribute__((aligned(16))) unsigned char ldsA[kValuTile * kARow];
    __shared__ __attribute__((aligned(16))) unsigned char ldsB[kValuTile * kBRow];

    const int tid = threadIdx.x;
    const int tq = tid >> 4;  // 0..15
    const int tr = tid & 15;  // 0..15
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kValuTile;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * kValuTile;

    float accf[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) accf[a][b] = 0.0f;

    for (int c = 0; c < chunks; ++c) {
        // ---- stage the chunk's planes: 16-byte pieces, (row, plane, half)
        for (int piece = tid; piece < kValuTile * SA * 2; piece += kValuBlock) {
            const int half = piece & 1;
            const int pl = (piece >> 1) % SA;
            const int row = (piece >> 1) / SA;
            const int64_t q = q0 + row;
            const int w = c * 4 + half * 2;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (q < Q) {
                // words are 8-byte aligned only (W64 may be odd): two 8-byte loads
                const uint2* src = reinterpret_cast<const uint2*>(A32 + ((static_cast<size_t>(q) * SA + pl) * W64 + w) * 2);
                if (w < W64) { const uint2 t0 = src[0]; v.x = t0.x; v.y = t0.y; }
                if (w + 1 < W64) { const uint2 t1 = src[1]; v.z = t1.x; v.w = t1.y; }
            }
            *reinterpret_cast<uint4*>(ldsA + row * kARow + pl * 32 + half * 16) = v;
        }
        for (int piece = tid; piece < kValuTile * SB * 2; piece += kValuBlock) {
            const int half = piece & 1;
            const int pl = (piece >> 1) % SB;
            const int row = (piece >> 1) / SB;
            const int64_t r = r0 + row;
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (kTiled) {
                // tiled word index: ((((r/16)*chunks + c)*SB + pl)*64 + g*16 + r%16), g = 2*half, 2*half+1
                if (r < ((R + 15) / 16) * 16) {
                    const size_t base = (((static_cast<size_t>(r >> 4) * chunks + c) * SB + pl) << 6) + (r & 15);
                    const uint2 t0 = *reinterpret_cast<const uint2*>(B32 + (base + (half * 2) * 16) * 2);
                    const uint2 t1 = *reinterpret_cast<const uint2*>(B32 + (base + (half * 2 + 1) * 16) * 2);
                    v = make_uint4(t0.x, t0.y, t1.x, t1.y);
                }
            } else if (r < R) {
                const int w = c * 4 + half * 2;
                const uint2* src = reinterpret_cast<const uint2*>(B32 + ((static_cast<size_t>(r) * SB + pl) * W64 + w) * 2);
                if (w < W64) { const uint2 t0 = src[0]; v.x = t0.x; v.y = t0.y; }
                if (w + 1 < W64) { const uint2 t1 = src[1]; v.z = t1.x; v.w = t1.y; }
            }
            *reinterpret_cast<uint4*>(ldsB + row * kBRow + pl * 32 + half * 16) = v;
        }
        __syncthreads();

        int I[4][4];
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) I[a][b] = 0;

#pragma unroll
        for (int half = 0; half < 2; ++half) {
            uint4 bk[4][SB];  // key planes of this half chunk stay in VGPRs
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int j = 0; j < SB; ++j)
                    bk[b][j] = *reinterpret_cast<const uint4*>(ldsB + (tr + 16 * b) * kBRow + j * 32 + half * 16);
#pragma unroll
            for (int i = 0; i < SA; ++i) {
                uint4 aq[4];
#pragma unroll
                for (int a = 0; a < 4; ++a)
                    aq[a] = *reinterpret_cast<const uint4*>(ldsA + (tq + 16 * a) * kARow + i * 32 + half * 16);
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        // Horner over key planes, top (negative) plane first
                        int t = 0;
#pragma unroll
                        for (int j = SB - 1; j >= 0; --j) {
                            int cnt = __popc(aq[a].x & bk[b][j].x);
                            cnt += __popc(aq[a].y & bk[b][j].y);
                            cnt += __popc(aq[a].z & bk[b][j].z);
                            cnt += __popc(aq[a].w & bk[b][j].w);
                            t = (j == SB - 1) ? -cnt : (t << 1) + cnt;
                        }
                        I[a][b] = (i == SA - 1) ? I[a][b] - (t << i) : I[a][b] + (t << i);
                    }
            }
        }

        const int cs = (qscale_stride == 1) ? 0 : c;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t q = q0 + tq + 16 * a;
            const float qs = (q < Q) ? qscale[q * qscale_stride + cs] : 0.0f;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                accf[a][b] = fmaf(static_cast<float>(I[a][b]), qs, accf[a][b]);
                if (kInts) {
                    const int64_t r = r0 + tr + 16 * b;
                    if (q < Q && r < R) chunk_ints[(static_cast<size_t>(q) * R + r) * chunks + c] = I[a][b];
                }
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const int64_t r = r0 + tr + 16 * b;
        if (r >= R) continue;
        const float bs = Bw[r * SB];
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t q = q0 + tq + 16 * a;
            if (q < Q) out[static_cast<size_t>(q) * R_total + r] = (accf[a][b] * bs) * scale_inv;
        }
    }
}

// Any Sa, Sb up to 16: one thread per output, planes read straight from global memory.
__global__ void dot_valu_generic_kernel(const unsigned long long* __restrict__ A, const float* __restrict__ qscale,
                                        int qscale_stride, int Sa, const unsigned long long* __restrict__ B,
                                        const float* __restrict__ Bw, int Sb, int W64, int chunks, int64_t R,
                                        int64_t Q, float scale_inv, int64_t R_total, float* __restrict__ out,
                                        int* __restrict__ chunk_ints) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= Q * R) return;
    const int64_t q = idx / R;
    const int64_t r = idx - q * R;
    const unsigned long long* Aq = A + static_cast<size_t>(q) * Sa * W64;
    const unsigned long long* Br = B + static_cast<size_t>(r) * Sb * W64;
    float acc = 0.0f;
    for (int c = 0; c < chunks; ++c) {
        int I = 0;
        for (int i = 0; i < Sa; ++i)
            for (int j = 0; j < Sb; ++j) {
                int cnt = 0;
                for (int w = c * 4; w < c * 4 + 4 && w < W64; ++w) cnt += __popcll(Aq[i * W64 + w] & Br[j * W64 + w]);
                const int v = cnt << (i + j);
                I = ((i == Sa - 1) != (j == Sb - 1)) ? I - v : I + v;
            }
        if (chunk_ints) chunk_ints[(static_cast<size_t>(q) * R + r) * chunks + c] = I;
        acc = fmaf(static_cast<float>(I), qscale[q * qscale_stride + ((qscale_stride == 1) ? 0 : c)], acc);
    }
    out[static_cast<size_t>(q) * R_total + r] = (acc * Bw[r * Sb]) * scale_inv;
}

static int launch_planes_to_int8(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out, hipStream_t st) {
    const int chunks = (W64 + 3) / 4;
    const int64_t total = rows * chunks * 8;
    if (total == 0) return BSI_OK;
    hipLaunchKernelGGL(planes_to_int8_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const uint32_t*>(words), rows, S, W64, chunks,
                       reinterpret_cast<uint32_t*>(out));
    BSI_LAUNCH_CHECK("planes_to_int8_kernel");
    return BSI_OK;
}

template <int SB, bool kTiled>
static void launch_mfma(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw, int Sb,
                        int W64, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                        float* out, int32_t* chunk_ints, hipStream_t st) {
    const dim3 grid(static_cast<unsigned>((R + kTileR - 1) / kTileR), static_cast<unsigned>((Q + kTileQ - 1) / kTileQ));
    constexpr int kLds = (kTileR + kTileQ) * kRowBytes;  // above the 64 KiB default: opt in once per kernel
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dot_mfma_kernel<SB, kTiled, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dot_mfma_kernel<SB, kTiled, false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        configured = true;
    }
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
    static bool configured = false;
    if (!configured) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dot_mfma_ws_kernel<SB, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&dot_mfma_ws_kernel<SB, false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        configured = true;
    }
    if (chunk_ints)
        hipLaunchKernelGGL((dot_mfma_ws_kernel<SB, true>), grid, dim3(kWsBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
    else
        hipLaunchKernelGGL((dot_mfma_ws_kernel<SB, false>), grid, dim3(kWsBlock), kLds, st, A8, qscale, stride,
                           reinterpret_cast<const unsigned long long*>(B), Bw, chunks, R, Q, down_shift, scale_inv,
                           R_total, out, chunk_ints);
}

template <bool kTiled>
static void launch_valu76(const uint64_t* A, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                          int W64, int chunks, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out,
                          int32_t* chunk_ints, hipStream_t st) {
    const dim3 grid(static_cast<unsigned>((R + kValuTile - 1) / kValuTile),
                    static_cast<unsigned>((Q + kValuTile - 1) / kValuTile));
    if (chunk_ints)
        hipLaunchKernelGGL((dot_valu_kernel<7, 6, kTiled, true>), grid, dim3(kValuBlock), 0, st,
                           reinterpret_cast<const uint32_t*>(A), qscale, stride, reinterpret_cast<const uint32_t*>(B),
                           Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints);
    else
        hipLaunchKernelGGL((dot_valu_kernel<7, 6, kTiled, false>), grid, dim3(kValuBlock), 0, st,
                           reinterpret_cast<const uint32_t*>(A), qscale, stride, reinterpret_cast<const uint32_t*>(B),
                           Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints);
}

}  // namespace bsi

using namespace bsi;

extern "C" int bsi_hip_tile_key_planes(const uint64_t* words, int64_t R, int Sb, int W64, uint64_t* out, void* stream) {
    BSI_REQUIRE(R >= 0 && Sb >= 1 && Sb <= 64 && W64 >= 1, "bad shape");
    if (R == 0) return BSI_OK;
    BSI_REQUIRE(words && out, "null pointer");
    const int chunks = (W64 + 3) / 4;
    const int64_t total = ((R + 15) / 16) * chunks * Sb * 64;
    hipLaunchKernelGGL(tile_key_planes_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       as_stream(stream), reinterpret_cast<const unsigned long long*>(words), R, Sb, W64, chunks,
                       total, reinterpret_cast<unsigned long long*>(out));
    BSI_LAUNCH_CHECK("tile_key_planes_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_planes_to_int8(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out, void* stream) {
    BSI_REQUIRE(rows >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(S >= 1 && S <= 8, "S must be in [1, 8] to fit int8");
    if (rows == 0) return BSI_OK;
    BSI_REQUIRE(words && out, "null pointer");
    return launch_planes_to_int8(words, rows, S, W64, out, as_stream(stream));
}

extern "C" size_t bsi_hip_dot_workspace_bytes(int64_t Q, int W64, int core) {
    if (core == BSI_CORE_VALU || Q <= 0 || W64 <= 0) return 0;
    return static_cast<size_t>(Q) * static_cast<size_t>((W64 + 3) / 4) * 256;
}

extern "C" int bsi_hip_dot(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                           int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R,
                           int64_t Q, float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core,
                           void* workspace, size_t workspace_bytes, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0, "negative Q or R");
    BSI_REQUIRE(W64 >= 1, "W64 must be >= 1");
    BSI_REQUIRE(Sa >= 1 && Sa <= 16 && Sb >= 1 && Sb <= 16, "Sa and Sb must be in [1, 16]");
    BSI_REQUIRE(R_total >= R, "R_total must be >= R");
    BSI_REQUIRE(b_layout == BSI_LAYOUT_CANONICAL || b_layout == BSI_LAYOUT_TILED16, "unknown key layout %d", b_layout);
    if (Q == 0 || R == 0) return BSI_OK;
    const int chunks = (W64 + 3) / 4;
    BSI_REQUIRE(A_chunk_scales != nullptr, "A_chunk_scales is required (pass a [Q,1] array of row scales if there are no chunk scales)");
    BSI_REQUIRE(A_scale_stride == chunks || A_scale_stride == 1,
                "chunk scale stride mismatch: got %d expected %d (or 1 for row scales)", A_scale_stride, chunks);
    BSI_REQUIRE(B && Bw && out, "null pointer");
    BSI_REQUIRE(A || A_ints8, "neither query planes nor int8 queries given");
    hipStream_t st = as_stream(stream);

    const bool mfma_ok = (Sa >= 2 && Sa <= 8 && Sb >= 2 && Sb <= 8);
    if (core == BSI_CORE_AUTO) core = mfma_ok ? BSI_CORE_MFMA : BSI_CORE_VALU;

    if (core == BSI_CORE_MFMA) {
        if (!mfma_ok) return fail(BSI_ERR_UNSUPPORTED, "MFMA core needs Sa, Sb in [2, 8] (got %d, %d)", Sa, Sb);
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
        const bool tiled = (b_layout == BSI_LAYOUT_TILED16);
        if (Sb == 6 && tiled) {
            launch_mfma_ws<6>(A8, A_chunk_scales, A_scale_stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
            BSI_LAUNCH_CHECK("dot_mfma_ws_kernel");
            return BSI_OK;
        }
        if (Sb == 6) {
            if (tiled) launch_mfma<6, true>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
            else launch_mfma<6, false>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        } else {
            if (tiled) launch_mfma<0, true>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
            else launch_mfma<0, false>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        }
        BSI_LAUNCH_CHECK("dot_mfma_kernel");
        return BSI_OK;
    }

    if (core != BSI_CORE_VALU) return fail(BSI_ERR_INVALID, "unknown core %d", core);
    BSI_REQUIRE(A != nullptr, "VALU core needs the query planes");
    if (Sa == 7 && Sb == 6) {
        if (b_layout == BSI_LAYOUT_TILED16)
            launch_valu76<true>(A, A_chunk_scales, A_scale_stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
        else
            launch_valu76<false>(A, A_chunk_scales, A_scale_stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
        BSI_LAUNCH_CHECK("dot_valu_kernel");
        return BSI_OK;
    }
    if (b_layout != BSI_LAYOUT_CANONICAL)
        return fail(BSI_ERR_UNSUPPORTED, "generic VALU kernel reads canonical key planes only");
    const int64_t total = Q * R;
    hipLaunchKernelGGL(dot_valu_generic_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const unsigned long long*>(A), A_chunk_scales, A_scale_stride, Sa,
                       reinterpret_cast<const unsigned long long*>(B), Bw, Sb, W64, chunks, R, Q, scale_inv, R_total,
                       out, chunk_ints);
    BSI_LAUNCH_CHECK("dot_valu_generic_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_dot_timed(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales,
                                 int A_scale_stride, int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw,
                                 int Sb, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out, int core,
                                 void* workspace, size_t workspace_bytes, int iters, float* mean_us, void* stream) {
    BSI_REQUIRE(iters >= 1 && mean_us, "iters must be >= 1 and mean_us non-null");
    hipStream_t st = as_stream(stream);
    hipEvent_t e0, e1;
    BSI_HIP_CHECK(hipEventCreate(&e0));
    BSI_HIP_CHECK(hipEventCreate(&e1));
    int rc = BSI_OK;
    hipEventRecord(e0, st);
    for (int i = 0; i < iters && rc == BSI_OK; ++i)
        rc = bsi_hip_dot(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                         R_total, out, nullptr, core, workspace, workspace_bytes, stream);
    hipEventRecord(e1, st);
    hipError_t se = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (se == hipSuccess) se = hipEventElapsedTime(&ms, e0, e1);
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    if (rc != BSI_OK) return rc;
    if (se != hipSuccess) return fail(BSI_ERR_HIP, "event timing failed: %s", hipGetErrorString(se));
    *mean_us = ms * 1000.0f / static_cast<float>(iters);
    return BSI_OK;
}
