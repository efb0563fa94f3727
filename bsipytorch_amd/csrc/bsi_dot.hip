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
#include "bsi_common.h"

#include <type_traits>

namespace bsi {

// The scale of a key row as the fixed-bit dots use it: the magnitude of its slice-0 weight, 2^shift_r.  (With a
// single key slice, slice 0 is the sign slice and its weight is negative; the sign of every product is already in
// the plane signs s_ij the kernels apply.)
__device__ __forceinline__ float key_factor(float slice0_weight) { return fabsf(slice0_weight); }


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

// (a & m) | (b & ~m) in one v_bitop3_b32 (truth table of S0 = 0xF0, S1 = 0xCC, S2 = 0xAA)
__device__ __forceinline__ uint32_t bsel(uint32_t a, uint32_t b, uint32_t m) {
    return __builtin_amdgcn_bitop3_b32(a, b, m, 0xE4);
}

// The same transpose for six planes sitting in rows 2..7 (rows 0 and 1 are zero), in its three
// butterfly stages (14 + 16 + 16 operations) so that callers can put other work between them:
// y[t] byte m = (value of element 8m + t) << 2.  p0..p5 are the planes.
__device__ __forceinline__ void t6_stage1(uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t p4, uint32_t p5,
                                          uint32_t (&x)[8]) {
    // rows: x2 = p0, x3 = p1, x4 = p2, x5 = p3, x6 = p4, x7 = p5; swap the 4x4 blocks of rows (s, s+4)
    x[0] = (p2 << 4) & 0xF0F0F0F0u; x[4] = p2 & 0xF0F0F0F0u;
    x[1] = (p3 << 4) & 0xF0F0F0F0u; x[5] = p3 & 0xF0F0F0F0u;
    x[2] = bsel(p0, p4 << 4, 0x0F0F0F0Fu); x[6] = bsel(p0 >> 4, p4, 0x0F0F0F0Fu);
    x[3] = bsel(p1, p5 << 4, 0x0F0F0F0Fu); x[7] = bsel(p1 >> 4, p5, 0x0F0F0F0Fu);
}
__device__ __forceinline__ void t6_stage2(const uint32_t (&x)[8], uint32_t (&a)[8]) {  // 2x2 blocks of rows (s, s+2)
    a[0] = bsel(x[0], x[2] << 2, 0x33333333u); a[2] = bsel(x[0] >> 2, x[2], 0x33333333u);
    a[1] = bsel(x[1], x[3] << 2, 0x33333333u); a[3] = bsel(x[1] >> 2, x[3], 0x33333333u);
    a[4] = bsel(x[4], x[6] << 2, 0x33333333u); a[6] = bsel(x[4] >> 2, x[6], 0x33333333u);
    a[5] = bsel(x[5], x[7] << 2, 0x33333333u); a[7] = bsel(x[5] >> 2, x[7], 0x33333333u);
}
__device__ __forceinline__ void t6_stage3(const uint32_t (&a)[8], uint32_t (&y)[8]) {  // single bits of rows (s, s+1)
    y[0] = bsel(a[0], a[1] << 1, 0x55555555u); y[1] = bsel(a[0] >> 1, a[1], 0x55555555u);
    y[2] = bsel(a[2], a[3] << 1, 0x55555555u); y[3] = bsel(a[2] >> 1, a[3], 0x55555555u);
    y[4] = bsel(a[4], a[5] << 1, 0x55555555u); y[5] = bsel(a[4] >> 1, a[5], 0x55555555u);
    y[6] = bsel(a[6], a[7] << 1, 0x55555555u); y[7] = bsel(a[6] >> 1, a[7], 0x55555555u);
}
__device__ __forceinline__ void transpose_6planes(uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3, uint32_t p4,
                                                  uint32_t p5, uint32_t (&y)[8]) {
    uint32_t x[8], a[8];
    t6_stage1(p0, p1, p2, p3, p4, p5, x);
    t6_stage2(x, a);
    t6_stage3(a, y);
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
                                      uint32_t* __restrict__ out32, int tiled) {
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
    // row-major [rows][chunks * 256], or tiled [rows / 64][2 chunks half-chunks][64 rows][128 bytes]: the 32 bytes
    // of column `col` are bytes 32 (col % 4) .. of half-chunk col / 4 of the row
    const size_t at = tiled ? ((static_cast<size_t>(row >> 6) * (2 * chunks) + (col >> 2)) * 8192 +
                               static_cast<size_t>(row & 63) * 128 + static_cast<size_t>(col & 3) * 32) / 4
                            : (static_cast<size_t>(row) * cols + col) * 8;
    uint4* dst = reinterpret_cast<uint4*>(out32 + at);
    dst[0] = make_uint4(y[0], y[1], y[2], y[3]);
    dst[1] = make_uint4(y[4], y[5], y[6], y[7]);
}

// Planes of two's-complement values of any width -> int8 digit images for the matrix cores:
// value = sum_j digit_j * 128^j with digits 0 .. n-2 the unsigned 7-bit groups of planes and digit n-1 the
// remaining top planes, sign-extended.  out[j][row][chunks * 256] in the same in-chunk element order as
// planes_to_int8_kernel (no pre-shift).  One thread per (digit, row, 32-bit column).
__global__ void planes_to_digits_kernel(const uint32_t* __restrict__ words32, int64_t rows, int S, int W64, int chunks,
                                        int ndig, uint32_t* __restrict__ out32) {
    const int cols = chunks * 8;
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<int64_t>(ndig) * rows * cols) return;
    const int col = static_cast<int>(idx % cols);
    const int64_t t = idx / cols;
    const int64_t row = t % rows;
    const int j = static_cast<int>(t / rows);
    const bool top = (j == ndig - 1);
    uint32_t y[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        int plane = 7 * j + s;
        if (top && plane >= S) plane = S - 1;  // sign extension of the top digit
        const bool have = (s < 7 || top) && plane < S && col < 2 * W64;
        y[s] = have ? words32[(static_cast<size_t>(row) * S + plane) * (2 * W64) + col] : 0u;
    }
    transpose8x8(y);
    uint4* dst = reinterpret_cast<uint4*>(out32 + (static_cast<size_t>(t) * cols + col) * 8);
    dst[0] = make_uint4(y[0], y[1], y[2], y[3]);
    dst[1] = make_uint4(y[4], y[5], y[6], y[7]);
}

// out[q, idx[r]] = float(sum_{i,j} I[i Q + q, j R + r] * 2^(7 (i + j) - preshift) * Aw[q, 0] * Bw[r, 0]) * scale_inv
// (+ bias[r]): the digit products of the int32 GEMM put back together, exactly, in float64.
__global__ void digits_combine_kernel(const int* __restrict__ I, int nq, int nk, int64_t Q, int64_t R, int preshift,
                                      const float* __restrict__ Aw, int Sa, const float* __restrict__ Bw, int Sb,
                                      const long long* __restrict__ key_indices, float scale_inv, int64_t R_total,
                                      const float* __restrict__ bias, float* __restrict__ out) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= Q * R) return;
    const int64_t q = idx / R, r = idx - q * R;
    const int64_t ld = static_cast<int64_t>(nk) * R;
    double acc = 0.0;
    for (int i = 0; i < nq; ++i)
        for (int j = 0; j < nk; ++j)
            acc += ldexp(static_cast<double>(I[(static_cast<int64_t>(i) * Q + q) * ld + static_cast<int64_t>(j) * R + r]),
                         7 * (i + j) - preshift);
    acc = acc * static_cast<double>(Aw[q * Sa]) * static_cast<double>(Bw[r * Sb]);
    const int64_t col = key_indices ? key_indices[r] : r;
    float v = static_cast<float>(acc) * scale_inv;
    if (bias != nullptr) v = v + bias[r];
    out[q * R_total + col] = v;
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

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() would also
// drain the vector-memory counter, i.e. stall every iteration on the producers' prefetch loads.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// LDS buffer of one chunk: int8 key rows (padded, written through registers), int8 query rows
// (unpadded, 16-byte columns XOR-swizzled by row & 15, written by direct global->LDS loads) and
// the chunk scales of the 128 queries (64 floats per producer wave, the upper 32 unused).
constexpr int kWsQOff = kTileR * kRowBytes;
constexpr int kWsScaleOff = kWsQOff + kTileQ * 256;
constexpr int kWsStage = kWsScaleOff + 4 * 64 * 4;  // bytes of one LDS buffer

#define BSI_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define BSI_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

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

// ------------------------------------------------------------------ MFMA core on the cached int8 key image
//
// Compute-bound shapes (hundreds of query rows) pay for the plane -> int8 recombination of the keys
// on the vector ALU in every workgroup that touches a key tile.  A keyset can therefore carry,
// next to its packed planes, the recombined int8 image of the same integers (built once by
// bsi_hip_planes_to_int8, 1 byte per weight); this kernel contracts that image with the int8
// query image.
//   * workgroup = 128 keys x 128 queries over all chunks; 8 MFMA waves of 64 keys x 32 queries
//     and 4 loader waves (one per SIMD).  Only the loader waves issue global loads: a wave that
//     issues them blocks while the memory queue is full, which the MFMA waves must never do;
//   * LDS is a ring of four half-chunk stages (keys 128 x 128 B + queries 128 x 128 B = 32 KiB
//     each), filled by buffer loads that write LDS directly (a loader wave issues 4 + 4 per
//     stage, 1 KiB each); the 16-byte columns of a row are XOR-swizzled with (row >> 1) & 7 so
//     that the 16 rows a ds_read_b128 touches hit distinct banks;
//   * loads of half h+3 are issued when half h starts; the wait before the barrier that ends half
//     h only covers the loads of half h+1, so two stages stay in flight across barriers;
//   * the fp32 epilogue of chunk c-1 (one cvt + one fma per output and chunk, in chunk order)
//     is interleaved element by element with the MFMAs of chunk c (two accumulator sets).
typedef __amdgpu_buffer_rsrc_t bsi_rsrc;
__device__ __forceinline__ bsi_rsrc make_rsrc(const void* base, size_t bytes) {
    const size_t capped = bytes > 0x7FFFFFFFull ? 0x7FFFFFFFull : bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(capped), 0x00020000);
}
// 64 lanes x 16 bytes from `r` (byte offset lane_off per lane + wave_off) to 1 KiB of LDS at dst (wave-uniform)
__device__ __forceinline__ void load16_to_lds(bsi_rsrc r, uint32_t lane_off, uint32_t wave_off, unsigned char* dst) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, BSI_LDS_PTR(dst), 16, static_cast<int>(lane_off),
                                             static_cast<int>(wave_off), 0, 0);
}

// Peak probe for the int8-image kernel's operand path: every workgroup (one per CU) streams an L2-resident region
// into LDS with the same LDS-direct buffer loads the kernel's loader waves use, 96 KiB in flight per CU (the kernel's
// three stages), all CUs at once.  Nothing reads the LDS copy; the figure is what the path from L2 through the CU's
// vector memory unit into LDS delivers -- with kWaves issuing waves of kSlots loads in flight each, in contiguous
// 1 KiB pieces or (kRows) in the kernel's own pieces of 8 rows x 128 bytes out of 128 rows.
constexpr int kProbeLdsWaves = 8, kProbeLdsSlots = 12;
template <int kWaves, int kSlots, bool kRows>
__global__ __launch_bounds__(kWaves * 64) void probe_l2_lds_kernel(const unsigned char* __restrict__ buf,
                                                                   size_t region_bytes, int regions, int passes) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const bsi_rsrc r = make_rsrc(buf + static_cast<size_t>(blockIdx.x % regions) * region_bytes, region_bytes);
    const int pieces = static_cast<int>(region_bytes / 1024);
    // kRows: the region is 128 rows of region_bytes / 128 bytes; a piece is 8 rows x 128 bytes (the kernel's stage loads)
    const uint32_t rowbytes = static_cast<uint32_t>(region_bytes / 128);
    const uint32_t lane_off = kRows ? static_cast<uint32_t>(lane >> 3) * rowbytes + static_cast<uint32_t>(lane & 7) * 16
                                    : static_cast<uint32_t>(lane) * 16;
    int slot = 0;
    for (int pass = 0; pass < passes; ++pass)
        for (int p = wave; p < pieces; p += kWaves) {
            const uint32_t wave_off = kRows ? static_cast<uint32_t>(p & 15) * 8 * rowbytes + static_cast<uint32_t>(p >> 4) * 128
                                            : static_cast<uint32_t>(p) * 1024;
            load16_to_lds(r, lane_off, wave_off, lds + (wave * kSlots + slot) * 1024);
            slot = (slot + 1 == kSlots) ? 0 : slot + 1;
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kSlots - 1) : "memory");
        }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Tile configuration: TM keys x TN queries per workgroup (128 x 128, 128 x 64, 64 x 64 or 64 x 32; the smaller
// ones for grids that would leave CUs without a workgroup), MFMA waves arranged 2 (keys) x kWavesN (queries),
// each WM x WN tiles of 16 x 16; one loader wave per (up to) 64 operand rows.
static std::atomic<int> g_i8_tile{0};  // 0 = by grid size; 128, 12864 (128 keys x 64 queries) or 64 force a tile
static std::atomic<int> g_digits_route{0};  // bsi_hip_dot_digits: 0 = by cost, 1 = stacked digits + combine pass, 2 = in-accumulator

#ifndef BSI_I8_WN_RULE
#define BSI_I8_WN_RULE ((TM == 128 && TN == 128) ? 2 : 1)
#endif
template <int TM, int TN>
struct I8Cfg {
    static constexpr int kTM = TM, kTN = TN;
    static constexpr int kWM = TM / 32;                // 16-key tiles per wave (2 waves along the keys)
    // 16-query tiles per wave: two for the 128 x 128 tile (eight MFMA waves of 64 x 32), one for the smaller tiles, which
    // would otherwise run on four MFMA waves or fewer -- one per SIMD, and a single wave cannot issue its MFMAs, the chain
    // and the operand reads fast enough to keep its SIMD's matrix pipe busy
    static constexpr int kWN = BSI_I8_WN_RULE;
    static constexpr int kWavesN = TN / (16 * kWN);    // waves along the queries
    static constexpr int kConsumers = 2 * kWavesN;
    static constexpr int kGroups = (TM + TN) / 8;      // groups of 8 operand rows (1 KiB per half-chunk) in a stage
    // loader waves: one per SIMD (the more waves issue a stage's loads, the faster it comes) -- but two for the
    // 64 x 64 tile, measured: on one machine 512 x 2048 x 8192 takes 17.4 us with two and 18.7 with four (with four
    // or with eight MFMA waves alike), while the 64 x 32 and 128 x 64 tiles gain 5 to 10 % from four
    static constexpr int kLoaders = (TM == 64 && TN == 64) ? 2 : 4;
    static constexpr int kLoads = (kGroups + kLoaders - 1) / kLoaders;  // loads per loader wave and stage
    static constexpr int kBlock = (kConsumers + kLoaders) * 64;
    static constexpr int kOperandK = TM * 128;         // bytes of the key tile of one half-chunk
    static constexpr int kStage = (TM + TN) * 128;     // keys then queries
    static constexpr int kScaleBytes = 4 * kLoaders * 256;  // chunk scales: ring of 4 chunks x loader regions x 64 floats
    static constexpr int kEpilogueBytes = 2 * TM * 4;  // the tile's key factors, then its biases (chain modes)
    static constexpr int kLds = 4 * kStage + kScaleBytes + kEpilogueBytes;
};

// Timeline build (make TIMELINE=1, -DBSI_TIMELINE): one MFMA wave and one loader wave of every workgroup of
// dot_mfma_i8_kernel stamp the 100 MHz wall clock at the points below, 8 slots per workgroup (the first
// kTimelineWorkgroups of the grid); bsi_hip_timeline_read copies them out.  The ordinary build has none of this.
constexpr int kTimelineWorkgroups = 8192;
enum TimelineStamp {
    kStampMfmaEntry = 0, kStampFirstStage = 1, kStampLoopDone = 2, kStampStored = 3, kStampLoaderEntry = 4,
    kStampLoaderDone = 5, kStampFirstIssue = 6, kStampThreeIssued = 7
};
#ifdef BSI_TIMELINE
__device__ unsigned long long g_timeline[kTimelineWorkgroups * 8];
#define BSI_STAMP(slot)                                                                    \
    {                                                                                      \
        const unsigned wg_ = blockIdx.y * gridDim.x + blockIdx.x;                          \
        if (lane == 0 && wg_ < kTimelineWorkgroups) g_timeline[wg_ * 8 + (slot)] = wall_clock64(); \
    }
#else
#define BSI_STAMP(slot)
#endif

// A loader wave of the int8-image kernels (lw = its number among the C::kLoaders loader waves; `consumers` MFMA
// waves share the workgroup's barriers with it): 8 of the stage's groups of 8 rows (the TM key rows, then the TN
// query rows: a load moves 1 KiB = 8 rows x 128 bytes), plus the chunk scales of 64 queries once per chunk.
template <typename C, bool kSum>
__device__ __forceinline__ void i8_loader_wave(unsigned char* __restrict__ lds, int lw, int lane,
                                               const int8_t* __restrict__ A8, const float* __restrict__ qscale,
                                               int qscale_stride, const int8_t* __restrict__ K8,
                                               const float* __restrict__ Bw, int Sb, int chunks, int halves, int64_t R,
                                               int64_t Q, int64_t r0, int64_t q0, size_t rowbytes,
                                               const float* __restrict__ bias, int ndig, long long dig_stride,
                                               int key_tiled, const unsigned char* __restrict__ warm,
                                               long long warm_lines) {
    constexpr int TM = C::kTM, TN = C::kTN;
    constexpr int L = C::kLoaders, NI = C::kLoads, KG = TM / 8, QG = TN / 8;
    // The key groups and the query groups both divide evenly among the loader waves: every loader moves KG / L key
    // groups, then QG / L query groups, so which operand a load belongs to is known at compile time.
    static_assert(KG % L == 0 && QG % L == 0 && NI == KG / L + QG / L, "loads per loader wave");
    unsigned char* const scale_lds = lds + 4 * C::kStage;  // [chunk & 3][loader][64] floats
    // The prologue below is kept short on purpose: it runs on one wave per SIMD while the whole workgroup waits for
    // the first stage.  No row is clamped: a load that starts past its operand's end reads nothing (buffer bounds),
    // and whatever such a row or query leaves in LDS only reaches outputs past R or Q, which are never stored.
    // tiled keys: blocks of 64 rows x 128 bytes per half-chunk, 2 chunks of them per 64-row tile; rows past R
    // are zero padding inside the last block
    const uint32_t rowbytes32 = static_cast<uint32_t>(chunks) << 8;
    const uint32_t kblock = static_cast<uint32_t>(chunks) << 14;  // bytes of a 64-row tile of the tiled image
    const bsi_rsrc rk = key_tiled ? make_rsrc(K8 + static_cast<size_t>(r0 / 64) * kblock,
                                              static_cast<size_t>((R + 63) / 64 - r0 / 64) * kblock)
                                  : make_rsrc(K8 + static_cast<size_t>(r0) * rowbytes,
                                              static_cast<size_t>(R - r0) * rowbytes);
    const bsi_rsrc rq = make_rsrc(A8 + static_cast<size_t>(q0) * rowbytes,
                                  static_cast<size_t>(Q - q0) * rowbytes +
                                      (kSum ? static_cast<size_t>(ndig - 1) * static_cast<size_t>(dig_stride) : 0));
    // A load moves group g of the stage: 8 rows x 128 bytes; lane = (row lr of the group, 16-byte column lc), and the
    // logical column that lands in LDS column lc of row 8 g + lr is lc ^ (((8 g + lr) >> 1) & 7) = lc ^ (4 (g & 1) +
    // (lr >> 1)).  Per lane: the offset inside the group, for either parity of g and for either layout; per load
    // (scalar): the offset of its group.
    const uint32_t lr = static_cast<uint32_t>(lane) >> 3, lc = static_cast<uint32_t>(lane) & 7;
    uint32_t voff[NI], goff[NI];
    bool is_key[NI];  // known at compile time once the loops are unrolled
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        is_key[i] = i < KG / L;
        const int gg = is_key[i] ? lw + L * i : lw + L * (i - KG / L);  // group of its operand
        const uint32_t col = (lc ^ (static_cast<uint32_t>(gg & 1) * 4 + (lr >> 1))) * 16;
        const bool tiled = is_key[i] && key_tiled;
        voff[i] = (tiled ? lr * 128 : lr * rowbytes32) + col;
        goff[i] = tiled ? static_cast<uint32_t>(gg >> 3) * kblock + static_cast<uint32_t>(gg & 7) * 1024
                        : static_cast<uint32_t>(gg) * 8 * rowbytes32;
    }
    const uint32_t kstep_bytes = key_tiled ? 8192u : 128u;  // from one half-chunk of a key row to the next
    // scales: loader wave lw fetches the 64 queries of group lw % (TN / 64) (waves fetching the same group
    // write their own regions, so that every loader wave has the same number of loads in flight)
    const bsi_rsrc rs = make_rsrc(qscale + q0 * qscale_stride, static_cast<size_t>(Q - q0) * qscale_stride * 4);
    const uint32_t soff = static_cast<uint32_t>((lw % (TN >= 64 ? TN / 64 : 1)) * 64 + lane) * static_cast<uint32_t>(qscale_stride) * 4;
    const int sstep = (qscale_stride == 1) ? 0 : 4;
    // issue() is called for h = 0, 1, 2, ... in order; in the sum mode (next_c, next_dg) follow the chunk and
    // the digit (counted from the top one) of the half-chunk to come
    int next_c = 0, next_dg = 0;
    uint32_t so_k = 0, so_q = 0;
    auto issue = [&](int h) {  // stage of half-chunk h (clamped to the last) into its ring slot
        const int hc = h < halves ? h : halves - 1;
        if (kSum) {
            if (h < halves) {
                const uint32_t half = static_cast<uint32_t>(next_c) * 2 + static_cast<uint32_t>(h & 1);
                so_k = half * kstep_bytes;
                so_q = half * 128 + static_cast<uint32_t>(ndig - 1 - next_dg) * static_cast<uint32_t>(dig_stride);
                if (h & 1) {
                    if (++next_c == chunks) {
                        next_c = 0;
                        ++next_dg;
                    }
                }
            }
        } else {
            so_q = static_cast<uint32_t>(hc) * 128;
            so_k = static_cast<uint32_t>(hc) * kstep_bytes;
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int g = i < KG / L ? lw + L * i : KG + lw + L * (i - KG / L);  // group of the stage
            load16_to_lds(is_key[i] ? rk : rq, voff[i], goff[i] + (is_key[i] ? so_k : so_q),
                          lds + (h & 3) * C::kStage + g * 1024);
        }
        if (!kSum && (h & 1)) {  // with the second half of chunk c = h / 2: its scales
            const int c = hc >> 1;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs, BSI_LDS_PTR(scale_lds + ((c & 3) * C::kLoaders + lw) * 256), 4, static_cast<int>(soff),
                c * sstep, 0, 0);
        }
    };
    if (lw == 0) BSI_STAMP(kStampFirstIssue);
    issue(0);
    issue(1);
    issue(2);
    if (lw == 0) BSI_STAMP(kStampThreeIssued);
    // The epilogue's operands, staged once per workgroup behind the first three stages: the slice-0 weight (key
    // factor) and the bias of the tile's TM keys, 64 rows per load.  (Fetched per lane at the end they are 32
    // vector-memory instructions for every MFMA wave, all queued in front of the output stores.)  Every loader wave
    // issues kEpi of them -- wrapping around where they do not divide evenly -- so that the waits below count the
    // same for all.  Rows past R, and the biases of a call without one, read nothing and give 0 (buffer bounds).
    constexpr int kEpi = kSum ? 0 : (2 * (TM / 64) + L - 1) / L;
    if (!kSum) {
        const bsi_rsrc wrs = make_rsrc(Bw + static_cast<size_t>(r0) * Sb, static_cast<size_t>(R - r0) * Sb * sizeof(float));
        const bsi_rsrc brs = make_rsrc(bias != nullptr ? bias + r0 : Bw,
                                       bias != nullptr ? static_cast<size_t>(R - r0) * sizeof(float) : 0);
        unsigned char* const epi = lds + 4 * C::kStage + C::kScaleBytes;
#pragma unroll
        for (int k = 0; k < kEpi; ++k) {
            const int j = (lw + L * k) % (2 * (TM / 64));
            const bool is_bias = j >= TM / 64;
            const int blk = is_bias ? j - TM / 64 : j;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(is_bias ? brs : wrs,
                                                     BSI_LDS_PTR(epi + (is_bias ? TM * 4 : 0) + blk * 256), 4,
                                                     (blk * 64 + lane) * (is_bias ? 4 : Sb * 4), 0, 0, 0);
        }
    }
    // stage 0 landed (stage 1 + scales + stage 2 + the epilogue operands may be in flight)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NI + (kSum ? 0 : 1) + kEpi) : "memory");
    lds_barrier();
    for (int h = 0; h < halves; ++h) {
        if (h + 3 < halves) {
            issue(h + 3);  // its slot was released by the barrier that ended half h - 1
            // stage h + 1 (and the scales issued right behind it) landed; stages h + 2, h + 3 and one
            // scale load, 2 NI + 1 instructions, may still be in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NI + (kSum ? 0 : 1)) : "memory");
        } else if (h + 3 == halves) {
            // nothing left to issue (a copy of the last stage here, as the prologue does for a single chunk, would
            // queue 96 KiB of loads in front of every workgroup's output stores); the last stage and its
            // scales may be in flight
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NI + (kSum ? 0 : 1)) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        lds_barrier();
    }
    if (warm_lines > 0) {
        // one lane per 128-byte line, 64 lines per load; this loader wave's share of the region.  The values
        // are summed only so that the loads stay; the store below never happens.
        const long long waves = static_cast<long long>(gridDim.x) * gridDim.y * C::kLoaders;
        const long long mine = (static_cast<long long>(blockIdx.y) * gridDim.x + blockIdx.x) * C::kLoaders + lw;
        const long long per = (warm_lines + waves - 1) / waves;
        const long long first = mine * per;
        const long long last = (first + per < warm_lines) ? first + per : warm_lines;
        unsigned sum = 0;
        for (long long l = first + lane; l < last; l += 64)
            sum += *reinterpret_cast<const volatile unsigned*>(warm + l * 128);
        if (sum == 0x5ca1ab1eu && warm_lines < 0) scale_lds[lane] = 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may still be writing LDS when the workgroup ends
}

// One k-step (64 of a chunk's 256 elements) of an MFMA wave: WM WN MFMAs on the operands in (ka, qb), one
// epilogue element of the previous chunk (held in `prev`) behind each MFMA, and behind the first WM + WN of them
// the reads of the NEXT k-step's operands into (ka_n, qb_n), so that the LDS latency of every k-step hides
// behind the MFMAs of the one before it -- also across the barrier between two stages of the ring.
// KS: k-step of the chunk (0..3); krow_n / qrow_n: the wave's rows of the next k-step's stage, column included.
// kMode: kI8Chain (fp32 chunk-scale chain), kI8Ints (the same, and the per-chunk integers are stored) or kI8Sum
// (plain int32 sum over all chunks: no scales, no epilogue).
constexpr int kI8Chain = 0, kI8Ints = 1, kI8Sum = 2;
template <int WM, int WN, int KS, int kMode>
__device__ __forceinline__ void i8_kstep(const v4i (&ka)[WM], const v4i (&qb)[WN], v4i (&ka_n)[WM], v4i (&qb_n)[WN],
                                         const unsigned char* __restrict__ krow_n,
                                         const unsigned char* __restrict__ qrow_n, v4i (&acc)[WM][WN],
                                         const v4i (&prev)[WM][WN], float (&accf)[WM][WN][4],
                                         const float (&qs_prev)[WN], int* __restrict__ ints_prev,
                                         const int64_t (&int_off)[WM][WN], const int (&int_rows)[WM], int down_shift,
                                         int chunks) {
    static_assert(WM + WN <= 2 * WM * WN, "two operand reads behind each MFMA of a k-step");
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const int t = a * WN + b;
            constexpr bool kInts = (kMode == kI8Ints);
            const v4i c0 = (KS == 0 && kMode != kI8Sum) ? (v4i){0, 0, 0, 0} : acc[a][b];
            acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[a], qb[b], c0, 0, 0, 0);
            if (kMode != kI8Sum) {
                const int idx = KS * (WM * WN) + t, tt = idx >> 2, e = idx & 3, ea = tt / WN, eb = tt % WN;
                accf[ea][eb][e] = fmaf(static_cast<float>(prev[ea][eb][e]), qs_prev[eb], accf[ea][eb][e]);
                if (kInts && ints_prev != nullptr && int_off[ea][eb] >= 0 && e < int_rows[ea])
                    ints_prev[int_off[ea][eb] + static_cast<int64_t>(e) * chunks] = prev[ea][eb][e] >> down_shift;
            }
            // reads 2 t and 2 t + 1 of the next k-step, in the order its MFMAs first need them: ka[0], qb[0..],
            // ka[1..].  Two per MFMA: the last of them is then issued more than half a k-step before the barrier
            // that may follow this k-step, which has to wait for all of them before it releases their stage.
#pragma unroll
            for (int r = 2 * t; r < 2 * t + 2; ++r) {
                if (r == 0) ka_n[0] = *reinterpret_cast<const v4i*>(krow_n);
                else if (r <= WN) qb_n[r - 1] = *reinterpret_cast<const v4i*>(qrow_n + (r - 1) * 16 * 128);
                else if (r < WM + WN) ka_n[r - WN] = *reinterpret_cast<const v4i*>(krow_n + (r - WN) * 16 * 128);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
}

// The output tile of an MFMA wave (WM x WN tiles of 16 keys x 16 queries; lane (ln, lg) holds keys 4 lg .. + 3 of
// query ln of each) stored in whole 128-byte lines.  Stored as it lies, a store instruction writes 64 bytes per query
// (4 lanes x 16 bytes): half a line.  Here neighbouring query lanes first swap one of two vertically adjacent tiles
// (a, a + 1), so that the even lane holds keys 0 .. 15 of both queries and the odd lane keys 16 .. 31; a store then
// writes, for one query of the pair, 8 lanes x 16 bytes = the 32 consecutive keys of a line.  Only for a tile that
// lies wholly inside the output and whose lines are aligned; returns false (nothing stored) otherwise.  stream_out: nontemporal stores.
template <int WM, int WN>
__device__ __forceinline__ bool i8_store_lines(const float (&v)[WM][WN][4], float* __restrict__ out, int64_t R_total,
                                               int64_t rw, int64_t qw, int64_t R, int64_t Q, int ln, int lg,
                                               bool stream_out) {
    static_assert(WM % 2 == 0, "tiles are paired along the keys");
    const bool whole = rw + WM * 16 <= R && qw + WN * 16 <= Q && (R_total & 31) == 0 && (rw & 31) == 0 &&
                       (reinterpret_cast<uintptr_t>(out) & 127) == 0;
    if (!whole) return false;
    const bool odd = (ln & 1) != 0;
#pragma unroll
    for (int a = 0; a < WM; a += 2)
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            float x[4], y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float give = odd ? v[a][b][e] : v[a + 1][b][e];
                // quad_perm [1, 0, 3, 2]: the value of the neighbouring query lane
                const float got = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(give), 0xB1, 0xF, 0xF, false));
                x[e] = odd ? got : v[a][b][e];       // the pair's even query: keys 16 (odd lane) + 4 lg ..
                y[e] = odd ? v[a + 1][b][e] : got;   // the pair's odd query
            }
            const int64_t qe = qw + b * 16 + (ln & ~1);
            float* dst = out + static_cast<size_t>(qe) * R_total + rw + a * 16 + (odd ? 16 : 0) + lg * 4;
            if (stream_out) {  // the output leaves the caches as it is written
                typedef float v4f __attribute__((ext_vector_type(4)));
                __builtin_nontemporal_store((v4f){x[0], x[1], x[2], x[3]}, reinterpret_cast<v4f*>(dst));
                __builtin_nontemporal_store((v4f){y[0], y[1], y[2], y[3]}, reinterpret_cast<v4f*>(dst + R_total));
            } else {
                *reinterpret_cast<float4*>(dst) = make_float4(x[0], x[1], x[2], x[3]);
                *reinterpret_cast<float4*>(dst + R_total) = make_float4(y[0], y[1], y[2], y[3]);
            }
        }
    return true;
}

template <int TM, int TN, int kMode>
__global__ __launch_bounds__((I8Cfg<TM, TN>::kBlock)) void dot_mfma_i8_kernel(
    const int8_t* __restrict__ A8, const float* __restrict__ qscale, int qscale_stride,
    const int8_t* __restrict__ K8,  // int8 key image [R, chunks * 256]
    const float* __restrict__ Bw, int Sb, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv,
    int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints, const float* __restrict__ bias,
    int ndig, long long dig_stride, const long long* __restrict__ key_indices, int key_tiled,
    const unsigned char* __restrict__ warm, long long warm_lines, int out_stream) {
    // out_stream: the float outputs of whole tiles go out with nontemporal stores (they leave the caches as they are
    // written) instead of plain ones (they stay for the kernel that reads them next).
    // warm / warm_lines: an optional region of 128-byte lines (the keys the NEXT dot will read) that the loader
    // waves touch once they have issued their last stage, so that it sits in the memory-side cache by the time
    // that dot runs.  (Issued any earlier, from any wave, these long misses hold up the stage loads queued behind
    // them in the CU's vector memory path: measured 40 % slower.)
    // key_tiled: K8 is the tiled image [ceil(R / 64)][2 chunks][64 rows][128 bytes] (a workgroup's key rows of one
    // half-chunk are contiguous, so cold keys stream from HBM in whole pages) instead of row-major [R][chunks * 256].
    // kI8Sum only: A8 holds ndig digit images of the queries, dig_stride bytes apart, lowest digit first; the
    // chunk loop runs over them from the top digit down and the accumulators are shifted left by 7 between two
    // digits (Horner), so that they end as sum_d (sum_i digit_i[q, d] 128^i) K8[r, d].  With chunk_ints the int32
    // sums are stored there ([Q, R_total]); without, out[q, idx[r]] = float(sum * 2^-down_shift * qscale[q *
    // qscale_stride] * Bw[r * Sb]) * scale_inv (+ bias[r]), the product formed in float64.
    using C = I8Cfg<TM, TN>;
    constexpr int WM = C::kWM, WN = C::kWN;
    constexpr bool kInts = (kMode == kI8Ints), kSum = (kMode == kI8Sum);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // C::kLds

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * TM;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * TN;
    const size_t rowbytes = static_cast<size_t>(chunks) * 256;
    const int vchunks = kSum ? chunks * ndig : chunks;  // chunks of the loop: every digit image runs over all chunks
    const int halves = vchunks * 2;
    unsigned char* const scale_lds = lds + 4 * C::kStage;  // [chunk & 3][loader][64] floats

    if (wave >= C::kConsumers) {
        if (wave == C::kConsumers) BSI_STAMP(kStampLoaderEntry);
        i8_loader_wave<C, kSum>(lds, wave - C::kConsumers, lane, A8, qscale, qscale_stride, K8, Bw, Sb, chunks, halves, R,
                                     Q, r0, q0, rowbytes, bias, ndig, dig_stride, key_tiled, warm, warm_lines);
        if (wave == C::kConsumers) BSI_STAMP(kStampLoaderDone);
        return;
    }
    if (wave == 0) BSI_STAMP(kStampMfmaEntry);

    // ---- MFMA waves
    const int wr = wave & 1, wq = wave >> 1;  // half of the keys, group of 32 queries
    const int ln = lane & 15, lg = lane >> 4;
    const int krow_off = (wr * (WM * 16) + ln) * 128;
    const int qrow_off = C::kOperandK + (wq * (WN * 16) + ln) * 128;
    int pcol[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) pcol[kk] = ((kk * 4 + lg) ^ (ln >> 1)) * 16;
    float accf[WM][WN][4];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;
    v4i acc0[WM][WN], acc1[WM][WN];
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b) acc0[a][b] = acc1[a][b] = (v4i){0, 0, 0, 0};
    // the MFMA accumulators hold 2^down_shift times the integer dot; the chain runs on them unscaled
    // (a power of two commutes with every rounding) and the factor is taken out once at the end
    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
    int64_t int_off[WM][WN];
    int int_rows[WM];
#pragma unroll
    for (int a = 0; a < WM; ++a) {
        const int64_t r = r0 + wr * (WM * 16) + a * 16 + lg * 4;
        int_rows[a] = static_cast<int>((R - r) < 4 ? (R - r) : 4);
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
            int_off[a][b] = (kInts && q < Q && r < R) ? (q * R + r) * chunks : -1;
        }
    }
    // chunk scales of the lane's query columns, from the loaders' ring: region g holds queries 64 g .. + 63
    const int qfirst = wq * (WN * 16);
    const unsigned char* sread = scale_lds + (qfirst >> 6) * 256 + ((qfirst & 63) + ln) * 4;
    float qsa[WN], qsb[WN];  // scales of even / odd chunks
#pragma unroll
    for (int b = 0; b < WN; ++b) qsa[b] = qsb[b] = 0.0f;
#define BSI_I8_SCALES(dst, c)                                                                                  \
    {                                                                                                          \
        _Pragma("unroll") for (int b = 0; b < WN; ++b) dst[b] =                                                \
            *reinterpret_cast<const float*>(sread + ((c) & 3) * (C::kLoaders * 256) + b * 64);                 \
    }
    // The k-steps run one behind their operand reads: k-step j's MFMAs cover the reads of k-step j + 1.  A
    // stage (half-chunk, two k-steps) is released to the loaders by the barrier that follows the k-step in
    // which its last operands were read (the even ones); the same barrier tells that the next stage has landed.
    v4i ka[2][WM], qb[2][WN];  // operand sets of even / odd k-steps
#define BSI_I8_KSTEP(KS, nslot, acc, prev, qs, ip)                                                                  \
    i8_kstep<WM, WN, KS, kMode>(ka[(KS) & 1], qb[(KS) & 1], ka[((KS) + 1) & 1], qb[((KS) + 1) & 1],                 \
                                lds + (nslot) * C::kStage + krow_off + pcol[((KS) + 1) & 1],                        \
                                lds + (nslot) * C::kStage + qrow_off + pcol[((KS) + 1) & 1], acc, prev, accf, qs,   \
                                ip, int_off, int_rows, down_shift, chunks);
    // a chunk whose halves sit in ring slots s0, s0 + 1; nslot: slot of the next chunk's first half
#define BSI_I8_CHUNK(s0, nslot, acc, prev, qs, ip)                                                                  \
    BSI_I8_KSTEP(0, s0, acc, prev, qs, ip);                                                                         \
    lds_barrier();                                                                                                  \
    BSI_I8_KSTEP(1, (s0) + 1, acc, prev, qs, ip);                                                                   \
    BSI_I8_KSTEP(2, (s0) + 1, acc, prev, qs, ip);                                                                   \
    lds_barrier();                                                                                                  \
    BSI_I8_KSTEP(3, nslot, acc, prev, qs, ip);

    lds_barrier();  // stage 0 is there
    if (wave == 0) BSI_STAMP(kStampFirstStage);
#pragma unroll
    for (int t = 0; t < WM; ++t) ka[0][t] = *reinterpret_cast<const v4i*>(lds + krow_off + t * 16 * 128 + pcol[0]);
#pragma unroll
    for (int t = 0; t < WN; ++t) qb[0][t] = *reinterpret_cast<const v4i*>(lds + qrow_off + t * 16 * 128 + pcol[0]);
    __builtin_amdgcn_sched_barrier(0);
    // sum mode: before the first chunk of every digit but the top one, the sums so far move up by one digit
    int to_next_digit = chunks;
#define BSI_I8_HORNER()                                                               \
    if (kSum && ndig > 1) {                                                           \
        if (to_next_digit == 0) {                                                     \
            _Pragma("unroll") for (int a = 0; a < WM; ++a)                            \
                _Pragma("unroll") for (int b = 0; b < WN; ++b)                        \
                    _Pragma("unroll") for (int e = 0; e < 4; ++e) acc0[a][b][e] <<= 7; \
            to_next_digit = chunks;                                                   \
        }                                                                             \
        --to_next_digit;                                                              \
    }
    int c = 0;
    for (; c + 1 < vchunks; c += 2) {
        int* const ip = (!kSum && c > 0) ? chunk_ints + (c - 1) : nullptr;
        // even chunk c -> acc0, ring slots 0 and 1; epilogue of chunk c-1 (acc1, scales qsb)
        BSI_I8_HORNER();
        BSI_I8_CHUNK(0, 2, acc0, acc1, qsb, ip);
        if (!kSum) BSI_I8_SCALES(qsa, c);  // landed with the second half of chunk c
        // odd chunk c+1 -> acc1, ring slots 2 and 3; epilogue of chunk c (acc0, scales qsa)
        if (kSum) {
            BSI_I8_HORNER();
            BSI_I8_CHUNK(2, 0, acc0, acc1, qsb, ip);  // int32 sum: one accumulator set over all chunks
        } else {
            BSI_I8_CHUNK(2, 0, acc1, acc0, qsa, chunk_ints + c);
            BSI_I8_SCALES(qsb, c + 1);
        }
    }
    bool last_in_acc0 = false;
    if (c < vchunks) {  // odd number of chunks: one more even chunk; its halves sit in slots 0 and 1
        int* const ip = (!kSum && c > 0) ? chunk_ints + (c - 1) : nullptr;
        BSI_I8_HORNER();
        BSI_I8_CHUNK(0, 2, acc0, acc1, qsb, ip);
        if (!kSum) BSI_I8_SCALES(qsa, c);
        last_in_acc0 = true;
    }
    // the last k-step read ahead into a stage that does not exist (the loaders fill it with a copy of the last
    // one); nothing uses those operands
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (wave == 0) BSI_STAMP(kStampLoopDone);
#undef BSI_I8_HORNER
#undef BSI_I8_CHUNK
#undef BSI_I8_KSTEP
#undef BSI_I8_SCALES
    if (kSum && chunk_ints != nullptr) {  // the plain integer sums, int32 [Q, R_total]
#pragma unroll
        for (int a = 0; a < WM; ++a) {
            const int64_t rb = r0 + wr * (WM * 16) + a * 16 + lg * 4;
#pragma unroll
            for (int b = 0; b < WN; ++b) {
                const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
                if (q >= Q) continue;
                int* dst = chunk_ints + static_cast<size_t>(q) * R_total + rb;
                if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                    *reinterpret_cast<v4i*>(dst) = acc0[a][b];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (rb + e < R) dst[e] = acc0[a][b][e];
                }
            }
        }
        return;
    }
    if (kSum) {  // float(sum * 2^-down_shift * query factor * key factor) * scale_inv (+ bias), the product in float64
        const double down2 = __longlong_as_double(static_cast<long long>(1023 - down_shift) << 52);
        double qf[WN];
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
            qf[b] = (q < Q) ? static_cast<double>(qscale[q * qscale_stride]) * down2 : 0.0;
        }
        if (key_indices == nullptr) {
            // identity key order: the key factors and biases of all the wave's rows in one round trip (buffer loads:
            // rows past R and a missing bias read nothing and give 0), then four outputs per store
            float kfv[WM][4], biv[WM][4];
            const bsi_rsrc wrs = make_rsrc(Bw, static_cast<size_t>(R) * Sb * sizeof(float));
            const bsi_rsrc brs = make_rsrc(bias != nullptr ? bias : Bw, bias != nullptr ? static_cast<size_t>(R) * sizeof(float) : 0);
#pragma unroll
            for (int a = 0; a < WM; ++a) {
                const int rb = static_cast<int>(r0 + wr * (WM * 16) + a * 16 + lg * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    kfv[a][e] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(wrs, (rb + e) * Sb * 4, 0, 0));
                    biv[a][e] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(brs, (rb + e) * 4, 0, 0));
                }
            }
#pragma unroll
            for (int a = 0; a < WM; ++a)
#pragma unroll
                for (int b = 0; b < WN; ++b)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float v = static_cast<float>(static_cast<double>(acc0[a][b][e]) * qf[b] * static_cast<double>(kfv[a][e])) * scale_inv;
                        if (bias != nullptr) v = v + biv[a][e];
                        accf[a][b][e] = v;
                    }
            if (i8_store_lines<WM, WN>(accf, out, R_total, r0 + wr * (WM * 16), q0 + wq * (WN * 16), R, Q, ln, lg, out_stream != 0)) return;
#pragma unroll
            for (int a = 0; a < WM; ++a) {
                const int64_t rb = r0 + wr * (WM * 16) + a * 16 + lg * 4;
#pragma unroll
                for (int b = 0; b < WN; ++b) {
                    const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
                    if (q >= Q) continue;
                    float* dst = out + static_cast<size_t>(q) * R_total + rb;
                    if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                        *reinterpret_cast<float4*>(dst) = make_float4(accf[a][b][0], accf[a][b][1], accf[a][b][2], accf[a][b][3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (rb + e < R) dst[e] = accf[a][b][e];
                    }
                }
            }
            return;
        }
#pragma unroll
        for (int a = 0; a < WM; ++a) {
            const int64_t rb = r0 + wr * (WM * 16) + a * 16 + lg * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t r = rb + e;
                if (r >= R) continue;
                const double kf = static_cast<double>(Bw[r * Sb]);
                const float bi = bias != nullptr ? bias[r] : 0.0f;
                const int64_t col = key_indices ? key_indices[r] : r;
#pragma unroll
                for (int b = 0; b < WN; ++b) {
                    const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
                    if (q >= Q) continue;
                    float v = static_cast<float>(static_cast<double>(acc0[a][b][e]) * qf[b] * kf) * scale_inv;
                    if (bias != nullptr) v = v + bi;
                    out[static_cast<size_t>(q) * R_total + col] = v;
                }
            }
        }
        return;
    }
    // epilogue of the last chunk
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = last_in_acc0 ? acc0[a][b][e] : acc1[a][b][e];
                const float qsv = last_in_acc0 ? qsa[b] : qsb[b];
                accf[a][b][e] = fmaf(static_cast<float>(v), qsv, accf[a][b][e]);
                if (kInts && int_off[a][b] >= 0 && e < int_rows[a])
                    chunk_ints[int_off[a][b] + static_cast<int64_t>(e) * chunks + (chunks - 1)] = v >> down_shift;
            }
    // The key factors and biases of the wave's rows, from the copy the loader waves staged in LDS when the workgroup
    // started (0 for rows past R and for a call without bias): two 16-byte reads per 16-key tile.
    float bs[WM][4], bi[WM][4];
    {
        const float* epi = reinterpret_cast<const float*>(lds + 4 * C::kStage + C::kScaleBytes);
#pragma unroll
        for (int a = 0; a < WM; ++a) {
            const int rl = wr * (WM * 16) + a * 16 + lg * 4;  // row of the tile
            const float4 w4 = *reinterpret_cast<const float4*>(epi + rl);
            const float4 b4 = *reinterpret_cast<const float4*>(epi + TM + rl);
            bs[a][0] = key_factor(w4.x), bs[a][1] = key_factor(w4.y), bs[a][2] = key_factor(w4.z), bs[a][3] = key_factor(w4.w);
            bi[a][0] = b4.x, bi[a][1] = b4.y, bi[a][2] = b4.z, bi[a][3] = b4.w;
        }
    }
#pragma unroll
    for (int a = 0; a < WM; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // (acc * key scale) * scale_inv, then + bias: each step rounded on its own, as separate kernels would
                float v = ((accf[a][b][e] * down) * bs[a][e]) * scale_inv;
                if (bias != nullptr) v = v + bi[a][e];
                accf[a][b][e] = v;
            }
    if (!i8_store_lines<WM, WN>(accf, out, R_total, r0 + wr * (WM * 16), q0 + wq * (WN * 16), R, Q, ln, lg, out_stream != 0)) {
#pragma unroll
        for (int a = 0; a < WM; ++a) {
            const int64_t rb = r0 + wr * (WM * 16) + a * 16 + lg * 4;
#pragma unroll
            for (int b = 0; b < WN; ++b) {
                const int64_t q = q0 + wq * (WN * 16) + b * 16 + ln;
                if (q >= Q) continue;
                float* dst = out + static_cast<size_t>(q) * R_total + rb;
                if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                    *reinterpret_cast<float4*>(dst) = make_float4(accf[a][b][0], accf[a][b][1], accf[a][b][2], accf[a][b][3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (rb + e < R) dst[e] = accf[a][b][e];
                }
            }
        }
    }
#ifdef BSI_TIMELINE
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stamp below: the outputs have left the wave
    if (wave == 0) BSI_STAMP(kStampStored);
#endif
}

// ------------------------------------------------------------------ int8 image, one accumulator set per MFMA wave
//
// The same workgroup tile (128 keys x 128 queries), ring and epilogue as dot_mfma_i8_kernel<128, 128>, with MFMA waves
// that keep ONE int32 accumulator set instead of two.  Without a second set to park a finished chunk in, the chain
// step of chunk c (one cvt + one fma per output) runs on the accumulators in place, between a tile's last MFMA of
// chunk c (k-step 3) and its first of chunk c + 1 (k-step 0, which starts from zero and overwrites it): two
// elements behind each MFMA of k-step 3 from its third MFMA on, three behind each of the first MFMAs of the next
// k-step 0, always of tiles whose turn to be overwritten has not come.  The 32 registers this frees per wave let four
// MFMA waves of 64 keys x 64 queries (WN = 4 query tiles; one wave per SIMD, 256 registers each) do the work of eight
// of 64 x 32: an MFMA wave's operand reads are (64 + 64) x 64 bytes per 64 x 64 x 64 MACs instead of (64 + 32) x 64
// per 64 x 32 x 64, a third fewer LDS bytes per MAC.  (The same scheme on eight MFMA waves of 64 x 32 with eight
// loader waves needs 16 waves of at most 128 registers; it spills and is slower, so it is not built.)
template <int WN>
struct I8WDump {  // where a lane's accumulators go in the [Q, R, chunks] dump (parity checks): element (a, b, e) at
    int64_t base, qstep;  // base + b * qstep + (a * 16 + e) * chunks, for the query columns of qmask and the
    int rows[4];          // first rows[a] key rows of tile a
    unsigned qmask;
};
template <int WN, bool kInts>
__device__ __forceinline__ void i8w_chain(int first, int count, const v4i (&acc)[4][WN], float (&accf)[4][WN][4],
                                          const float (&qs)[WN], int* __restrict__ ints_at, const I8WDump<WN>& dump,
                                          int down_shift, int chunks) {
#pragma unroll
    for (int i = first; i < first + count; ++i) {
        if (i >= 16 * WN) break;
        const int tile = i >> 2, e = i & 3, a = tile / WN, b = tile % WN;
        accf[a][b][e] = fmaf(static_cast<float>(acc[a][b][e]), qs[b], accf[a][b][e]);
        if (kInts && ints_at != nullptr && ((dump.qmask >> b) & 1u) && e < dump.rows[a])
            ints_at[dump.base + b * dump.qstep + static_cast<int64_t>(a * 16 + e) * chunks] = acc[a][b][e] >> down_shift;
    }
}

// One k-step of such an MFMA wave: 4 WN MFMAs (tile t = WN a + b), the reads of the next k-step's 4 + WN operand
// tiles behind the first of them, and the chain elements that fall to this k-step (see above).  qs_cur / ints_cur:
// scales and accumulator dump of the chunk being computed (used by k-step 3); qs_prev / ints_prev: of the chunk
// before it (used by k-step 0).
template <int WN, int KS, bool kInts>
__device__ __forceinline__ void i8w_kstep(const v4i (&ka)[4], const v4i (&qb)[WN], v4i (&ka_n)[4], v4i (&qb_n)[WN],
                                          const unsigned char* __restrict__ krow_n,
                                          const unsigned char* __restrict__ qrow_n, v4i (&acc)[4][WN],
                                          float (&accf)[4][WN][4], const float (&qs_cur)[WN], const float (&qs_prev)[WN],
                                          int* __restrict__ ints_cur, int* __restrict__ ints_prev, const I8WDump<WN>& dump,
                                          int down_shift, int chunks) {
    constexpr int NT = 4 * WN;            // tiles of the wave
    constexpr int kLate = 2 * (NT - 2);   // chain elements k-step 3 takes care of; the rest fall to the next k-step 0
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int a = t / WN, b = t % WN;
        const v4i c0 = (KS == 0) ? (v4i){0, 0, 0, 0} : acc[a][b];
        acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ka[a], qb[b], c0, 0, 0, 0);
        // read number t of the next k-step, in the order its MFMAs first need them: ka[0], qb[0 ..], ka[1 ..]
        if (t == 0) ka_n[0] = *reinterpret_cast<const v4i*>(krow_n);
        else if (t <= WN) qb_n[t - 1] = *reinterpret_cast<const v4i*>(qrow_n + (t - 1) * 16 * 128);
        else if (t < 4 + WN) ka_n[t - WN] = *reinterpret_cast<const v4i*>(krow_n + (t - WN) * 16 * 128);
        if (KS == 0 && kLate + 3 * t < 4 * NT)  // three elements of the previous chunk, of tiles above t
            i8w_chain<WN, kInts>(kLate + 3 * t, 3, acc, accf, qs_prev, ints_prev, dump, down_shift, chunks);
        if (KS == 3 && t >= 2)  // two elements of this chunk, of tiles finished two MFMAs ago or earlier
            i8w_chain<WN, kInts>(2 * (t - 2), 2, acc, accf, qs_cur, ints_cur, dump, down_shift, chunks);
        __builtin_amdgcn_sched_barrier(0);
    }
}

template <int WN>
struct I8WCfg {
    static_assert(WN == 4, "four MFMA waves of 64 x 64");
    using Tile = I8Cfg<128, 128>;  // LDS layout and loader waves
    static constexpr int kWavesN = 128 / (16 * WN);      // MFMA waves along the queries (2 along the keys)
    static constexpr int kConsumers = 2 * kWavesN;
    static constexpr int kBlock = (kConsumers + Tile::kLoaders) * 64;
};

template <int WN, bool kInts>
__global__ __launch_bounds__((I8WCfg<WN>::kBlock)) void dot_mfma_i8w_kernel(
    const int8_t* __restrict__ A8, const float* __restrict__ qscale, int qscale_stride, const int8_t* __restrict__ K8,
    const float* __restrict__ Bw, int Sb, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv,
    int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints, const float* __restrict__ bias,
    int key_tiled, const unsigned char* __restrict__ warm, long long warm_lines, int out_stream) {
    constexpr int TM = 128, TN = 128;
    using W = I8WCfg<WN>;
    using C = typename W::Tile;
    constexpr int kNE = 16 * WN;          // chain elements per lane and chunk
    constexpr int kLate = 2 * (4 * WN - 2);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // C::kLds

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t r0 = static_cast<int64_t>(blockIdx.x) * TM;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * TN;
    const size_t rowbytes = static_cast<size_t>(chunks) * 256;
    const int halves = chunks * 2;
    unsigned char* const scale_lds = lds + 4 * C::kStage;

    if (wave >= W::kConsumers) {
        i8_loader_wave<C, false>(lds, wave - W::kConsumers, lane, A8, qscale, qscale_stride, K8, Bw, Sb, chunks, halves, R, Q,
                                 r0, q0, rowbytes, bias, 1, 0, key_tiled, warm, warm_lines);
        return;
    }

    // ---- MFMA waves: wr = half of the keys, wq = group of 16 WN queries
    const int wr = wave & 1, wq = wave >> 1;
    const int ln = lane & 15, lg = lane >> 4;
    const int krow_off = (wr * 64 + ln) * 128;
    const int qrow_off = C::kOperandK + (wq * (16 * WN) + ln) * 128;
    int pcol[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) pcol[kk] = ((kk * 4 + lg) ^ (ln >> 1)) * 16;
    float accf[4][WN][4];
    v4i acc[4][WN];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            acc[a][b] = (v4i){0, 0, 0, 0};
#pragma unroll
            for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;
        }
    const float down = __uint_as_float(static_cast<uint32_t>(127 - down_shift) << 23);
    I8WDump<WN> dump;
    {
        const int64_t rl = r0 + wr * 64 + lg * 4, ql = q0 + wq * (16 * WN) + ln;  // the lane's first key row and query column
        dump.base = (ql * R + rl) * chunks;
        dump.qstep = 16 * R * chunks;
        dump.qmask = 0;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t left = R - (rl + a * 16);
            dump.rows[a] = static_cast<int>(left < 0 ? 0 : (left < 4 ? left : 4));
        }
#pragma unroll
        for (int b = 0; b < WN; ++b)
            if (kInts && ql + b * 16 < Q) dump.qmask |= 1u << b;
    }
    // chunk scales of the lane's query columns, from the loaders' ring: 64 queries per region, region g = queries 64 g ..
    const int qfirst = wq * (16 * WN);
    const unsigned char* sread = scale_lds + (qfirst >> 6) * 256 + ((qfirst & 63) + ln) * 4;
    float qsa[WN], qsb[WN];  // scales of even / odd chunks (all zero before the first chunk: its "previous" chain adds 0)
#pragma unroll
    for (int b = 0; b < WN; ++b) qsa[b] = qsb[b] = 0.0f;
#define BSI_I8W_SCALES(dst, c)                                                                         \
    {                                                                                                  \
        _Pragma("unroll") for (int b = 0; b < WN; ++b) dst[b] =                                        \
            *reinterpret_cast<const float*>(sread + ((c) & 3) * (C::kLoaders * 256) + b * 64);         \
    }
    v4i ka[2][4], qb[2][WN];  // operand sets of even / odd k-steps
#define BSI_I8W_KSTEP(KS, nslot, qc, qp, ic, ip)                                                                    \
    i8w_kstep<WN, KS, kInts>(ka[(KS) & 1], qb[(KS) & 1], ka[((KS) + 1) & 1], qb[((KS) + 1) & 1],                    \
                             lds + (nslot) * C::kStage + krow_off + pcol[((KS) + 1) & 1],                           \
                             lds + (nslot) * C::kStage + qrow_off + pcol[((KS) + 1) & 1], acc, accf, qc, qp, ic, ip, \
                             dump, down_shift, chunks);
    // a chunk whose halves sit in ring slots s0, s0 + 1; nslot: slot of the next chunk's first half; qc / qp: this
    // chunk's and the previous chunk's scales.  This chunk's scales have landed with its second half, which the
    // first barrier announces.
#define BSI_I8W_CHUNK(s0, nslot, qc, qp, ic, ip, c)                                                                 \
    BSI_I8W_KSTEP(0, s0, qc, qp, ic, ip);                                                                           \
    lds_barrier();                                                                                                  \
    BSI_I8W_SCALES(qc, c);                                                                                          \
    BSI_I8W_KSTEP(1, (s0) + 1, qc, qp, ic, ip);                                                                     \
    BSI_I8W_KSTEP(2, (s0) + 1, qc, qp, ic, ip);                                                                     \
    lds_barrier();                                                                                                  \
    BSI_I8W_KSTEP(3, nslot, qc, qp, ic, ip);

    lds_barrier();  // stage 0 is there
#pragma unroll
    for (int t = 0; t < 4; ++t) ka[0][t] = *reinterpret_cast<const v4i*>(lds + krow_off + t * 16 * 128 + pcol[0]);
#pragma unroll
    for (int t = 0; t < WN; ++t) qb[0][t] = *reinterpret_cast<const v4i*>(lds + qrow_off + t * 16 * 128 + pcol[0]);
    __builtin_amdgcn_sched_barrier(0);
    int c = 0;
    for (; c + 1 < chunks; c += 2) {
        // even chunk c: ring slots 0 and 1, scales qsa; the chain elements of chunk c - 1 left for its k-step 0 use qsb
        BSI_I8W_CHUNK(0, 2, qsa, qsb, chunk_ints + c, (c > 0 ? chunk_ints + (c - 1) : nullptr), c);
        // odd chunk c + 1: ring slots 2 and 3, scales qsb
        BSI_I8W_CHUNK(2, 0, qsb, qsa, chunk_ints + c + 1, chunk_ints + c, c + 1);
    }
    bool last_even = false;
    if (c < chunks) {  // odd number of chunks: one more even chunk
        BSI_I8W_CHUNK(0, 2, qsa, qsb, chunk_ints + c, (c > 0 ? chunk_ints + (c - 1) : nullptr), c);
        last_even = true;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the last k-step read ahead into a stage nothing uses
#undef BSI_I8W_CHUNK
#undef BSI_I8W_KSTEP
#undef BSI_I8W_SCALES
    // the chain elements of the last chunk that its k-step 3 left
    if (last_even) i8w_chain<WN, kInts>(kLate, kNE - kLate, acc, accf, qsa, chunk_ints + (chunks - 1), dump, down_shift, chunks);
    else i8w_chain<WN, kInts>(kLate, kNE - kLate, acc, accf, qsb, chunk_ints + (chunks - 1), dump, down_shift, chunks);
    // key factors and biases from the copy the loader waves staged in LDS
    float bs[4][4], bi[4][4];
    {
        const float* epi = reinterpret_cast<const float*>(lds + 4 * C::kStage + C::kScaleBytes);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int rl = wr * 64 + a * 16 + lg * 4;
            const float4 w4 = *reinterpret_cast<const float4*>(epi + rl);
            const float4 b4 = *reinterpret_cast<const float4*>(epi + TM + rl);
            bs[a][0] = key_factor(w4.x), bs[a][1] = key_factor(w4.y), bs[a][2] = key_factor(w4.z), bs[a][3] = key_factor(w4.w);
            bi[a][0] = b4.x, bi[a][1] = b4.y, bi[a][2] = b4.z, bi[a][3] = b4.w;
        }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < WN; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = ((accf[a][b][e] * down) * bs[a][e]) * scale_inv;
                if (bias != nullptr) v = v + bi[a][e];
                accf[a][b][e] = v;
            }
    if (i8_store_lines<4, WN>(accf, out, R_total, r0 + wr * 64, q0 + wq * (16 * WN), R, Q, ln, lg, out_stream != 0)) return;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int64_t rb = r0 + wr * 64 + a * 16 + lg * 4;
#pragma unroll
        for (int b = 0; b < WN; ++b) {
            const int64_t q = q0 + wq * (16 * WN) + b * 16 + ln;
            if (q >= Q) continue;
            float* dst = out + static_cast<size_t>(q) * R_total + rb;
            if (rb + 3 < R && ((reinterpret_cast<uintptr_t>(dst) & 15) == 0)) {
                *reinterpret_cast<float4*>(dst) = make_float4(accf[a][b][0], accf[a][b][1], accf[a][b][2], accf[a][b][3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (rb + e < R) dst[e] = accf[a][b][e];
            }
        }
    }
}

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
// The epilogue's operands (the key's slice-0 weight and, optionally, its bias), requested when the kernel starts
// instead of after the chain, where two dependent cache misses would end every workgroup.  Buffer loads: a lane
// without an output, or a call without bias, reads nothing and gets 0; no branch, so the loads stay where they
// are written.
struct EpilogueOperands {
    float bw, bias;
};
__device__ __forceinline__ EpilogueOperands load_epilogue_operands(const float* Bw, const float* bias, int64_t R, bool valid,
                                                                   int64_t r) {
    const bsi_rsrc wr = make_rsrc(Bw, static_cast<size_t>(R) * 6 * sizeof(float));
    const bsi_rsrc br = make_rsrc(bias != nullptr ? bias : Bw, bias != nullptr ? static_cast<size_t>(R) * sizeof(float) : 0);
    EpilogueOperands e;
    e.bw = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(wr, valid ? static_cast<int>(r * 24) : -1, 0, 0));
    e.bias = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(br, valid ? static_cast<int>(r * 4) : -1, 0, 0));
    return e;
}

// The fp32 chain of one output over chunks [c0, c1): accf = fmaf(float(I_c), scale_c * down, accf) in chunk order,
// eight chunks' integers and scales fetched ahead of their eight dependent steps (fetched one step at a time the
// chain costs an LDS or cache round trip per chunk: 4 us of a 17 us kernel at 64 chunks).  int_at(c) / scale_at(c)
// read chunk c's integer and chunk scale; the arithmetic and its order are those of the one-step loop.
template <typename IntAt, typename ScaleAt>
__device__ __forceinline__ float chain_chunks(float accf, int c0, int c1, float down, IntAt int_at, ScaleAt scale_at) {
    int c = c0;
    for (; c + 8 <= c1; c += 8) {
        int v[8];
        float sc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = int_at(c + u);
            sc[u] = scale_at(c + u);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) accf = fmaf(static_cast<float>(v[u]), sc[u] * down, accf);
    }
    for (; c < c1; ++c) accf = fmaf(static_cast<float>(int_at(c)), scale_at(c) * down, accf);
    return accf;
}

constexpr int kStreamMaxQ = 32;        // above this the 128 x 128 tiled kernel takes over
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
        const float bs = key_factor(Bw[r * SB]);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int64_t q = q0 + tq + 16 * a;
            if (q < Q) out[static_cast<size_t>(q) * R_total + r] = (accf[a][b] * bs) * scale_inv;
        }
    }
}

// Any Sa, Sb up to 63 (where the reference clamps its fixed-bit flags, bsi_vector_cuda.cpp:256-262): one thread per
// output, planes read straight from global memory.  The chunk's integer is summed modulo 2^64 (a term shifted by 64
// or more is a multiple of 2^64), which is the integer dot of the chunk whenever that fits 64 bits; the per-chunk
// integers stored for parity checks are its low 32 bits.  tiled: the key planes are in
// the tiled16 layout (word (r, j, 4 c + g) at (((r / 16) chunks + c) Sb + j) 64 + 16 g + r % 16) instead of [R, Sb, W64].
__global__ void dot_valu_generic_kernel(const unsigned long long* __restrict__ A, const float* __restrict__ qscale,
                                        int qscale_stride, int Sa, const unsigned long long* __restrict__ B,
                                        const float* __restrict__ Bw, int Sb, int W64, int chunks, int64_t R,
                                        int64_t Q, float scale_inv, int64_t R_total, float* __restrict__ out,
                                        int* __restrict__ chunk_ints, int tiled) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= Q * R) return;
    const int64_t q = idx / R;
    const int64_t r = idx - q * R;
    const unsigned long long* Aq = A + static_cast<size_t>(q) * Sa * W64;
    const unsigned long long* Br = B + static_cast<size_t>(r) * Sb * W64;
    const unsigned long long* Bt = B + static_cast<size_t>(r >> 4) * chunks * Sb * 64 + (r & 15);  // the row's 16-key tile
    float acc = 0.0f;
    for (int c = 0; c < chunks; ++c) {
        unsigned long long I = 0ULL;
        for (int i = 0; i < Sa; ++i)
            for (int j = 0; j < Sb; ++j) {
                int cnt = 0;
                for (int w = c * 4; w < c * 4 + 4 && w < W64; ++w) {
                    const unsigned long long bw = tiled ? Bt[(static_cast<size_t>(c) * Sb + j) * 64 + (w & 3) * 16] : Br[j * W64 + w];
                    cnt += __popcll(Aq[i * W64 + w] & bw);
                }
                const unsigned long long v = (i + j < 64) ? static_cast<unsigned long long>(cnt) << (i + j) : 0ULL;
                I = ((i == Sa - 1) != (j == Sb - 1)) ? I - v : I + v;
            }
        if (chunk_ints) chunk_ints[(static_cast<size_t>(q) * R + r) * chunks + c] = static_cast<int>(I);
        acc = fmaf(static_cast<float>(static_cast<long long>(I)), qscale[q * qscale_stride + ((qscale_stride == 1) ? 0 : c)], acc);
    }
    out[static_cast<size_t>(q) * R_total + r] = (acc * key_factor(Bw[r * Sb])) * scale_inv;
}

// Weighted-slice dot for operands whose slice weights are arbitrary floats (the decimal builder's
// data-dependent slice counts, or fixed-bit operands without chunk scales):
//   out[q, idx[r]] = float(sum over i, j, w of popcount(A[q,i,w] & B[r,j,w]) * double(Aw[q,i] * Bw[r,j])) * scale_inv
// The coefficient is the float32 product; the sum runs in float64, exact while it stays below 2^53 (every
// term is an integer times a power of two for the builders' weights), so the result does not depend on
// the order of the terms.  Workgroup = 32 queries x 32 keys, 2 x 2 outputs per thread, WB words of every
// slice staged through LDS per step.  Any Sa, Sb in [1, 64].
template <int WB, bool kTiled>
__global__ __launch_bounds__(256) void dot_weighted_kernel(
    const unsigned long long* __restrict__ A, const float* __restrict__ Aw, int Sa, int W64,
    const unsigned long long* __restrict__ B, const float* __restrict__ Bw, int Sb, int chunks, int64_t R, int64_t Q,
    const long long* __restrict__ key_indices, float scale_inv, int64_t R_total, float* __restrict__ out,
    double* __restrict__ out64) {
    extern __shared__ __attribute__((aligned(16))) unsigned char wlds[];
    const int strideA = Sa * WB + 1, strideB = Sb * WB + 1;  // in 64-bit words; odd, so rows start in different banks
    unsigned long long* As = reinterpret_cast<unsigned long long*>(wlds);  // [32][strideA]
    unsigned long long* Bs = As + 32 * strideA;                            // [32][strideB]
    float* Aws = reinterpret_cast<float*>(Bs + 32 * strideB);              // [32][Sa]
    float* Bws = Aws + 32 * Sa;                                            // [32][Sb]
    const int tid = threadIdx.x;
    const int tq = tid >> 4, tr = tid & 15;
    const int64_t q0 = static_cast<int64_t>(blockIdx.y) * 32, r0 = static_cast<int64_t>(blockIdx.x) * 32;
    for (int idx = tid; idx < 32 * Sa; idx += 256) {
        const int64_t q = q0 + idx / Sa;
        Aws[idx] = q < Q ? Aw[q * Sa + idx % Sa] : 0.0f;
    }
    for (int idx = tid; idx < 32 * Sb; idx += 256) {
        const int64_t r = r0 + idx / Sb;
        Bws[idx] = r < R ? Bw[r * Sb + idx % Sb] : 0.0f;
    }
    double acc[2][2] = {{0.0, 0.0}, {0.0, 0.0}};
    for (int w0 = 0; w0 < W64; w0 += WB) {
        __syncthreads();  // the previous step's reads are done (and, first time, nothing)
        for (int idx = tid; idx < 32 * Sa * WB; idx += 256) {
            const int m = idx / (Sa * WB), rem = idx - m * (Sa * WB);
            const int i = rem / WB, w = w0 + rem % WB;
            const int64_t q = q0 + m;
            As[m * strideA + rem] = (q < Q && w < W64) ? A[(q * Sa + i) * W64 + w] : 0ULL;
        }
        for (int idx = tid; idx < 32 * Sb * WB; idx += 256) {
            const int m = idx / (Sb * WB), rem = idx - m * (Sb * WB);
            const int j = rem / WB, w = w0 + rem % WB;
            const int64_t r = r0 + m;
            unsigned long long v = 0ULL;
            if (r < R && w < W64)
                v = kTiled ? B[((((r >> 4) * chunks + (w >> 2)) * Sb + j) * 64) + (w & 3) * 16 + (r & 15)]
                           : B[(r * Sb + j) * W64 + w];
            Bs[m * strideB + rem] = v;
        }
        __syncthreads();
        for (int i = 0; i < Sa; ++i) {
            unsigned long long a0[WB], a1[WB];
#pragma unroll
            for (int w = 0; w < WB; ++w) {
                a0[w] = As[tq * strideA + i * WB + w];
                a1[w] = As[(tq + 16) * strideA + i * WB + w];
            }
            const float aw0 = Aws[tq * Sa + i], aw1 = Aws[(tq + 16) * Sa + i];
            for (int j = 0; j < Sb; ++j) {
                const unsigned long long* b0 = Bs + tr * strideB + j * WB;
                const unsigned long long* b1 = Bs + (tr + 16) * strideB + j * WB;
                int c00 = 0, c01 = 0, c10 = 0, c11 = 0;
#pragma unroll
                for (int w = 0; w < WB; ++w) {
                    const unsigned long long x0 = b0[w], x1 = b1[w];
                    c00 += __popcll(a0[w] & x0);
                    c01 += __popcll(a0[w] & x1);
                    c10 += __popcll(a1[w] & x0);
                    c11 += __popcll(a1[w] & x1);
                }
                const float bw0 = Bws[tr * Sb + j], bw1 = Bws[(tr + 16) * Sb + j];
                acc[0][0] += static_cast<double>(c00) * static_cast<double>(aw0 * bw0);
                acc[0][1] += static_cast<double>(c01) * static_cast<double>(aw0 * bw1);
                acc[1][0] += static_cast<double>(c10) * static_cast<double>(aw1 * bw0);
                acc[1][1] += static_cast<double>(c11) * static_cast<double>(aw1 * bw1);
            }
        }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int64_t q = q0 + tq + 16 * a, r = r0 + tr + 16 * b;
            if (q < Q && r < R) {
                const int64_t col = key_indices ? key_indices[r] : r;
                if (out64 != nullptr) out64[q * R_total + col] = acc[a][b];  // the exact weighted sum itself
                else out[q * R_total + col] = static_cast<float>(acc[a][b]) * scale_inv;
            }
        }
}

// out[q, r] += bias[r] for the kernels that do not add the bias in their own epilogue
__global__ void add_bias_kernel(float* __restrict__ out, const float* __restrict__ bias, int64_t Q, int64_t R,
                                int64_t R_total) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= Q * R) return;
    const int64_t q = i / R, r = i - q * R;
    out[q * R_total + r] = out[q * R_total + r] + bias[r];
}

__global__ void zero_uint4_kernel(uint4* __restrict__ p, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

static int launch_planes_to_int8(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out, hipStream_t st,
                                 int tiled = 0) {
    const int chunks = (W64 + 3) / 4;
    const int64_t total = rows * chunks * 8;
    if (total == 0) return BSI_OK;
    if (tiled && (rows & 63) != 0) {  // the rows that pad the last 64-row tile read as zeros
        const size_t tile_bytes = static_cast<size_t>(chunks) * 2 * 8192;
        hipLaunchKernelGGL(zero_uint4_kernel, dim3(static_cast<unsigned>((tile_bytes / 16 + 255) / 256)), dim3(256), 0, st,
                           reinterpret_cast<uint4*>(out + static_cast<size_t>(rows >> 6) * tile_bytes), tile_bytes / 16);
        BSI_LAUNCH_CHECK("zero_uint4_kernel");
    }
    hipLaunchKernelGGL(planes_to_int8_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const uint32_t*>(words), rows, S, W64, chunks,
                       reinterpret_cast<uint32_t*>(out), tiled);
    BSI_LAUNCH_CHECK("planes_to_int8_kernel");
    return BSI_OK;
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

// Set by bsi_hip_dot_bias_warm around its launch: the region the int8-image kernel should touch for the next dot.
static thread_local const void* g_warm_ptr = nullptr;
static thread_local size_t g_warm_bytes = 0;
// How the int8-image kernels store their output.  The entry points of a linear layer (bsi_hip_dot_bias,
// bsi_hip_dot_bias_warm, bsi_hip_linear) set t_layer_output around their launch: the next kernel of the model reads
// that output, so it is stored plainly and stays in the caches.  The dot entry points proper stream it out with
// nontemporal stores: the dirty lines then do not wait in the L2s for the write-back at the kernel's end (1.2 us less
// for the 16 MiB of Q512 R8192).  Measured both ways: streamed layer outputs cost an OPT-1.3B-shaped prefill 2 %
// (4.89 -> 5.00 ms replayed), plain dot outputs cost the standalone dot 8 %.  BSI_OPT_OUTPUT_STORES overrides.
static thread_local int t_layer_output = 0;
static std::atomic<int> g_output_stores{0};  // 0 = by entry point, 1 = always plain, 2 = always nontemporal
static int stream_output() {
    const int forced = g_output_stores.load(std::memory_order_relaxed);
    if (forced != 0) return forced == 2 ? 1 : 0;
    return t_layer_output ? 0 : 1;
}

template <int TM, int TN, int kMode>
static void launch_mfma_i8_tm(const int8_t* A8, const float* qscale, int stride, const int8_t* K8, const float* Bw,
                              int Sb, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv,
                              int64_t R_total, float* out, int32_t* chunk_ints, const float* bias, hipStream_t st,
                              int ndig, long long dig_stride, const long long* key_indices, int key_tiled) {
    using C = I8Cfg<TM, TN>;
    const dim3 grid(static_cast<unsigned>((R + TM - 1) / TM), static_cast<unsigned>((Q + TN - 1) / TN));
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_i8_kernel<TM, TN, kMode>), C::kLds);
    hipLaunchKernelGGL((dot_mfma_i8_kernel<TM, TN, kMode>), grid, dim3(C::kBlock), C::kLds, st, A8, qscale, stride, K8,
                       Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, ndig, dig_stride,
                       key_indices, key_tiled, static_cast<const unsigned char*>(g_warm_ptr),
                       static_cast<long long>(g_warm_bytes / 128), stream_output());
}

// Sum mode (ndig >= 1 digit images of the queries; int32 sums into chunk_ints when given, else the float epilogue)
// or, with ndig == 0, the chain with or without stored integers.
template <int TM, int TN>
static void launch_mfma_i8_t(int ndig, long long dig_stride, const long long* key_indices, int key_tiled, const int8_t* A8,
                             const float* qscale, int stride, const int8_t* K8, const float* Bw, int Sb, int chunks,
                             int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total, float* out,
                             int32_t* chunk_ints, const float* bias, hipStream_t st) {
    if (ndig > 0)
        launch_mfma_i8_tm<TM, TN, kI8Sum>(A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total,
                                          out, chunk_ints, bias, st, ndig, dig_stride, key_indices, key_tiled);
    else if (chunk_ints)
        launch_mfma_i8_tm<TM, TN, kI8Ints>(A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total,
                                           out, chunk_ints, bias, st, 1, 0, nullptr, key_tiled);
    else
        launch_mfma_i8_tm<TM, TN, kI8Chain>(A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv,
                                            R_total, out, chunk_ints, bias, st, 1, 0, nullptr, key_tiled);
}

// The 128 x 128 tile on four MFMA waves of 64 x 64 with one accumulator set, and four loader waves (tile 1284; chain
// modes only).
template <int WN>
static void launch_mfma_i8w(const int8_t* A8, const float* qscale, int stride, const int8_t* K8, const float* Bw, int Sb,
                            int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total, float* out,
                            int32_t* chunk_ints, const float* bias, hipStream_t st, int key_tiled) {
    using W = I8WCfg<WN>;
    using C = typename W::Tile;
    const dim3 grid(static_cast<unsigned>((R + 127) / 128), static_cast<unsigned>((Q + 127) / 128));
    static LdsOptIn once0, once1;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_i8w_kernel<WN, false>), C::kLds);
    lds_opt_in(once1, reinterpret_cast<const void*>(&dot_mfma_i8w_kernel<WN, true>), C::kLds);
    const unsigned char* warm = static_cast<const unsigned char*>(g_warm_ptr);
    const long long warm_lines = static_cast<long long>(g_warm_bytes / 128);
    if (chunk_ints)
        hipLaunchKernelGGL((dot_mfma_i8w_kernel<WN, true>), grid, dim3(W::kBlock), C::kLds, st, A8, qscale, stride, K8, Bw, Sb,
                           chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, key_tiled, warm, warm_lines,
                           stream_output());
    else
        hipLaunchKernelGGL((dot_mfma_i8w_kernel<WN, false>), grid, dim3(W::kBlock), C::kLds, st, A8, qscale, stride, K8, Bw, Sb,
                           chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, key_tiled, warm, warm_lines,
                           stream_output());
}

// Tile choice.  The 128 x 128 tile moves the fewest operand bytes per MAC and is the fastest whenever its grid
// covers the 256 CUs (one workgroup per CU at a time) -- measured up to several rounds of 256.  A smaller grid
// leaves CUs idle that smaller tiles would use: a workgroup's time per half-chunk is about 1 : 0.63 : 0.35 : 0.31
// for 128 x 128 : 128 x 64 : 64 x 64 : 64 x 32, so take the least (rounds of 256 workgroups x time), the larger
// tile on a tie.  g_i8_tile forces a tile (tuning and tests).
static int choose_i8_tile(int64_t R, int64_t Q, int64_t* cost_out = nullptr) {
    const int64_t n128 = ((R + 127) / 128) * ((Q + 127) / 128);
    if (cost_out) *cost_out = ((n128 + 255) / 256) * 100;
    if (const int forced = g_i8_tile.load(std::memory_order_relaxed)) return forced;
    if (n128 > 256) return 128;
    const int64_t cost[4] = {100, ((((R + 127) / 128) * ((Q + 63) / 64) + 255) / 256) * 63,
                             ((((R + 63) / 64) * ((Q + 63) / 64) + 255) / 256) * 35,
                             ((((R + 63) / 64) * ((Q + 31) / 32) + 255) / 256) * 31};
    const int tiles[4] = {128, 12864, 64, 6432};
    int best = 0;
    for (int i = 1; i < 4; ++i)
        if (cost[i] < cost[best]) best = i;
    if (cost_out) *cost_out = cost[best];
    return tiles[best];
}

static void launch_mfma_i8(const int8_t* A8, const float* qscale, int stride, const int8_t* K8, const float* Bw, int Sb,
                           int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                           float* out, int32_t* chunk_ints, const float* bias, hipStream_t st, int key_tiled = 0,
                           int ndig = 0, long long dig_stride = 0, const long long* key_indices = nullptr) {
    const int tile = choose_i8_tile(R, Q);
    if (tile == 1284 && ndig == 0) {
        launch_mfma_i8w<4>(A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias,
                           st, key_tiled);
        return;
    }
#define BSI_I8_ARGS ndig, dig_stride, key_indices, key_tiled, A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, st
    if (tile == 128 || tile == 1284) launch_mfma_i8_t<128, 128>(BSI_I8_ARGS);
    else if (tile == 12864) launch_mfma_i8_t<128, 64>(BSI_I8_ARGS);
    else if (tile == 64) launch_mfma_i8_t<64, 64>(BSI_I8_ARGS);
    else launch_mfma_i8_t<64, 32>(BSI_I8_ARGS);
#undef BSI_I8_ARGS
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

extern "C" size_t bsi_hip_int8_tiled_bytes(int64_t rows, int W64) {
    if (rows <= 0 || W64 <= 0) return 0;
    return static_cast<size_t>((rows + 63) / 64) * static_cast<size_t>((W64 + 3) / 4) * 2 * 8192;
}

extern "C" int bsi_hip_planes_to_int8_tiled(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out,
                                            void* stream) {
    BSI_REQUIRE(rows >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(S >= 1 && S <= 8, "S must be in [1, 8] (got %d)", S);
    if (rows == 0) return BSI_OK;
    BSI_REQUIRE(words && out, "null pointer");
    return launch_planes_to_int8(words, rows, S, W64, out, as_stream(stream), /*tiled=*/1);
}

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
            // two key tiles per workgroup halve the query re-reads once there are enough tiles to fill the GPU
            const bool two = (R + 15) / 16 >= 1024;
#define BSI_STREAM_ARGS A8, A_chunk_scales, A_scale_stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, st
            if (Q <= 16) { if (two) launch_mfma_stream<1, 2>(BSI_STREAM_ARGS); else launch_mfma_stream<1, 1>(BSI_STREAM_ARGS); }
            else { if (two) launch_mfma_stream<2, 2>(BSI_STREAM_ARGS); else launch_mfma_stream<2, 1>(BSI_STREAM_ARGS); }
#undef BSI_STREAM_ARGS
            BSI_LAUNCH_CHECK("dot_mfma_stream_kernel");
            *bias_fused = true;
            return BSI_OK;
        }
        if (Sb == 6 && tiled) {
            launch_mfma_ws<6>(A8, A_chunk_scales, A_scale_stride, B, Bw, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
            BSI_LAUNCH_CHECK("dot_mfma_ws_kernel");
            return BSI_OK;
        }
        if (Sb == 6) {  // canonical planes (the tiled ones went to the kernels above)
            launch_mfma<6, false>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        } else {
            if (tiled) launch_mfma<0, true>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
            else launch_mfma<0, false>(A8, A_chunk_scales, A_scale_stride, B, Bw, Sb, W64, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, st);
        }
        BSI_LAUNCH_CHECK("dot_mfma_kernel");
        return BSI_OK;
    }

    if (core != BSI_CORE_VALU) return fail(BSI_ERR_INVALID, "unknown core %d", core);
    if (b_layout == BSI_LAYOUT_INT8 || b_layout == BSI_LAYOUT_INT8_TILED)
        return fail(BSI_ERR_UNSUPPORTED, "the popcount core reads key planes, not the int8 image");
    BSI_REQUIRE(A != nullptr, "VALU core needs the query planes");
    if (Sa == 7 && Sb == 6) {
        if (b_layout == BSI_LAYOUT_TILED16)
            launch_valu76<true>(A, A_chunk_scales, A_scale_stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
        else
            launch_valu76<false>(A, A_chunk_scales, A_scale_stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
        BSI_LAUNCH_CHECK("dot_valu_kernel");
        return BSI_OK;
    }
    const int64_t total = Q * R;
    BSI_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, "too many outputs for one launch of the any-width kernel");
    hipLaunchKernelGGL(dot_valu_generic_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const unsigned long long*>(A), A_chunk_scales, A_scale_stride, Sa,
                       reinterpret_cast<const unsigned long long*>(B), Bw, Sb, W64, chunks, R, Q, scale_inv, R_total,
                       out, chunk_ints, b_layout == BSI_LAYOUT_TILED16 ? 1 : 0);
    BSI_LAUNCH_CHECK("dot_valu_generic_kernel");
    return BSI_OK;
}

static int dot_with_bias(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride,
                         int Sa, int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                         float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core, void* workspace,
                         size_t workspace_bytes, void* stream, const float* bias) {
    bool fused = false;
    const int rc = dot_launch(A, A_ints8, A_chunk_scales, A_scale_stride, Sa, W64, B, b_layout, Bw, Sb, R, Q, scale_inv,
                              R_total, out, chunk_ints, core, workspace, workspace_bytes, stream, bias, &fused);
    if (rc != BSI_OK || bias == nullptr || fused || Q == 0 || R == 0) return rc;
    const int64_t total = Q * R;
    hipLaunchKernelGGL(add_bias_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                       out, bias, Q, R, R_total);
    BSI_LAUNCH_CHECK("add_bias_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_add_bias(float* out, const float* bias, int64_t Q, int64_t R, int64_t R_total, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0 && R_total >= R, "bad shape");
    if (Q == 0 || R == 0) return BSI_OK;
    BSI_REQUIRE(out && bias, "null pointer");
    const int64_t total = Q * R;
    hipLaunchKernelGGL(add_bias_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, as_stream(stream),
                       out, bias, Q, R, R_total);
    BSI_LAUNCH_CHECK("add_bias_kernel");
    return BSI_OK;
}

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

template <int WB, bool kTiled>
static int launch_dot_weighted(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B, const float* Bw,
                               int Sb, int64_t R, int64_t Q, const int64_t* key_indices, float scale_inv,
                               int64_t R_total, float* out, double* out64, hipStream_t st) {
    const size_t lds = static_cast<size_t>(32) * ((Sa * WB + 1) + (Sb * WB + 1)) * 8 + static_cast<size_t>(32) * (Sa + Sb) * 4;
    if (lds > 150 * 1024) return fail(BSI_ERR_UNSUPPORTED, "slice counts %d + %d do not fit the LDS tile", Sa, Sb);
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_weighted_kernel<WB, kTiled>), 150 * 1024);
    const dim3 grid(static_cast<unsigned>((R + 31) / 32), static_cast<unsigned>((Q + 31) / 32));
    hipLaunchKernelGGL((dot_weighted_kernel<WB, kTiled>), grid, dim3(256), lds, st,
                       reinterpret_cast<const unsigned long long*>(A), Aw, Sa, W64,
                       reinterpret_cast<const unsigned long long*>(B), Bw, Sb, (W64 + 3) / 4, R, Q,
                       reinterpret_cast<const long long*>(key_indices), scale_inv, R_total, out, out64);
    BSI_LAUNCH_CHECK("dot_weighted_kernel");
    return BSI_OK;
}

static int dot_weighted_impl(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B, int b_layout,
                             const float* Bw, int Sb, int64_t R, int64_t Q, const int64_t* key_indices, float scale_inv,
                             int64_t R_total, float* out, double* out64, void* stream) {
    BSI_REQUIRE(R >= 0 && Q >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(Sa >= 1 && Sa <= 64 && Sb >= 1 && Sb <= 64, "slice counts must be in [1, 64] (got %d, %d)", Sa, Sb);
    BSI_REQUIRE(R_total >= R, "R_total (%lld) < R (%lld)", static_cast<long long>(R_total), static_cast<long long>(R));
    BSI_REQUIRE(b_layout == BSI_LAYOUT_CANONICAL || b_layout == BSI_LAYOUT_TILED16,
                "the weighted dot reads key planes (canonical or tiled16), got layout %d", b_layout);
    BSI_REQUIRE((Q + 31) / 32 <= 65535, "too many query rows for one launch");
    if (R == 0 || Q == 0) return BSI_OK;
    BSI_REQUIRE(A && Aw && B && Bw && (out || out64), "null pointer");
    hipStream_t st = as_stream(stream);
    const bool tiled = b_layout == BSI_LAYOUT_TILED16;
    // 8 words of every slice per step while that fits 60 KiB of LDS, else 2
#define BSI_WEIGHTED_GO(WB, T) \
    launch_dot_weighted<WB, T>(A, Aw, Sa, W64, B, Bw, Sb, R, Q, key_indices, scale_inv, R_total, out, out64, st)
    if (Sa + Sb <= 28) return tiled ? BSI_WEIGHTED_GO(8, true) : BSI_WEIGHTED_GO(8, false);
    return tiled ? BSI_WEIGHTED_GO(2, true) : BSI_WEIGHTED_GO(2, false);
#undef BSI_WEIGHTED_GO
}

extern "C" int bsi_hip_dot_weighted(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B,
                                    int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                                    const int64_t* key_indices, float scale_inv, int64_t R_total, float* out,
                                    void* stream) {
    return dot_weighted_impl(A, Aw, Sa, W64, B, b_layout, Bw, Sb, R, Q, key_indices, scale_inv, R_total, out, nullptr, stream);
}

extern "C" int bsi_hip_dot_weighted_f64(const uint64_t* A, const float* Aw, int Sa, int W64, const uint64_t* B,
                                        int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                                        const int64_t* key_indices, int64_t R_total, double* out, void* stream) {
    return dot_weighted_impl(A, Aw, Sa, W64, B, b_layout, Bw, Sb, R, Q, key_indices, 1.0f, R_total, nullptr, out, stream);
}

extern "C" int bsi_hip_planes_to_int8_digits(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out,
                                             void* stream) {
    BSI_REQUIRE(rows >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(S >= 1 && S <= 64, "S must be in [1, 64] (got %d)", S);
    if (rows == 0) return BSI_OK;
    BSI_REQUIRE(words && out, "null pointer");
    const int chunks = (W64 + 3) / 4, ndig = (S + 6) / 7;
    const int64_t total = static_cast<int64_t>(ndig) * rows * chunks * 8;
    BSI_REQUIRE((total + 255) / 256 <= 0x7fffffffLL, "too large for one launch");
    hipLaunchKernelGGL(planes_to_digits_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       as_stream(stream), reinterpret_cast<const uint32_t*>(words), rows, S, W64, chunks, ndig,
                       reinterpret_cast<uint32_t*>(out));
    BSI_LAUNCH_CHECK("planes_to_digits_kernel");
    return BSI_OK;
}

extern "C" size_t bsi_hip_dot_digits_workspace_bytes(int64_t Q, int nq, int64_t R, int nk) {
    if (Q <= 0 || R <= 0 || nq <= 0 || nk <= 0) return 0;
    return static_cast<size_t>(nq) * static_cast<size_t>(Q) * static_cast<size_t>(nk) * static_cast<size_t>(R) * 4;
}

extern "C" int bsi_hip_dot_digits(const int8_t* A_digits, int nq, const float* Aw, int Sa, const int8_t* K_digits, int nk,
                                  int preshift, const float* Bw, int Sb, int W64, int64_t R, int64_t Q,
                                  const int64_t* key_indices, float scale_inv, int64_t R_total, const float* bias,
                                  float* out, void* workspace, size_t workspace_bytes, int k_tiled, void* stream) {
    BSI_REQUIRE(R >= 0 && Q >= 0 && W64 >= 1, "bad shape");
    BSI_REQUIRE(nq >= 1 && nq <= 10 && nk >= 1 && nk <= 10, "digit counts must be in [1, 10] (got %d, %d)", nq, nk);
    BSI_REQUIRE(k_tiled == 0 || nk == 1, "a tiled key image is a single digit");
    BSI_REQUIRE(Sa >= 1 && Sb >= 1 && preshift >= 0 && preshift <= 14, "bad slice counts or preshift");
    BSI_REQUIRE(R_total >= R, "R_total (%lld) < R (%lld)", static_cast<long long>(R_total), static_cast<long long>(R));
    // |sum| <= 256 chunks' worth of 128 * 128 per element: int32 holds D up to 2^17 elements
    BSI_REQUIRE(W64 <= 2048, "more than 2^17 elements per row could overflow the int32 sums (W64 = %d)", W64);
    if (R == 0 || Q == 0) return BSI_OK;
    BSI_REQUIRE(A_digits && Aw && K_digits && Bw && out, "null pointer");
    const int64_t Qd = static_cast<int64_t>(nq) * Q, Rd = static_cast<int64_t>(nk) * R;
    BSI_REQUIRE((Qd + 31) / 32 <= 65535, "too many query rows for one launch");
    hipStream_t st = as_stream(stream);
    const int chunks = (W64 + 3) / 4;
    const long long dig_stride = static_cast<long long>(Q) * chunks * 256;
    // One key digit: the query digits are put back together in the accumulator (shift by 7 between digits) and the
    // epilogue writes the floats -- if int32 holds sum_d |query value| |key digit|: query bits (Sa - 1 + preshift
    // when nq == 1, as the image is pre-shifted) + 7 key bits + log2(elements) <= 31, and the digit images lie
    // within reach of a 32-bit buffer offset.
    int log2_elems = 0;
    while ((1LL << log2_elems) < static_cast<long long>(chunks) * 256) ++log2_elems;
    const int qbits = (nq == 1) ? 7 : (Sa - 1);
    const int kbits = (preshift == 0 && Sb <= 7) ? (Sb - 1) : 7;
    const bool can_fold = nk == 1 && qbits + kbits + log2_elems <= 31 && static_cast<long long>(nq) * dig_stride < (1LL << 31);
    // folding runs nq times the chunks on the grid of Q rows; stacking runs the chunks once on the grid of nq Q rows
    // and then reads the int32 products back (about 3 us + 4 bytes per product at 4 TB/s; one cost unit of the tile
    // model is about 0.012 us per chunk)
    int64_t cost_fold = 0, cost_stack = 0;
    const int tile_fold = choose_i8_tile(R, Q, &cost_fold);
    const int tile_stack = choose_i8_tile(Rd, Qd, &cost_stack);
    // without the chain's epilogue to overlap, the 64-key tiles come out about 1.3 times their modelled cost
    const double us_fold = 0.012 * static_cast<double>(cost_fold) * chunks * nq * ((tile_fold == 64 || tile_fold == 6432) ? 1.3 : 1.0);
    const double us_stack = 0.012 * static_cast<double>(cost_stack) * chunks * ((tile_stack == 64 || tile_stack == 6432) ? 1.3 : 1.0) + 3.0 +
                            static_cast<double>(nq * nk + 1) * static_cast<double>(Q) * static_cast<double>(R) * 4.0 / 4.0e6;
    const int route = g_digits_route.load(std::memory_order_relaxed);
    const bool fold = route == 2 || (route == 0 && (nq == 1 || us_fold <= us_stack));
    if (can_fold && fold) {
        launch_mfma_i8(A_digits, Aw, Sa, K_digits, Bw, Sb, chunks, R, Q, preshift, scale_inv, R_total, out, nullptr, bias,
                       st, k_tiled, nq, dig_stride, reinterpret_cast<const long long*>(key_indices));
        BSI_LAUNCH_CHECK("dot_mfma_i8_kernel (int32 sum, digits recombined in the accumulator)");
        return BSI_OK;
    }
    const size_t need = bsi_hip_dot_digits_workspace_bytes(Q, nq, R, nk);
    BSI_REQUIRE(workspace != nullptr && workspace_bytes >= need, "workspace too small: %zu < %zu bytes", workspace_bytes,
                need);
    // else one int8 GEMM over the stacked digits: I[i Q + q, j R + r] = sum_d A_i[q, d] K_j[r, d]
    launch_mfma_i8(A_digits, Bw, 1, K_digits, Bw, 1, chunks, Rd, Qd, 0, 1.0f, Rd, nullptr,
                   reinterpret_cast<int32_t*>(workspace), nullptr, st, k_tiled, 1, 0, nullptr);
    BSI_LAUNCH_CHECK("dot_mfma_i8_kernel (int32 sum)");
    const int64_t total = Q * R;
    hipLaunchKernelGGL(digits_combine_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const int*>(workspace), nq, nk, Q, R, preshift, Aw, Sa, Bw, Sb,
                       reinterpret_cast<const long long*>(key_indices), scale_inv, R_total, bias, out);
    BSI_LAUNCH_CHECK("digits_combine_kernel");
    return BSI_OK;
}

extern "C" int bsi_hip_probe_l2_to_lds(const void* buf, size_t bytes, int loader_pattern, double* bytes_per_s, void* stream) {
    BSI_REQUIRE(buf && bytes_per_s, "null pointer");
    constexpr size_t kRegion = 256 * 1024;
    constexpr int kRegions = 8, kPasses = 64;
    BSI_REQUIRE(bytes >= kRegion * kRegions, "the probe streams %zu bytes of the buffer", kRegion * kRegions);
    hipStream_t st = as_stream(stream);
    int dev = 0, cus = 0;
    BSI_HIP_CHECK(hipGetDevice(&dev));
    BSI_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int lds = kProbeLdsWaves * kProbeLdsSlots * 1024;
    BSI_REQUIRE(loader_pattern >= 0 && loader_pattern <= 3, "loader_pattern must be 0, 1, 2 or 3");
    static LdsOptIn once0, once1, once2, once3;
    lds_opt_in(once0, reinterpret_cast<const void*>(&probe_l2_lds_kernel<8, 12, false>), lds);
    lds_opt_in(once1, reinterpret_cast<const void*>(&probe_l2_lds_kernel<4, 24, true>), lds);
    lds_opt_in(once2, reinterpret_cast<const void*>(&probe_l2_lds_kernel<4, 24, false>), lds);
    lds_opt_in(once3, reinterpret_cast<const void*>(&probe_l2_lds_kernel<8, 12, true>), lds);
    hipEvent_t e0, e1;
    BSI_HIP_CHECK(hipEventCreate(&e0));
    if (hipError_t ec = hipEventCreate(&e1); ec != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BSI_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(ec));
    }
    float best = 1e30f;
    hipError_t err = hipSuccess;
    for (int rep = 0; rep < 4 && err == hipSuccess; ++rep) {  // the first repetition also brings the regions into L2
        (void)hipEventRecord(e0, st);
        if (loader_pattern == 1)
            hipLaunchKernelGGL((probe_l2_lds_kernel<4, 24, true>), dim3(static_cast<unsigned>(cus)), dim3(4 * 64), lds, st,
                               static_cast<const unsigned char*>(buf), kRegion, kRegions, kPasses);
        else if (loader_pattern == 2)
            hipLaunchKernelGGL((probe_l2_lds_kernel<4, 24, false>), dim3(static_cast<unsigned>(cus)), dim3(4 * 64), lds, st,
                               static_cast<const unsigned char*>(buf), kRegion, kRegions, kPasses);
        else if (loader_pattern == 3)
            hipLaunchKernelGGL((probe_l2_lds_kernel<8, 12, true>), dim3(static_cast<unsigned>(cus)), dim3(8 * 64), lds, st,
                               static_cast<const unsigned char*>(buf), kRegion, kRegions, kPasses);
        else
            hipLaunchKernelGGL((probe_l2_lds_kernel<8, 12, false>), dim3(static_cast<unsigned>(cus)), dim3(8 * 64), lds, st,
                               static_cast<const unsigned char*>(buf), kRegion, kRegions, kPasses);
        (void)hipEventRecord(e1, st);
        err = hipEventSynchronize(e1);
        float ms = 0.0f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (rep > 0 && ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return fail(BSI_ERR_HIP, "probe timing failed: %s", hipGetErrorString(err));
    BSI_LAUNCH_CHECK("probe_l2_lds_kernel");
    *bytes_per_s = static_cast<double>(cus) * kRegion * kPasses / (best * 1e-3);
    return BSI_OK;
}

extern "C" int bsi_hip_timeline_read(unsigned long long* stamps_host, int workgroups) {
    BSI_REQUIRE(stamps_host && workgroups >= 1 && workgroups <= kTimelineWorkgroups, "workgroups must be 1 .. %d",
                kTimelineWorkgroups);
#ifdef BSI_TIMELINE
    BSI_HIP_CHECK(hipDeviceSynchronize());
    BSI_HIP_CHECK(hipMemcpyFromSymbol(stamps_host, HIP_SYMBOL(g_timeline), sizeof(unsigned long long) * 8 * workgroups));
    void* dev = nullptr;  // cleared, so that the next read shows which workgroups have run since
    BSI_HIP_CHECK(hipGetSymbolAddress(&dev, HIP_SYMBOL(g_timeline)));
    BSI_HIP_CHECK(hipMemset(dev, 0, sizeof(unsigned long long) * 8 * kTimelineWorkgroups));
    return BSI_OK;
#else
    return fail(BSI_ERR_INVALID, "this library was built without the timeline stamps (make TIMELINE=1 builds one with)");
#endif
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
