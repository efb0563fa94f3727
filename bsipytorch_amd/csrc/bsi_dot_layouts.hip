// Operand layouts of the dot: canonical key planes -> tiled16 planes, planes -> int8 images (fixed-bit values
// shifted to the top of the byte, or 7-bit digits of wider values).  See bsi_dot.hip for the dot itself.
#include "bsi_dot_device.h"
#include "bsi_dot_internal.h"

namespace bsi {

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

__global__ void zero_uint4_kernel(uint4* __restrict__ p, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = make_uint4(0u, 0u, 0u, 0u);
}

int launch_planes_to_int8(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out, hipStream_t st,
                                 int tiled) {
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
