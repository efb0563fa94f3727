// The popcount kernels of the dot: the 7 x 6 bit kernel on the vector ALU, the kernel for any slice counts, the
// weighted-slice kernel of decimal-mode operands, and the bias pass for kernels that do not fuse it.
#include "bsi_dot_device.h"
#include "bsi_dot_internal.h"

namespace bsi {

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

void launch_valu76(bool tiled, const uint64_t* A, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                   int W64, int chunks, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out,
                   int32_t* chunk_ints, hipStream_t st) {
    if (tiled) launch_valu76<true>(A, qscale, stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
    else launch_valu76<false>(A, qscale, stride, B, Bw, W64, chunks, R, Q, scale_inv, R_total, out, chunk_ints, st);
}

void launch_valu_generic(const uint64_t* A, const float* qscale, int stride, int Sa, const uint64_t* B, const float* Bw,
                         int Sb, int W64, int chunks, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out,
                         int32_t* chunk_ints, int tiled, hipStream_t st) {
    const int64_t total = Q * R;
    hipLaunchKernelGGL(dot_valu_generic_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st,
                       reinterpret_cast<const unsigned long long*>(A), qscale, stride, Sa,
                       reinterpret_cast<const unsigned long long*>(B), Bw, Sb, W64, chunks, R, Q, scale_inv, R_total,
                       out, chunk_ints, tiled);
}

void launch_add_bias(float* out, const float* bias, int64_t Q, int64_t R, int64_t R_total, hipStream_t st) {
    const int64_t total = Q * R;
    hipLaunchKernelGGL(add_bias_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, st, out, bias, Q, R,
                       R_total);
}

}  // namespace bsi

using namespace bsi;

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

extern "C" int bsi_hip_add_bias(float* out, const float* bias, int64_t Q, int64_t R, int64_t R_total, void* stream) {
    BSI_REQUIRE(Q >= 0 && R >= 0 && R_total >= R, "bad shape");
    if (Q == 0 || R == 0) return BSI_OK;
    BSI_REQUIRE(out && bias, "null pointer");
    launch_add_bias(out, bias, Q, R, R_total, as_stream(stream));
    BSI_LAUNCH_CHECK("add_bias_kernel");
    return BSI_OK;
}
