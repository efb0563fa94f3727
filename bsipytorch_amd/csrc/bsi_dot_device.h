// Device-side helpers shared by the dot kernels' translation units: bit transposes between planes and int8 bytes,
// buffer descriptors and LDS-direct loads, the workgroup barrier that waits for LDS traffic only, the epilogue
// operands and the fp32 chain over chunks.
#pragma once
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

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() would also
// drain the vector-memory counter, i.e. stall every iteration on the producers' prefetch loads.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define BSI_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define BSI_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

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

}  // namespace bsi
