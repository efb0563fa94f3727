// Shared host/device helpers of libbsi_hip.so (gfx950 only, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../include/bsi_hip.h"

#define BSI_WAVE 64
#define BSI_CHUNK_ELEMS 256
#define BSI_CHUNK_WORDS 4

namespace bsi {

// ---- error plumbing: every extern "C" entry returns a code and leaves a message here ----
std::string& last_error_ref();
int fail(int code, const char* fmt, ...);

#define BSI_REQUIRE(cond, ...)                                   \
    do {                                                         \
        if (!(cond)) return ::bsi::fail(BSI_ERR_INVALID, __VA_ARGS__); \
    } while (0)

#define BSI_HIP_CHECK(expr)                                                                          \
    do {                                                                                             \
        hipError_t _e = (expr);                                                                      \
        if (_e != hipSuccess)                                                                        \
            return ::bsi::fail(BSI_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
    } while (0)

// A kernel's opt-in to more than 64 KiB of dynamic LDS, done once per kernel and device.  Any number of threads may
// launch the kernel at the same time (the worst case is that two of them set the attribute); a failure is kept for
// the launch check that follows, which reports it instead of the launch error it would cause.
struct LdsOptIn {
    std::atomic<uint64_t> devices{0};  // bit d: done on device d (devices past 63 set it on every launch)
};
hipError_t& pending_config_error();
inline void lds_opt_in(LdsOptIn& once, const void* kernel, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t{1} << dev) : 0;
    if (e == hipSuccess && bit != 0 && (once.devices.load(std::memory_order_acquire) & bit) != 0) return;
    if (e == hipSuccess) e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) once.devices.fetch_or(bit, std::memory_order_release);
    else pending_config_error() = e;
}

// After a kernel launch: surface launch-configuration errors immediately.
#define BSI_LAUNCH_CHECK(name)                                                                       \
    do {                                                                                             \
        hipError_t _c = ::bsi::pending_config_error();                                               \
        ::bsi::pending_config_error() = hipSuccess;                                                  \
        hipError_t _e = hipGetLastError();                                                           \
        if (_c != hipSuccess)                                                                        \
            return ::bsi::fail(BSI_ERR_HIP, "LDS opt-in of %s failed: %s", name, hipGetErrorString(_c)); \
        if (_e != hipSuccess)                                                                        \
            return ::bsi::fail(BSI_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(_e)); \
    } while (0)

static inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---- device helpers ----

template <typename T>
__device__ __forceinline__ float load_as_float(const T* p, int64_t i);
template <>
__device__ __forceinline__ float load_as_float<float>(const float* p, int64_t i) { return p[i]; }
template <>
__device__ __forceinline__ float load_as_float<__half>(const __half* p, int64_t i) { return __half2float(p[i]); }
template <>
__device__ __forceinline__ float load_as_float<__hip_bfloat16>(const __hip_bfloat16* p, int64_t i) {
    // bf16 is the top half of an fp32
    const uint16_t raw = reinterpret_cast<const uint16_t*>(p)[i];
    return __uint_as_float(static_cast<uint32_t>(raw) << 16);
}

// round half away from zero of x (x = (double)(float)v * 10^dec); the multiply is done by the
// caller with __dmul_rn so that it is never contracted with the + 0.5
// Values the conversion cannot hold are given what the reference's own conversion gives them on its hardware (the C++
// cast is undefined there; cvt.rzi.s64.f64 saturates and turns a NaN into -2^63): magnitudes of 2^63 and more,
// the infinities included, become +-(2^63 - 1), a NaN becomes -2^63.
__device__ __forceinline__ long long magnitude_to_ll(double y) {  // y >= 0
    return y >= 9223372036854775808.0 ? 9223372036854775807LL : static_cast<long long>(y);
}
__device__ __forceinline__ long long round_half_away(double x) {
    if (x != x) return static_cast<long long>(0x8000000000000000ULL);
    if (x >= 0.0) return magnitude_to_ll(floor(__dadd_rn(x, 0.5)));
    return -magnitude_to_ll(floor(__dadd_rn(-x, 0.5)));
}

__device__ __forceinline__ long long round_scaled(float f, double dec_scale) {
    return round_half_away(__dmul_rn(static_cast<double>(f), dec_scale));
}

__device__ __forceinline__ unsigned long long uabs_ll(long long v) {
    return v >= 0 ? static_cast<unsigned long long>(v) : 0ULL - static_cast<unsigned long long>(v);  // -2^63 -> 2^63
}

// bits needed for max_abs minus the magnitude bits available; optional outlier clipping
__device__ __forceinline__ int compute_shift(unsigned long long max_abs, double sum_abs, int count, int fixed_bits,
                                             float clip_k) {
    if (fixed_bits <= 0) return 0;
    int bits = 0;
    if (clip_k > 0.0f && count > 0) {
        double effective = static_cast<double>(max_abs);
        const double mean_abs = sum_abs / static_cast<double>(count);
        const double clip_max = mean_abs * static_cast<double>(clip_k);
        if (clip_max < effective) effective = clip_max;
        if (effective > 0.0) {
            int e = 0;
            (void)frexp(effective, &e);
            bits = e;
        }
    } else {
        bits = (max_abs > 0ULL) ? (64 - __clzll(static_cast<long long>(max_abs))) : 0;
    }
    int shift = bits - (fixed_bits - 1);
    if (shift < 0) shift = 0;
    if (shift > 62) shift = 62;
    return shift;
}

__device__ __forceinline__ long long shift_clamp(long long v, int shift, long long qmin, long long qmax) {
    const unsigned long long av = uabs_ll(v);
    const unsigned long long round_add = (shift > 0) ? (1ULL << (shift - 1)) : 0ULL;
    const unsigned long long q = (av + round_add) >> shift;
    long long out = (v < 0) ? -static_cast<long long>(q) : static_cast<long long>(q);
    if (out < qmin) out = qmin;
    if (out > qmax) out = qmax;
    return out;
}

// |round half away from zero of x * scale| for an integer scale of at most 127 and |x| < 2^23, in a dozen 32-bit
// integer instructions.  With |x| = m * 2^(ex - 150) (24-bit m, hidden bit included) the product M = m * scale is
// exact in 31 bits, and the float64 route (exact product, + 0.5, floor) equals (M + half) >> s with s = 150 - ex;
// s >= 32 gives 0 (denormals land there too, so their missing hidden bit does not matter).  Checked against the
// float64 route on every float.  |x| >= 2^23, infinities and NaNs set `big` and are left to the 64-bit routine.
__device__ __forceinline__ unsigned scaled_magnitude_u32(float x, unsigned scale, bool& big) {
    const unsigned bits = __float_as_uint(x) & 0x7fffffffu;
    const unsigned ex = bits >> 23;
    const unsigned M = __umul24((bits & 0x7fffffu) | 0x800000u, scale);
    big = big || ex >= 150u;
    const unsigned s = 150u - ex;
    const unsigned r = (M + (1u << ((s - 1u) & 31u))) >> (s & 31u);
    return (s >= 32u) ? 0u : r;
}

// Largest v of the wave in every lane's return value (all 64 lanes active): four DPP steps inside each row of 16
// lanes, then the four rows through scalar registers.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
#define BSI_DPP_MAX(ctrl)                                                                                      \
    {                                                                                                          \
        const unsigned o = static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), ctrl, 0xF, 0xF, false)); \
        v = o > v ? o : v;                                                                                     \
    }
    BSI_DPP_MAX(0xB1)   // quad_perm [1,0,3,2]
    BSI_DPP_MAX(0x4E)   // quad_perm [2,3,0,1]
    BSI_DPP_MAX(0x141)  // row_half_mirror
    BSI_DPP_MAX(0x140)  // row_mirror
#undef BSI_DPP_MAX
    const unsigned a = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(v), 0));
    const unsigned b = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(v), 16));
    const unsigned c = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(v), 32));
    const unsigned d = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(v), 48));
    const unsigned ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

extern std::atomic<int> g_build_items;  // BSI_OPT_BUILD_ITEMS (bsi_build.hip)

// 10^dec as an integer when scaled_magnitude_u32 can take it (at most 127), else 0: float64 arithmetic then.
static inline unsigned integer_decimal_scale(double dec_scale) {
    return (dec_scale >= 1.0 && dec_scale <= 127.0 && dec_scale == static_cast<double>(static_cast<unsigned>(dec_scale)))
               ? static_cast<unsigned>(dec_scale) : 0u;
}

// Position of element e (0..255) of a chunk inside the chunk's 256 int8 bytes in the MFMA core's
// order: element 32w + 8m + t sits at byte 32w + 4t + m (see planes_to_int8_kernel in bsi_dot_layouts.hip).
__device__ __forceinline__ int mfma_byte_pos(int e) {
    const int w = e >> 5, r = e & 31;
    const int m = r >> 3, t = r & 7;
    return (w << 5) + (t << 2) + m;
}

// wave64 butterfly reductions (every lane ends with the result)
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(v, off, BSI_WAVE);
        if (o > v) v = o;
    }
    return v;
}
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, BSI_WAVE);
    return v;
}
__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, BSI_WAVE);
    return v;
}

// One wave expands one EWAH stream (in[0 .. in_len), [marker][literals...] with marker = run_bit | run_len << 1 |
// literal_count << 33) into dst[0 .. wpad): W decoded words, zeros after them.  Bounds as the reference decoder's
// (bsi_ops/csrc/cuda/bsi_cuda_kernels_ewah.cuh:5-33): output clipped at W words, input at in_len, the rest zero.
// dst may be global memory or LDS.  The markers form a chain; the wave follows it through a window of 64 stream
// words held one per lane, so stepping to the next marker is a lane broadcast, not a dependent memory load.
// Call it with all 64 lanes active and wave-uniform arguments.
__device__ __forceinline__ void ewah_expand_wave(const unsigned long long* __restrict__ in, int in_len, int W,
                                                 unsigned long long* __restrict__ dst, int wpad, int lane) {
    int idx = 0, o = 0, win_at = 0;
    unsigned long long win = (lane < in_len) ? in[lane] : 0ULL;
    while (idx < in_len && o < W) {
        if (idx - win_at >= BSI_WAVE) {
            win_at = idx;
            win = (win_at + lane < in_len) ? in[win_at + lane] : 0ULL;
        }
        const int at = __builtin_amdgcn_readfirstlane(idx - win_at);
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<unsigned>(win)), at));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<unsigned>(win >> 32)), at));
        ++idx;
        const unsigned long long run_val = (lo & 1u) ? ~0ULL : 0ULL;
        const unsigned run_len = (lo >> 1) | (hi << 31);   // bits 1..32 of the marker
        const unsigned lit = hi >> 1;                      // bits 33..63
        const int n_run = static_cast<int>(run_len < static_cast<unsigned>(W - o) ? run_len : static_cast<unsigned>(W - o));
        for (int k = lane; k < n_run; k += BSI_WAVE) dst[o + k] = run_val;
        o += n_run;
        int n_lit = static_cast<int>(lit < static_cast<unsigned>(W - o) ? lit : static_cast<unsigned>(W - o));
        if (n_lit > in_len - idx) n_lit = in_len - idx;
        for (int k = lane; k < n_lit; k += BSI_WAVE) dst[o + k] = in[idx + k];
        o += n_lit;
        idx += n_lit;
        if (static_cast<unsigned>(n_lit) < lit) break;     // clipped: the reference loop stops here too
    }
    for (int k = o + lane; k < wpad; k += BSI_WAVE) dst[k] = 0ULL;
}

}  // namespace bsi
