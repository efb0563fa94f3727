// A model of the int8-image dot kernel's chunk loop, without the library: what the matrix pipes, the LDS operand reads,
// the stage loads and the workgroup barrier cost each other on one CU.
//
// One workgroup per CU (forced by its LDS size).  Eight "MFMA waves" run the kernel's k-step over and over on static
// LDS contents -- 8 v_mfma_i32_16x16x64_i8, 8 chain elements (one cvt + one fma), kReads 16-byte operand reads per lane
// that feed the next k-step's operands -- and four "loader waves" stream an L2-resident region into another part of
// LDS with LDS-direct 16-byte buffer loads, up to kFlight + 8 loads in flight per wave.  Optionally all twelve waves meet
// at a workgroup barrier once per half-chunk (two k-steps, eight loads per loader wave: a 32 KiB stage per CU), as in the
// kernel.  Every wave reads the shader cycle counter and the 100 MHz wall clock around its loop; printed: cycles per
// MFMA and SIMD (16 = the pipe's rate), cycles and microseconds per 32 KiB stage (512 cycles = 64 bytes per cycle), and
// the shader clock the two counters imply.  Machines whose shader clock settles lower under this load show fewer cycles
// per stage for the same time: part of the stage's way is clocked by the memory side, not by the CU.
//
//   make -C bsipytorch_amd/csrc ../benchmarks/loop_model && bsipytorch_amd/benchmarks/loop_model
#include <hip/hip_runtime.h>

#include <cstdio>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

#define CHECK(x)                                                                          \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)

constexpr int kLdsBytes = 136 * 1024;   // 32 KiB of operands + a 96 KiB ring for the loaders + slack: one workgroup per CU
constexpr size_t kRegion = 256 * 1024;  // what a workgroup's loaders stream, over and over (8 regions: L2-resident)

template <bool kLoaders, bool kBarrier, int kReads, int kPrio, bool kMfma, int kFlight>
__global__ __launch_bounds__(768) void loop_model(int* sink, int ksteps, unsigned long long* cycles,
                                                  const unsigned char* buf) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int i = threadIdx.x; i < 32768 / 4; i += 768) reinterpret_cast<int*>(lds)[i] = (i * 2654435761u) & 0x3f3f3f3f;
    __syncthreads();
    if (wave >= 8) {  // loader waves: 8 loads of 1 KiB per half-chunk each
        if (!kLoaders && !kBarrier) return;
        const rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(buf) + (blockIdx.x % 8) * kRegion, 0,
                                                           static_cast<int>(kRegion), 0x00020000);
        unsigned off = 0;
        if (kPrio) __builtin_amdgcn_s_setprio(kPrio);
        const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
        for (int h = 0; h < ksteps / 2; ++h) {
            if (kLoaders) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int block = ((h & 3) * 32 + (wave - 8) * 8 + i) % 96;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void*)(lds + 32768 + block * 1024),
                                                             16, lane * 16, off, 0, 0);
                    off += 1024;
                    if (off + 1024 > kRegion) off = 0;
                }
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kFlight) : "memory");
            }
            if (kBarrier) asm volatile("s_barrier" ::: "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
        if (lane == 0) {
            atomicMax(&cycles[1], t1 - t0);
            atomicMax(&cycles[3], w1 - w0);
        }
        return;
    }
    // MFMA waves: 64 keys x 32 queries each, the kernel's XOR-swizzled 128-byte rows
    const int ln = lane & 15, lg = lane >> 4;
    const unsigned char* base = lds + ((wave & 1) * 64 + ln) * 128 + ((lg ^ (ln >> 1)) & 7) * 16;
    v4i ka[2][4], qb[2][2], acc[4][2], prev[4][2];
    float accf[4][2][4];
    for (int a = 0; a < 4; ++a) {
        ka[0][a] = ka[1][a] = *reinterpret_cast<const v4i*>(base + a * 2048);
        for (int b = 0; b < 2; ++b) {
            acc[a][b] = (v4i){0, 0, 0, 0};
            prev[a][b] = (v4i){a, b, 3, 4};
            for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.f;
        }
    }
    for (int b = 0; b < 2; ++b) qb[0][b] = qb[1][b] = *reinterpret_cast<const v4i*>(base + 16384 + b * 2048);
    const float sc = 1.0f + (lane & 3);
    const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int ks = 0; ks < ksteps; ks += 2) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            v4i(&kc)[4] = ka[half];
            v4i(&qc)[2] = qb[half];
            v4i(&kn)[4] = ka[half ^ 1];
            v4i(&qn)[2] = qb[half ^ 1];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int a = t >> 1, b = t & 1;
                if (kMfma) acc[a][b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(kc[a], qc[b], acc[a][b], 0, 0, 0);
                else __builtin_amdgcn_s_sleep(1);
                const int e = t & 3, ta = (t >> 2) * 2, tb = half;
                if (kMfma) accf[ta][tb][e] = fmaf(static_cast<float>(prev[ta][tb][e]), sc, accf[ta][tb][e]);
                if (t < kReads) {
                    const v4i r = *reinterpret_cast<const v4i*>(base + (t < 4 ? t * 2048 : 16384 + (t - 4) * 2048));
                    if (t < 4) kn[t] = r;
                    else qn[t - 4] = r;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kBarrier && half == 0) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    int sum = 0;
    float fs = 0;
    for (int a = 0; a < 4; ++a)
        for (int b = 0; b < 2; ++b) {
            sum += acc[a][b][0] + acc[a][b][3];
            for (int e = 0; e < 4; ++e) fs += accf[a][b][e];
        }
    if (sum == 0x7FFFFFFF || fs == 1.2345f) sink[0] = sum;  // never: keeps the results alive
    if (lane == 0) {
        atomicMax(&cycles[0], t1 - t0);
        atomicMax(&cycles[2], w1 - w0);
    }
}

template <bool kLoaders, bool kBarrier, int kReads = 6, int kPrio = 0, bool kMfma = true, int kFlight = 16>
static int run(int* sink, unsigned long long* cycles, const unsigned char* buf, int cus, const char* name) {
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&loop_model<kLoaders, kBarrier, kReads, kPrio, kMfma, kFlight>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
    const int ksteps = 4096;
    unsigned long long h[4] = {0, 0, 0, 0};
    for (int rep = 0; rep < 2; ++rep) {  // the first repetition brings the regions into L2
        CHECK(hipMemset(cycles, 0, 32));
        hipLaunchKernelGGL((loop_model<kLoaders, kBarrier, kReads, kPrio, kMfma, kFlight>), dim3(cus), dim3(768), kLdsBytes, 0,
                           sink, ksteps, cycles, buf);
        CHECK(hipDeviceSynchronize());
        CHECK(hipMemcpy(h, cycles, 32, hipMemcpyDeviceToHost));
    }
    printf("%-58s", name);
    if (kMfma) printf(" %5.1f cycles per MFMA and SIMD", static_cast<double>(h[0]) / (ksteps * 8.0 * 2));
    else printf(" %30s", "");
    if (kLoaders) printf("  %4.0f cycles = %.3f us per 32 KiB stage (%.1f B/clk/CU)", static_cast<double>(h[1]) / (ksteps / 2),
                         static_cast<double>(h[3]) / 100.0 / (ksteps / 2), 32768.0 * (ksteps / 2) / static_cast<double>(h[1]));
    const double ghz = kMfma ? static_cast<double>(h[0]) / (static_cast<double>(h[2]) * 10.0)
                             : static_cast<double>(h[1]) / (static_cast<double>(h[3]) * 10.0);
    printf("  [shader clock %.2f GHz]\n", ghz);
    return 0;
}

int main() {
    int* sink;
    unsigned long long* cycles;
    unsigned char* buf;
    int cus = 0;
    CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    CHECK(hipMalloc(&sink, 64));
    CHECK(hipMalloc(&cycles, 32));
    CHECK(hipMalloc(&buf, 8 * kRegion));
    CHECK(hipMemset(buf, 1, 8 * kRegion));
    int rc = 0;
    rc |= run<false, false>(sink, cycles, buf, cus, "MFMA waves alone");
    rc |= run<true, false>(sink, cycles, buf, cus, "+ loader waves streaming, no barrier");
    rc |= run<false, true>(sink, cycles, buf, cus, "+ a barrier per half-chunk, no loads");
    rc |= run<true, true>(sink, cycles, buf, cus, "+ loader waves and the barrier per half-chunk");
    rc |= run<true, false, 4>(sink, cycles, buf, cus, "loaders, no barrier, 4 operand reads per k-step");
    rc |= run<true, false, 0>(sink, cycles, buf, cus, "loaders, no barrier, no operand reads");
    rc |= run<true, false, 0, 0, false>(sink, cycles, buf, cus, "loaders next to sleeping waves");
    rc |= run<true, false, 6, 0, true, 40>(sink, cycles, buf, cus, "loaders with up to 48 loads in flight each, no barrier");
    rc |= run<true, false, 6, 3>(sink, cycles, buf, cus, "loader waves at s_setprio 3, no barrier");
    rc |= run<true, true, 6, 3>(sink, cycles, buf, cus, "loader waves at s_setprio 3, barrier per half-chunk");
    return rc;
}
