// Error plumbing, device info and the peak probes of libbsi_hip.so.
#include "bsi_common.h"

namespace bsi {

std::string& last_error_ref() {
    static thread_local std::string msg;
    return msg;
}

hipError_t& pending_config_error() {
    static thread_local hipError_t e = hipSuccess;
    return e;
}

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error_ref() = buf;
    return code;
}

typedef int v4i __attribute__((ext_vector_type(4)));

// 8 independent v_and + v_bcnt(accumulate) chains per lane
__global__ void probe_valu_kernel(unsigned* __restrict__ sink, unsigned seed, int iters) {
    unsigned a = seed ^ (threadIdx.x * 2654435761u), b = a * 40503u + 1u;
    unsigned c0 = 0, c1 = 0, c2 = 0, c3 = 0, c4 = 0, c5 = 0, c6 = 0, c7 = 0;
    for (int i = 0; i < iters; ++i) {
        c0 += __popc(a & (b + c4));
        c1 += __popc(b & (a + c5));
        c2 += __popc(a & (b ^ c6));
        c3 += __popc(b & (a ^ c7));
        c4 += __popc(a & (b | c0));
        c5 += __popc(b & (a | c1));
        c6 += __popc(a & (b - c2));
        c7 += __popc(b & (a - c3));
    }
    const unsigned s = c0 + c1 + c2 + c3 + c4 + c5 + c6 + c7;
    if (s == 0xFFFFFFFFu) sink[0] = s;
}

__global__ void probe_mfma_kernel(int* __restrict__ sink, int seed, int iters, int random_operands) {
    v4i a = {seed + (int)threadIdx.x, seed, 3, 5}, b = {7, seed, 11, (int)threadIdx.x};
    if (random_operands) {
        // pseudo-random bytes shaped like the dot's images: 6-bit values << 2 against 7-bit values << 1
        unsigned s = (threadIdx.x + 1u + blockIdx.x * 977u) * 2654435761u + static_cast<unsigned>(seed);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s = s * 1664525u + 1013904223u;
            a[j] = static_cast<int>((s >> 4) & 0xfcfcfcfcu);
            s = s * 1664525u + 1013904223u;
            b[j] = static_cast<int>((s >> 4) & 0xfefefefeu);
        }
    }
    v4i c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, a, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(b, b, c3, 0, 0, 0);
    }
    const int s = c0[0] + c1[1] + c2[2] + c3[3];
    if (s == 0x7FFFFFFF) sink[0] = s;
}

__global__ void probe_read_kernel(const uint4* __restrict__ buf, size_t n16, unsigned* __restrict__ sink) {
    unsigned acc = 0;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) {
        const uint4 v = buf[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x12345678u) sink[0] = acc;
}

template <typename F>
static int time_launch(hipStream_t st, int reps, float* ms_best, F&& launch) {
    hipEvent_t e0, e1;
    BSI_HIP_CHECK(hipEventCreate(&e0));
    if (hipError_t ec = hipEventCreate(&e1); ec != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(BSI_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(ec));
    }
    float best = 1e30f;
    hipError_t err = hipSuccess;
    for (int r = 0; r < reps && err == hipSuccess; ++r) {
        err = hipEventRecord(e0, st);
        if (err != hipSuccess) break;
        launch();
        err = hipEventRecord(e1, st);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        float ms = 0.0f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) return fail(BSI_ERR_HIP, "probe timing failed: %s", hipGetErrorString(err));
    *ms_best = best;
    return BSI_OK;
}

}  // namespace bsi

using namespace bsi;

extern "C" int bsi_hip_stream_capture_id(void* stream, unsigned long long* id) {
    BSI_REQUIRE(id != nullptr, "null pointer");
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    BSI_HIP_CHECK(hipStreamGetCaptureInfo(bsi::as_stream(stream), &status, &cid));
    *id = status == hipStreamCaptureStatusActive ? cid : 0;
    return BSI_OK;
}

extern "C" const char* bsi_hip_version(void) { return "bsi_hip gfx950 0.1 (" __DATE__ ")"; }

extern "C" const char* bsi_hip_last_error(void) { return last_error_ref().c_str(); }

extern "C" int bsi_hip_device_info(char* arch, int arch_len, int* cu_count, int* lds_bytes) {
    int dev = 0;
    BSI_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    BSI_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (arch && arch_len > 0) snprintf(arch, static_cast<size_t>(arch_len), "%s", prop.gcnArchName);
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (lds_bytes) *lds_bytes = static_cast<int>(prop.sharedMemPerBlockOptin ? prop.sharedMemPerBlockOptin : prop.sharedMemPerBlock);
    return BSI_OK;
}

extern "C" int bsi_hip_probe_valu_popcount(double* lane_ops_per_s, void* stream) {
    BSI_REQUIRE(lane_ops_per_s, "null pointer");
    hipStream_t st = as_stream(stream);
    unsigned* sink = nullptr;
    BSI_HIP_CHECK(hipMalloc(&sink, 64));
    const int iters = 4096, blocks = 256 * 16, threads = 256;
    float ms = 0.0f;
    int rc = time_launch(st, 5, &ms, [&] {
        hipLaunchKernelGGL(probe_valu_kernel, dim3(blocks), dim3(threads), 0, st, sink, 12345u, iters);
    });
    (void)hipFree(sink);
    if (rc) return rc;
    // per iteration: 8 v_and + 8 v_bcnt that the dot would issue (the feeding add/xor/or ops are not counted)
    *lane_ops_per_s = static_cast<double>(blocks) * threads * iters * 16.0 / (ms * 1e-3);
    return BSI_OK;
}

extern "C" int bsi_hip_probe_mfma_i8(double* ops_per_s, void* stream) {
    return bsi_hip_probe_mfma_i8_operands(0, ops_per_s, stream);
}

extern "C" int bsi_hip_probe_mfma_i8_operands(int random_operands, double* ops_per_s, void* stream) {
    BSI_REQUIRE(ops_per_s, "null pointer");
    BSI_REQUIRE(random_operands == 0 || random_operands == 1, "random_operands must be 0 or 1");
    hipStream_t st = as_stream(stream);
    int* sink = nullptr;
    BSI_HIP_CHECK(hipMalloc(&sink, 64));
    const int iters = 4096, blocks = 256 * 8, threads = 256;
    float ms = 0.0f;
    int rc = time_launch(st, 5, &ms, [&] {
        hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(threads), 0, st, sink, 3, iters, random_operands);
    });
    (void)hipFree(sink);
    if (rc) return rc;
    const double waves = static_cast<double>(blocks) * (threads / 64);
    *ops_per_s = waves * iters * 4.0 * (2.0 * 16 * 16 * 64) / (ms * 1e-3);
    return BSI_OK;
}

extern "C" int bsi_hip_probe_stream_read(const void* buf, size_t bytes, double* bytes_per_s, void* stream) {
    BSI_REQUIRE(buf && bytes_per_s && bytes >= 16, "bad arguments");
    hipStream_t st = as_stream(stream);
    unsigned* sink = nullptr;
    BSI_HIP_CHECK(hipMalloc(&sink, 64));
    const size_t n16 = bytes / 16;
    float ms = 0.0f;
    int rc = time_launch(st, 5, &ms, [&] {
        hipLaunchKernelGGL(probe_read_kernel, dim3(256 * 16), dim3(256), 0, st, static_cast<const uint4*>(buf), n16, sink);
    });
    (void)hipFree(sink);
    if (rc) return rc;
    *bytes_per_s = static_cast<double>(n16) * 16.0 / (ms * 1e-3);
    return BSI_OK;
}
