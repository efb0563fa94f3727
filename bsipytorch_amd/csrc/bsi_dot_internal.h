// Host-side interface between the translation units of the dot (all in namespace bsi): the launchers each kernel
// family exports, and the process-wide options and per-thread launch state that the int8-image launchers read.
#pragma once
#include "bsi_common.h"

#include <atomic>

namespace bsi {

constexpr int kStreamMaxQ = 32;  // the few-rows kernels take up to this many query rows; above, the tiled kernels

// ---- bsi_dot_layouts.hip: canonical planes -> int8 image (value << (8 - S)), row-major or in 64-row tiles
int launch_planes_to_int8(const uint64_t* words, int64_t rows, int S, int W64, int8_t* out, hipStream_t st, int tiled = 0);

// ---- bsi_dot_planes.hip: the matrix-core kernels that read key PLANES (canonical or tiled16) and recombine them in
// the workgroup; returns the name of the kernel it launched, for the launch check
const char* launch_mfma_planes(bool tiled, const int8_t* A8, const float* qscale, int stride, const uint64_t* B,
                               const float* Bw, int Sb, int W64, int chunks, int64_t R, int64_t Q, int down_shift,
                               float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, hipStream_t st);

// ---- bsi_dot_i8.hip: the kernels on the int8 image of the keys
extern std::atomic<int> g_i8_tile;        // 0 = by grid size; 128, 1284, 12864, 64 or 6432 force a tile (tuning and tests)
extern std::atomic<int> g_digits_route;   // bsi_hip_dot_digits: 0 = by cost, 1 = stacked digits + combine pass, 2 = in-accumulator
extern std::atomic<int> g_output_stores;  // 0 = by entry point, 1 = always plain, 2 = always nontemporal
// Set by bsi_hip_dot_bias_warm around its launch: the region the int8-image kernel should touch for the next dot.
extern thread_local const void* g_warm_ptr;
extern thread_local size_t g_warm_bytes;
// Set by the entry points of a linear layer around their launch: the next kernel of the model reads that output.
extern thread_local int t_layer_output;
int choose_i8_tile(int64_t R, int64_t Q, int64_t* cost_out = nullptr);
// D-split of the chain-mode int8-image dot (bsi_hip_dot_attach_split_scratch): the calling thread's scratch region
// (counters of kSplitCounterBytes, then the segments' partial sums) and the device it lies on; the option
// BSI_OPT_I8_SPLIT; the choice itself (tile 128 / 12864 and *segments, or 0).
constexpr size_t kSplitCounterBytes = BSI_SPLIT_COUNTER_BYTES;
constexpr int64_t kSplitMaxTiles = BSI_SPLIT_MAX_TILES;  // then two running totals (BSI_SPLIT_STAT_*)
static_assert((kSplitMaxTiles + 2) * sizeof(unsigned) <= kSplitCounterBytes, "counters and totals fit their area");
extern thread_local unsigned char* t_split_scratch;
extern thread_local size_t t_split_bytes;
extern thread_local int t_split_device;
extern std::atomic<int> g_i8_split;
int choose_i8_split(int64_t R, int64_t Q, int chunks, int* segments);
void launch_mfma_i8(const int8_t* A8, const float* qscale, int stride, const int8_t* K8, const float* Bw, int Sb,
                    int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total, float* out,
                    int32_t* chunk_ints, const float* bias, hipStream_t st,
                    int key_tiled = 0, int ndig = 0, long long dig_stride = 0, const long long* key_indices = nullptr);

// ---- bsi_dot_few_rows.hip: the plane-streaming kernel for up to kStreamMaxQ query rows on 6-plane tiled keys
// (query tiles and key tiles per workgroup chosen from Q and R)
void launch_mfma_stream_by_shape(const int8_t* A8, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                                 int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                                 float* out, int32_t* chunk_ints, const float* bias, hipStream_t st);

// ---- bsi_dot_valu.hip: the popcount kernels
void launch_valu76(bool tiled, const uint64_t* A, const float* qscale, int stride, const uint64_t* B, const float* Bw,
                   int W64, int chunks, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out,
                   int32_t* chunk_ints, hipStream_t st);
void launch_valu_generic(const uint64_t* A, const float* qscale, int stride, int Sa, const uint64_t* B, const float* Bw,
                         int Sb, int W64, int chunks, int64_t R, int64_t Q, float scale_inv, int64_t R_total, float* out,
                         int32_t* chunk_ints, int tiled, hipStream_t st);
void launch_add_bias(float* out, const float* bias, int64_t Q, int64_t R, int64_t R_total, hipStream_t st);

// ---- bsi_dot.hip: validation, kernel selection and launch of the fixed-bit dot, bias included
int dot_with_bias(const uint64_t* A, const int8_t* A_ints8, const float* A_chunk_scales, int A_scale_stride, int Sa,
                  int W64, const uint64_t* B, int b_layout, const float* Bw, int Sb, int64_t R, int64_t Q,
                  float scale_inv, int64_t R_total, float* out, int32_t* chunk_ints, int core, void* workspace,
                  size_t workspace_bytes, void* stream, const float* bias);

}  // namespace bsi
