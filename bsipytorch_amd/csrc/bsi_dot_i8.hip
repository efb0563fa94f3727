// The matrix-core dot on the cached int8 image of the keys (the compute-bound calls), its probe of the L2 -> LDS
// path, the timeline stamps, and the decimal-mode dot on int8 digit images that runs on the same kernel.
#include "bsi_dot_device.h"
#include "bsi_dot_internal.h"

namespace bsi {

// process-wide options set through bsi_hip_set_option (meanings beside their declarations in bsi_dot_internal.h)
std::atomic<int> g_i8_tile{0};
std::atomic<int> g_digits_route{0};

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
    // D-split launches: one flag word per MFMA wave (a prefix of its chain came near the exactness limit), then the
    // workgroup's decision (kSplitLeave / kSplitCombine / kSplitRedo)
    static constexpr int kSplitFlagBytes = 64;
    static constexpr int kLdsSplit = kLds + kSplitFlagBytes;
    static_assert(kConsumers < 15, "flag words of the MFMA waves, then the decision word");
};
constexpr int kSplitLeave = 0, kSplitCombine = 1, kSplitRedo = 2;

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
__device__ unsigned long long g_timeline_cycles[kTimelineWorkgroups * 8];  // the shader-clock counter at the same points
#define BSI_STAMP(slot)                                                                    \
    {                                                                                      \
        const unsigned wg_ = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x; \
        if (lane == 0 && wg_ < kTimelineWorkgroups) {                                      \
            g_timeline[wg_ * 8 + (slot)] = wall_clock64();                                 \
            g_timeline_cycles[wg_ * 8 + (slot)] = clock64();                               \
        }                                                                                  \
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
                                               const float* __restrict__ Bw, int Sb, int chunks, int first_chunk,
                                               int halves, int64_t R, int64_t Q, int64_t r0, int64_t q0, size_t rowbytes,
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
    // the first stage.  No row is clamped: the offset of a lane's ROW (group and row inside it) travels in the
    // per-lane offset of the buffer load, which the hardware compares with the descriptor's size, so a row past its
    // operand's end reads nothing; whatever such a row or query leaves in LDS only reaches outputs past R or Q, which
    // are never stored.  The wave-uniform offset of the load carries the position INSIDE the row only (the
    // half-chunk), so nothing depends on whether that offset takes part in the range check.
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
    // the offset of its group.
    const uint32_t lr = static_cast<uint32_t>(lane) >> 3, lc = static_cast<uint32_t>(lane) & 7;
    uint32_t voff[NI];
    bool is_key[NI];  // known at compile time once the loops are unrolled
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        is_key[i] = i < KG / L;
        const int gg = is_key[i] ? lw + L * i : lw + L * (i - KG / L);  // group of its operand
        const uint32_t col = (lc ^ (static_cast<uint32_t>(gg & 1) * 4 + (lr >> 1))) * 16;
        const bool tiled = is_key[i] && key_tiled;
        voff[i] = (tiled ? lr * 128 : lr * rowbytes32) + col +
                  (tiled ? static_cast<uint32_t>(gg >> 3) * kblock + static_cast<uint32_t>(gg & 7) * 1024
                         : static_cast<uint32_t>(gg) * 8 * rowbytes32);
    }
    const uint32_t kstep_bytes = key_tiled ? 8192u : 128u;  // from one half-chunk of a key row to the next
    // scales: loader wave lw fetches the 64 queries of group lw % (TN / 64) (waves fetching the same group
    // write their own regions, so that every loader wave has the same number of loads in flight)
    const bsi_rsrc rs = make_rsrc(qscale + q0 * qscale_stride, static_cast<size_t>(Q - q0) * qscale_stride * 4);
    const uint32_t soff = static_cast<uint32_t>((lw % (TN >= 64 ? TN / 64 : 1)) * 64 + lane) * static_cast<uint32_t>(qscale_stride) * 4;
    const int sstep = (qscale_stride == 1) ? 0 : 4;
    // issue() is called for h = 0, 1, 2, ... in order, h counted from the first half of chunk first_chunk (the
    // workgroup's share of the row in a D-split launch, else 0); in the sum mode (next_c, next_dg) follow the chunk
    // and the digit (counted from the top one) of the half-chunk to come
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
            so_q = static_cast<uint32_t>(hc + 2 * first_chunk) * 128;
            so_k = static_cast<uint32_t>(hc + 2 * first_chunk) * kstep_bytes;
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int g = i < KG / L ? lw + L * i : KG + lw + L * (i - KG / L);  // group of the stage
            load16_to_lds(is_key[i] ? rk : rq, voff[i], is_key[i] ? so_k : so_q,
                          lds + (h & 3) * C::kStage + g * 1024);
        }
        if (!kSum && (h & 1)) {  // with the second half of chunk c = h / 2: its scales
            const int c = hc >> 1;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs, BSI_LDS_PTR(scale_lds + ((c & 3) * C::kLoaders + lw) * 256), 4, static_cast<int>(soff),
                (c + first_chunk) * sstep, 0, 0);
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
        const long long waves = static_cast<long long>(gridDim.x) * gridDim.y * gridDim.z * C::kLoaders;
        const long long mine = ((static_cast<long long>(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * C::kLoaders + lw;
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
#ifndef BSI_SPLIT_TRACK
#define BSI_SPLIT_TRACK kSplit
#endif
template <int WM, int WN, int KS, int kMode, bool kTrack>
__device__ __forceinline__ void i8_kstep(const v4i (&ka)[WM], const v4i (&qb)[WN], v4i (&ka_n)[WM], v4i (&qb_n)[WN],
                                         const unsigned char* __restrict__ krow_n,
                                         const unsigned char* __restrict__ qrow_n, v4i (&acc)[WM][WN],
                                         const v4i (&prev)[WM][WN], float (&accf)[WM][WN][4],
                                         const float (&qs_prev)[WN], int* __restrict__ ints_prev,
                                         const int64_t (&int_off)[WM][WN], const int (&int_rows)[WM], int down_shift,
                                         int chunks, float& peak) {
    // kTrack (D-split launches): `peak` follows the largest magnitude the lane's chain values take, two of them per
    // three-input maximum
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
                if (kTrack && (e & 1)) peak = fmaxf(fmaxf(peak, fabsf(accf[ea][eb][e - 1])), fabsf(accf[ea][eb][e]));
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

template <int TM, int TN, int kMode, bool kSplit>
__global__ __launch_bounds__((I8Cfg<TM, TN>::kBlock)) void dot_mfma_i8_kernel(
    const int8_t* __restrict__ A8, const float* __restrict__ qscale, int qscale_stride,
    const int8_t* __restrict__ K8,  // int8 key image [R, chunks * 256]
    const float* __restrict__ Bw, int Sb, int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv,
    int64_t R_total, float* __restrict__ out, int* __restrict__ chunk_ints, const float* __restrict__ bias,
    int ndig, long long dig_stride, const long long* __restrict__ key_indices, int key_tiled,
    const unsigned char* __restrict__ warm, long long warm_lines, int out_stream, float* __restrict__ split_partials,
    unsigned* __restrict__ split_counters, float split_limit, int split_shape) {
    // kSplit (chain mode only): a D-split launch.  gridDim.z workgroups share an output tile, each running the chain
    // over its own run of chunks from zero.  All operands of the chain are integers (times one power of two), so
    // as long as no value the chain takes exceeds 2^24 of its unit nothing is ever rounded, the value after every
    // chunk is the exact sum so far, and sums of the segments' results in any order equal the one sequential chain over
    // all chunks bit for bit.  Each workgroup follows the largest magnitude its chain values take; with every
    // segment's peak at most split_limit = 2^24 units / gridDim.z, every prefix of the sequential chain is at most
    // 2^24 units as well, which proves the equality.  A workgroup stores its partial sums to split_partials, then
    // counts itself in at split_counters[tile] (bit 16 and up: segments whose peak went over the limit); the last
    // one to arrive adds the others' sums to its own and writes the outputs -- or, if any segment went over the
    // limit, runs the whole tile again over all chunks in order.  It leaves the counter at zero.
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
    // Which tile (and, in a D-split launch, which segment) this workgroup computes.  A D-split launch is a 1-D grid:
    // key tile fastest, then query tile, then segment, so that workgroups which share a key tile and a run of chunks
    // are neighbours (a grid that gave every XCD one segment of a few key tiles was measured and is no faster).
    int bx = static_cast<int>(blockIdx.x), by = static_cast<int>(blockIdx.y), seg = 0, nseg = 1, tiles_x = static_cast<int>(gridDim.x);
    if (kSplit) {
        tiles_x = split_shape & 1023;
        const int tiles_y = (split_shape >> 10) & 1023;
        nseg = split_shape >> 20;
        const int id = static_cast<int>(blockIdx.x);
        bx = id % tiles_x;
        by = (id / tiles_x) % tiles_y;
        seg = id / (tiles_x * tiles_y);
    }
    const int64_t r0 = static_cast<int64_t>(bx) * TM;
    const int64_t q0 = static_cast<int64_t>(by) * TN;
    const size_t rowbytes = static_cast<size_t>(chunks) * 256;
    static_assert(!kSplit || kMode == kI8Chain, "only the plain chain splits D");
    const int vchunks = kSum ? chunks * ndig : chunks;  // chunks of the loop: every digit image runs over all chunks
    // the workgroup's run of chunks: all of them, or segment seg of nseg
    const int first_chunk = kSplit ? (chunks * seg) / nseg : 0;
    const int my_chunks = kSplit ? (chunks * (seg + 1)) / nseg - first_chunk : vchunks;
    unsigned char* const scale_lds = lds + 4 * C::kStage;  // [chunk & 3][loader][64] floats
    // kSplit: [MFMA wave] flags, [15] = decision
    volatile __attribute__((address_space(3))) int* const split_flags =
        reinterpret_cast<volatile __attribute__((address_space(3))) int*>(BSI_LDS_PTR(lds + C::kLds));

    if (wave >= C::kConsumers) {
        if (wave == C::kConsumers) BSI_STAMP(kStampLoaderEntry);
        i8_loader_wave<C, kSum>(lds, wave - C::kConsumers, lane, A8, qscale, qscale_stride, K8, Bw, Sb, chunks, first_chunk,
                                my_chunks * 2, R, Q, r0, q0, rowbytes, bias, ndig, dig_stride, key_tiled, warm, warm_lines);
        if (kSplit) {
            lds_barrier();  // the MFMA waves have stored their partial sums
            lds_barrier();  // the decision is in LDS
            if (__builtin_amdgcn_readfirstlane(split_flags[15]) == kSplitRedo)
                i8_loader_wave<C, kSum>(lds, wave - C::kConsumers, lane, A8, qscale, qscale_stride, K8, Bw, Sb, chunks, 0,
                                        chunks * 2, R, Q, r0, q0, rowbytes, bias, ndig, dig_stride, key_tiled, nullptr, 0);
        }
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
    i8_kstep<WM, WN, KS, kMode, BSI_SPLIT_TRACK>(ka[(KS) & 1], qb[(KS) & 1], ka[((KS) + 1) & 1], qb[((KS) + 1) & 1],         \
                                lds + (nslot) * C::kStage + krow_off + pcol[((KS) + 1) & 1],                        \
                                lds + (nslot) * C::kStage + qrow_off + pcol[((KS) + 1) & 1], acc, prev, accf, qs,   \
                                ip, int_off, int_rows, down_shift, chunks, peak);
    // a chunk whose halves sit in ring slots s0, s0 + 1; nslot: slot of the next chunk's first half
#define BSI_I8_CHUNK(s0, nslot, acc, prev, qs, ip)                                                                  \
    BSI_I8_KSTEP(0, s0, acc, prev, qs, ip);                                                                         \
    lds_barrier();                                                                                                  \
    BSI_I8_KSTEP(1, (s0) + 1, acc, prev, qs, ip);                                                                   \
    BSI_I8_KSTEP(2, (s0) + 1, acc, prev, qs, ip);                                                                   \
    lds_barrier();                                                                                                  \
    BSI_I8_KSTEP(3, nslot, acc, prev, qs, ip);

    float peak = 0.0f;      // kSplit: the largest magnitude the lane's chain values have taken
    int run_chunks = my_chunks;
    bool last_in_acc0 = false;
#pragma nounroll
    for (int pass = 0;; ++pass) {  // one pass; a D-split launch's last workgroup of a tile may need a second over all chunks
    if (kSplit && pass > 0) {
#pragma unroll
        for (int a = 0; a < WM; ++a)
#pragma unroll
            for (int b = 0; b < WN; ++b) {
                acc0[a][b] = acc1[a][b] = (v4i){0, 0, 0, 0};
#pragma unroll
                for (int e = 0; e < 4; ++e) accf[a][b][e] = 0.0f;
            }
#pragma unroll
        for (int b = 0; b < WN; ++b) qsa[b] = qsb[b] = 0.0f;
    }
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
    for (; c + 1 < run_chunks; c += 2) {
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
    last_in_acc0 = false;
    if (c < run_chunks) {  // odd number of chunks: one more even chunk; its halves sit in slots 0 and 1
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
    if (!kSplit) break;
    if (kSplit) {
        // the chain step of the run's last chunk
#pragma unroll
        for (int a = 0; a < WM; ++a)
#pragma unroll
            for (int b = 0; b < WN; ++b)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = last_in_acc0 ? acc0[a][b][e] : acc1[a][b][e];
                    accf[a][b][e] = fmaf(static_cast<float>(v), last_in_acc0 ? qsa[b] : qsb[b], accf[a][b][e]);
                    peak = fmaxf(peak, fabsf(accf[a][b][e]));
                }
        if (pass > 0) break;  // the whole row in order: these are the sequential chain's values
        typedef float v4f __attribute__((ext_vector_type(4)));
        // (formed here, from values the compiler cannot see through, so that no address of the partial sums is
        // computed ahead of the chunk loop and held in registers the loop has none to spare of)
        int lane_late = lane, tile_late = by * tiles_x + bx;
        asm volatile("" : "+v"(lane_late), "+s"(tile_late));
        const size_t tile = static_cast<size_t>(tile_late);
        constexpr size_t kWaveVecs = static_cast<size_t>(WM) * WN * 64;  // 16-byte pieces of an MFMA wave's outputs
        v4f* const parts = reinterpret_cast<v4f*>(split_partials) + tile * nseg * (C::kConsumers * kWaveVecs);
        {
            v4f* mine = parts + (static_cast<size_t>(seg) * C::kConsumers + wave) * kWaveVecs + lane_late;
#pragma unroll
            for (int a = 0; a < WM; ++a)
#pragma unroll
                for (int b = 0; b < WN; ++b)
                    __builtin_nontemporal_store((v4f){accf[a][b][0], accf[a][b][1], accf[a][b][2], accf[a][b][3]},
                                                mine + (a * WN + b) * 64);
        }
        const int wave_over = (__builtin_amdgcn_ballot_w64(!(peak <= split_limit)) != 0) ? 1 : 0;  // any lane of the wave
        if (lane == 0) split_flags[wave] = wave_over;
        // This wave's partial sums have reached the L2 (stores are counted down once the L2 has them).  One lane of
        // the workgroup then makes the whole workgroup's stores visible to the device (a release fence writes back
        // the L2's dirty lines, whichever wave wrote them) before it counts the workgroup in: one write-back per
        // workgroup.  Fences from every wave, and fences that also invalidate, cost the launch ten times the split's gain.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        lds_barrier();
        if (wave == 0 && lane == 0) {
            unsigned any = 0;
            for (int w = 0; w < C::kConsumers; ++w) any |= static_cast<unsigned>(split_flags[w]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            const unsigned old = __hip_atomic_fetch_add(split_counters + tile, 1u + (any ? 0x10000u : 0u), __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT);
            int decision = kSplitLeave;
            if ((old & 0xFFFFu) == static_cast<unsigned>(nseg - 1)) {  // the tile's last workgroup
                // what the other workgroups stored before they counted themselves in, not what this CU's caches
                // may hold of an earlier launch: the invalidation is the CU's, so it serves the waves that load
                // behind the barrier below
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the invalidation has been carried out, not just issued
                decision = ((old >> 16) != 0 || any != 0) ? kSplitRedo : kSplitCombine;
                __hip_atomic_store(split_counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
                // running totals behind the tile counters: tiles combined, tiles computed again
                __hip_atomic_fetch_add(split_counters + kSplitMaxTiles + (decision == kSplitRedo ? 1 : 0), 1u,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            split_flags[15] = decision;
        }
        lds_barrier();
        const int decision = __builtin_amdgcn_readfirstlane(split_flags[15]);
        if (decision == kSplitLeave) return;
        if (decision == kSplitCombine) {
            for (int sg = 0; sg < nseg; ++sg) {
                if (sg == seg) continue;
                const v4f* theirs = parts + (static_cast<size_t>(sg) * C::kConsumers + wave) * kWaveVecs + lane_late;
#pragma unroll
                for (int a = 0; a < WM; ++a)
#pragma unroll
                    for (int b = 0; b < WN; ++b) {
                        const v4f v = __builtin_nontemporal_load(theirs + (a * WN + b) * 64);
#pragma unroll
                        for (int e = 0; e < 4; ++e) accf[a][b][e] += v[e];  // exact: see the head of the kernel
                    }
            }
            break;
        }
        run_chunks = chunks;  // kSplitRedo: the loader waves fill the ring from chunk 0 again
    }
    }  // passes
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
    // epilogue of the last chunk (a D-split launch has done it above)
    if (!kSplit)
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
        i8_loader_wave<C, false>(lds, wave - W::kConsumers, lane, A8, qscale, qscale_stride, K8, Bw, Sb, chunks, 0, halves, R, Q,
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

// Set by bsi_hip_dot_bias_warm around its launch: the region the int8-image kernel should touch for the next dot.
thread_local const void* g_warm_ptr = nullptr;
thread_local size_t g_warm_bytes = 0;
// How the int8-image kernels store their output.  The entry points of a linear layer (bsi_hip_dot_bias,
// bsi_hip_dot_bias_warm, bsi_hip_linear) set t_layer_output around their launch: the next kernel of the model reads
// that output, so it is stored plainly and stays in the caches.  The dot entry points proper stream it out with
// nontemporal stores: the dirty lines then do not wait in the L2s for the write-back at the kernel's end (1.2 us less
// for the 16 MiB of Q512 R8192).  Measured both ways: streamed layer outputs cost an OPT-1.3B-shaped prefill 2 %
// (4.89 -> 5.00 ms replayed), plain dot outputs cost the standalone dot 8 %.  BSI_OPT_OUTPUT_STORES overrides.
thread_local int t_layer_output = 0;
std::atomic<int> g_output_stores{0};  // 0 = by entry point, 1 = always plain, 2 = always nontemporal
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
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_i8_kernel<TM, TN, kMode, false>), C::kLds);
    hipLaunchKernelGGL((dot_mfma_i8_kernel<TM, TN, kMode, false>), grid, dim3(C::kBlock), C::kLds, st, A8, qscale, stride, K8,
                       Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total, out, chunk_ints, bias, ndig, dig_stride,
                       key_indices, key_tiled, static_cast<const unsigned char*>(g_warm_ptr),
                       static_cast<long long>(g_warm_bytes / 128), stream_output(), static_cast<float*>(nullptr),
                       static_cast<unsigned*>(nullptr), 0.0f, 0);
}

// The D-split launch of the chain mode: `segments` workgroups per output tile, each over its own run of chunks (see
// the head of dot_mfma_i8_kernel).  scratch: the calling thread's attached split scratch (counters, then partial sums).
template <int TM, int TN>
static void launch_mfma_i8_split(int segments, unsigned char* scratch, const int8_t* A8, const float* qscale, int stride,
                                 const int8_t* K8, const float* Bw, int Sb, int chunks, int64_t R, int64_t Q, int down_shift,
                                 float scale_inv, int64_t R_total, float* out, const float* bias, hipStream_t st,
                                 int key_tiled) {
    using C = I8Cfg<TM, TN>;
    const int tiles_x = static_cast<int>((R + TM - 1) / TM), tiles_y = static_cast<int>((Q + TN - 1) / TN);
    const dim3 grid(static_cast<unsigned>(tiles_x * tiles_y * segments));
    const int split_shape = tiles_x | (tiles_y << 10) | (segments << 20);
    // every segment's chain values stay at or below 2^(24 + down_shift) / segments (rounded down to a power of two)
    int log2_segments = 0;
    while ((1 << log2_segments) < segments) ++log2_segments;
    const float limit = __builtin_ldexpf(1.0f, 24 + down_shift - log2_segments);
    static LdsOptIn once0;
    lds_opt_in(once0, reinterpret_cast<const void*>(&dot_mfma_i8_kernel<TM, TN, kI8Chain, true>), C::kLdsSplit);
    hipLaunchKernelGGL((dot_mfma_i8_kernel<TM, TN, kI8Chain, true>), grid, dim3(C::kBlock), C::kLdsSplit, st, A8, qscale,
                       stride, K8, Bw, Sb, chunks, R, Q, down_shift, scale_inv, R_total, out, static_cast<int*>(nullptr), bias,
                       1, 0LL, static_cast<const long long*>(nullptr), key_tiled,
                       static_cast<const unsigned char*>(g_warm_ptr), static_cast<long long>(g_warm_bytes / 128),
                       stream_output(), reinterpret_cast<float*>(scratch + kSplitCounterBytes),
                       reinterpret_cast<unsigned*>(scratch), limit, split_shape);
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
int choose_i8_tile(int64_t R, int64_t Q, int64_t* cost_out) {
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

// D-split choice for a chain-mode call whose grid leaves most CUs idle: the 128 x 128 or 128 x 64 tile with `segments`
// workgroups per tile over runs of chunks, if the calling thread has attached a scratch region that holds the
// partial sums and the modelled time beats the best unsplit tile.  The model, in microseconds, from measurements on
// the MI355X: a workgroup's half-chunk costs 0.0045 us per unit of choose_i8_tile's scale; the partial sums' way
// through memory (stores, one write-back fence per workgroup, the counter, the last workgroup's loads) costs about
// 2 + 0.9 x segments + 0.5 per MiB of partial sums.  That overhead is why shapes like Q512 x R2048 x D8192 stay
// unsplit (16.3 us on 64 x 64 tiles against 22.6 - 26.5 split), and why grids of a few tiles over long rows split
// (Q128 x R512 x D16384: 20.0 -> 13.6 us; Q64 x R256 x D32768: 37.0 -> 17.3; Q256 x R1024 x D16384: 24.9 -> 18.3).
// Returns the tile (128 or 12864) and sets *segments, or 0 for no split.  g_i8_split: 0 = by this model, 1 = never,
// n >= 2 = n segments on the forced tile (g_i8_tile 128 or 12864; 128 x 128 otherwise) whenever the scratch allows it.
thread_local unsigned char* t_split_scratch = nullptr;
thread_local size_t t_split_bytes = 0;
thread_local int t_split_device = -1;
std::atomic<int> g_i8_split{0};
constexpr double kCostUnitUs = 0.0045;
constexpr int kSplitMinChunks = 2;  // chunks per segment at least
constexpr int kSplitMaxSegments = 64;

static size_t split_scratch_need(int64_t tiles, int segments, int TM, int TN) {
    return kSplitCounterBytes + static_cast<size_t>(tiles) * segments * TM * TN * sizeof(float);
}

int choose_i8_split(int64_t R, int64_t Q, int chunks, int* segments) {
    *segments = 1;
    const int mode = g_i8_split.load(std::memory_order_relaxed);
    if (mode == 1 || t_split_scratch == nullptr) return 0;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev != t_split_device) return 0;
    const int64_t kr = (R + 127) / 128;
    const int64_t tiles_of[2] = {kr * ((Q + 127) / 128), kr * ((Q + 63) / 64)};
    const int tile_id[2] = {128, 12864}, tn_of[2] = {128, 64}, unit[2] = {100, 63};
    if (mode >= 2) {
        const int forced = g_i8_tile.load(std::memory_order_relaxed);
        const int i = forced == 12864 ? 1 : 0;
        const int seg = mode < chunks ? mode : chunks;
        if (seg < 2 || tiles_of[i] > kSplitMaxTiles || split_scratch_need(tiles_of[i], seg, 128, tn_of[i]) > t_split_bytes) return 0;
        *segments = seg;
        return tile_id[i];
    }
    if (tiles_of[0] >= 128) return 0;  // half the GPU busy on the large tile: nothing to gain
    int64_t unsplit = 0;
    (void)choose_i8_tile(R, Q, &unsplit);
    double best_us = kCostUnitUs * static_cast<double>(unsplit) * chunks * 2;
    int best = 0;
    for (int i = 0; i < 2; ++i) {
        const int64_t n = tiles_of[i];
        if (n > 128) continue;
        int max_seg = static_cast<int>(256 / n);
        if (max_seg > kSplitMaxSegments) max_seg = kSplitMaxSegments;
        if (max_seg > chunks / kSplitMinChunks) max_seg = chunks / kSplitMinChunks;
        for (int seg = 2; seg <= max_seg; ++seg) {
            const size_t need = split_scratch_need(n, seg, 128, tn_of[i]);
            if (need > t_split_bytes) break;
            const int64_t run = (chunks + seg - 1) / seg;  // chunks of the longest segment
            const double us = kCostUnitUs * unit[i] * static_cast<double>(run) * 2 + 2.0 + 0.9 * seg +
                              0.5 * static_cast<double>(need - kSplitCounterBytes) / (1 << 20);
            if (us < best_us) {
                best_us = us;
                best = tile_id[i];
                *segments = seg;
            }
        }
    }
    return best;
}

void launch_mfma_i8(const int8_t* A8, const float* qscale, int stride, const int8_t* K8, const float* Bw, int Sb,
                           int chunks, int64_t R, int64_t Q, int down_shift, float scale_inv, int64_t R_total,
                           float* out, int32_t* chunk_ints, const float* bias, hipStream_t st, int key_tiled,
                           int ndig, long long dig_stride, const long long* key_indices) {
    if (ndig == 0 && chunk_ints == nullptr) {
        int segments = 1;
        const int split_tile = choose_i8_split(R, Q, chunks, &segments);
        if (split_tile == 128) {
            launch_mfma_i8_split<128, 128>(segments, t_split_scratch, A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift,
                                           scale_inv, R_total, out, bias, st, key_tiled);
            return;
        }
        if (split_tile == 12864) {
            launch_mfma_i8_split<128, 64>(segments, t_split_scratch, A8, qscale, stride, K8, Bw, Sb, chunks, R, Q, down_shift,
                                          scale_inv, R_total, out, bias, st, key_tiled);
            return;
        }
    }
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

}  // namespace bsi

using namespace bsi;

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

extern "C" int bsi_hip_timeline_read_cycles(unsigned long long* cycles_host, int workgroups) {
    BSI_REQUIRE(cycles_host && workgroups >= 1 && workgroups <= kTimelineWorkgroups, "workgroups must be 1 .. %d",
                kTimelineWorkgroups);
#ifdef BSI_TIMELINE
    BSI_HIP_CHECK(hipDeviceSynchronize());
    BSI_HIP_CHECK(hipMemcpyFromSymbol(cycles_host, HIP_SYMBOL(g_timeline_cycles), sizeof(unsigned long long) * 8 * workgroups));
    return BSI_OK;
#else
    return fail(BSI_ERR_INVALID, "this library was built without the timeline stamps (make TIMELINE=1 builds one with)");
#endif
}
