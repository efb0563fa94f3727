/*
 * bsi_oracle.c -- CPU restatement of the reference's fixed-bit BSI tensor-dot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may include, link or call this
 * file: it is the checker that the HIP kernels are compared against (tests, the smoke
 * check and the CPU-baseline leg of the benchmark).  It is written straight from the
 * reference's device sources, one function per cited block, with plain scalar loops so
 * that it can be read against them.  The reference has no CPU implementation of this
 * path (its CPU functions sit behind an un-vendored submodule and never knew fixed-bit
 * chunk scaling), so there is nothing of the reference's to compile instead.
 *
 * How each function is pinned (tests/test_oracle_*.py, none of them re-types the formula):
 *   round_half_away      exact decimal arithmetic (python `decimal`, ROUND_HALF_UP on |x|)
 *   compute_shift        python int.bit_length(), exhaustive over max_abs
 *   shift_clamp          exact rationals (python `fractions`), exhaustive over (r, s)
 *   pack                 reconstruction of every element from its bit-planes
 *   ewah_*               hand-built streams from the documented RLW layout, round trips,
 *                        size pass == emitted length
 *   dot_fixed            the integer-dot identity  I[q,r,c] = sum_d a[q,d]*b[r,d]  (numpy
 *                        int64 matmul on the quantised ints), exact-rational replay of the
 *                        fp32 chain on small cases, and the reference print-scripts' known
 *                        answers ([1,2,3,4].[4,3,2,1] = 20, ...) at decimal_places = 0
 *
 * All citations are relative to the reference tree: bsi_ops/csrc/cuda/...
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define BSI_CHUNK_ELEMS 256 /* elements per scale chunk: bsi_cuda_kernels_quant.cuh:170 */
#define BSI_CHUNK_WORDS 4   /* 64-bit words per chunk: bsi_cuda_kernels_dot.cuh:1306 */

/* bsi_cuda_kernels_quant.cuh:24-29 (bsi_round_half_away_to_ll).  The cast there is undefined for values an int64
 * cannot hold; on the reference's hardware it is cvt.rzi.s64.f64, which saturates and turns a NaN into -2^63.  That
 * is written out here: magnitudes of 2^63 and more (the infinities included) give +-(2^63 - 1), a NaN (which fails
 * x >= 0 and takes the second branch, where the negation of -2^63 wraps) gives -2^63. */
static int64_t magnitude_to_ll(double y) { /* y >= 0 */
    return y >= 9223372036854775808.0 ? INT64_MAX : (int64_t)y;
}
int64_t bsi_oracle_round_half_away(double x) {
    if (x != x) return INT64_MIN;
    if (x >= 0.0) return magnitude_to_ll(floor(x + 0.5));
    return -magnitude_to_ll(floor(-x + 0.5));
}

/* bsi_cuda_kernels_quant.cuh:110-121 (quantize_round_to_int64_batch_kernel):
 * value -> float -> double, times 10^dec, round half away from zero. */
void bsi_oracle_round_to_int64(const float* x, int64_t n, int decimal_places, int64_t* out) {
    const double dec_scale = pow(10.0, (double)decimal_places); /* bsi_vector_cuda.cpp:443 */
    for (int64_t i = 0; i < n; ++i) out[i] = bsi_oracle_round_half_away((double)x[i] * dec_scale);
}

static uint64_t uabs64(int64_t v) { return v >= 0 ? (uint64_t)v : 0 - (uint64_t)v; } /* quant.cuh:31-33; -2^63 -> 2^63 */

/* bsi_cuda_kernels_quant.cuh:82-108 (bsi_compute_shift) */
int bsi_oracle_compute_shift(uint64_t max_abs, double sum_abs, int count, int fixed_bits, float clip_k) {
    if (fixed_bits <= 0) return 0;
    int bits = 0;
    if (clip_k > 0.0f && count > 0) {
        double effective = (double)max_abs;
        const double mean_abs = sum_abs / (double)count;
        const double clip_max = mean_abs * (double)clip_k;
        if (clip_max < effective) effective = clip_max;
        if (effective > 0.0) {
            int e = 0;
            (void)frexp(effective, &e);
            bits = e;
        }
    } else {
        bits = (max_abs > 0) ? (64 - __builtin_clzll(max_abs)) : 0;
    }
    int shift = bits - (fixed_bits - 1);
    if (shift < 0) shift = 0;
    if (shift > 62) shift = 62;
    return shift;
}

/* bsi_cuda_kernels_quant.cuh:205-226 (apply_row_shift_clamp_kernel body; the same lines are
 * inlined at :378-399 and :450-475): rounded signed right shift, then clamp to fixed_bits. */
int64_t bsi_oracle_shift_clamp(int64_t v, int shift, int fixed_bits) {
    const uint64_t av = uabs64(v);
    const uint64_t round_add = (shift > 0) ? (1ULL << (shift - 1)) : 0ULL;
    const uint64_t q = (av + round_add) >> shift;
    int64_t out = (v < 0) ? -(int64_t)q : (int64_t)q;
    const int64_t qmax = ((int64_t)1 << (fixed_bits - 1)) - 1;
    const int64_t qmin = -((int64_t)1 << (fixed_bits - 1));
    if (out < qmin) out = qmin;
    if (out > qmax) out = qmax;
    return out;
}

/*
 * Fixed-bit quantiser for a [Q, d] batch.
 *   chunk_scale != 0 : per (row, 256-element chunk) shift -- queries
 *                      quant.cuh:291-341 (shift/scale pass) + :414-488 (quantise pass)
 *   chunk_scale == 0 : per row shift -- keys, and queries when W64 % 4 != 0
 *                      quant.cuh:255-289 + :343-412; ATen twin bsi_vector_cuda.cpp:658-743
 * Outputs: ints [Q, d] quantised values, shifts/scales [Q, chunks] or [Q].
 * An empty chunk (start >= d) gets shift 0, scale 1 (quant.cuh:307-314).
 */
void bsi_oracle_quantize_fixed(const float* x, int64_t Q, int64_t d, int decimal_places, int fixed_bits,
                               int chunk_scale, float clip_k, int64_t* ints, int32_t* shifts, float* scales) {
    const double dec_scale = pow(10.0, (double)decimal_places);
    const int64_t chunks = chunk_scale ? (d + BSI_CHUNK_ELEMS - 1) / BSI_CHUNK_ELEMS : 1;
    const int64_t span = chunk_scale ? BSI_CHUNK_ELEMS : d;
    for (int64_t q = 0; q < Q; ++q) {
        for (int64_t c = 0; c < chunks; ++c) {
            const int64_t start = c * span;
            int64_t valid = d - start;
            if (valid > span) valid = span;
            if (valid < 0) valid = 0;
            uint64_t max_abs = 0;
            double sum_abs = 0.0;
            for (int64_t e = 0; e < valid; ++e) {
                const int64_t r = bsi_oracle_round_half_away((double)x[q * d + start + e] * dec_scale);
                const uint64_t av = uabs64(r);
                if (av > max_abs) max_abs = av;
                sum_abs += (double)av;
            }
            const int shift = (valid > 0) ? bsi_oracle_compute_shift(max_abs, sum_abs, (int)valid, fixed_bits, clip_k) : 0;
            shifts[q * chunks + c] = shift;
            scales[q * chunks + c] = (float)(1ULL << shift);
            for (int64_t e = 0; e < valid; ++e) {
                const int64_t r = bsi_oracle_round_half_away((double)x[q * d + start + e] * dec_scale);
                ints[q * d + start + e] = bsi_oracle_shift_clamp(r, shift, fixed_bits);
            }
        }
    }
}

/* bsi_cuda_kernels_pack.cuh:129-174 (pack_bits_all_ballot_multi_kernel_batch_oneshot):
 * words [Q, slices, W]; bit b of word w of slice s = bit s of (uint64(v[64w+b]) & mask);
 * elements past d contribute 0. */
void bsi_oracle_pack(const int64_t* ints, int64_t Q, int64_t d, int slices, int64_t W, uint64_t* words) {
    const uint64_t mask = (slices >= 64) ? ~0ULL : ((1ULL << slices) - 1ULL);
    memset(words, 0, (size_t)(Q * slices * W) * sizeof(uint64_t));
    for (int64_t q = 0; q < Q; ++q)
        for (int64_t e = 0; e < d; ++e) {
            const uint64_t v = (uint64_t)ints[q * d + e] & mask;
            for (int s = 0; s < slices; ++s)
                if ((v >> s) & 1ULL) words[(q * slices + s) * W + (e >> 6)] |= 1ULL << (e & 63);
        }
}

/* bsi_cuda.cpp:217-236 (weight_for_meta / make_slice_weights_cuda): 2^(offset+idx),
 * negated for the top slice of a two's-complement vector. */
void bsi_oracle_slice_weights(int S, int offset, int twos, float* out) {
    for (int i = 0; i < S; ++i) {
        const int sh = offset + i;
        long double w = (sh >= 0) ? ldexpl(1.0L, sh) : 0.0L;
        if (twos && i == S - 1) w = -w;
        out[i] = (float)w;
    }
}

/* ---------------- EWAH ---------------- */

/* bsi_cuda_kernels_ewah.cuh:47-69 + :84-102: per-slice density -> compress flag. */
void bsi_oracle_compress_flags(const uint64_t* words, int S, int W, double threshold, int32_t* flags) {
    for (int s = 0; s < S; ++s) {
        uint64_t cnt = 0;
        for (int w = 0; w < W; ++w) cnt += (uint64_t)__builtin_popcountll(words[(size_t)s * W + w]);
        const double total_bits = (double)W * 64.0;
        double p = (total_bits > 0.0) ? ((double)cnt / total_bits) : 0.0;
        if (p < 0.0) p = 0.0;
        if (p > 1.0) p = 1.0;
        const double a = pow(1.0 - p, 128.0);
        const double b = pow(p, 128.0);
        const double M = 1.0 - a - b;
        flags[s] = (M <= threshold) ? 1 : 0;
    }
}

/* Shared walk of bsi_cuda_kernels_ewah.cuh:118-162 (size) and :178-232 (emit): one marker
 * word per (run, literal span); out == NULL gives the size pass.
 * Marker = run_bit | run_len << 1 | lit_count << 33 (:221-226). */
static uint64_t ewah_walk(const uint64_t* base, int W, int compress, uint64_t* out) {
    uint64_t o = 0;
    int idx = 0;
    while (idx < W) {
        int run_len = 0, run_bit = 0;
        if (compress) {
            const uint64_t v = base[idx];
            if (v == 0ULL || v == ~0ULL) {
                run_bit = (v == ~0ULL) ? 1 : 0;
                int k = idx;
                while (k < W && base[k] == v) ++k;
                run_len = k - idx;
                idx = k;
            }
        }
        int lit_count = 0;
        const int lit_start = idx;
        while (idx < W) {
            const uint64_t v = base[idx];
            if (compress && (v == 0ULL || v == ~0ULL)) break;
            ++lit_count;
            ++idx;
        }
        if (out) {
            out[o] = (uint64_t)run_bit | (((uint64_t)run_len & 0xFFFFFFFFULL) << 1) | ((uint64_t)lit_count << 33);
            for (int k = 0; k < lit_count; ++k) out[o + 1 + k] = base[lit_start + k];
        }
        o += 1ULL + (uint64_t)lit_count;
    }
    return o;
}

void bsi_oracle_ewah_size(const uint64_t* words, int S, int W, const int32_t* flags, uint64_t* sizes) {
    for (int s = 0; s < S; ++s) sizes[s] = ewah_walk(words + (size_t)s * W, W, flags[s], NULL);
}

void bsi_oracle_ewah_emit(const uint64_t* words, int S, int W, const int32_t* flags, const uint64_t* off,
                          uint64_t* out, int32_t* out_len) {
    for (int s = 0; s < S; ++s) out_len[s] = (int32_t)ewah_walk(words + (size_t)s * W, W, flags[s], out + off[s]);
}

/* bsi_cuda_kernels_ewah.cuh:5-33 (ewah_decompress_kernel) */
void bsi_oracle_ewah_decompress(const uint64_t* in, int in_len, int W, uint64_t* out) {
    int idx = 0, o = 0;
    while (idx < in_len && o < W) {
        const uint64_t rlw = in[idx++];
        const int running_bit = (int)(rlw & 1ULL);
        const uint32_t run_len = (uint32_t)((rlw >> 1) & 0xFFFFFFFFULL);
        const uint32_t lit_words = (uint32_t)(rlw >> 33);
        const uint64_t run_val = running_bit ? ~0ULL : 0ULL;
        for (uint32_t k = 0; k < run_len && o < W; ++k) out[o++] = run_val;
        for (uint32_t k = 0; k < lit_words && o < W && idx < in_len; ++k) out[o++] = in[idx++];
    }
    while (o < W) out[o++] = 0ULL;
}

/* ---------------- dot ---------------- */

/*
 * bsi_cuda_kernels_dot.cuh:1384-1542 (fixed76 chunk-scale kernel, generalised to any Sa/Sb
 * with the same sign rule) + bsi_cuda.cpp:710-711 (scale_inv):
 *   I[q,r,c] = sum_{i<Sa} sum_{j<Sb} sgn(i,j) * (popc(A[q,i,4c..4c+3] & B[r,j,4c..4c+3]) << (i+j))
 *              sgn = -1 iff (i == Sa-1) xor (j == Sb-1)                       (:1474-1477)
 *   acc      = fmaf((float)I, qscale[q,c] * bscale[r], acc)                   (:1516-1523)
 *   out[q,r] = acc * scale_inv                                                (:1533-1540)
 * qscale is read at q*qscale_stride + c; bscale[r] is the reference's Bw[r*Sb + 0] (:1339-1340).
 * A partial last chunk (W % 4 != 0) reads the missing words as zero.
 * chunk_ints (may be NULL) receives I as int32 [Q, R, chunks]; out (may be NULL) the fp32 result
 * with row stride R_total.
 */
void bsi_oracle_dot_fixed(const uint64_t* A, const float* qscale, int64_t qscale_stride, int Sa, int W,
                          const uint64_t* B, const float* bscale, int Sb, int64_t R, int64_t Q, float scale_inv,
                          int64_t R_total, int32_t* chunk_ints, float* out) {
    const int chunks = (W + BSI_CHUNK_WORDS - 1) / BSI_CHUNK_WORDS;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        const uint64_t* Br = B + (size_t)r * Sb * W;
        for (int64_t q = 0; q < Q; ++q) {
            const uint64_t* Aq = A + (size_t)q * Sa * W;
            float acc = 0.0f;
            for (int c = 0; c < chunks; ++c) {
                const int w0 = c * BSI_CHUNK_WORDS;
                const int w1 = (w0 + BSI_CHUNK_WORDS < W) ? w0 + BSI_CHUNK_WORDS : W;
                /* summed modulo 2^64 (a term shifted by 64 or more is a multiple of 2^64): the chunk's integer dot
                 * whenever that fits 64 bits, and the reference's int32 for its 7 x 6 bits (|I| <= 2^19) */
                uint64_t I = 0;
                for (int i = 0; i < Sa; ++i)
                    for (int j = 0; j < Sb; ++j) {
                        uint64_t cnt = 0;
                        for (int w = w0; w < w1; ++w)
                            cnt += (uint64_t)__builtin_popcountll(Aq[(size_t)i * W + w] & Br[(size_t)j * W + w]);
                        const uint64_t v = (i + j < 64) ? cnt << (i + j) : 0;
                        if ((i == Sa - 1) != (j == Sb - 1)) I -= v; else I += v;
                    }
                if (chunk_ints) chunk_ints[((size_t)q * R + r) * chunks + c] = (int32_t)(uint32_t)I;
                acc = fmaf((float)(int64_t)I, qscale[q * qscale_stride + c] * bscale[r], acc);
            }
            if (out) out[(size_t)q * R_total + r] = acc * scale_inv;
        }
    }
}

int bsi_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
