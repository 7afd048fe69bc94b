/* blocked_join.c -- the CPU baseline: a cache-blocked brute-force Euclidean join in GEMM form.
 *
 * TEST / MEASUREMENT INFRASTRUCTURE ONLY: built into liboracle.so, called by tests/ (pinned against the
 * difference-form FP64 checker of fasted_oracle.c) and by the cpu_baseline leg of bench.py.  The shipped
 * library never links or loads it.
 *
 * Pair definition: the reference's (source/warpMma.cuh:241-267) -- every ordered pair (q, c) with
 * s_q + s_c - 2 q.c <= eps^2, i = j included, no padding -- evaluated in FP64 or in FP32 on the FP16
 * points widened to that type.  The reference has no CPU path of its own ("We do not compare to CPU
 * algorithms", icpp_paper/main.tex:479); this is what a host-only user would run instead of the GPU join.
 *
 * Structure (the usual three-level blocking of a dense contraction):
 *   query block   up to 1536 rows, widened and packed once as panels [k][6 rows]
 *   candidate block of 128 rows per thread (OpenMP dynamic), its K slices of 256 widened and packed as
 *                 [k][128 columns] (L2-resident)
 *   micro-kernel  6 x 2 vectors of accumulators in registers, one broadcast + two loads + twelve FMAs per k
 *   then the distance test on the block's 1536 x 128 products.
 * The micro-kernel is written with GCC vector types and compiled twice: 256-bit (x86-64-v3) and, where the
 * host has it, 512-bit (AVX-512F), chosen at run time.
 *
 * This file includes itself four times (REAL = double / float, vector = 32 / 64 bytes).
 */
#ifndef BJ_INSTANCE

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

float oracle_f16_to_f32(uint16_t h); /* fasted_oracle.c */

enum { BJ_MR = 6, BJ_NC = 128, BJ_KC = 256, BJ_MC = 1536 };

typedef struct {
    int *q, *c;
    size_t n, cap;
} bj_pairs;

static void bj_push(bj_pairs *v, int q, int c) {
    if (v->n == v->cap) {
        v->cap = v->cap ? v->cap * 2 : 4096;
        v->q = (int *)realloc(v->q, v->cap * sizeof(int));
        v->c = (int *)realloc(v->c, v->cap * sizeof(int));
    }
    v->q[v->n] = q;
    v->c[v->n] = c;
    ++v->n;
}

static float bj_half_table[65536];
static int bj_half_table_ready = 0;
static void bj_init_table(void) {
    if (bj_half_table_ready) return;
    for (unsigned i = 0; i < 65536u; ++i) bj_half_table[i] = oracle_f16_to_f32((uint16_t)i);
    bj_half_table_ready = 1;
}

static double bj_now(void) {
#ifdef _OPENMP
    return omp_get_wtime();
#else
    return 0.0;
#endif
}

#define BJ_INSTANCE 1
#define REAL double
#define VBYTES 32
#define FN(x) x##_f64_v256
#define TARGET
#include "blocked_join.c"
#undef REAL
#undef VBYTES
#undef FN
#undef TARGET

#define REAL float
#define VBYTES 32
#define FN(x) x##_f32_v256
#define TARGET
#include "blocked_join.c"
#undef REAL
#undef VBYTES
#undef FN
#undef TARGET

#define REAL double
#define VBYTES 64
#define FN(x) x##_f64_v512
#define TARGET __attribute__((target("avx512f,avx512vl,avx512dq,avx512bw,fma")))
#include "blocked_join.c"
#undef REAL
#undef VBYTES
#undef FN
#undef TARGET

#define REAL float
#define VBYTES 64
#define FN(x) x##_f32_v512
#define TARGET __attribute__((target("avx512f,avx512vl,avx512dq,avx512bw,fma")))
#include "blocked_join.c"
#undef REAL
#undef VBYTES
#undef FN
#undef TARGET

/* 512-bit vectors when the host has them (0 forces 256-bit, for tests that want both paths run) */
static int bj_vector_bits = -1;
int oracle_blocked_join_vector_bits(int force) {
    if (force == 256 || force == 512) bj_vector_bits = force;
    if (bj_vector_bits < 0) {
        __builtin_cpu_init();
        bj_vector_bits = __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512vl") ? 512 : 256;
    }
    if (bj_vector_bits == 512 && !__builtin_cpu_supports("avx512f")) bj_vector_bits = 256;
    return bj_vector_bits;
}

/* Joins `nq` query rows with `nc` candidate rows (FP16 bit patterns, `d` columns, row strides `ldq`, `ldc`
 * halves).  precision: 64 or 32.  Pairs are reported as (q_offset + row, c_offset + row), in no particular
 * order, up to `cap` of them (out_q / out_c may be NULL with cap 0: count only); the return value counts all.
 * *seconds receives the wall time of the call (widening, packing, contraction and test). */
unsigned long long oracle_blocked_join(const uint16_t *queries, size_t nq, size_t ldq, const uint16_t *cands, size_t nc,
                                       size_t ldc, size_t d, double eps, int precision, int q_offset, int c_offset,
                                       int *out_q, int *out_c, unsigned long long cap, double *seconds) {
    bj_init_table();
    const int bits = oracle_blocked_join_vector_bits(0);
    const double t0 = bj_now();
    unsigned long long found;
    if (precision == 64)
        found = bits == 512 ? bj_join_f64_v512(queries, nq, ldq, cands, nc, ldc, d, eps, q_offset, c_offset, out_q, out_c, cap)
                            : bj_join_f64_v256(queries, nq, ldq, cands, nc, ldc, d, eps, q_offset, c_offset, out_q, out_c, cap);
    else
        found = bits == 512 ? bj_join_f32_v512(queries, nq, ldq, cands, nc, ldc, d, eps, q_offset, c_offset, out_q, out_c, cap)
                            : bj_join_f32_v256(queries, nq, ldq, cands, nc, ldc, d, eps, q_offset, c_offset, out_q, out_c, cap);
    if (seconds) *seconds = bj_now() - t0;
    return found;
}

#else /* ---- one instance: REAL, VBYTES, FN, TARGET ------------------------------------------------ */

typedef REAL FN(vreal) __attribute__((vector_size(VBYTES), aligned(VBYTES)));
#define VT FN(vreal)
#define VL ((int)(VBYTES / sizeof(REAL)))

/* rows [r0, r0 + rows) of the queries -> panels of BJ_MR rows: Ap[panel][k][BJ_MR], missing rows zero;
 * also their squared norms */
TARGET static void FN(bj_pack_queries)(const uint16_t *q, size_t ld, size_t r0, size_t rows, size_t d, REAL *Ap, REAL *norms) {
    const size_t panels = (rows + BJ_MR - 1) / BJ_MR;
#pragma omp parallel for schedule(static)
    for (long long p = 0; p < (long long)panels; ++p) {
        REAL *dst = Ap + (size_t)p * d * BJ_MR;
        for (int i = 0; i < BJ_MR; ++i) {
            const size_t r = (size_t)p * BJ_MR + i;
            REAL s = 0;
            if (r < rows) {
                const uint16_t *src = q + (r0 + r) * ld;
                for (size_t k = 0; k < d; ++k) {
                    const REAL x = (REAL)bj_half_table[src[k]];
                    dst[k * BJ_MR + i] = x;
                    s += x * x;
                }
            } else {
                for (size_t k = 0; k < d; ++k) dst[k * BJ_MR + i] = 0;
            }
            norms[r] = s;
        }
    }
}

/* K slice [k0, k0 + kc) of candidate rows [c0, c0 + cols) -> Bp[k][BJ_NC], missing columns zero */
TARGET static void FN(bj_pack_candidates)(const uint16_t *c, size_t ld, size_t c0, size_t cols, size_t k0, size_t kc, REAL *Bp) {
    for (size_t j = 0; j < BJ_NC; ++j) {
        if (j < cols) {
            const uint16_t *src = c + (c0 + j) * ld + k0;
            for (size_t k = 0; k < kc; ++k) Bp[k * BJ_NC + j] = (REAL)bj_half_table[src[k]];
        } else {
            for (size_t k = 0; k < kc; ++k) Bp[k * BJ_NC + j] = 0;
        }
    }
}

/* Ct[6][2 vectors] += Ap panel (kc x 6) . Bp (kc x 2 vectors) */
TARGET static inline void FN(bj_micro)(const REAL *restrict ap, const REAL *restrict bp, size_t kc, REAL *restrict ct) {
    VT acc[BJ_MR][2];
    for (int i = 0; i < BJ_MR; ++i) {
        acc[i][0] = *(const VT *)(ct + (size_t)i * BJ_NC);
        acc[i][1] = *(const VT *)(ct + (size_t)i * BJ_NC + VL);
    }
    for (size_t k = 0; k < kc; ++k) {
        const VT b0 = *(const VT *)(bp + k * BJ_NC), b1 = *(const VT *)(bp + k * BJ_NC + VL);
#pragma GCC unroll 6
        for (int i = 0; i < BJ_MR; ++i) {
            const REAL a = ap[k * BJ_MR + i];
            acc[i][0] += a * b0;
            acc[i][1] += a * b1;
        }
    }
    for (int i = 0; i < BJ_MR; ++i) {
        *(VT *)(ct + (size_t)i * BJ_NC) = acc[i][0];
        *(VT *)(ct + (size_t)i * BJ_NC + VL) = acc[i][1];
    }
}

TARGET static unsigned long long FN(bj_join)(const uint16_t *queries, size_t nq, size_t ldq, const uint16_t *cands, size_t nc,
                                             size_t ldc, size_t d, double eps, int q_offset, int c_offset, int *out_q,
                                             int *out_c, unsigned long long cap) {
    const REAL eps2 = (REAL)(eps * eps);
    const size_t cblocks = (nc + BJ_NC - 1) / BJ_NC;
    const size_t mcPad = ((BJ_MC + BJ_MR - 1) / BJ_MR) * BJ_MR;
    REAL *Ap = (REAL *)aligned_alloc(64, mcPad * d * sizeof(REAL));
    REAL *qn = (REAL *)aligned_alloc(64, ((mcPad * sizeof(REAL) + 63) / 64) * 64);
    int nthreads = 1;
#ifdef _OPENMP
    nthreads = omp_get_max_threads();
#endif
    bj_pairs *lists = (bj_pairs *)calloc((size_t)nthreads, sizeof(bj_pairs));
    unsigned long long *counts = (unsigned long long *)calloc((size_t)nthreads, sizeof(unsigned long long));
    const int keep = out_q != NULL && out_c != NULL && cap > 0;

    for (size_t q0 = 0; q0 < nq; q0 += BJ_MC) {
        const size_t rows = nq - q0 < BJ_MC ? nq - q0 : BJ_MC;
        const size_t panels = (rows + BJ_MR - 1) / BJ_MR;
        FN(bj_pack_queries)(queries, ldq, q0, rows, d, Ap, qn);
#pragma omp parallel
        {
            int tid = 0;
#ifdef _OPENMP
            tid = omp_get_thread_num();
#endif
            REAL *Bp = (REAL *)aligned_alloc(64, (size_t)BJ_KC * BJ_NC * sizeof(REAL));
            REAL *Ct = (REAL *)aligned_alloc(64, mcPad * BJ_NC * sizeof(REAL));
            REAL cn[BJ_NC];
#pragma omp for schedule(dynamic, 1)
            for (long long cb = 0; cb < (long long)cblocks; ++cb) {
                const size_t c0 = (size_t)cb * BJ_NC;
                const size_t cols = nc - c0 < BJ_NC ? nc - c0 : BJ_NC;
                memset(Ct, 0, panels * BJ_MR * BJ_NC * sizeof(REAL));
                for (size_t j = 0; j < BJ_NC; ++j) cn[j] = 0;
                for (size_t k0 = 0; k0 < d; k0 += BJ_KC) {
                    const size_t kc = d - k0 < BJ_KC ? d - k0 : BJ_KC;
                    FN(bj_pack_candidates)(cands, ldc, c0, cols, k0, kc, Bp);
                    for (size_t k = 0; k < kc; ++k)
                        for (size_t j = 0; j < BJ_NC; ++j) cn[j] += Bp[k * BJ_NC + j] * Bp[k * BJ_NC + j];
                    for (size_t p = 0; p < panels; ++p) {
                        const REAL *ap = Ap + (p * d + k0) * BJ_MR;
                        for (size_t jr = 0; jr < BJ_NC; jr += 2 * VL)
                            FN(bj_micro)(ap, Bp + jr, kc, Ct + p * BJ_MR * BJ_NC + jr);
                    }
                }
                /* the test of the reference: (s_q + s_c) - 2 q.c <= eps^2 */
                for (size_t r = 0; r < rows; ++r) {
                    const REAL sq = qn[r];
                    const REAL *row = Ct + r * BJ_NC;
                    for (size_t j = 0; j < cols; ++j) {
                        const REAL d2 = (sq + cn[j]) - (REAL)2 * row[j];
                        if (d2 <= eps2) {
                            ++counts[tid];
                            if (keep) bj_push(&lists[tid], q_offset + (int)(q0 + r), c_offset + (int)(c0 + j));
                        }
                    }
                }
            }
            free(Bp);
            free(Ct);
        }
    }
    unsigned long long found = 0, written = 0;
    for (int t = 0; t < nthreads; ++t) {
        found += counts[t];
        for (size_t i = 0; i < lists[t].n && written < cap; ++i, ++written) {
            out_q[written] = lists[t].q[i];
            out_c[written] = lists[t].c[i];
        }
        free(lists[t].q);
        free(lists[t].c);
    }
    free(lists);
    free(counts);
    free(Ap);
    free(qn);
    return found;
}

#undef VT
#undef VL
#endif
