/*
 * fasted_oracle.c -- CPU restatement of the FaSTED epsilon self-join hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker: it is linked or loaded by the
 * test-suite, by the smoke check and by the CPU-baseline leg of the benchmark, and by
 * nothing else.  The shipped library never calls into it and has no CPU fallback.
 *
 * Every function cites the reference source (paths relative to the reference checkout)
 * whose behaviour it restates.  Plain C11 + OpenMP, no GPU, no third-party code.
 *
 * Parity status of each function (what pins it is in tests/test_oracle_*.py):
 *   oracle_f32_to_f16 / oracle_quantize   pinned: numpy float16 on all 65536 halves + ties,
 *                                          and the reference's own half.hpp via oracle/_ref
 *   oracle_exponential_points             pinned: golden FP16 bits from the reference's
 *                                          generator built in oracle/_ref
 *   oracle_build_padded                   pinned: same, padded shape + zero fill
 *   oracle_sum_squared_rz / _rn / _f64    pinned: closed form on integer rows (the reference's
 *                                          tests/python/sumSquared/sumSquared.py pattern),
 *                                          RZ <= exact <= RZ + D ulp invariant
 *   oracle_raster_coord                   pinned: permutation + 8x8 locality properties
 *   oracle_pairs_get_space                pinned: closed-form found/stored under overflow
 *   oracle_self_join_f64 / _f32           pinned: textbook brute force on tiny inputs, the
 *                                          identity/increasing fixtures of main.cu:86-131
 *   oracle_pair_stats                     pinned: the expected PairsStats of the reference's
 *                                          results/scripts/test_accuracy.py cases
 *   tensor-core accumulation order        PARITY UNPINNED at bit level: the A100's internal
 *                                          MMA rounding is hardware behaviour no reference
 *                                          test fixes; set-level parity is judged against
 *                                          FP64 through the relative 1e-3 epsilon band.
 */
#include <fenv.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#pragma STDC FENV_ACCESS ON

/* ------------------------------------------------------------------------------------
 * Quantisation: double -> float -> half, round-to-nearest-even at both steps.
 * Follows DataLoader/PointListBuilder.hpp:57-73 (castValue) and the IEEE branch of
 * DataLoader/half.hpp:907-937 (float2half_impl) with HALF_ROUND_STYLE 1 (half.hpp:373-375).
 * ---------------------------------------------------------------------------------- */
uint16_t oracle_f32_to_f16(float value) {
    uint32_t f;
    memcpy(&f, &value, 4);
    uint32_t sign = (f >> 16) & 0x8000u;
    f &= 0x7FFFFFFFu;
    if (f >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (f > 0x7F800000u ? (0x200u | ((f >> 13) & 0x3FFu)) : 0u));
    if (f >= 0x47800000u) /* >= 65536: overflow to inf under RNE */
        return (uint16_t)(sign | 0x7C00u);
    if (f >= 0x38800000u) { /* normal half */
        uint32_t v = sign | (((f >> 23) - 112u) << 10) | ((f >> 13) & 0x3FFu);
        uint32_t g = (f >> 12) & 1u, s = (f & 0xFFFu) != 0u;
        return (uint16_t)(v + (g & (s | v)));
    }
    if (f >= 0x33000000u) { /* subnormal half */
        int i = 125 - (int)(f >> 23);
        uint32_t m = (f & 0x7FFFFFu) | 0x800000u;
        uint32_t v = sign | (m >> (i + 1));
        uint32_t g = (m >> i) & 1u, s = (m & ((1u << i) - 1u)) != 0u;
        return (uint16_t)(v + (g & (s | v)));
    }
    return (uint16_t)sign; /* underflow to signed zero */
}

float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, out;
    if (e == 0) {
        if (m == 0) {
            out = sign;
        } else { /* subnormal: normalise */
            int sh = 0;
            while (!(m & 0x400u)) {
                m <<= 1;
                ++sh;
            }
            m &= 0x3FFu;
            out = sign | ((uint32_t)(113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        out = sign | 0x7F800000u | (m << 13);
    } else {
        out = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &out, 4);
    return f;
}

void oracle_quantize(const double *in, size_t n, uint16_t *out) {
    for (size_t i = 0; i < n; ++i) out[i] = oracle_f32_to_f16((float)in[i]);
}

void oracle_widen(const uint16_t *in, size_t n, double *out) {
    for (size_t i = 0; i < n; ++i) out[i] = (double)oracle_f16_to_f32(in[i]);
}

/* ------------------------------------------------------------------------------------
 * Seeded exponential generator.
 * Follows DataLoader/ExponentialPointGenerator.hpp:11 (SEED 2137834274) and :35-57
 * (draw until 0 <= v <= max).  std::mt19937 is the standard MT19937; libstdc++'s
 * std::exponential_distribution<double> returns -log(1 - u)/lambda with
 * u = generate_canonical<double,53>(gen) = (lo + hi * 2^32) / 2^64 from two draws
 * (lo first), clamped below 1.
 * ---------------------------------------------------------------------------------- */
typedef struct {
    uint32_t mt[624];
    int idx;
} mt19937_t;

static void mt_seed(mt19937_t *g, uint32_t seed) {
    g->mt[0] = seed;
    for (int i = 1; i < 624; ++i) g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
    g->idx = 624;
}

static uint32_t mt_next(mt19937_t *g) {
    if (g->idx >= 624) {
        for (int i = 0; i < 624; ++i) {
            uint32_t y = (g->mt[i] & 0x80000000u) | (g->mt[(i + 1) % 624] & 0x7FFFFFFFu);
            g->mt[i] = g->mt[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908B0DFu : 0u);
        }
        g->idx = 0;
    }
    uint32_t y = g->mt[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9D2C5680u;
    y ^= (y << 15) & 0xEFC60000u;
    y ^= y >> 18;
    return y;
}

static double mt_canonical53(mt19937_t *g) {
    double lo = (double)mt_next(g);
    double hi = (double)mt_next(g);
    double r = (lo + hi * 4294967296.0) / 18446744073709551616.0;
    if (r >= 1.0) r = nextafter(1.0, 0.0);
    return r;
}

#define ORACLE_REFERENCE_SEED 2137834274u

/* Writes n*d doubles, row-major, exactly the sequence the reference generator yields. */
void oracle_exponential_points(int n, int d, double lambda, double max_value, double *out) {
    mt19937_t g;
    mt_seed(&g, ORACLE_REFERENCE_SEED);
    for (size_t i = 0; i < (size_t)n * (size_t)d; ++i) {
        double v;
        do {
            v = -log(1.0 - mt_canonical53(&g)) / lambda;
        } while (v < 0.0 || v > max_value);
        out[i] = v;
    }
}

/* ------------------------------------------------------------------------------------
 * Padded FP16 point list.
 * Follows DataLoader/PointListBuilder.hpp:132-192 (build): every point is quantised,
 * its dimensions zero-padded to a multiple of dim_factor, then all-zero points are
 * appended until the count is a multiple of points_factor.  Returns padded sizes; `out`
 * must hold n_pad*d_pad halves (call with out == NULL to query the sizes only).
 * ---------------------------------------------------------------------------------- */
static int round_up_multiple(int v, int m) { return (int)(ceil(1.0 * v / m) * m); }

void oracle_build_padded(const double *in, int n, int d, int dim_factor, int points_factor, uint16_t *out,
                         int *n_pad, int *d_pad) {
    int dp = round_up_multiple(d, dim_factor);
    int np = round_up_multiple(n, points_factor);
    *n_pad = np;
    *d_pad = dp;
    if (!out) return;
    memset(out, 0, (size_t)np * dp * sizeof(uint16_t));
    for (int i = 0; i < n; ++i)
        for (int k = 0; k < d; ++k) out[(size_t)i * dp + k] = oracle_f32_to_f16((float)in[(size_t)i * d + k]);
}

/* ------------------------------------------------------------------------------------
 * Squared norms.
 * oracle_sum_squared_rz follows sumSquared.cuh:34-40 (SumSquareHalf2: x*x and y*y in
 * FP32 -- exact, 11-bit significands -- added with round-toward-zero) and :53-73
 * (SquaredSumsKernel launched with ONE thread per point, :98-100, so the fold over the
 * half2 pairs is strictly sequential, each add round-toward-zero).
 * _rn is the same fold with round-to-nearest; _f64 is the exact-to-double value.
 * ---------------------------------------------------------------------------------- */
void oracle_sum_squared_rz(const uint16_t *pts, size_t n, size_t d, float *sums) {
    int saved = fegetround();
    fesetround(FE_TOWARDZERO);
    for (size_t i = 0; i < n; ++i) {
        volatile float acc = 0.0f;
        for (size_t k = 0; k < d; k += 2) {
            float x = oracle_f16_to_f32(pts[i * d + k]);
            float y = (k + 1 < d) ? oracle_f16_to_f32(pts[i * d + k + 1]) : 0.0f;
            volatile float xx = x * x, yy = y * y; /* exact */
            volatile float pair = xx + yy;         /* RZ */
            acc = acc + pair;                      /* RZ */
        }
        sums[i] = acc;
    }
    fesetround(saved);
}

void oracle_sum_squared_rn(const uint16_t *pts, size_t n, size_t d, float *sums) {
    for (size_t i = 0; i < n; ++i) {
        volatile float acc = 0.0f;
        for (size_t k = 0; k < d; k += 2) {
            float x = oracle_f16_to_f32(pts[i * d + k]);
            float y = (k + 1 < d) ? oracle_f16_to_f32(pts[i * d + k + 1]) : 0.0f;
            volatile float pair = x * x + y * y;
            acc = acc + pair;
        }
        sums[i] = acc;
    }
}

void oracle_sum_squared_f64(const uint16_t *pts, size_t n, size_t d, double *sums) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)n; ++i) {
        double acc = 0.0;
        for (size_t k = 0; k < d; ++k) {
            double x = (double)oracle_f16_to_f32(pts[(size_t)i * d + k]);
            acc += x * x;
        }
        sums[i] = acc;
    }
}

/* ------------------------------------------------------------------------------------
 * On-demand rasterizer: chunk index -> tile origin.
 * Follows rasterizer/onDemandRasterizer.cuh:50-71 (initialize) and :78-108 (nextChunk):
 * indices are dealt in raster squares of raster_size x raster_size tiles, squares in
 * row-major order, tiles row-major inside a square.  Returns 0 when idx is past the end
 * (the reference's nullopt), 1 otherwise.
 * ---------------------------------------------------------------------------------- */
int oracle_raster_coord(unsigned long long idx, unsigned long long chunk_rows, unsigned long long chunk_cols,
                        unsigned int raster_size, int tile_m, int tile_n, int *row, int *col) {
    unsigned long long max_chunks = chunk_rows * chunk_cols;
    if (idx >= max_chunks) return 0;
    unsigned long long area = (unsigned long long)raster_size * raster_size;
    unsigned long long raster_cols = chunk_cols / raster_size;
    unsigned long long rc = idx / area;
    unsigned int base_row = (unsigned int)((rc / raster_cols) * raster_size);
    unsigned int base_col = (unsigned int)((rc % raster_cols) * raster_size);
    unsigned long long local = idx % area;
    unsigned int lr = (unsigned int)(local / raster_size), lc = (unsigned int)(local % raster_size);
    *row = (int)((base_row + lr) * (unsigned int)tile_m);
    *col = (int)((base_col + lc) * (unsigned int)tile_n);
    return 1;
}

/* ------------------------------------------------------------------------------------
 * Pair buffer reservation model.
 * Follows pair.cuh:123-133 (getSpace): `found` always advances by n; the request is
 * stored (and `stored` advances) only when old+n <= max_pairs.  Returns the slot index or
 * -1 for the reference's nullptr.
 * ---------------------------------------------------------------------------------- */
long long oracle_pairs_get_space(unsigned long long *found, unsigned long long *stored, unsigned long long max_pairs,
                                 unsigned int n) {
    unsigned long long old = *found;
    *found += n;
    if (old + n > max_pairs) return -1;
    *stored += n;
    return (long long)old;
}

/* ------------------------------------------------------------------------------------
 * Brute-force self-joins.  Pair definition follows warpMma.cuh:241-267 and
 * findPairs.cuh:678: ordered pairs (q,c), q==c included, both (q,c) and (c,q), kept when
 * d^2 <= eps^2, only for q,c < n (padding excluded).  Output order is row-major (q then
 * c), which is the order pair.cuh:39-45,151-158 sorts into.
 *
 * oracle_self_join_f64: ground truth.  d^2 = sum_k (x_k - y_k)^2 in FP64 on the
 *   FP16-quantised coordinates, compared with eps*eps in FP64.
 * oracle_self_join_f32: the reference's arithmetic model.  s_i from the caller (RZ sums to
 *   mirror sumSquared.cuh), acc = sequential FP32 dot product, d^2 = (s_q + s_c) - 2*acc
 *   in FP32 (warpMma.cuh:241-242), compared with (float)(eps*eps) (findPairs.cuh:678).
 *
 * Both return the number of pairs found; up to `cap` pairs are written to out_q/out_c.
 * `d` is the row stride in halves (padded dimensionality).
 * ---------------------------------------------------------------------------------- */
static void widen_rows_f32(const uint16_t *pts, size_t n, size_t d, float *dst) {
#pragma omp parallel for schedule(static)
    for (long long i = 0; i < (long long)(n * d); ++i) dst[i] = oracle_f16_to_f32(pts[i]);
}

typedef struct {
    int *q, *c;
    size_t n, cap;
} pairvec;

static void pv_push(pairvec *v, int q, int c) {
    if (v->n == v->cap) {
        v->cap = v->cap ? v->cap * 2 : 1024;
        v->q = (int *)realloc(v->q, v->cap * sizeof(int));
        v->c = (int *)realloc(v->c, v->cap * sizeof(int));
    }
    v->q[v->n] = q;
    v->c[v->n] = c;
    ++v->n;
}

/* mode 0: FP64 difference form; mode 1: FP32 reference model.  Rows [q0, q1) are the
 * queries (all n points are candidates), so a bounded sample of the full join can be
 * timed or checked. */
static unsigned long long join_rows(const uint16_t *pts, size_t n, size_t d, double eps, const float *sums, int mode,
                                    size_t q0, size_t q1, int *out_q, int *out_c, unsigned long long cap) {
    float *w = (float *)malloc(n * d * sizeof(float));
    widen_rows_f32(pts, n, d, w);
    const double eps2_d = eps * eps;
    const float eps2_f = (float)(eps * eps);
    size_t nq = q1 - q0;
    pairvec *rows = (pairvec *)calloc(nq, sizeof(pairvec));
#pragma omp parallel for schedule(dynamic, 4)
    for (long long qi = 0; qi < (long long)nq; ++qi) {
        size_t q = q0 + (size_t)qi;
        const float *x = w + q * d;
        for (size_t c = 0; c < n; ++c) {
            const float *y = w + c * d;
            int hit;
            if (mode == 0) {
                double acc = 0.0;
                for (size_t k = 0; k < d; ++k) {
                    double t = (double)x[k] - (double)y[k];
                    acc += t * t;
                }
                hit = acc <= eps2_d;
            } else {
                float acc = 0.0f;
                for (size_t k = 0; k < d; ++k) acc += x[k] * y[k];
                float d2 = (sums[q] + sums[c]) - (2.0f * acc);
                hit = d2 <= eps2_f;
            }
            if (hit) pv_push(&rows[qi], (int)q, (int)c);
        }
    }
    unsigned long long found = 0;
    for (size_t qi = 0; qi < nq; ++qi) {
        for (size_t j = 0; j < rows[qi].n; ++j) {
            if (found < cap) {
                out_q[found] = rows[qi].q[j];
                out_c[found] = rows[qi].c[j];
            }
            ++found;
        }
        free(rows[qi].q);
        free(rows[qi].c);
    }
    free(rows);
    free(w);
    return found;
}

unsigned long long oracle_self_join_f64(const uint16_t *pts, size_t n, size_t d, double eps, int *out_q, int *out_c,
                                        unsigned long long cap) {
    return join_rows(pts, n, d, eps, NULL, 0, 0, n, out_q, out_c, cap);
}

unsigned long long oracle_self_join_f64_rows(const uint16_t *pts, size_t n, size_t d, double eps, size_t q0, size_t q1,
                                             int *out_q, int *out_c, unsigned long long cap) {
    return join_rows(pts, n, d, eps, NULL, 0, q0, q1, out_q, out_c, cap);
}

unsigned long long oracle_self_join_f32(const uint16_t *pts, size_t n, size_t d, double eps, const float *sums,
                                        int *out_q, int *out_c, unsigned long long cap) {
    return join_rows(pts, n, d, eps, sums, 1, 0, n, out_q, out_c, cap);
}

/* FP64 Euclidean distance of each listed pair (for the epsilon-band classifier). */
void oracle_pair_distances_f64(const uint16_t *pts, size_t d, const int *q, const int *c, size_t npairs, double *dist) {
#pragma omp parallel for schedule(static)
    for (long long p = 0; p < (long long)npairs; ++p) {
        const uint16_t *x = pts + (size_t)q[p] * d, *y = pts + (size_t)c[p] * d;
        double acc = 0.0;
        for (size_t k = 0; k < d; ++k) {
            double t = (double)oracle_f16_to_f32(x[k]) - (double)oracle_f16_to_f32(y[k]);
            acc += t * t;
        }
        dist[p] = sqrt(acc);
    }
}

/* ------------------------------------------------------------------------------------
 * Merge-walk comparison of two row-major-sorted pair lists.
 * Follows results/scripts/compute_accuracy.py:70-130 (compute_pair_stats): counts pairs
 * in both lists, only in the right list, only in the left list.  stats[0..4] =
 * {both, right_only, left_only, left_total, right_total}.  When only_q/only_c/only_side
 * are non-NULL the one-sided pairs are written there (side 0 = left only, 1 = right only),
 * up to only_cap.
 * ---------------------------------------------------------------------------------- */
void oracle_pair_stats(const int *lq, const int *lc, size_t nl, const int *rq, const int *rc, size_t nr,
                       unsigned long long stats[5], int *only_q, int *only_c, int *only_side, size_t only_cap) {
    size_t i = 0, j = 0, both = 0, lo = 0, ro = 0, w = 0;
    while (i < nl || j < nr) {
        int side;
        if (i < nl && j < nr) {
            if (lq[i] == rq[j] && lc[i] == rc[j]) {
                ++both;
                ++i;
                ++j;
                continue;
            }
            side = (lq[i] < rq[j] || (lq[i] == rq[j] && lc[i] < rc[j])) ? 0 : 1;
        } else {
            side = (i < nl) ? 0 : 1;
        }
        if (side == 0) {
            if (only_q && w < only_cap) {
                only_q[w] = lq[i];
                only_c[w] = lc[i];
                only_side[w] = 0;
                ++w;
            }
            ++lo;
            ++i;
        } else {
            if (only_q && w < only_cap) {
                only_q[w] = rq[j];
                only_c[w] = rc[j];
                only_side[w] = 1;
                ++w;
            }
            ++ro;
            ++j;
        }
    }
    stats[0] = both;
    stats[1] = ro;
    stats[2] = lo;
    stats[3] = nl;
    stats[4] = nr;
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
