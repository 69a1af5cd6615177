/*
 * Per-word CPU restatement of the reference's signature / log-signature algorithms.
 *
 * TEST INFRASTRUCTURE ONLY: built by oracle/build.py into oracle/liboracle_words.so and loaded by
 * oracle/words_oracle.py from the test-suite, the smoke check and the CPU-baseline leg of the
 * benchmark.  The shipped library never links or calls it.
 *
 * Every routine walks one word at a time exactly as the corresponding reference kernel does with
 * one thread per word; the loops are written for a CPU (plain C, OpenMP over the batch).
 * Compiled twice, with -DREAL=double -DSUF=_f64 and -DREAL=float -DSUF=_f32.
 *
 * Parity status: every function below is pinned by tests/test_oracle_math.py against closed forms,
 * brute-force iterated sums and the level-tensor formulation in oracle/tensor_oracle.py.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL double
#define SUF _f64
#endif
#define CAT2(a, b) a##b
#define CAT(a, b) CAT2(a, b)
#define FN(name) CAT(name, SUF)

#define MAX_DEPTH 12

/* word code -> letters, first letter most significant
 * (src/pathsig/utils/word_mappings.cuh:17-28, src/pathsig/projections.py:101-105) */
static void decode_word(uint64_t code, int degree, int64_t d, int *letters) {
    for (int pos = degree - 1; pos >= 0; --pos) {
        letters[pos] = (int)(code % (uint64_t)d);
        code /= (uint64_t)d;
    }
}

/* compensated accumulation (src/pathsig/forward/sig_kernels.cu:51-66) */
static inline void kahan_add(volatile REAL *sum, REAL to_add, volatile REAL *comp) {
    volatile REAL y = to_add - *comp;
    volatile REAL t = *sum + y;
    *comp = (t - *sum) - y;
    *sum = t;
}

/* One Horner/Chen step on the prefixes of one word: p <- p (x) exp(sign*dx)
 * (src/pathsig/forward/sig_kernels.cu:139-152; with sign=-1 and no compensation it is the
 * roll-back of src/pathsig/backward/sig_backward_kernels.cu:187-201).  top = highest level updated. */
static inline void chen_step(REAL *p, REAL *comp, const int *letters, const REAL *dx, int top, REAL sign) {
    for (int m = top; m > 0; --m) {
        REAL h = 0;
        for (int k = 0; k <= m - 1; ++k) {
            const REAL scale = sign * dx[letters[k]] * ((REAL)1 / (REAL)(m - k));
            h = scale * (p[k] + h);
        }
        if (comp) kahan_add(&p[m], h, &comp[m]);
        else p[m] += h;
    }
}

typedef struct {
    int64_t size;          /* words at this level              */
    int64_t offset;        /* first output column of the level */
    const int64_t *codes;  /* NULL: dense, code == index       */
} level_plan;

/* Output layout: levels concatenated; a level is dense (d^k columns, code == column) when its size
 * is d^k, otherwise its columns follow the stored codes, which are concatenated over the non-full
 * levels only (src/pathsig/forward/sig_launch.cu:171-206). */
static int64_t plan_levels(int64_t d, int depth, const int64_t *level_sizes, const int64_t *codes, level_plan *plan) {
    int64_t off = 0, enc = 0, dpow = 1;
    for (int k = 1; k <= depth; ++k) {
        dpow *= d;
        int64_t size = level_sizes ? level_sizes[k] : dpow;
        plan[k].size = size;
        plan[k].offset = off;
        plan[k].codes = NULL;
        if (level_sizes && size != dpow) {
            plan[k].codes = codes + enc;
            enc += size;
        }
        off += size;
    }
    return off;
}

/* A1: forward signature (src/pathsig/forward/sig_kernels.cu:79-157). */
int FN(ow_sig_forward)(const REAL *path, REAL *sig, int64_t B, int64_t L, int64_t d, int depth,
                       const int64_t *level_sizes, const int64_t *codes,
                       const int32_t *windows, int64_t W) {
    if (depth < 1 || depth > MAX_DEPTH || L < 2) return -1;
    level_plan plan[MAX_DEPTH + 1];
    const int64_t S = plan_levels(d, depth, level_sizes, codes, plan);
    const int64_t nwin = windows ? W : 1;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t w = 0; w < nwin; ++w) {
            const int64_t start = windows ? windows[2 * w] : 0;
            const int64_t end = windows ? windows[2 * w + 1] : L;
            const int64_t steps = end - start - 1;
            const REAL *x = path + (b * L + start) * d;
            REAL *out = sig + (b * nwin + w) * S;
            REAL *dx = (REAL *)malloc(sizeof(REAL) * (size_t)d);
            for (int deg = 1; deg <= depth; ++deg) {
                for (int64_t i = 0; i < plan[deg].size; ++i) {
                    const uint64_t code = plan[deg].codes ? (uint64_t)plan[deg].codes[i] : (uint64_t)i;
                    int letters[MAX_DEPTH];
                    decode_word(code, deg, d, letters);
                    REAL p[MAX_DEPTH + 1] = {0}, comp[MAX_DEPTH + 1] = {0};
                    p[0] = 1;
                    for (int64_t t = 0; t < steps; ++t) {
                        for (int k = 0; k < deg; ++k) {
                            const int a = letters[k];
                            dx[a] = x[(t + 1) * d + a] - x[t * d + a];
                        }
                        chen_step(p, comp, letters, dx, deg, (REAL)1);
                    }
                    out[plan[deg].offset + i] = p[deg];
                }
            }
            free(dx);
        }
    }
    return 0;
}

/* A2 + A3: signature backward (src/pathsig/backward/sig_backward_kernels.cu:61-343 and :347-377;
 * prefix initialisation policy of src/pathsig/backward/sig_backward_launch.cu:206-221,267). */
int FN(ow_sig_backward)(const REAL *path, const REAL *sig, const REAL *grad_sig, REAL *grad_path,
                        int64_t B, int64_t L, int64_t d, int depth,
                        const int64_t *level_sizes, const int64_t *codes,
                        const int32_t *windows, int64_t W) {
    if (depth < 1 || depth > MAX_DEPTH || L < 2) return -1;
    level_plan plan[MAX_DEPTH + 1];
    const int64_t S = plan_levels(d, depth, level_sizes, codes, plan);
    const int64_t nwin = windows ? W : 1;
    /* a level may read its prefixes from the saved signature only while all lower levels are dense */
    int recompute[MAX_DEPTH + 1];
    {
        int flag = 0;
        int64_t dpow = 1;
        for (int k = 1; k <= depth; ++k) {
            dpow *= d;
            recompute[k] = flag;
            if (plan[k].size == 0 || plan[k].size != dpow) flag = 1;
        }
    }
#pragma omp parallel for schedule(dynamic)
    for (int64_t b = 0; b < B; ++b) {
        REAL *ginc = (REAL *)calloc((size_t)((L - 1) * d), sizeof(REAL));
        REAL *dx = (REAL *)malloc(sizeof(REAL) * (size_t)d);
        for (int64_t w = 0; w < nwin; ++w) {
            const int64_t start = windows ? windows[2 * w] : 0;
            const int64_t end = windows ? windows[2 * w + 1] : L;
            const int64_t steps = end - start - 1;
            const REAL *x = path + (b * L + start) * d;
            const REAL *s = sig + (b * nwin + w) * S;
            const REAL *g = grad_sig + (b * nwin + w) * S;
            REAL *gi = ginc + start * d;
            for (int deg = 1; deg <= depth; ++deg) {
                for (int64_t i = 0; i < plan[deg].size; ++i) {
                    const uint64_t code = plan[deg].codes ? (uint64_t)plan[deg].codes[i] : (uint64_t)i;
                    int letters[MAX_DEPTH];
                    decode_word(code, deg, d, letters);
                    const REAL gval = g[plan[deg].offset + i];
                    REAL pref[MAX_DEPTH + 1] = {0}, suf[MAX_DEPTH + 1] = {0}, lg[MAX_DEPTH];
                    pref[0] = 1;
                    suf[0] = 1;
                    if (recompute[deg]) { /* :134-157 */
                        for (int64_t t = 0; t < steps; ++t) {
                            for (int k = 0; k < deg; ++k) dx[letters[k]] = x[(t + 1) * d + letters[k]] - x[t * d + letters[k]];
                            chen_step(pref, NULL, letters, dx, deg - 1, (REAL)1);
                        }
                    } else { /* :158-171: dense offsets sum_{j<k} d^j + code(prefix) */
                        uint64_t off = 0, dpow = (uint64_t)d, pw = 0;
                        for (int lvl = 1; lvl < deg; ++lvl) {
                            pw = pw * (uint64_t)d + (uint64_t)letters[lvl - 1];
                            pref[lvl] = s[off + pw];
                            off += dpow;
                            dpow *= (uint64_t)d;
                        }
                    }
                    pref[deg] = s[plan[deg].offset + i]; /* :173 */
                    for (int64_t t = steps - 1; t >= 0; --t) {
                        for (int k = 0; k < deg; ++k) dx[letters[k]] = x[(t + 1) * d + letters[k]] - x[t * d + letters[k]];
                        chen_step(pref, NULL, letters, dx, deg, (REAL)-1); /* :187-201 */
                        /* :204-253  prefix x (product of increments over a segment, one factor removed) x suffix */
                        for (int q = 0; q < deg; ++q) lg[q] = 0;
                        for (int pl = 0; pl < deg; ++pl) {
                            const REAL pv = pref[pl];
                            REAL prev_prod = 1;
                            for (int lp = pl; lp < deg; ++lp) {
                                if (lp > pl) prev_prod *= dx[letters[lp - 1]] * ((REAL)1 / (REAL)(lp - pl + 1));
                                REAL tp = prev_prod;
                                REAL tg = tp * suf[deg - lp - 1];
                                int denom = lp - pl + 2;
                                for (int pos = lp + 1; pos < deg; ++pos, ++denom) {
                                    tp *= dx[letters[pos]] * ((REAL)1 / (REAL)denom);
                                    tg += tp * suf[deg - pos - 1];
                                }
                                lg[lp] += tg * pv;
                            }
                        }
                        for (int q = 0; q < deg; ++q) gi[t * d + letters[q]] += lg[q] * gval; /* :286-318 */
                        /* :321-339  suffix <- exp(dx) (x) suffix */
                        for (int m = deg - 1; m > 0; --m) {
                            const int base = deg - m;
                            REAL h = 0;
                            for (int pp = m; pp >= 1; --pp) {
                                const REAL scale = dx[letters[base + pp - 1]] * ((REAL)1 / (REAL)pp);
                                h = scale * (suf[m - pp] + h);
                            }
                            suf[m] += h;
                        }
                    }
                }
            }
        }
        /* :347-377 increment gradient -> path gradient */
        REAL *gp = grad_path + b * L * d;
        for (int64_t t = 0; t < L; ++t)
            for (int64_t j = 0; j < d; ++j) {
                if (t == 0) gp[j] = -ginc[j];
                else if (t == L - 1) gp[t * d + j] = ginc[(L - 2) * d + j];
                else gp[t * d + j] = ginc[(t - 1) * d + j] - ginc[t * d + j];
            }
        free(dx);
        free(ginc);
    }
    return 0;
}

/* hybrid layout of the two log-signature ops: levels < depth dense, top level `top_size` columns
 * taken from top_codes unless full (src/pathsig/forward/sig_launch.cu:300-312). */
static int64_t plan_hybrid(int64_t d, int depth, int64_t top_size, const int64_t *top_codes, level_plan *plan) {
    int64_t off = 0, dpow = 1;
    for (int k = 1; k <= depth; ++k) {
        dpow *= d;
        plan[k].size = (k == depth) ? top_size : dpow;
        plan[k].offset = off;
        plan[k].codes = (k == depth && top_size != dpow) ? top_codes : NULL;
        off += plan[k].size;
    }
    return off;
}

/* A6: signature -> log-signature and the P cache (src/pathsig/forward/sig_kernels.cu:161-241). */
int FN(ow_logsig_forward)(const REAL *sig, REAL *P, REAL *logsig, int64_t rows, int64_t d, int depth,
                          int64_t top_size, const int64_t *top_codes) {
    if (depth < 1 || depth > MAX_DEPTH) return -1;
    level_plan plan[MAX_DEPTH + 1];
    const int64_t S = plan_hybrid(d, depth, top_size, top_codes, plan);
#pragma omp parallel for schedule(dynamic)
    for (int64_t r = 0; r < rows; ++r) {
        const REAL *s = sig + r * S;
        REAL *Pr = P + r * S * depth;
        REAL *lg = logsig + r * S;
        memset(Pr, 0, sizeof(REAL) * (size_t)(S * depth));
        for (int deg = 1; deg <= depth; ++deg) { /* ascending: level n reads P rows of lower levels */
            for (int64_t i = 0; i < plan[deg].size; ++i) {
                const uint64_t code = plan[deg].codes ? (uint64_t)plan[deg].codes[i] : (uint64_t)i;
                int letters[MAX_DEPTH];
                decode_word(code, deg, d, letters);
                REAL sufv[MAX_DEPTH + 1];
                uint64_t pind[MAX_DEPTH + 1];
                uint64_t lo = 0, dpow = 1, pw = 0;
                for (int k = 1; k < deg; ++k) { /* :197-207 */
                    dpow *= (uint64_t)d;
                    pw = pw * (uint64_t)d + (uint64_t)letters[k - 1];
                    pind[k] = pw + lo;
                    sufv[k] = s[lo + code % dpow];
                    lo += dpow;
                }
                pind[deg] = (uint64_t)(plan[deg].offset + i);
                sufv[deg] = s[pind[deg]];
                const uint64_t Poff = pind[deg] * (uint64_t)depth;
                Pr[Poff] = sufv[deg];
                REAL acc = sufv[deg];
                for (int m = 2; m <= deg; ++m) { /* :221-238 */
                    REAL pv = 0;
                    for (int k = m - 1; k < deg; ++k) pv += Pr[pind[k] * (uint64_t)depth + (uint64_t)(m - 2)] * sufv[deg - k];
                    const REAL coeff = (m & 1) ? ((REAL)1 / (REAL)m) : -((REAL)1 / (REAL)m);
                    acc += coeff * pv;
                    Pr[Poff + (uint64_t)(m - 1)] = pv;
                }
                lg[pind[deg]] = acc;
            }
        }
    }
    return 0;
}

/* A7: adjoint of A6 (src/pathsig/backward/sig_backward_kernels.cu:381-477, levels descending as in
 * src/pathsig/backward/sig_backward_launch.cu:426-456). */
int FN(ow_logsig_backward)(const REAL *sig, const REAL *P, const REAL *glogsig, REAL *gsig, int64_t rows,
                           int64_t d, int depth, int64_t top_size, const int64_t *top_codes) {
    if (depth < 1 || depth > MAX_DEPTH) return -1;
    level_plan plan[MAX_DEPTH + 1];
    const int64_t S = plan_hybrid(d, depth, top_size, top_codes, plan);
#pragma omp parallel for schedule(dynamic)
    for (int64_t r = 0; r < rows; ++r) {
        const REAL *s = sig + r * S;
        const REAL *Pr = P + r * S * depth;
        const REAL *gl = glogsig + r * S;
        REAL *gs = gsig + r * S;
        REAL *gP = (REAL *)calloc((size_t)(S * depth), sizeof(REAL));
        memset(gs, 0, sizeof(REAL) * (size_t)S);
        for (int deg = depth; deg >= 1; --deg) {
            for (int64_t i = 0; i < plan[deg].size; ++i) {
                const uint64_t code = plan[deg].codes ? (uint64_t)plan[deg].codes[i] : (uint64_t)i;
                int letters[MAX_DEPTH];
                decode_word(code, deg, d, letters);
                uint64_t pind[MAX_DEPTH + 1], sind[MAX_DEPTH + 1];
                uint64_t lo = 0, dpow = 1, pw = 0;
                for (int k = 1; k < deg; ++k) {
                    dpow *= (uint64_t)d;
                    pw = pw * (uint64_t)d + (uint64_t)letters[k - 1];
                    pind[k] = pw + lo;
                    sind[k] = lo + code % dpow;
                    lo += dpow;
                }
                const uint64_t wg = (uint64_t)(plan[deg].offset + i);
                REAL gPv[MAX_DEPTH];
                for (int m = 1; m <= deg; ++m) { /* :449-455 */
                    const REAL coeff = (m & 1) ? ((REAL)1 / (REAL)m) : -((REAL)1 / (REAL)m);
                    gPv[m - 1] = coeff * gl[wg] + gP[wg * (uint64_t)depth + (uint64_t)(m - 1)];
                }
                gs[wg] += gPv[0]; /* :458 */
                for (int m = 2; m <= deg; ++m) { /* :460-476 */
                    for (int k = m - 1; k < deg; ++k) {
                        const uint64_t pi = pind[k], si = sind[deg - k];
                        gP[pi * (uint64_t)depth + (uint64_t)(m - 2)] += gPv[m - 1] * s[si];
                        gs[si] += gPv[m - 1] * Pr[pi * (uint64_t)depth + (uint64_t)(m - 2)];
                    }
                }
            }
        }
        free(gP);
    }
    return 0;
}
