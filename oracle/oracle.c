/*
 * CPU oracle for the three operator families: row softmax (plain and
 * padding-masked), LayerNorm (y, mean, rstd) and GEMM (fp32, and fp16/bf16
 * inputs with wide accumulation).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared with; it is never part of the product path.  Only the tests, the
 * smoke check and the CPU-baseline leg of the benchmark load it.
 *
 * Every function restates the arithmetic the reference intends, with float
 * (or half) inputs and outputs and DOUBLE internal arithmetic, and cites the
 * reference lines it follows.  The reference's device code has arithmetic
 * bugs (scalar Subtract returns a+b, common/functors.h:164-170; WelfordMerge
 * divides M2 by count-1 inside every merge, nn_operators/layernorm/
 * layernorm.h:48); those are not reproduced: the oracle computes the
 * mathematically intended operator.
 *
 * Pinning: the reference holds no golden vectors for softmax or LayerNorm and
 * only the identity known-answer inputs (nn_operators/gemm/main.cu:217-235)
 * for GEMM.  The oracle is therefore pinned by closed forms, invariants,
 * brute force in long double and library routines (tests/test_oracle_*.py).
 *
 * Plain C99 + optional OpenMP (parallel over rows).
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void oracle_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------ */
/* half / bfloat16 conversions (bit-level, round-to-nearest-even)           */
/* ------------------------------------------------------------------------ */

static double f16_bits_to_double(uint16_t h) {
    int sign = (h >> 15) & 1;
    int exp = (h >> 10) & 0x1f;
    int man = h & 0x3ff;
    double v;
    if (exp == 0) {
        v = ldexp((double)man, -24);
    } else if (exp == 31) {
        v = man ? NAN : INFINITY;
    } else {
        v = ldexp((double)(man | 0x400), exp - 25);
    }
    return sign ? -v : v;
}

/* double -> binary16, one rounding (nearest, ties to even), overflow -> inf */
static uint16_t double_to_f16_bits(double d) {
    uint16_t sign = (uint16_t)(signbit(d) ? 0x8000u : 0u);
    if (isnan(d)) return (uint16_t)(sign | 0x7e00u);
    double a = fabs(d);
    if (isinf(a)) return (uint16_t)(sign | 0x7c00u);
    if (a == 0.0) return sign;
    int e;
    (void)frexp(a, &e);           /* a = m * 2^e, m in [0.5,1) => a in [2^(e-1), 2^e) */
    int unbiased = e - 1;
    double q;                      /* a expressed in units of the target ulp */
    int biased;
    if (unbiased < -14) {          /* subnormal range: ulp = 2^-24 */
        q = ldexp(a, 24);
        biased = 0;
    } else {
        q = ldexp(a, 10 - unbiased);   /* in [1024, 2048) */
        biased = unbiased + 15;
    }
    double r = nearbyint(q);       /* default rounding mode: ties-to-even */
    uint32_t bits;
    if (biased == 0) {
        bits = (uint32_t)r;        /* may carry into exponent 1: correct */
    } else {
        bits = ((uint32_t)biased << 10) + ((uint32_t)r - 1024u);
    }
    if (bits >= 0x7c00u) bits = 0x7c00u;
    return (uint16_t)(sign | bits);
}

static double bf16_bits_to_double(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return (double)f;
}

static uint16_t double_to_bf16_bits(double d) {
    if (isnan(d)) return 0x7fc0u;
    /* bf16 keeps 8 significand bits; round the double directly */
    uint16_t sign = (uint16_t)(signbit(d) ? 0x8000u : 0u);
    double a = fabs(d);
    if (isinf(a)) return (uint16_t)(sign | 0x7f80u);
    if (a == 0.0) return sign;
    int e;
    (void)frexp(a, &e);
    int unbiased = e - 1;
    double q;
    int biased;
    if (unbiased < -126) {
        q = ldexp(a, 133);         /* ulp of bf16 subnormal = 2^-133 */
        biased = 0;
    } else {
        q = ldexp(a, 7 - unbiased);    /* in [128, 256) */
        biased = unbiased + 127;
    }
    double r = nearbyint(q);
    uint32_t bits;
    if (biased == 0) bits = (uint32_t)r;
    else bits = ((uint32_t)biased << 7) + ((uint32_t)r - 128u);
    if (bits >= 0x7f80u) bits = 0x7f80u;
    return (uint16_t)(sign | bits);
}

ORACLE_API void oracle_f16_to_f64(const uint16_t *in, double *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f16_bits_to_double(in[i]);
}
ORACLE_API void oracle_f64_to_f16(const double *in, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = double_to_f16_bits(in[i]);
}
ORACLE_API void oracle_bf16_to_f64(const uint16_t *in, double *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_bits_to_double(in[i]);
}
ORACLE_API void oracle_f64_to_bf16(const double *in, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = double_to_bf16_bits(in[i]);
}

/* ------------------------------------------------------------------------ */
/* Row softmax                                                              */
/* ------------------------------------------------------------------------ */

#define ORACLE_MASK_VALUE (-10000.0)

/*
 * Row softmax along the last dimension of a row-major [rows, cols] matrix.
 * Follows nn_operators/softmax/softmax.h:32-57: running max initialised to
 * -FLT_MAX (:33), max over the row (:35-42), exp(x - max) and its sum
 * (:45-52), divide (:54-57).  "x - max" is the intended operator; the
 * reference's Subtract functor adds instead (common/functors.h:168).
 *
 * Padding mask (not in the reference): when valid_len is non-NULL, row r
 * belongs to sequence r / rows_per_seq and every column j >= valid_len[seq]
 * takes the value -10000 before the softmax.
 */
ORACLE_API int oracle_softmax_f32(const float *in, float *out, int64_t rows, int64_t cols,
                                  const int32_t *valid_len, int64_t rows_per_seq) {
    if (rows < 0 || cols <= 0) return 1;
    if (valid_len && rows_per_seq <= 0) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *x = in + r * cols;
        float *y = out + r * cols;
        int64_t vl = cols;
        if (valid_len) {
            vl = valid_len[r / rows_per_seq];
            if (vl < 0) vl = 0;
            if (vl > cols) vl = cols;
        }
        double mx = -(double)FLT_MAX;
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? (double)x[j] : ORACLE_MASK_VALUE;
            if (v > mx) mx = v;
        }
        double sum = 0.0;
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? (double)x[j] : ORACLE_MASK_VALUE;
            sum += exp(v - mx);
        }
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? (double)x[j] : ORACLE_MASK_VALUE;
            y[j] = (float)(exp(v - mx) / sum);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* LayerNorm                                                                */
/* ------------------------------------------------------------------------ */

/*
 * LayerNorm over the last dimension, two passes in double.
 * y = (x - mean) * rsqrt(var + eps) [* gamma + beta]
 * (nn_operators/layernorm/layernorm.h:184-195, with the intended x - mean).
 * var divides by N (unbiased == 0) or N - 1 (unbiased != 0; the reference's
 * intent at layernorm.h:48).  mean, rstd, gamma, beta may be NULL.
 * A row holding a NaN or an infinity has no statistics: the sum of squared
 * deviations is NaN (inf - inf), so rstd and y are NaN, and mean is reported as
 * NaN too (the reference's streaming update makes its mean NaN as soon as an
 * element follows an infinity: d = x - mu = -inf, mu += d/n, layernorm.h:16-18).
 */
ORACLE_API int oracle_layernorm_f32(const float *in, float *out, float *mean_out, float *rstd_out,
                                    const float *gamma, const float *beta,
                                    int64_t rows, int64_t cols, double eps, int unbiased) {
    if (rows < 0 || cols <= 0) return 1;
    if (unbiased && cols < 2) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *x = in + r * cols;
        double s = 0.0;
        for (int64_t j = 0; j < cols; ++j) s += (double)x[j];
        double mean = s / (double)cols;
        double m2 = 0.0;
        for (int64_t j = 0; j < cols; ++j) {
            double d = (double)x[j] - mean;
            m2 += d * d;
        }
        double var = m2 / (double)(unbiased ? cols - 1 : cols);
        if (isnan(m2)) mean = NAN;
        double rstd = 1.0 / sqrt(var + eps);
        if (out) {
            float *y = out + r * cols;
            for (int64_t j = 0; j < cols; ++j) {
                double v = ((double)x[j] - mean) * rstd;
                if (gamma) v *= (double)gamma[j];
                if (beta) v += (double)beta[j];
                y[j] = (float)v;
            }
        }
        if (mean_out) mean_out[r] = (float)mean;
        if (rstd_out) rstd_out[r] = (float)rstd;
    }
    return 0;
}

/*
 * The same two operators on 16-bit storage (binary16 or bfloat16 bit patterns; gamma and beta
 * in the same type): inputs are widened exactly, the arithmetic is the double arithmetic above,
 * and the result is rounded once to the storage type.  out64 (optional) receives the unrounded
 * values.  The reference carries half specialisations of its functors for this case
 * (common/functors.h:71-77,105-111).
 */
static double bits16_to_double(uint16_t b, int bf16) { return bf16 ? bf16_bits_to_double(b) : f16_bits_to_double(b); }
static uint16_t double_to_bits16(double d, int bf16) { return bf16 ? double_to_bf16_bits(d) : double_to_f16_bits(d); }

ORACLE_API int oracle_softmax_16(const uint16_t *in, uint16_t *out, double *out64, int64_t rows, int64_t cols,
                                 const int32_t *valid_len, int64_t rows_per_seq, int bf16) {
    if (rows < 0 || cols <= 0) return 1;
    if (valid_len && rows_per_seq <= 0) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const uint16_t *x = in + r * cols;
        int64_t vl = cols;
        if (valid_len) {
            vl = valid_len[r / rows_per_seq];
            if (vl < 0) vl = 0;
            if (vl > cols) vl = cols;
        }
        double mx = -(double)FLT_MAX;
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? bits16_to_double(x[j], bf16) : ORACLE_MASK_VALUE;
            if (v > mx) mx = v;
        }
        double sum = 0.0;
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? bits16_to_double(x[j], bf16) : ORACLE_MASK_VALUE;
            sum += exp(v - mx);
        }
        for (int64_t j = 0; j < cols; ++j) {
            double v = j < vl ? bits16_to_double(x[j], bf16) : ORACLE_MASK_VALUE;
            double y = exp(v - mx) / sum;
            if (out64) out64[r * cols + j] = y;
            if (out) out[r * cols + j] = double_to_bits16(y, bf16);
        }
    }
    return 0;
}

ORACLE_API int oracle_layernorm_16(const uint16_t *in, uint16_t *out, double *out64, float *mean_out,
                                   float *rstd_out, const uint16_t *gamma, const uint16_t *beta, int64_t rows,
                                   int64_t cols, double eps, int unbiased, int bf16) {
    if (rows < 0 || cols <= 0) return 1;
    if (unbiased && cols < 2) return 1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const uint16_t *x = in + r * cols;
        double s = 0.0;
        for (int64_t j = 0; j < cols; ++j) s += bits16_to_double(x[j], bf16);
        double mean = s / (double)cols;
        double m2 = 0.0;
        for (int64_t j = 0; j < cols; ++j) {
            double d = bits16_to_double(x[j], bf16) - mean;
            m2 += d * d;
        }
        double var = m2 / (double)(unbiased ? cols - 1 : cols);
        if (isnan(m2)) mean = NAN;
        double rstd = 1.0 / sqrt(var + eps);
        for (int64_t j = 0; j < cols; ++j) {
            double v = (bits16_to_double(x[j], bf16) - mean) * rstd;
            if (gamma) v *= bits16_to_double(gamma[j], bf16);
            if (beta) v += bits16_to_double(beta[j], bf16);
            if (out64) out64[r * cols + j] = v;
            if (out) out[r * cols + j] = double_to_bits16(v, bf16);
        }
        if (mean_out) mean_out[r] = (float)mean;
        if (rstd_out) rstd_out[r] = (float)rstd;
    }
    return 0;
}

/* Welford triplets in float, as the reference keeps them (count is a float). */
static void welford_update_f32(float *count, float *mean, float *m2, float v) {
    /* nn_operators/layernorm/layernorm.h:13-23 */
    *count += 1.0f;
    float delta = v - *mean;
    *mean += delta / *count;
    float delta2 = v - *mean;
    *m2 += delta * delta2;
}

static void welford_merge_f32(float *ca, float *ma, float *m2a, float cb, float mb, float m2b) {
    /* nn_operators/layernorm/layernorm.h:36-47 (Chan merge); line 48's
     * division of M2 by count-1 inside the merge is the bug left out. */
    float cab = *ca + cb;
    if (cab == 0.0f) return;
    float delta = mb - *ma;
    float cb_over = cb / cab;
    float m2 = *m2a + m2b + delta * delta * (*ca) * cb_over;
    *ca = cab;
    *ma += delta * cb_over;
    *m2a = m2;
}

/*
 * Float-only restatement with the reference's lane structure: `lanes` lanes,
 * each owning vec_len-wide vectors at column (lane + lanes*k)*vec_len
 * (layernorm.h:172-179), one Welford triplet per vector slot, slots folded
 * in-lane (layernorm.h:68-75), lanes merged by a halving tree
 * (layernorm.h:56-61).  It exists to test the merge algebra; the parity
 * oracle is oracle_layernorm_f32.
 */
ORACLE_API int oracle_layernorm_welford_f32(const float *in, float *out, float *mean_out,
                                            float *rstd_out, const float *gamma, const float *beta,
                                            int64_t rows, int64_t cols, float eps, int unbiased,
                                            int lanes, int vec_len) {
    if (rows < 0 || cols <= 0 || lanes <= 0 || lanes > 1024 || vec_len <= 0 || vec_len > 16) return 1;
    if (cols % vec_len) return 1;
    if (lanes & (lanes - 1)) return 1;
    const int64_t nvec = cols / vec_len;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *x = in + r * cols;
        float lc[1024], lm[1024], l2[1024];
        for (int l = 0; l < lanes; ++l) {
            float c[16] = {0}, m[16] = {0}, s[16] = {0};
            for (int64_t v = l; v < nvec; v += lanes)
                for (int e = 0; e < vec_len; ++e)
                    welford_update_f32(&c[e], &m[e], &s[e], x[v * vec_len + e]);
            for (int e = 1; e < vec_len; ++e) welford_merge_f32(&c[0], &m[0], &s[0], c[e], m[e], s[e]);
            lc[l] = c[0]; lm[l] = m[0]; l2[l] = s[0];
        }
        for (int off = lanes / 2; off > 0; off >>= 1)
            for (int l = 0; l < off; ++l)
                welford_merge_f32(&lc[l], &lm[l], &l2[l], lc[l + off], lm[l + off], l2[l + off]);
        float mean = lm[0];
        float var = l2[0] / (float)(unbiased ? cols - 1 : cols);
        float rstd = 1.0f / sqrtf(var + eps);
        if (out) {
            float *y = out + r * cols;
            for (int64_t j = 0; j < cols; ++j) {
                float v = (x[j] - mean) * rstd;
                if (gamma) v *= gamma[j];
                if (beta) v += beta[j];
                y[j] = v;
            }
        }
        if (mean_out) mean_out[r] = mean;
        if (rstd_out) rstd_out[r] = rstd;
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* GEMM                                                                     */
/* ------------------------------------------------------------------------ */

/*
 * D[M,N] = alpha * A[M,K] * B[K,N] + beta * C[M,N], all row-major fp32,
 * sequential-k dot product (the commented CPU loop of
 * nn_operators/gemm/main.cu:162-167) accumulated in double; epilogue of
 * nn_operators/gemm/simt_gemm.h:325-373 (D = acc + C when C is given, else
 * acc) generalised with alpha/beta.  C may be NULL (treated as beta = 0).
 * absprod (may be NULL) receives sum_k |A_ik| |B_kj|, the scale of the
 * summation-order error bound.
 */
ORACLE_API int oracle_sgemm_f32(int64_t m, int64_t n, int64_t k, double alpha, const float *A,
                                const float *B, double beta, const float *C, float *D,
                                double *absprod) {
    if (m < 0 || n < 0 || k < 0) return 1;
#pragma omp parallel
    {
    double *acc = (double *)__builtin_malloc(sizeof(double) * 2 * (size_t)(n > 0 ? n : 1));
    double *aacc = acc + n;
#pragma omp for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t j = 0; j < n; ++j) { acc[j] = 0.0; aacc[j] = 0.0; }
        for (int64_t kk = 0; kk < k; ++kk) {
            double a = (double)A[i * k + kk];
            const float *brow = B + kk * n;
            double fa = fabs(a);
            for (int64_t j = 0; j < n; ++j) {
                double b = (double)brow[j];
                acc[j] += a * b;
                aacc[j] += fa * fabs(b);
            }
        }
        for (int64_t j = 0; j < n; ++j) {
            double v = alpha * acc[j];
            if (C && beta != 0.0) v += beta * (double)C[i * n + j];
            D[i * n + j] = (float)v;
            if (absprod) absprod[i * n + j] = aacc[j];
        }
    }
    __builtin_free(acc);
    }
    return 0;
}

/*
 * Tensor-core-path GEMM: A [M,K] row-major, B logical [K,N] stored row-major
 * (b_col_major == 0, the reference layout, nn_operators/gemm/
 * tensor_core_gemm.h:178) or column-major (b_col_major != 0: memory [N][K]),
 * C/D [M,N] row-major.  Inputs and outputs are binary16 (is_bf16 == 0) or
 * bfloat16 bit patterns; products and sums are exact in double up to its own
 * rounding; one final rounding to the 16-bit type.  d64 (may be NULL)
 * receives the unrounded double result, absprod as above.
 */
/* Epilogue activations: 0 none; 1 GELU(x) = x/2 (1 + erf(x / sqrt 2)); 2 its tanh form
 * x/2 (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))). */
static double apply_activation(double x, int act) {
    if (act == 1) return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440));
    if (act == 2) return 0.5 * x * (1.0 + tanh(0.79788456080286535588 * (x + 0.044715 * x * x * x)));
    return x;
}

/* D = act(alpha A B + beta C + bias[n]): the epilogue of the feed-forward up-projection that the
 * 16384 x 3072 x 768 configuration stands for.  bias (may be NULL) is a 16-bit vector of length n. */
ORACLE_API int oracle_gemm_16_bias_act(int64_t m, int64_t n, int64_t k, double alpha, const uint16_t *A,
                                       const uint16_t *B, int b_col_major, double beta, const uint16_t *C,
                                       const uint16_t *bias, int act, uint16_t *D, int is_bf16, double *d64,
                                       double *absprod) {
    if (m < 0 || n < 0 || k < 0 || act < 0 || act > 2) return 1;
    /* widen B once into [N][K] doubles so the inner loop is contiguous */
    double *Bt = (double *)__builtin_malloc(sizeof(double) * (size_t)(n * k > 0 ? n * k : 1));
    if (!Bt) return 2;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; ++j)
        for (int64_t kk = 0; kk < k; ++kk) {
            uint16_t bits = b_col_major ? B[j * k + kk] : B[kk * n + j];
            Bt[j * k + kk] = is_bf16 ? bf16_bits_to_double(bits) : f16_bits_to_double(bits);
        }
#pragma omp parallel
    {
    double *arow = (double *)__builtin_malloc(sizeof(double) * (size_t)(k > 0 ? k : 1));
#pragma omp for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t kk = 0; kk < k; ++kk)
            arow[kk] = is_bf16 ? bf16_bits_to_double(A[i * k + kk]) : f16_bits_to_double(A[i * k + kk]);
        for (int64_t j = 0; j < n; ++j) {
            const double *bcol = Bt + j * k;
            double acc = 0.0, aacc = 0.0;
            for (int64_t kk = 0; kk < k; ++kk) {
                acc += arow[kk] * bcol[kk];
                aacc += fabs(arow[kk] * bcol[kk]);
            }
            double v = alpha * acc;
            if (C && beta != 0.0) {
                uint16_t cb = C[i * n + j];
                v += beta * (is_bf16 ? bf16_bits_to_double(cb) : f16_bits_to_double(cb));
            }
            if (bias) v += is_bf16 ? bf16_bits_to_double(bias[j]) : f16_bits_to_double(bias[j]);
            v = apply_activation(v, act);
            if (D) D[i * n + j] = is_bf16 ? double_to_bf16_bits(v) : double_to_f16_bits(v);
            if (d64) d64[i * n + j] = v;
            if (absprod) absprod[i * n + j] = aacc;
        }
    }
    __builtin_free(arow);
    }
    __builtin_free(Bt);
    return 0;
}

ORACLE_API int oracle_gemm_16(int64_t m, int64_t n, int64_t k, double alpha, const uint16_t *A,
                              const uint16_t *B, int b_col_major, double beta, const uint16_t *C,
                              uint16_t *D, int is_bf16, double *d64, double *absprod) {
    return oracle_gemm_16_bias_act(m, n, k, alpha, A, B, b_col_major, beta, C, NULL, 0, D, is_bf16, d64, absprod);
}
