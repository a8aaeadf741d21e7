/*
 * CPU oracle for the dense GEMM path  C[M,N] = A[M,K] . B[N,K]^T  (A, B, C row-major,
 * 16-bit float storage, fp32 accumulation).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are compared
 * with and the CPU baseline that is timed beside them.  Nothing on the product path may
 * link, import or call it.
 *
 * It restates, in plain C, the arithmetic of the reference project's host-side files:
 *   reference.h:5-46      reference_cpu_gemm      -> orc_reference_cpu_gemm*()
 *   reference.h:49-76     reference_gpu_gemm_kernel (same contract, k>=K zero filled)
 *                                                  -> orc_naive_gemm()
 *   common.h:283-307      random_fill / arange_fill / constant_fill -> orc_fill_*()
 *   common.h:367-397      assert_allclose         -> orc_allclose_count()
 *   matmul_h100_optimal.cu:86-108  randomize_matrix / verify_matrix
 *                                                  -> orc_fill_normal(), orc_absdiff_count()
 *
 * The reference's own header cannot be compiled in this image (it includes <cuda.h>,
 * <cuda_fp16.h>, <curand_kernel.h>), so no reference build exists beside this file.  What
 * pins each function (closed forms, exact-integer fills, brute force, float64 BLAS, an
 * independent bf16 rounding implementation) is listed with the tests in
 * tests/test_oracle.py.  The seeded generators (orc_fill_uniform/normal) are this
 * project's own and have no counterpart in the reference, whose generators are unseeded
 * rand() and a library-defined std::normal_distribution.
 *
 * Storage types: dtype 0 = bfloat16, dtype 1 = IEEE binary16.  Both are passed as
 * uint16_t bit patterns.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_BF16 0
#define ORC_FP16 1

/* ------------------------------------------------------------------ 16-bit floats -- */

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* bfloat16 -> float is exact: the 16 bits are the top half of the binary32 pattern. */
float orc_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* float -> bfloat16, round to nearest, ties to even; NaN stays a (quiet) NaN.
 * This is what `(__nv_bfloat16)float_value` does in reference.h:40. */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float orc_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* float -> binary16, round to nearest even, overflow to inf, gradual underflow. */
uint16_t orc_f32_to_fp16(float f) {
    uint32_t u = f32_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);           /* NaN */
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* >= 65520 -> inf */
    if (a < 0x38800000u) {                                            /* below 2^-14 */
        if (a < 0x33000000u) return sign;                             /* < 2^-25 -> 0 */
        /* subnormal half: scale so that the integer part is the 10-bit mantissa */
        float v = bits_to_f32(a) * 16777216.0f;                       /* * 2^24, exact */
        float r = nearbyintf(v);                                      /* RNE by default */
        return (uint16_t)(sign | (uint16_t)r);
    }
    uint32_t lsb = (a >> 13) & 1u;
    a += 0xfffu + lsb;
    return (uint16_t)(sign | (uint16_t)((a - 0x38000000u) >> 13));
}

static inline float to_f32(uint16_t h, int dtype) {
    return dtype == ORC_BF16 ? orc_bf16_to_f32(h) : orc_fp16_to_f32(h);
}
static inline uint16_t from_f32(float f, int dtype) {
    return dtype == ORC_BF16 ? orc_f32_to_bf16(f) : orc_f32_to_fp16(f);
}

void orc_to_f32_array(const uint16_t* src, float* dst, size_t n, int dtype) {
    for (size_t i = 0; i < n; ++i) dst[i] = to_f32(src[i], dtype);
}
void orc_from_f32_array(const float* src, uint16_t* dst, size_t n, int dtype) {
    for (size_t i = 0; i < n; ++i) dst[i] = from_f32(src[i], dtype);
}

/* -------------------------------------------------------------- seeded generators -- */
/* Counter based: element i of stream s under seed is a pure function of (seed, s, i), so
 * any slice of any matrix can be regenerated anywhere, in any order, on any thread count. */

static inline uint64_t mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
uint64_t orc_rng_u64(uint64_t seed, uint64_t stream, uint64_t index) {
    return mix64(mix64(seed ^ (stream * 0xd1342543de82ef95ull)) + index);
}

/* i.i.d. uniform on the 2^24-point grid of [-1, 1), then rounded to the storage type. */
void orc_fill_uniform(uint16_t* dst, size_t n, uint64_t seed, uint64_t stream, int dtype) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t r = orc_rng_u64(seed, stream, i);
        float u = (float)(r >> 40) * (1.0f / 16777216.0f);     /* [0,1), exact */
        dst[i] = from_f32(2.0f * u - 1.0f, dtype);
    }
}

/* i.i.d. N(0, sigma^2) by Box-Muller in double, rounded once to the storage type.
 * Plays the part of randomize_matrix (matmul_h100_optimal.cu:86-92, N(0,1)). */
void orc_fill_normal(uint16_t* dst, size_t n, uint64_t seed, uint64_t stream, float sigma,
                     int dtype) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint64_t r = orc_rng_u64(seed, stream, i);
        double u1 = ((double)(r >> 40) + 1.0) * (1.0 / 16777216.0);          /* (0,1] */
        double u2 = (double)(r & 0xffffffull) * (1.0 / 16777216.0);          /* [0,1) */
        double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
        dst[i] = from_f32((float)(z * (double)sigma), dtype);
    }
}

/* random_fill (common.h:283-290): value = (r % 1000 * 1 / 100 % 10) - 5, an integer in
 * [-5, 4].  The reference draws r from unseeded rand(); here r comes from the counter
 * generator so the fill is reproducible. */
void orc_fill_randint(uint16_t* dst, size_t n, uint64_t seed, uint64_t stream, int dtype) {
    for (size_t i = 0; i < n; ++i) {
        int r = (int)(orc_rng_u64(seed, stream, i) >> 33);       /* 0 .. 2^31-1 like rand() */
        dst[i] = from_f32((float)(r % 1000 * 1 / 100 % 10 - 5.0), dtype);
    }
}
/* arange_fill (common.h:292-299): value = i % bound. */
void orc_fill_arange(uint16_t* dst, size_t n, int bound, int dtype) {
    for (size_t i = 0; i < n; ++i) dst[i] = from_f32((float)((int)(i % (size_t)bound)), dtype);
}
/* constant_fill (common.h:301-307). */
void orc_fill_constant(uint16_t* dst, size_t n, float value, int dtype) {
    uint16_t v = from_f32(value, dtype);
    for (size_t i = 0; i < n; ++i) dst[i] = v;
}

/* --------------------------------------------------------------- reference GEMM ---- */

/* One 64x64 output tile exactly as reference.h:19-43 computes it: a 64x64 fp32
 * accumulator block, k advanced in blocks of 32, inside a block kk ascending, then jj,
 * then ii innermost; reads wrap modulo M and N; the store is predicated and writes
 * (CType)(acc * alpha + beta)  -- beta is a scalar added to every element, not beta*C. */
static void ref_tile_faithful(int M, int N, int K, const uint16_t* hA, const uint16_t* hB,
                              uint16_t* golden, float* golden_acc, float alpha, float beta,
                              int dtype, int i, int j) {
    float accum[64 * 64];
    memset(accum, 0, sizeof accum);
    for (int k = 0; k < K; k += 32) {
        for (int kk = 0; kk < 32; ++kk) {
            if (k + kk >= K) break;
            for (int jj = 0; jj < 64; ++jj) {
                for (int ii = 0; ii < 64; ++ii) {
                    float a = to_f32(hA[(size_t)((i + ii) % M) * K + k + kk], dtype);
                    float b = to_f32(hB[(size_t)((j + jj) % N) * K + k + kk], dtype);
                    float p = a * b;
                    accum[ii * 64 + jj] = accum[ii * 64 + jj] + p;
                }
            }
        }
    }
    for (int ii = 0; ii < 64; ++ii) {
        for (int jj = 0; jj < 64; ++jj) {
            if (i + ii < M && j + jj < N) {
                size_t o = (size_t)(i + ii) * N + j + jj;
                float scaled = accum[ii * 64 + jj] * alpha;
                float v = scaled + beta;
                if (golden) golden[o] = from_f32(v, dtype);
                if (golden_acc) golden_acc[o] = accum[ii * 64 + jj];
            }
        }
    }
}

/* Same value for every element as ref_tile_faithful -- each C[i][j] is still one fp32
 * accumulator fed in ascending k, one rounding per addition -- but the operands are
 * converted to fp32 once and the loop nest is k / ii / jj with jj contiguous, which the
 * compiler vectorises.  Element results do not depend on the order in which *different*
 * elements are visited, so the two routines agree bit for bit (tested). */
static void ref_tile_fast(int M, int N, int K, const uint16_t* hA, const uint16_t* hB,
                          uint16_t* golden, float* golden_acc, float alpha, float beta,
                          int dtype, int i, int j) {
    enum { KB = 256 };
    float accum[64 * 64];
    float at[KB * 64], bt[KB * 64];               /* [kk][ii] and [kk][jj] */
    memset(accum, 0, sizeof accum);
    for (int k = 0; k < K; k += KB) {
        int kn = K - k < KB ? K - k : KB;
        for (int ii = 0; ii < 64; ++ii) {
            const uint16_t* row = hA + (size_t)((i + ii) % M) * K + k;
            for (int kk = 0; kk < kn; ++kk) at[kk * 64 + ii] = to_f32(row[kk], dtype);
        }
        for (int jj = 0; jj < 64; ++jj) {
            const uint16_t* row = hB + (size_t)((j + jj) % N) * K + k;
            for (int kk = 0; kk < kn; ++kk) bt[kk * 64 + jj] = to_f32(row[kk], dtype);
        }
        for (int kk = 0; kk < kn; ++kk) {
            const float* bp = bt + kk * 64;
            for (int ii = 0; ii < 64; ++ii) {
                float a = at[kk * 64 + ii];
                float* acc = accum + ii * 64;
                for (int jj = 0; jj < 64; ++jj) acc[jj] = acc[jj] + a * bp[jj];
            }
        }
    }
    for (int ii = 0; ii < 64; ++ii) {
        for (int jj = 0; jj < 64; ++jj) {
            if (i + ii < M && j + jj < N) {
                size_t o = (size_t)(i + ii) * N + j + jj;
                float scaled = accum[ii * 64 + jj] * alpha;
                float v = scaled + beta;
                if (golden) golden[o] = from_f32(v, dtype);
                if (golden_acc) golden_acc[o] = accum[ii * 64 + jj];
            }
        }
    }
}

/* reference_cpu_gemm (reference.h:5-46), whole matrix.  The reference puts
 * `omp parallel for` on both tile loops; with nested parallelism off (the OpenMP default)
 * only the ceil(M/64) row-tile iterations would run in parallel, i.e. one thread when
 * M <= 64.  Tiles are independent, so the two loops are collapsed here; results do not
 * depend on it.  fast = 0 runs the loop nest in the reference's own order.
 * C and Cacc may each be NULL; Cacc receives the raw fp32 accumulators. */
void orc_reference_cpu_gemm(int M, int N, int K, const uint16_t* A, const uint16_t* B,
                            uint16_t* C, float* Cacc, float alpha, float beta, int dtype,
                            int fast) {
    int tm = (M + 63) / 64, tn = (N + 63) / 64;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int ti = 0; ti < tm; ++ti)
        for (int tj = 0; tj < tn; ++tj) {
            if (fast) ref_tile_fast(M, N, K, A, B, C, Cacc, alpha, beta, dtype, ti * 64, tj * 64);
            else ref_tile_faithful(M, N, K, A, B, C, Cacc, alpha, beta, dtype, ti * 64, tj * 64);
        }
}

/* The same routine restricted to a list of 64x64 tiles (tile_ij = {ti0, tj0, ti1, tj1, ...}
 * in units of tiles).  Only those tiles of C / Cacc are written.  Because every tile of
 * reference.h is computed independently, a sampled tile holds exactly the values the full
 * run would hold. */
void orc_reference_cpu_gemm_tiles(int M, int N, int K, const uint16_t* A, const uint16_t* B,
                                  uint16_t* C, float* Cacc, float alpha, float beta,
                                  int dtype, int fast, const int* tile_ij, int ntiles) {
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntiles; ++t) {
        int i = tile_ij[2 * t] * 64, j = tile_ij[2 * t + 1] * 64;
        if (i >= M || j >= N) continue;
        if (fast) ref_tile_fast(M, N, K, A, B, C, Cacc, alpha, beta, dtype, i, j);
        else ref_tile_faithful(M, N, K, A, B, C, Cacc, alpha, beta, dtype, i, j);
    }
}

/* The contract of reference_gpu_gemm_kernel (reference.h:49-76) as a plain triple loop:
 * one accumulator per element, k ascending, terms with k >= K are zero, predicated store.
 * It is the second, independent statement of the GEMM the reference holds; the tests use
 * it as a brute-force cross-check of the tiled routine above. */
void orc_naive_gemm(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C,
                    float alpha, float beta, int dtype) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) {
                float p = to_f32(A[(size_t)m * K + k], dtype) * to_f32(B[(size_t)n * K + k], dtype);
                acc = acc + p;
            }
            float scaled = acc * alpha;
            C[(size_t)m * N + n] = from_f32(scaled + beta, dtype);
        }
}

/* ------------------------------------------------------------------- checkers ------ */

/* assert_allclose (common.h:367-397) without the abort: an element is an error when
 * |r - g| > rtol * |g| (pure relative: g == 0 tolerates nothing).  Returns the error
 * count; *avg_diff = mean |r-g| over the failing elements (0 if none); *n_inf counts
 * infinities in either array (the reference asserts there are none). */
long long orc_allclose_count(const uint16_t* res, const uint16_t* golden, size_t n, float rtol,
                             int dtype, double* avg_diff, long long* n_inf) {
    long long errors = 0, infs = 0;
    double total = 0.0;
    for (size_t i = 0; i < n; ++i) {
        float r = to_f32(res[i], dtype), g = to_f32(golden[i], dtype);
        if (isinf(r) || isinf(g)) ++infs;
        if (fabsf(r - g) > rtol * fabsf(g)) { ++errors; total += fabsf(r - g); }
    }
    if (avg_diff) *avg_diff = errors ? total / (double)errors : 0.0;
    if (n_inf) *n_inf = infs;
    return errors;
}

/* verify_matrix (matmul_h100_optimal.cu:94-108): the difference of the two 16-bit values
 * is itself rounded to the storage type, and the element fails when |diff| > 0.1.
 * Returns the index of the first failing element or -1. */
long long orc_absdiff_first_fail(const uint16_t* ref, const uint16_t* out, size_t n,
                                 float thresh, int dtype) {
    for (size_t i = 0; i < n; ++i) {
        float d = to_f32(from_f32(to_f32(ref[i], dtype) - to_f32(out[i], dtype), dtype), dtype);
        if (fabs((double)d) > (double)thresh) return (long long)i;
    }
    return -1;
}

double orc_max_abs(const uint16_t* x, size_t n, int dtype) {
    double m = 0.0;
#pragma omp parallel for reduction(max : m) schedule(static)
    for (size_t i = 0; i < n; ++i) {
        double v = fabs((double)to_f32(x[i], dtype));
        if (v > m) m = v;
    }
    return m;
}

/* The acceptance tolerance of this build (not a reference function):
 *     |out - ref| <= rel * |ref| + abs_coef * sqrt(K) * max|a| * max|b|
 * with rel = 2^-7 and abs_coef = 1e-3 in every caller.  Compares only the elements of the
 * listed 64x64 tiles when tile_ij != NULL, all elements otherwise.  NaN anywhere counts as
 * a violation.  report[0] = violations, [1] = max |err|, [2] = max |err| / bound,
 * [3] = elements compared, [4] = the absolute term of the bound. */
long long orc_check_tolerance(int M, int N, int K, const uint16_t* out, const uint16_t* ref,
                              double max_a, double max_b, double rel, double abs_coef,
                              int dtype, const int* tile_ij, int ntiles, double* report) {
    double abs_term = abs_coef * sqrt((double)K) * max_a * max_b;
    long long bad = 0, cmp = 0;
    double max_err = 0.0, max_ratio = 0.0;
    int tm = (M + 63) / 64, tn = (N + 63) / 64;
    int total = tile_ij ? ntiles : tm * tn;
#pragma omp parallel for schedule(static) reduction(+ : bad, cmp) reduction(max : max_err, max_ratio)
    for (int t = 0; t < total; ++t) {
        int ti = tile_ij ? tile_ij[2 * t] : t / tn;
        int tj = tile_ij ? tile_ij[2 * t + 1] : t % tn;
        for (int i = ti * 64; i < ti * 64 + 64 && i < M; ++i)
            for (int j = tj * 64; j < tj * 64 + 64 && j < N; ++j) {
                double o = (double)to_f32(out[(size_t)i * N + j], dtype);
                double r = (double)to_f32(ref[(size_t)i * N + j], dtype);
                double err = fabs(o - r);
                double bound = rel * fabs(r) + abs_term;
                ++cmp;
                if (!(err <= bound)) { ++bad; continue; }
                if (err > max_err) max_err = err;
                if (bound > 0 && err / bound > max_ratio) max_ratio = err / bound;
            }
    }
    if (report) {
        report[0] = (double)bad; report[1] = max_err; report[2] = max_ratio;
        report[3] = (double)cmp; report[4] = abs_term;
    }
    return bad;
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
