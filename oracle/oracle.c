/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's host-side
 * goldens for the CSR SpMV / SpMM path, used by tests/, by the smoke test and
 * by the cpu_baseline leg of bench.py as the checker / baseline.  The product
 * (libops_sparse.so) never links, loads or calls anything in this file.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference tree).  Plain C99, no dependencies; built by oracle/Makefile into
 * oracle/liboracle.so.
 *
 * What pins each function (tests/test_oracle.py):
 *   oracle_spmv_f64 / oracle_spmm_f64   brute force against a dense fp64
 *        matmul, diagonal / identity closed forms, A*e_j = column j, empty A,
 *        alpha = 0, linearity, the reference README's 4x3 * 3x2 known answer,
 *        SpMM column j == SpMV on B[:, j], layout / transpose equivalences
 *   oracle_spmv_f32 / oracle_spmm_f32   same cases (exact on small integers),
 *        agreement with the fp64 oracle inside the reference's own tolerances
 *   oracle_f32_to_f16 / oracle_f16_to_f32   exhaustive 65 536-pattern round
 *        trip and comparison with numpy's IEEE half conversion
 *   oracle_mere_mare   hand-computed 3-element vectors
 *   oracle_fill_*      the reference generator itself (oracle/_ref, built
 *        from test/frame/fill.h) where present, and committed fixture hashes
 *   oracle_spmm22_*    (the arch22 SpMM program's random_col / generate_*_csr)
 *        a second statement of the same recipe in Python over numpy's MT19937
 *        stream; row lengths, value formula, Zipf shares and distinctness as
 *        closed forms; the engine itself is the one pinned by oracle_fill_*
 *   oracle_glibc_rand_stream / oracle_spmm35_random_csr   the host's own
 *        libc (srand / rand through ctypes) on eight seeds; row lengths,
 *        ascending distinct columns, value grid, the first row by hand
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ SpMV */

/*
 * fp64 oracle: z = alpha * (A x) + beta * y with everything widened to double
 * and one final rounding to float.  Follows SpMVOpGolden,
 * test/spmv_op/spmv_op_golden.h:24-75, which does the same through an Eigen
 * SparseMatrix<double>; duplicates in a row are summed (Eigen's
 * setFromTriplets sums them too), cols <= 0 gives beta * y (:39-46).
 * y may alias z.
 */
void oracle_spmv_f64(int64_t rows, int64_t cols, const int32_t *rowptr, const int32_t *colind, const float *val,
                     const float *x, const float *y, float alpha, float beta, float *z)
{
    for (int64_t i = 0; i < rows; ++i) {
        double sum = 0.0;
        if (cols > 0) {
            for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
                sum += (double)val[p] * (double)x[colind[p]];
            }
        }
        /* beta == 0 must not read y: the library treats y as write-only then. */
        double r = (double)alpha * sum;
        if (beta != 0.0f) {
            r += (double)beta * (double)y[i];
        }
        z[i] = (float)r;
    }
}

/*
 * The reference's fp32 CPU golden, as written: float accumulation in stored
 * order, z = alpha * sum + beta * y.  SpmvCpu, test/spmv/arch22/spmv_test.cpp:156-173.
 * (beta * y is evaluated even for beta == 0, as in the reference.)
 */
void oracle_spmv_f32(int64_t rows, const int32_t *rowptr, const int32_t *colind, const float *val, const float *x,
                     const float *y, float alpha, float beta, float *z)
{
    for (int64_t i = 0; i < rows; ++i) {
        float sum = 0.0f;
        for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
            sum += val[p] * x[colind[p]];
        }
        z[i] = alpha * sum + beta * y[i];
    }
}

/* The same loop with its rows shared out among `threads` OpenMP threads (rows are independent: the results
 * are those of oracle_spmv_f32 bit for bit).  The all-cores CPU baseline of the benchmark. */
void oracle_spmv_f32_threads(int64_t rows, const int32_t *rowptr, const int32_t *colind, const float *val,
                             const float *x, const float *y, float alpha, float beta, float *z, int threads)
{
#pragma omp parallel for schedule(static, 4096) num_threads(threads)
    for (int64_t i = 0; i < rows; ++i) {
        float sum = 0.0f;
        for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
            sum += val[p] * x[colind[p]];
        }
        z[i] = alpha * sum + beta * y[i];
    }
}

/*
 * Transposed fp32 golden: z = beta * y, then z[col] += (alpha * x[row]) * val
 * row by row.  SpmvTransCpu, test/spmv/arch22/spmv_test.cpp:177-197.
 */
void oracle_spmv_trans_f32(int64_t rows, int64_t cols, const int32_t *rowptr, const int32_t *colind,
                           const float *val, const float *x, const float *y, float alpha, float beta, float *z)
{
    for (int64_t j = 0; j < cols; ++j) {
        z[j] = beta * y[j];
    }
    for (int64_t i = 0; i < rows; ++i) {
        const float xv = alpha * x[i];
        if (xv == 0.0f) {
            continue;
        }
        for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
            z[colind[p]] = z[colind[p]] + xv * val[p];
        }
    }
}

/* Transposed product with fp64 accumulation per output element (no reference
 * counterpart; the fp64 analogue of the function above, used as the oracle
 * for op = T).  `acc` is caller-provided scratch of `cols` doubles. */
void oracle_spmv_trans_f64(int64_t rows, int64_t cols, const int32_t *rowptr, const int32_t *colind,
                           const float *val, const float *x, const float *y, float alpha, float beta, float *z,
                           double *acc)
{
    for (int64_t j = 0; j < cols; ++j) {
        acc[j] = 0.0;
    }
    for (int64_t i = 0; i < rows; ++i) {
        for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
            acc[colind[p]] += (double)val[p] * (double)x[i];
        }
    }
    for (int64_t j = 0; j < cols; ++j) {
        double r = (double)alpha * acc[j];
        if (beta != 0.0f) {
            r += (double)beta * (double)y[j];
        }
        z[j] = (float)r;
    }
}

/* int32 golden: SpmvCpu<int32_t>, same file, CompT = int32_t (wrap-around
 * arithmetic done in uint32 to stay defined in C). */
void oracle_spmv_i32(int64_t rows, const int32_t *rowptr, const int32_t *colind, const int32_t *val,
                     const int32_t *x, const int32_t *y, int32_t alpha, int32_t beta, int32_t *z)
{
    for (int64_t i = 0; i < rows; ++i) {
        uint32_t sum = 0;
        for (int32_t p = rowptr[i]; p < rowptr[i + 1]; ++p) {
            sum += (uint32_t)val[p] * (uint32_t)x[colind[p]];
        }
        z[i] = (int32_t)((uint32_t)alpha * sum + (uint32_t)beta * (uint32_t)y[i]);
    }
}

/* ------------------------------------------------------------------ SpMM */

/* Index formulas of B and C for every (order, opB) combination:
 * SpmmCpuFp32, test/spmm/arch35/spmm_test.cpp:141-156 — identical to the
 * device kernel, sparse/spmm/arch35/spmm_kernel.cpp:155-168, :215-219. */
static int64_t b_index(int64_t c, int64_t j, int64_t ldb, int b_row_major, int trans_b)
{
    if (!trans_b) {
        return b_row_major ? c * ldb + j : j * ldb + c;
    }
    return b_row_major ? j * ldb + c : c * ldb + j;
}
static int64_t c_index(int64_t r, int64_t j, int64_t ldc, int c_row_major)
{
    return c_row_major ? r * ldc + j : j * ldc + r;
}

/* The reference's fp32 SpMM golden as written (loop order r, j, p; float
 * accumulate; C = alpha * acc + beta * C_old, C_old read unconditionally).
 * SpmmCpuFp32, test/spmm/arch35/spmm_test.cpp:125-161; with row-major
 * operands and ldb = ldc = n it is spmm_csr_cpu,
 * test/spmm/arch22/spmm_test.cpp:133-147. */
void oracle_spmm_f32(int64_t m, int64_t n, const int32_t *rowptr, const int32_t *colind, const float *val,
                     const float *B, int64_t ldb, int b_row_major, int trans_b, float *C, int64_t ldc,
                     int c_row_major, float alpha, float beta)
{
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (int32_t p = rowptr[r]; p < rowptr[r + 1]; ++p) {
                acc += val[p] * B[b_index(colind[p], j, ldb, b_row_major, trans_b)];
            }
            const int64_t ci = c_index(r, j, ldc, c_row_major);
            C[ci] = alpha * acc + beta * C[ci];
        }
    }
}

/* oracle_spmm_f32 with its rows shared out among `threads` OpenMP threads (same results bit for bit). */
void oracle_spmm_f32_threads(int64_t m, int64_t n, const int32_t *rowptr, const int32_t *colind, const float *val,
                             const float *B, int64_t ldb, int b_row_major, int trans_b, float *C, int64_t ldc,
                             int c_row_major, float alpha, float beta, int threads)
{
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads)
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t j = 0; j < n; ++j) {
            float acc = 0.0f;
            for (int32_t p = rowptr[r]; p < rowptr[r + 1]; ++p) {
                acc += val[p] * B[b_index(colind[p], j, ldb, b_row_major, trans_b)];
            }
            const int64_t ci = c_index(r, j, ldc, c_row_major);
            C[ci] = alpha * acc + beta * C[ci];
        }
    }
}

/* fp64-accumulated SpMM oracle (the SpMM analogue of oracle_spmv_f64; the
 * reference's golden template for it is the Eigen fp64 product in
 * agent/skills/repo-test-develop/references/test/{op}/op_golden.h:80-120).
 * C is not read when beta == 0. */
void oracle_spmm_f64(int64_t m, int64_t n, const int32_t *rowptr, const int32_t *colind, const float *val,
                     const float *B, int64_t ldb, int b_row_major, int trans_b, float *C, int64_t ldc,
                     int c_row_major, float alpha, float beta)
{
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t j = 0; j < n; ++j) {
            double acc = 0.0;
            for (int32_t p = rowptr[r]; p < rowptr[r + 1]; ++p) {
                acc += (double)val[p] * (double)B[b_index(colind[p], j, ldb, b_row_major, trans_b)];
            }
            const int64_t ci = c_index(r, j, ldc, c_row_major);
            double out = (double)alpha * acc;
            if (beta != 0.0f) {
                out += (double)beta * (double)C[ci];
            }
            C[ci] = (float)out;
        }
    }
}

/* Same oracle with the loops ordered r, p, j for row-major B and C, so that it
 * finishes in seconds on large cases; arithmetic per element is identical to
 * oracle_spmm_f64 (each C element still sums its products in stored order).
 * `acc` is scratch of n doubles. */
void oracle_spmm_f64_rowmajor(int64_t m, int64_t n, const int32_t *rowptr, const int32_t *colind, const float *val,
                              const float *B, int64_t ldb, float *C, int64_t ldc, float alpha, float beta,
                              double *acc)
{
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t j = 0; j < n; ++j) {
            acc[j] = 0.0;
        }
        for (int32_t p = rowptr[r]; p < rowptr[r + 1]; ++p) {
            const double v = (double)val[p];
            const float *brow = B + (int64_t)colind[p] * ldb;
            for (int64_t j = 0; j < n; ++j) {
                acc[j] += v * (double)brow[j];
            }
        }
        for (int64_t j = 0; j < n; ++j) {
            double out = (double)alpha * acc[j];
            if (beta != 0.0f) {
                out += (double)beta * (double)C[r * ldc + j];
            }
            C[r * ldc + j] = (float)out;
        }
    }
}

/* int8 golden: int32 accumulate, alpha * acc + beta * C_old in int32.
 * SpmmCpuInt8, test/spmm/arch35/spmm_test.cpp:163-200.  The device kernel
 * evaluates the epilogue in int64 and saturates (spmm_kernel.cpp:251-266);
 * `saturate` != 0 restates that variant. */
void oracle_spmm_i8(int64_t m, int64_t n, const int32_t *rowptr, const int32_t *colind, const int8_t *val,
                    const int8_t *B, int64_t ldb, int b_row_major, int trans_b, int32_t *C, int64_t ldc,
                    int c_row_major, int32_t alpha, int32_t beta, int saturate)
{
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t j = 0; j < n; ++j) {
            uint32_t acc = 0;
            for (int32_t p = rowptr[r]; p < rowptr[r + 1]; ++p) {
                acc += (uint32_t)((int32_t)val[p] * (int32_t)B[b_index(colind[p], j, ldb, b_row_major, trans_b)]);
            }
            const int64_t ci = c_index(r, j, ldc, c_row_major);
            if (saturate) {
                int64_t wide = (int64_t)alpha * (int64_t)(int32_t)acc;
                if (beta != 0) {
                    wide += (int64_t)beta * (int64_t)C[ci];
                }
                if (wide > 2147483647LL) wide = 2147483647LL;
                if (wide < -2147483648LL) wide = -2147483648LL;
                C[ci] = (int32_t)wide;
            } else {
                C[ci] = (int32_t)((uint32_t)alpha * acc + (uint32_t)beta * (uint32_t)C[ci]);
            }
        }
    }
}

/* ------------------------------------------------------------- fp16 bits */

/* Round-to-nearest-even float -> IEEE half bits, with subnormals, overflow to
 * infinity and NaN kept.  Fp32ToFp16Bits, test/spmm/arch35/spmm_test.cpp:303-348. */
uint16_t oracle_f32_to_f16(float v)
{
    uint32_t bits;
    memcpy(&bits, &v, sizeof bits);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const uint32_t raw_exp = (bits >> 23) & 0xFFu;
    const int32_t exp = (int32_t)raw_exp - 127;
    const uint32_t mant = bits & 0x007FFFFFu;
    if (raw_exp == 0xFFu) {
        return (uint16_t)(sign | 0x7C00u | (mant != 0u ? 0x0200u : 0u));
    }
    if (exp >= 16) {
        return (uint16_t)(sign | 0x7C00u);
    }
    if (exp >= -14) {
        uint32_t res = ((uint32_t)(exp + 15) << 10) | (mant >> 13);
        const uint32_t rem = mant & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (res & 1u))) {
            res += 1u; /* may carry into the exponent, up to infinity */
        }
        return (uint16_t)(sign | res);
    }
    if (exp >= -25) {
        const uint32_t sig = 0x00800000u | mant;
        const uint32_t shift = (uint32_t)(-exp - 1); /* 14..24 */
        uint32_t frac = sig >> shift;
        const uint32_t rem = sig & ((1u << shift) - 1u);
        const uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (frac & 1u))) {
            frac += 1u;
        }
        return (uint16_t)(sign | frac);
    }
    return (uint16_t)sign;
}

/* Fp16BitsToFp32, test/spmm/arch35/spmm_test.cpp:350-373.  One deliberate
 * difference: for subnormal inputs the reference ORs the normalised mantissa
 * including its leading 1 into the word (:361), which lands on the exponent's
 * lowest bit and doubles the result whenever that bit was 0.  Here the leading
 * 1 is masked off, which is the IEEE value; for normal numbers, zero, Inf and
 * NaN (all the reference's tests exercise) the two agree bit for bit. */
float oracle_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x03FFu;
    uint32_t f;
    if (exp == 0) {
        if (mant == 0) {
            f = sign;
        } else {
            const uint32_t shift = (uint32_t)__builtin_clz(mant) - 21u;
            mant <<= shift;
            f = sign | ((1u + 127u - 15u - shift) << 23) | ((mant & 0x03FFu) << 13);
        }
    } else if (exp == 31) {
        f = sign | 0x7F800000u | (mant << 13);
    } else {
        f = sign | ((exp + 127u - 15u) << 23) | (mant << 13);
    }
    float v;
    memcpy(&v, &f, sizeof v);
    return v;
}

void oracle_f32_to_f16_array(const float *in, uint16_t *out, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        out[i] = oracle_f32_to_f16(in[i]);
    }
}
void oracle_f16_to_f32_array(const uint16_t *in, float *out, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        out[i] = oracle_f16_to_f32(in[i]);
    }
}

/* ---------------------------------------------------------------- verifier */

/* Mean / max relative error with the reference's floor in the denominator:
 * rel = |out - gold| / (|gold| + eps), eps = 2^-14 for the test framework
 * (MereMareStrategy, test/frame/verify.h:112-161, kEpsilon :153) and 1e-7 for
 * the SpMM test (VerifyFloat, test/spmm/arch35/spmm_test.cpp:202-252).
 * Elements that are bit-for-bit equal, or abnormal (NaN / Inf) on both sides,
 * are skipped; abnormal on one side only counts as a mismatch.
 * result[0] = MERE, result[1] = MARE, result[2] = mismatches, result[3] = counted. */
void oracle_mere_mare(const float *out, const float *gold, int64_t n, double eps, double *result)
{
    double sum = 0.0, mx = 0.0;
    int64_t mismatch = 0, counted = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float o = out[i], g = gold[i];
        const int oa = isnan(o) || isinf(o), ga = isnan(g) || isinf(g);
        if (o == g || (oa && ga)) {
            continue; /* skipped */
        }
        if (oa || ga) {
            ++mismatch;
            continue;
        }
        const double rel = fabs((double)(o - g)) / (fabs((double)g) + eps);
        sum += rel;
        if (rel > mx) mx = rel;
        ++counted;
    }
    result[0] = counted > 0 ? sum / (double)counted : 0.0;
    result[1] = mx;
    result[2] = (double)mismatch;
    result[3] = (double)counted;
}

/* -------------------------------------------------- reference generators */

/* std::mt19937 (the C++ standard fixes its output stream). */
typedef struct {
    uint32_t s[624];
    int idx;
} mt19937_t;

static void mt_seed(mt19937_t *g, uint32_t seed)
{
    g->s[0] = seed;
    for (int i = 1; i < 624; ++i) {
        g->s[i] = 1812433253u * (g->s[i - 1] ^ (g->s[i - 1] >> 30)) + (uint32_t)i;
    }
    g->idx = 624;
}

static uint32_t mt_next(mt19937_t *g)
{
    if (g->idx >= 624) {
        for (int i = 0; i < 624; ++i) {
            const uint32_t y = (g->s[i] & 0x80000000u) | (g->s[(i + 1) % 624] & 0x7fffffffu);
            g->s[i] = g->s[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        g->idx = 0;
    }
    uint32_t y = g->s[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

/* libstdc++ (GCC 11+) std::uniform_int_distribution<int32_t>(0, hi) on a
 * 32-bit engine: Lemire's multiply-shift with rejection. */
static int32_t uniform_int(mt19937_t *g, int32_t hi)
{
    const uint32_t range = (uint32_t)hi + 1u; /* hi < 2^31 - 1 here */
    uint64_t product = (uint64_t)mt_next(g) * (uint64_t)range;
    uint32_t low = (uint32_t)product;
    if (low < range) {
        const uint32_t threshold = (0u - range) % range;
        while (low < threshold) {
            product = (uint64_t)mt_next(g) * (uint64_t)range;
            low = (uint32_t)product;
        }
    }
    return (int32_t)(product >> 32);
}

/* libstdc++ std::uniform_real_distribution<float>(lo, hi): one engine draw,
 * generate_canonical<float, 24> = float(u) / 2^32 (clamped below 1), then
 * canonical * (hi - lo) + lo in float. */
static float uniform_real(mt19937_t *g, float lo, float hi)
{
    volatile float canon = (float)mt_next(g) / 4294967296.0f;
    if (canon >= 1.0f) {
        canon = nextafterf(1.0f, 0.0f);
    }
    volatile float scaled = canon * (hi - lo);
    return scaled + lo;
}

static int cmp_i32(const void *a, const void *b)
{
    const int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
    return (x > y) - (x < y);
}

/*
 * SparseFillGenerator(seed).setValueRange(lo, hi).setEmptyRowProb(p)
 *   .generateCsr(rows, cols, nnzHint) with nnzHint > 0
 * (test/frame/fill.h:55-111): every non-skipped row gets
 * min(nnzHint / rows, cols) distinct uniform columns (at most 4x that many
 * draws), sorted, then one value per entry.  Arrays must hold
 * rows * (nnzHint / rows) entries.  Returns nnz.
 * The binomial row-length path (nnzHint <= 0) is not restated.
 */
int64_t oracle_fill_csr(uint32_t seed, int64_t rows, int64_t cols, int64_t nnz_hint, double empty_row_prob,
                        double lo, double hi, int32_t *rowptr, int32_t *colind, float *val)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for (int64_t i = 0; i <= rows; ++i) {
        rowptr[i] = 0;
    }
    if (rows <= 0 || cols <= 0 || nnz_hint <= 0) {
        return 0;
    }
    int32_t *visited = (int32_t *)malloc(sizeof(int32_t) * (size_t)cols);
    for (int64_t c = 0; c < cols; ++c) {
        visited[c] = -1;
    }
    int64_t target = nnz_hint / (rows > 1 ? rows : 1);
    if (target > cols) target = cols;
    int32_t *rowcols = (int32_t *)malloc(sizeof(int32_t) * (size_t)(target > 0 ? target : 1));
    int64_t nnz = 0;
    for (int64_t i = 0; i < rows; ++i) {
        rowptr[i] = (int32_t)nnz;
        if (empty_row_prob > 0.0 && uniform_real(&g, 0.0f, 1.0f) < (float)empty_row_prob) {
            continue;
        }
        if (target <= 0) {
            continue;
        }
        int64_t have = 0, attempt = 0;
        while (have < target && attempt < target * 4) {
            const int32_t c = uniform_int(&g, (int32_t)cols - 1);
            if (visited[c] != (int32_t)i) {
                visited[c] = (int32_t)i;
                rowcols[have++] = c;
            }
            ++attempt;
        }
        qsort(rowcols, (size_t)have, sizeof(int32_t), cmp_i32);
        for (int64_t k = 0; k < have; ++k) {
            colind[nnz] = rowcols[k];
            val[nnz] = uniform_real(&g, (float)lo, (float)hi);
            ++nnz;
        }
    }
    rowptr[rows] = (int32_t)nnz;
    free(visited);
    free(rowcols);
    return nnz;
}

/* makeDenseFloat(size, lo, hi, seed), test/frame/fill.h:199-203. */
void oracle_fill_dense(uint32_t seed, int64_t n, double lo, double hi, float *out)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for (int64_t i = 0; i < n; ++i) {
        out[i] = uniform_real(&g, (float)lo, (float)hi);
    }
}

/* FNV-1a over a byte range, used to fingerprint generated arrays in fixtures. */
uint64_t oracle_fnv1a(const void *data, int64_t bytes)
{
    const unsigned char *p = (const unsigned char *)data;
    uint64_t h = 1469598103934665603ull;
    for (int64_t i = 0; i < bytes; ++i) {
        h ^= p[i];
        h *= 1099511628211ull;
    }
    return h;
}

/* ---------------------------------------------------------- CSR producers
 * Bit-exact integer / byte operations.  Pinned by: the reference's own goldens
 * compiled in place (oracle/_ref/libref_convert.so) where present; numpy
 * (bincount + cumsum, repeat, stable argsort) and scipy's CSR -> CSC on
 * random inputs; hand-written small cases (tests/test_oracle.py).
 */

/* Coo2CsrGolden, test/coo2csr/coo2csr_golden.h:44-77: count per row (rows
 * outside [0, m) ignored, unsigned subtraction of the base), prefix sum + base. */
void oracle_coo2csr(const int32_t *rowInd, int64_t nnz, int64_t m, int32_t base, int32_t *rowPtr)
{
    for (int64_t i = 0; i <= m; ++i) {
        rowPtr[i] = base;
    }
    if (nnz <= 0 || m <= 0) {
        return;
    }
    int32_t *count = (int32_t *)calloc((size_t)m, sizeof(int32_t));
    for (int64_t k = 0; k < nnz; ++k) {
        const int32_t row = (int32_t)((uint32_t)rowInd[k] - (uint32_t)base);
        if (row >= 0 && row < m) {
            ++count[row];
        }
    }
    int64_t run = 0;
    for (int64_t i = 0; i < m; ++i) {
        run += count[i];
        rowPtr[i + 1] = (int32_t)(run + base);
    }
    free(count);
}

/* Csr2CooGolden, test/csr2coo/csr2coo_golden.h:37-61: rowInd zero-filled, row i
 * written over [rowPtr[i], rowPtr[i+1]) - base; a row whose bounds leave
 * [0, nnz] or run backwards is skipped. */
void oracle_csr2coo(const int32_t *rowPtr, int64_t m, int64_t nnz, int32_t base, int32_t *rowInd)
{
    memset(rowInd, 0, sizeof(int32_t) * (size_t)(nnz > 0 ? nnz : 0));
    for (int64_t i = 0; i < m; ++i) {
        const int64_t s = (int64_t)rowPtr[i] - base, e = (int64_t)rowPtr[i + 1] - base;
        if (s < 0 || e > nnz || s > e) {
            continue;
        }
        for (int64_t j = s; j < e; ++j) {
            rowInd[j] = (int32_t)i + base;
        }
    }
}

/* csrsortGolden, test/csrsort/arch35/csrsort_golden.h:38-70: per row a stable
 * ascending sort of the (signed) column indices, perm moved the same way.
 * Stable insertion into a merge: plain bottom-up merge sort on index pairs. */
void oracle_csrsort(const int32_t *rowPtr, int64_t m, int32_t base, int32_t *colInd, int32_t *perm)
{
    for (int64_t r = 0; r < m; ++r) {
        const int64_t b = (int64_t)rowPtr[r] - base, len = (int64_t)rowPtr[r + 1] - base - b;
        if (len <= 1) {
            continue;
        }
        int32_t *block = (int32_t *)malloc(sizeof(int32_t) * (size_t)len * 4);
        int32_t *c0 = block, *p0 = c0 + len, *c1 = p0 + len, *p1 = c1 + len;
        memcpy(c0, colInd + b, sizeof(int32_t) * (size_t)len);
        memcpy(p0, perm + b, sizeof(int32_t) * (size_t)len);
        for (int64_t w = 1; w < len; w *= 2) {
            for (int64_t lo = 0; lo < len; lo += 2 * w) {
                const int64_t mid = lo + w < len ? lo + w : len, hi = lo + 2 * w < len ? lo + 2 * w : len;
                int64_t i = lo, j = mid, k = lo;
                while (i < mid && j < hi) {
                    if (c0[j] < c0[i]) {          /* strict: equal keys keep the left one first */
                        c1[k] = c0[j]; p1[k++] = p0[j++];
                    } else {
                        c1[k] = c0[i]; p1[k++] = p0[i++];
                    }
                }
                while (i < mid) { c1[k] = c0[i]; p1[k++] = p0[i++]; }
                while (j < hi) { c1[k] = c0[j]; p1[k++] = p0[j++]; }
            }
            int32_t *t = c0; c0 = c1; c1 = t;
            t = p0; p0 = p1; p1 = t;
        }
        memcpy(colInd + b, c0, sizeof(int32_t) * (size_t)len);
        memcpy(perm + b, p0, sizeof(int32_t) * (size_t)len);
        free(block);
    }
}

/* cscsortGolden, test/cscsort/arch35/cscsort_golden.h:30-70: the column-wise twin of csrsortGolden; a CSC matrix is
 * the CSR form of its transpose, so the same walk over colPtr does it. */
void oracle_cscsort(const int32_t *colPtr, int64_t n, int32_t base, int32_t *rowInd, int32_t *perm)
{
    oracle_csrsort(colPtr, n, base, rowInd, perm);
}

/* coosortGolden, test/coosort/arch35/coosort_golden.h:52-85: a stable sort of the (row, col, P) triples, signed
 * keys, by (row, col) when byRow != 0 and by (col, row) otherwise; P travels with its entry.  Bottom-up merge sort
 * that takes from the right run only when its key is strictly smaller. */
void oracle_coosort(int64_t nnz, int32_t byRow, int32_t *rows, int32_t *cols, int32_t *perm)
{
    if (nnz <= 1) {
        return;
    }
    int32_t *block = (int32_t *)malloc(sizeof(int32_t) * (size_t)nnz * 6);
    int32_t *a0 = block, *b0 = a0 + nnz, *p0 = b0 + nnz, *a1 = p0 + nnz, *b1 = a1 + nnz, *p1 = b1 + nnz;
    memcpy(a0, byRow ? rows : cols, sizeof(int32_t) * (size_t)nnz);  /* a: primary key, b: secondary */
    memcpy(b0, byRow ? cols : rows, sizeof(int32_t) * (size_t)nnz);
    memcpy(p0, perm, sizeof(int32_t) * (size_t)nnz);
    for (int64_t w = 1; w < nnz; w *= 2) {
        for (int64_t lo = 0; lo < nnz; lo += 2 * w) {
            const int64_t mid = lo + w < nnz ? lo + w : nnz, hi = lo + 2 * w < nnz ? lo + 2 * w : nnz;
            int64_t i = lo, j = mid, k = lo;
            while (i < mid && j < hi) {
                const int less = a0[j] != a0[i] ? a0[j] < a0[i] : b0[j] < b0[i];
                if (less) {
                    a1[k] = a0[j]; b1[k] = b0[j]; p1[k++] = p0[j++];
                } else {
                    a1[k] = a0[i]; b1[k] = b0[i]; p1[k++] = p0[i++];
                }
            }
            while (i < mid) { a1[k] = a0[i]; b1[k] = b0[i]; p1[k++] = p0[i++]; }
            while (j < hi) { a1[k] = a0[j]; b1[k] = b0[j]; p1[k++] = p0[j++]; }
        }
        int32_t *t = a0; a0 = a1; a1 = t;
        t = b0; b0 = b1; b1 = t;
        t = p0; p0 = p1; p1 = t;
    }
    memcpy(byRow ? rows : cols, a0, sizeof(int32_t) * (size_t)nnz);
    memcpy(byRow ? cols : rows, b0, sizeof(int32_t) * (size_t)nnz);
    memcpy(perm, p0, sizeof(int32_t) * (size_t)nnz);
    free(block);
}

/* Csr2CscGolden, test/csr2csc_ex2/csr2csc_ex2_golden.h:50-110: column counts,
 * exclusive prefix sum + base, then a row-major walk that drops every entry at
 * its column's next free slot (so rows ascend inside a column).  Values move
 * as raw items of valBytes bytes (0: structure only). */
void oracle_csr2csc(int64_t m, int64_t n, int64_t nnz, int32_t base, const int32_t *rowPtr, const int32_t *colInd,
                    const void *val, int32_t valBytes, int32_t *colPtr, int32_t *rowInd, void *cscVal)
{
    for (int64_t j = 0; j <= n; ++j) {
        colPtr[j] = base;
    }
    if (nnz <= 0) {
        return;
    }
    int32_t *next = (int32_t *)calloc((size_t)n + 1, sizeof(int32_t));
    for (int64_t k = 0; k < nnz; ++k) {
        ++next[colInd[k] - base];
    }
    for (int64_t j = 0; j < n; ++j) {
        colPtr[j + 1] = colPtr[j] + next[j];
    }
    for (int64_t j = 0; j < n; ++j) {
        next[j] = colPtr[j] - base;
    }
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t k = (int64_t)rowPtr[i] - base; k < (int64_t)rowPtr[i + 1] - base; ++k) {
            const int32_t dest = next[colInd[k] - base]++;
            rowInd[dest] = (int32_t)i + base;
            if (valBytes > 0) {
                memcpy((unsigned char *)cscVal + (size_t)dest * valBytes, (const unsigned char *)val + (size_t)k * valBytes,
                       (size_t)valBytes);
            }
        }
    }
    free(next);
}

/* ------------------------------ the SpMM test programs' seeded generators
 *
 * arch22 (test/spmm/arch22/spmm_test.cpp:42-131): random_col() draws from ONE
 * thread_local std::mt19937(42) through a fresh uniform_int_distribution<int>(0,
 * cols - 1) per call; the engine is never re-seeded, so the inputs of a case depend
 * on how many engine outputs the cases before it consumed.  The engine lives here
 * as a process-wide state with a counter of consumed outputs: oracle_spmm22_seek(n)
 * puts it where the reference's engine is after n outputs (seed 42, discard n).
 * fill_row_random_cols (:56-74) keeps a row's columns in the order drawn, rejects a
 * repeat by drawing again (an unordered_set there, a stamp array here: only
 * membership matters), and sets values[cur] = 0.1f + 0.0001f * cur. */
static mt19937_t g_spmm22;
static uint64_t g_spmm22_used = 0;
static int g_spmm22_ready = 0;

void oracle_spmm22_seek(uint64_t outputs)
{
    mt_seed(&g_spmm22, 42u);
    for (uint64_t i = 0; i < outputs; ++i) {
        (void)mt_next(&g_spmm22);
    }
    g_spmm22_used = outputs;
    g_spmm22_ready = 1;
}

uint64_t oracle_spmm22_outputs_used(void)
{
    return g_spmm22_used;
}

/* random_col (:42-51) */
static int32_t spmm22_random_col(uint64_t cols)
{
    if (!g_spmm22_ready) {
        oracle_spmm22_seek(0);
    }
    if (cols == 0) {
        return 0;
    }
    const uint32_t range = (uint32_t)cols;
    uint64_t product = (uint64_t)mt_next(&g_spmm22) * (uint64_t)range;
    g_spmm22_used++;
    uint32_t low = (uint32_t)product;
    if (low < range) {
        const uint32_t threshold = (0u - range) % range;
        while (low < threshold) {
            product = (uint64_t)mt_next(&g_spmm22) * (uint64_t)range;
            g_spmm22_used++;
            low = (uint32_t)product;
        }
    }
    return (int32_t)(product >> 32);
}

/* fill_row_random_cols (:56-74); stamp[c] == tag marks column c as used in this row */
static uint64_t spmm22_fill_row(uint64_t row_nnz, uint64_t cols, int32_t *indices, float *values, uint64_t cur,
                                int64_t *stamp, int64_t tag)
{
    for (uint64_t j = 0; j < row_nnz; ++j) {
        int32_t col;
        do {
            col = spmm22_random_col(cols);
        } while (stamp[col] == tag);
        stamp[col] = tag;
        if (indices != NULL) {
            indices[cur] = col;
            values[cur] = 0.1f + 0.0001f * (float)cur; /* 0.0001f * cur: cur converts to float first */
        }
        cur++;
    }
    return cur;
}

/* generate_random_csr (:76-93) when powerlaw == 0, generate_powerlaw_csr (:98-131) otherwise.  indices ==
 * NULL: nothing is stored, the engine is only moved on (offsets are still written when given).  Returns the
 * number of entries, or -1 when memory for the stamp array is short. */
int64_t oracle_spmm22_csr(int powerlaw, uint64_t rows, uint64_t cols, uint64_t nnz, int32_t *offsets, int32_t *indices,
                          float *values)
{
    if (offsets != NULL) {
        offsets[0] = 0;
    }
    if (rows == 0 || cols == 0) {
        return 0;
    }
    int64_t *stamp = (int64_t *)malloc(sizeof(int64_t) * cols);
    uint64_t *row_nnz = (uint64_t *)malloc(sizeof(uint64_t) * rows);
    if (stamp == NULL || row_nnz == NULL) {
        free(stamp);
        free(row_nnz);
        return -1;
    }
    for (uint64_t c = 0; c < cols; ++c) {
        stamp[c] = -1;
    }
    if (!powerlaw) {
        for (uint64_t i = 0; i < rows; ++i) {
            row_nnz[i] = nnz / rows + (i < nnz % rows ? 1 : 0);
        }
    } else {
        /* Zipf weights 1 / (i + 1), shares truncated, the remainder to the top rows, each capped at cols */
        double total = 0.0;
        for (uint64_t i = 0; i < rows; ++i) {
            total += 1.0 / (double)(i + 1);
        }
        uint64_t assigned = 0;
        for (uint64_t i = 0; i < rows; ++i) {
            row_nnz[i] = (uint64_t)((double)nnz * (1.0 / (double)(i + 1)) / total);
            assigned += row_nnz[i];
        }
        for (uint64_t i = 0; assigned < nnz && i < rows; ++i) {
            row_nnz[i]++;
            assigned++;
        }
        for (uint64_t i = 0; i < rows; ++i) {
            if (row_nnz[i] > cols) {
                row_nnz[i] = cols;
            }
        }
    }
    uint64_t cur = 0;
    for (uint64_t i = 0; i < rows; ++i) {
        cur = spmm22_fill_row(row_nnz[i], cols, indices, values, cur, stamp, (int64_t)i);
        if (offsets != NULL) {
            offsets[i + 1] = (int32_t)cur;
        }
    }
    free(stamp);
    free(row_nnz);
    return (int64_t)cur;
}

/* arch35 (test/spmm/arch35/spmm_test.cpp:91-123, seeds :964-975): std::srand(seed), then per row nnz / m
 * (+ 1 for the first nnz % m rows, capped at k) distinct columns std::rand() % k collected in a std::set
 * (so stored ascending), values -5 + 10 * (produced % 10001) / 10000.  std::rand() is glibc's here: the
 * TYPE_3 additive feedback generator r[i] = r[i-3] + r[i-31] over 32-bit words, seeded by the Lehmer
 * generator 16807 mod 2^31 - 1, the first 310 outputs dropped, each output shifted right by one. */
typedef struct {
    uint32_t r[34];
    int f, b; /* front and rear positions in the circular table of 31 words */
    uint32_t t[31];
} glibc_rand_t;

static void glibc_srand(glibc_rand_t *g, uint32_t seed)
{
    int32_t word = (int32_t)(seed == 0 ? 1 : seed);
    g->t[0] = (uint32_t)word;
    for (int i = 1; i < 31; ++i) {
        const int32_t hi = word / 127773, lo = word % 127773;
        word = 16807 * lo - 2836 * hi;
        if (word < 0) {
            word += 2147483647;
        }
        g->t[i] = (uint32_t)word;
    }
    g->f = 3;
    g->b = 0;
    for (int i = 0; i < 310; ++i) {
        g->t[g->f] += g->t[g->b];
        g->f = (g->f + 1) % 31;
        g->b = (g->b + 1) % 31;
    }
}

static int32_t glibc_rand(glibc_rand_t *g)
{
    g->t[g->f] += g->t[g->b];
    const int32_t out = (int32_t)(g->t[g->f] >> 1);
    g->f = (g->f + 1) % 31;
    g->b = (g->b + 1) % 31;
    return out;
}

/* The first `count` outputs of std::rand() after std::srand(seed) (glibc). */
void oracle_glibc_rand_stream(uint32_t seed, int64_t count, int32_t *out)
{
    glibc_rand_t g;
    glibc_srand(&g, seed);
    for (int64_t i = 0; i < count; ++i) {
        out[i] = glibc_rand(&g);
    }
}

int64_t oracle_spmm35_random_csr(uint32_t seed, int32_t m, int32_t k, int32_t nnz, int32_t *row_off, int32_t *col_ind,
                                 float *vals)
{
    for (int32_t i = 0; i <= (m > 0 ? m : 0); ++i) {
        row_off[i] = 0;
    }
    if (m <= 0 || k <= 0) {
        return 0;
    }
    glibc_rand_t g;
    glibc_srand(&g, seed);
    unsigned char *picked = (unsigned char *)calloc((size_t)k, 1);
    if (picked == NULL) {
        return -1;
    }
    int32_t produced = 0;
    for (int32_t i = 0; i < m; ++i) {
        int32_t row_nnz = nnz / m + (i < (nnz % m) ? 1 : 0);
        if (row_nnz > k) {
            row_nnz = k;
        }
        int32_t have = 0;
        while (have < row_nnz) {
            const int32_t c = glibc_rand(&g) % k;
            if (!picked[c]) {
                picked[c] = 1;
                have++;
            }
        }
        for (int32_t c = 0; c < k; ++c) { /* a std::set iterates in ascending order */
            if (picked[c]) {
                picked[c] = 0;
                col_ind[produced] = c;
                vals[produced] = -5.0f + 10.0f * (float)(produced % 10001) / 10000.0f;
                produced++;
            }
        }
        row_off[i + 1] = produced;
    }
    free(picked);
    return produced;
}
