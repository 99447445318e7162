/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the dense GEMM path.
 *
 * A plain-C restatement of the CPU reference GEMM and input generator that the
 * reference's own GPU tests compare against.  Only tests, the smoke check and
 * the benchmark's cpu_baseline leg may load this library; the product library
 * never links or calls it.
 *
 * Reference files followed (paths relative to the reference tree):
 *   test/test.hpp:33-54     init_matrix: std::mt19937 gen(1) constructed inside
 *                           the function (so every matrix sees the same stream),
 *                           std::uniform_real_distribution<float>(-1,1), values
 *                           drawn in logical (row outer, column inner) order and
 *                           stored through the layout's index map, cast to the
 *                           element type with round-to-nearest-even.
 *   test/test.hpp:59-129    hgemm_cpu (4 type combinations): i, j, k loops,
 *                           operands widened to fp32, float accumulator updated in
 *                           ascending k, one final cast to the C element type.
 *   test/test.hpp:134-215   calculate_cosine_similarity / verify_results and
 *                           their thresholds (0.995 half, 0.97 bf16).
 *   common/matrix.hpp:154-164  index map: row-major i*n+j, column-major j*m+i.
 *
 * Pinning (every function below is pinned; none is "parity unpinned"):
 *   - mt19937 + uniform: six-draw known answers recorded from the reference's
 *     generator under libstdc++ (tests/golden/oracle_kat.json).
 *   - gemm for all four type pairs and three layout triples: element values and
 *     FNV-1a-64 hashes of the raw C bytes recorded from the reference's C++
 *     oracle on its seeded inputs (same fixture file).
 *   - beyond the fixtures: identity/one-hot/all-ones closed forms, float64 brute
 *     force on tiny shapes, and torch.matmul in fp32 (tests/test_oracle.py).
 *
 * The reference's own translation unit cannot be compiled here as oracle/_ref:
 * test/test.hpp uses googletest's ASSERT_GT and googletest is not installed.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* 16-bit float conversions (software, round-to-nearest-even)          */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1fu;
    uint32_t man  = h & 0x3ffu;
    if(exp == 0)
    {
        if(man == 0)
            return bits_f32(sign);
        /* subnormal: value = man * 2^-24, exact in fp32 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if(exp == 31)
        return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t x    = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax   = x & 0x7fffffffu;
    if(ax >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
    if(ax >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if(ax < 0x38800000u) /* result is subnormal or zero: |f| < 2^-14 */
    {
        if(ax < 0x33000000u) /* |f| < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
            return sign;
        /* scale so that one unit = 2^-24, then round to nearest even */
        uint32_t e     = ax >> 23;            /* biased exponent, 102..112 */
        uint32_t m     = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;            /* 14..24 */
        uint32_t q     = m >> shift;
        uint32_t rem   = m & ((1u << shift) - 1u);
        uint32_t half  = 1u << (shift - 1u);
        if(rem > half || (rem == half && (q & 1u)))
            q++;
        return (uint16_t)(sign | q);
    }
    /* normal range */
    uint32_t rounded = ax + 0xfffu + ((ax >> 13) & 1u);
    return (uint16_t)(sign | ((rounded - 0x38000000u) >> 13));
}

float oracle_bf16_to_f32(uint16_t h)
{
    return bits_f32((uint32_t)h << 16);
}

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t x = f32_bits(f);
    if((x & 0x7fffffffu) > 0x7f800000u) /* nan: keep quiet */
        return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

/* dtype codes shared with the Python wrapper */
enum
{
    ORACLE_F16  = 0,
    ORACLE_BF16 = 1,
    ORACLE_F32  = 2
};
enum
{
    ORACLE_ROW = 0,
    ORACLE_COL = 1
};

static inline size_t idx2(size_t i, size_t j, size_t m, size_t n, int layout)
{
    /* common/matrix.hpp:154-164 */
    return layout == ORACLE_ROW ? i * n + j : j * m + i;
}

/* ------------------------------------------------------------------ */
/* mt19937 (32-bit Mersenne twister, the std::mt19937 parameter set)   */
/* ------------------------------------------------------------------ */

typedef struct
{
    uint32_t s[624];
    int      pos;
} mt19937_t;

static void mt_seed(mt19937_t* g, uint32_t seed)
{
    g->s[0] = seed;
    for(int i = 1; i < 624; ++i)
        g->s[i] = 1812433253u * (g->s[i - 1] ^ (g->s[i - 1] >> 30)) + (uint32_t)i;
    g->pos = 624;
}

static uint32_t mt_next(mt19937_t* g)
{
    if(g->pos >= 624)
    {
        for(int i = 0; i < 624; ++i)
        {
            uint32_t y = (g->s[i] & 0x80000000u) | (g->s[(i + 1) % 624] & 0x7fffffffu);
            uint32_t v = g->s[(i + 397) % 624] ^ (y >> 1);
            if(y & 1u)
                v ^= 0x9908b0dfu;
            g->s[i] = v;
        }
        g->pos = 0;
    }
    uint32_t y = g->s[g->pos++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

/* std::generate_canonical<float,24> over a 32-bit engine is one draw divided by
 * 2^32 in float arithmetic, clamped below 1; uniform_real_distribution maps it
 * as canonical*(hi-lo)+lo.  (test/test.hpp:37-38) */
static inline float mt_canonical(mt19937_t* g)
{
    float r = (float)mt_next(g) / 4294967296.0f;
    if(r >= 1.0f)
        r = 0.99999994f; /* nextafter(1,0) */
    return r;
}

void oracle_raw_draws(uint32_t seed, size_t count, uint32_t* out)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for(size_t i = 0; i < count; ++i)
        out[i] = mt_next(&g);
}

void oracle_uniform_draws(uint32_t seed, float lo, float hi, size_t count, float* out)
{
    mt19937_t g;
    mt_seed(&g, seed);
    for(size_t i = 0; i < count; ++i)
        out[i] = mt_canonical(&g) * (hi - lo) + lo;
}

static void store_elem(void* dst, size_t at, int dtype, float v)
{
    if(dtype == ORACLE_F16)
        ((uint16_t*)dst)[at] = oracle_f32_to_f16(v);
    else if(dtype == ORACLE_BF16)
        ((uint16_t*)dst)[at] = oracle_f32_to_bf16(v);
    else
        ((float*)dst)[at] = v;
}

/* dist: 0 = uniform[lo,hi) as the reference draws it (test/test.hpp:33-54 uses
 * lo=-1, hi=1, seed=1); 1 = normal(mean=lo, std=hi) by Box-Muller on pairs of
 * canonical draws (harness-only distribution, not part of the reference). */
void oracle_init_matrix(void* dst, size_t m, size_t n, int layout, int dtype, uint32_t seed,
                        int dist, float lo, float hi)
{
    mt19937_t g;
    mt_seed(&g, seed);
    float spare     = 0.0f;
    int   has_spare = 0;
    for(size_t i = 0; i < m; ++i)
    {
        for(size_t j = 0; j < n; ++j)
        {
            float v;
            if(dist == 0)
            {
                v = mt_canonical(&g) * (hi - lo) + lo;
            }
            else
            {
                if(has_spare)
                {
                    v         = spare;
                    has_spare = 0;
                }
                else
                {
                    float u1  = 1.0f - mt_canonical(&g); /* (0,1] */
                    float u2  = mt_canonical(&g);
                    float rad = sqrtf(-2.0f * logf(u1));
                    float ang = 6.28318530717958647692f * u2;
                    v         = rad * cosf(ang);
                    spare     = rad * sinf(ang);
                    has_spare = 1;
                }
                v = v * hi + lo;
            }
            store_elem(dst, idx2(i, j, m, n, layout), dtype, v);
        }
    }
}

/* ------------------------------------------------------------------ */
/* GEMM (test/test.hpp:59-129)                                         */
/* ------------------------------------------------------------------ */

static inline float load_elem(const void* src, size_t at, int dtype)
{
    if(dtype == ORACLE_F16)
        return oracle_f16_to_f32(((const uint16_t*)src)[at]);
    if(dtype == ORACLE_BF16)
        return oracle_bf16_to_f32(((const uint16_t*)src)[at]);
    return ((const float*)src)[at];
}

/* The literal triple loop, one thread: the slow, obviously-faithful form. */
void oracle_gemm_naive(void* C, const void* A, const void* B, size_t M, size_t N, size_t K,
                       int layout_c, int layout_a, int layout_b, int in_dtype, int out_dtype)
{
    for(size_t i = 0; i < M; ++i)
    {
        for(size_t j = 0; j < N; ++j)
        {
            float acc = 0.0f;
            for(size_t k = 0; k < K; ++k)
            {
                float a = load_elem(A, idx2(i, k, M, K, layout_a), in_dtype);
                float b = load_elem(B, idx2(k, j, K, N, layout_b), in_dtype);
                acc += a * b;
            }
            store_elem(C, idx2(i, j, M, N, layout_c), out_dtype, acc);
        }
    }
}

/* Fast form with identical per-element arithmetic: operands are widened once to
 * fp32 (A as [M][K], B as [K][N]) and a strip of JB output columns is carried
 * through the k loop together; each output still sees acc += a*b in ascending k
 * with separately rounded product and sum, so results are bit-identical to the
 * naive form.  Rows are split across threads. */
#define JB 64

typedef struct
{
    const float* Af;
    const float* Bf;
    void*        C;
    float*       S;
    size_t       M, N, K;
    size_t       row_begin, row_end;
    int          layout_c, out_dtype;
} gemm_job_t;

__attribute__((target_clones("avx512f", "avx2", "default"))) static void
    strip_kernel(const float* a_row, const float* Bf, size_t N, size_t K, size_t j0, size_t jn,
                 float* acc, float* sabs)
{
    for(size_t jj = 0; jj < JB; ++jj)
    {
        acc[jj]  = 0.0f;
        sabs[jj] = 0.0f;
    }
    if(jn == JB)
    {
        for(size_t k = 0; k < K; ++k)
        {
            const float  a = a_row[k];
            const float* b = Bf + k * N + j0;
            for(size_t jj = 0; jj < JB; ++jj)
            {
                float p = a * b[jj];
                acc[jj] += p;
                sabs[jj] += fabsf(p);
            }
        }
    }
    else
    {
        for(size_t k = 0; k < K; ++k)
        {
            const float  a = a_row[k];
            const float* b = Bf + k * N + j0;
            for(size_t jj = 0; jj < jn; ++jj)
            {
                float p = a * b[jj];
                acc[jj] += p;
                sabs[jj] += fabsf(p);
            }
        }
    }
}

static void* gemm_worker(void* arg)
{
    gemm_job_t* job = (gemm_job_t*)arg;
    float       acc[JB], sabs[JB];
    for(size_t i = job->row_begin; i < job->row_end; ++i)
    {
        const float* a_row = job->Af + i * job->K;
        for(size_t j0 = 0; j0 < job->N; j0 += JB)
        {
            size_t jn = job->N - j0 < JB ? job->N - j0 : JB;
            strip_kernel(a_row, job->Bf, job->N, job->K, j0, jn, acc, sabs);
            for(size_t jj = 0; jj < jn; ++jj)
            {
                store_elem(job->C, idx2(i, j0 + jj, job->M, job->N, job->layout_c), job->out_dtype,
                           acc[jj]);
                if(job->S)
                    job->S[i * job->N + j0 + jj] = sabs[jj];
            }
        }
    }
    return NULL;
}

/* C (M x N) = A (M x K) * B (K x N) for rows [row_begin, row_end) only; other
 * rows of C are left untouched.  S, if not NULL, receives sum_k |a_ik*b_kj| as a
 * row-major M x N fp32 matrix (the scale of the comparison tolerance).
 * Returns 0 on success. */
int oracle_gemm_rows(void* C, const void* A, const void* B, size_t M, size_t N, size_t K,
                     int layout_c, int layout_a, int layout_b, int in_dtype, int out_dtype,
                     size_t row_begin, size_t row_end, int nthreads, float* S)
{
    if(row_end > M)
        row_end = M;
    if(row_begin >= row_end || N == 0)
        return 0;
    size_t rows = row_end - row_begin;
    float* Af   = (float*)malloc(sizeof(float) * rows * (K ? K : 1));
    float* Bf   = (float*)malloc(sizeof(float) * (K ? K : 1) * N);
    if(!Af || !Bf)
    {
        free(Af);
        free(Bf);
        return -1;
    }
    for(size_t i = 0; i < rows; ++i)
        for(size_t k = 0; k < K; ++k)
            Af[i * K + k] = load_elem(A, idx2(row_begin + i, k, M, K, layout_a), in_dtype);
    for(size_t k = 0; k < K; ++k)
        for(size_t j = 0; j < N; ++j)
            Bf[k * N + j] = load_elem(B, idx2(k, j, K, N, layout_b), in_dtype);

    if(nthreads < 1)
        nthreads = 1;
    if((size_t)nthreads > rows)
        nthreads = (int)rows;
    pthread_t*  tids = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
    gemm_job_t* jobs = (gemm_job_t*)malloc(sizeof(gemm_job_t) * (size_t)nthreads);
    for(int t = 0; t < nthreads; ++t)
    {
        gemm_job_t* job = &jobs[t];
        job->Af         = Af - row_begin * K; /* rebased so that row i is at Af + i*K */
        job->Bf         = Bf;
        job->C          = C;
        job->S          = S;
        job->M          = M;
        job->N          = N;
        job->K          = K;
        job->row_begin  = row_begin + rows * (size_t)t / (size_t)nthreads;
        job->row_end    = row_begin + rows * (size_t)(t + 1) / (size_t)nthreads;
        job->layout_c   = layout_c;
        job->out_dtype  = out_dtype;
        if(nthreads == 1)
            gemm_worker(job);
        else
            pthread_create(&tids[t], NULL, gemm_worker, job);
    }
    if(nthreads > 1)
        for(int t = 0; t < nthreads; ++t)
            pthread_join(tids[t], NULL);
    free(tids);
    free(jobs);
    free(Af);
    free(Bf);
    return 0;
}

int oracle_gemm(void* C, const void* A, const void* B, size_t M, size_t N, size_t K, int layout_c,
                int layout_a, int layout_b, int in_dtype, int out_dtype, int nthreads, float* S)
{
    return oracle_gemm_rows(C, A, B, M, N, K, layout_c, layout_a, layout_b, in_dtype, out_dtype, 0,
                            M, nthreads, S);
}

/* ------------------------------------------------------------------ */
/* Verification helpers                                                */
/* ------------------------------------------------------------------ */

/* test/test.hpp:134-196: float accumulators, row-outer/column-inner order. */
float oracle_cosine_similarity(const void* gpu, const void* cpu, size_t m, size_t n, int layout,
                               int dtype)
{
    float dot = 0.0f, ng = 0.0f, nc = 0.0f;
    for(size_t i = 0; i < m; ++i)
        for(size_t j = 0; j < n; ++j)
        {
            size_t at = idx2(i, j, m, n, layout);
            float  g  = load_elem(gpu, at, dtype);
            float  c  = load_elem(cpu, at, dtype);
            dot += g * c;
            ng += g * g;
            nc += c * c;
        }
    if(ng < 1e-10f || nc < 1e-10f)
    {
        float mg = 0.0f, mc = 0.0f;
        for(size_t i = 0; i < m; ++i)
            for(size_t j = 0; j < n; ++j)
            {
                size_t at = idx2(i, j, m, n, layout);
                float  g  = fabsf(load_elem(gpu, at, dtype));
                float  c  = fabsf(load_elem(cpu, at, dtype));
                if(g > mg)
                    mg = g;
                if(c > mc)
                    mc = c;
            }
        float tol = dtype == ORACLE_BF16 ? 1e-2f : 1e-4f;
        return (mg < tol && mc < tol) ? 1.0f : 0.0f;
    }
    return dot / (sqrtf(ng) * sqrtf(nc));
}

/* test/test.hpp:199-215 thresholds */
float oracle_cosine_threshold(int dtype)
{
    return dtype == ORACLE_BF16 ? 0.97f : 0.995f;
}

/* FNV-1a, 64 bit, over raw bytes: pins the restatement bit for bit.  The offset
 * basis is a parameter because the recorded reference hashes were taken with the
 * basis 1469598103934665603 rather than the standard 0xcbf29ce484222325. */
uint64_t oracle_fnv1a64_basis(const void* data, size_t nbytes, uint64_t basis)
{
    const uint8_t* p = (const uint8_t*)data;
    uint64_t       h = basis;
    for(size_t i = 0; i < nbytes; ++i)
    {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

uint64_t oracle_fnv1a64(const void* data, size_t nbytes)
{
    return oracle_fnv1a64_basis(data, nbytes, 0xcbf29ce484222325ull);
}
