/*
 * CPU restatement of the reference's two-phase fp32 attention (its MKL/OpenMP path).
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker the HIP kernels are compared with and
 * the timed CPU baseline.  Nothing shipped links it or calls it.
 *
 * Follows cpp/chunk_attn/kernel_cpu_mkl.cpp of the reference:
 *   oracle_one_chunk   <- attn_one_chunk  (kernel_cpu_mkl.cpp:16-120)
 *   oracle_one_seq     <- attn_one_seq    (kernel_cpu_mkl.cpp:122-213)
 *   ca_oracle_seq_first   <- seq_first    (kernel_cpu_mkl.cpp:215-242)
 *   ca_oracle_chunk_first <- chunk_first  (kernel_cpu_mkl.cpp:245-353)
 * The chunk pointer of a ChunkInfo row is replaced by (slot, n_tokens): chunk i's K and V
 * are the [H, c, d] blocks at element offset slot*H*c*d of two flat fp32 pools
 * (chunk_allocator.cpp:43-55).
 *
 * GEMM / exp: the reference calls MKL (cblas_sgemm, vsExp, cblas_saxpby).  MKL is a
 * third-party dependency that is not vendored; the caller may hand in Fortran-ABI
 * `sgemm_` and `vsExp` entry points (the PyTorch wheel's libtorch_cpu.so exports MKL's)
 * through ca_oracle_set_blas(); without them plain C loops with the same semantics are used.
 *
 * Pinned by tests/test_oracle_attn.py against float64 textbook softmax attention
 * (the check the reference's own tests use, tests/test_chunk_attn_cpu.py:234-265,333-385),
 * closed forms (equal keys -> mean of V, one token -> v) and brute force on tiny inputs.
 */
#include <float.h>
#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

typedef void (*sgemm_fn)(const char*, const char*, const int*, const int*, const int*,
                         const float*, const float*, const int*, const float*, const int*,
                         const float*, float*, const int*);
typedef void (*vsexp_fn)(const int, const float*, float*);

static sgemm_fn g_sgemm = 0;
static vsexp_fn g_vsexp = 0;

void ca_oracle_set_blas(void* sgemm_ptr, void* vsexp_ptr) {
    g_sgemm = (sgemm_fn)sgemm_ptr;
    g_vsexp = (vsexp_fn)vsexp_ptr;
}

int ca_oracle_has_blas(void) { return g_sgemm != 0 && g_vsexp != 0; }

/* row-major C[M,N] = A[M,K] * B[N,K]^T   (cblas_sgemm NoTrans/Trans of the reference) */
static void gemm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                    float* C, int ldc) {
    if (g_sgemm) {
        const float one = 1.f, zero = 0.f;
        g_sgemm("T", "N", &N, &M, &K, &one, B, &ldb, A, &lda, &zero, C, &ldc);
        return;
    }
    for (int i = 0; i < M; i++)
        for (int j = 0; j < N; j++) {
            float s = 0.f;
            for (int k = 0; k < K; k++) s += A[i * lda + k] * B[j * ldb + k];
            C[i * ldc + j] = s;
        }
}

/* row-major C[M,N] = A[M,K] * B[K,N] + beta * C   (cblas_sgemm NoTrans/NoTrans) */
static void gemm_nn(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                    float beta, float* C, int ldc) {
    if (g_sgemm) {
        const float one = 1.f;
        g_sgemm("N", "N", &N, &M, &K, &one, B, &ldb, A, &lda, &beta, C, &ldc);
        return;
    }
    for (int i = 0; i < M; i++) {
        for (int j = 0; j < N; j++) C[i * ldc + j] = (beta == 0.f) ? 0.f : beta * C[i * ldc + j];
        for (int k = 0; k < K; k++) {
            float a = A[i * lda + k];
            for (int j = 0; j < N; j++) C[i * ldc + j] += a * B[k * ldb + j];
        }
    }
}

static void vexp(int n, float* x) {
    if (g_vsexp) {
        g_vsexp(n, x, x);
        return;
    }
    for (int i = 0; i < n; i++) x[i] = expf(x[i]);
}

/* kernel_cpu_mkl.cpp:16-120.  q,o point at row seq_begin of head h (row stride H*d);
 * wmax/wsum point at entry seq_begin of head h.  lock may be NULL. */
static void oracle_one_chunk(const float* q, const float* k, const float* v, float* o, int n,
                             int tokens, int H, int d, float d_sqrt, float* wmax, float* wsum,
                             omp_lock_t* lock) {
    if (tokens <= 0) return; /* :30-32 */
    float* w = (float*)malloc(sizeof(float) * (size_t)n * tokens);
    float* wmax_loc = (float*)malloc(sizeof(float) * n * 3);
    float* scale1 = wmax_loc + n;
    float* scale2 = scale1 + n;
    float* o_loc = (float*)malloc(sizeof(float) * (size_t)n * d);

    gemm_nt(n, tokens, d, q, d * H, k, d, w, tokens); /* :41-55 */
    for (int i = 0; i < n; i++) {                    /* :58-71 */
        float m = -FLT_MAX;
        for (int j = 0; j < tokens; j++) m = fmaxf(m, w[i * tokens + j]);
        for (int j = 0; j < tokens; j++) w[i * tokens + j] = (w[i * tokens + j] - m) / d_sqrt;
        vexp(tokens, w + i * tokens);
        wmax_loc[i] = m / d_sqrt;
    }
    gemm_nn(n, d, tokens, w, tokens, v, d, 0.f, o_loc, d); /* :74-88 */

    if (lock) omp_set_lock(lock);
    for (int i = 0; i < n; i++) { /* :93-98 */
        float m = fmaxf(wmax[i], wmax_loc[i]);
        scale1[i] = wmax_loc[i] - m;
        scale2[i] = wmax[i] - m;
        wmax[i] = m;
    }
    vexp(n, scale1);
    vexp(n, scale2);
    for (int i = 0; i < n; i++) { /* :103-107 saxpby */
        float* dst = o + (size_t)i * d * H;
        const float* src = o_loc + (size_t)i * d;
        for (int e = 0; e < d; e++) dst[e] = scale1[i] * src[e] + scale2[i] * dst[e];
    }
    for (int i = 0; i < n; i++) { /* :110-116 */
        float s = 0.f;
        for (int j = 0; j < tokens; j++) s += w[i * tokens + j];
        wsum[i] = scale1[i] * s + scale2[i] * wsum[i];
    }
    if (lock) omp_unset_lock(lock);
    free(w);
    free(wmax_loc);
    free(o_loc);
}

/* rows: n_rows x 4 ints (slot, n_tokens, seq_begin, seq_end) in get_chunks order.
 * q, out: [n_seqs, H, d] fp32.  kernel_cpu_mkl.cpp:245-353. */
int ca_oracle_chunk_first(const float* q, const float* kpool, const float* vpool,
                          const int* rows, int n_rows, int n_seqs, int H, int d, int c,
                          float* out, int n_threads) {
    const float d_sqrt = sqrtf((float)d);
    const size_t chunk_elems = (size_t)H * c * d;
    float* wmax = (float*)malloc(sizeof(float) * (size_t)H * n_seqs);
    float* wsum = (float*)malloc(sizeof(float) * (size_t)H * n_seqs);
    for (size_t i = 0; i < (size_t)H * n_seqs; i++) {
        wmax[i] = -FLT_MAX; /* numeric_limits<float>::lowest(), :248-249 */
        wsum[i] = 0.f;
    }
    memset(out, 0, sizeof(float) * (size_t)n_seqs * H * d); /* attention.cpp:69 */
    if (n_threads <= 0) n_threads = omp_get_max_threads();
    omp_set_dynamic(0); /* kernel_cpu_mkl.h:23-26 */

    if (H < n_threads) { /* :263-307 */
        omp_lock_t* locks = (omp_lock_t*)malloc(sizeof(omp_lock_t) * H);
        for (int h = 0; h < H; h++) omp_init_lock(&locks[h]);
        const int total = H * n_rows;
#pragma omp parallel for num_threads(n_threads)
        for (int i = 0; i < total; i++) {
            const int r = i / H, h = i % H;
            const int slot = rows[4 * r], tokens = rows[4 * r + 1];
            const int b = rows[4 * r + 2], e = rows[4 * r + 3];
            oracle_one_chunk(q + (size_t)h * d + (size_t)b * d * H,
                             kpool + slot * chunk_elems + (size_t)h * c * d,
                             vpool + slot * chunk_elems + (size_t)h * c * d,
                             out + (size_t)h * d + (size_t)b * d * H, e - b, tokens, H, d, d_sqrt,
                             wmax + (size_t)h * n_seqs + b, wsum + (size_t)h * n_seqs + b,
                             &locks[h]);
        }
        for (int h = 0; h < H; h++) omp_destroy_lock(&locks[h]);
        free(locks);
    } else { /* :308-351 */
#pragma omp parallel for num_threads(n_threads)
        for (int h = 0; h < H; h++) {
            for (int r = 0; r < n_rows; r++) {
                const int slot = rows[4 * r], tokens = rows[4 * r + 1];
                const int b = rows[4 * r + 2], e = rows[4 * r + 3];
                oracle_one_chunk(q + (size_t)h * d + (size_t)b * d * H,
                                 kpool + slot * chunk_elems + (size_t)h * c * d,
                                 vpool + slot * chunk_elems + (size_t)h * c * d,
                                 out + (size_t)h * d + (size_t)b * d * H, e - b, tokens, H, d,
                                 d_sqrt, wmax + (size_t)h * n_seqs + b,
                                 wsum + (size_t)h * n_seqs + b, 0);
            }
        }
    }
    for (int s = 0; s < n_seqs; s++) /* :352 */
        for (int h = 0; h < H; h++) {
            const float l = wsum[(size_t)h * n_seqs + s];
            float* o = out + ((size_t)s * H + h) * d;
            for (int e = 0; e < d; e++) o[e] /= l;
        }
    free(wmax);
    free(wsum);
    return 0;
}

/* kernel_cpu_mkl.cpp:122-213 */
static void oracle_one_seq(const float* q, int seq, int h, const float* kpool, const float* vpool,
                           const int* rows, int n_rows, float* o, int c, int H, int d,
                           float d_sqrt) {
    float* w = (float*)malloc(sizeof(float) * (size_t)c);
    float wmax = -FLT_MAX, wsum = 0.f;
    const size_t chunk_elems = (size_t)H * c * d;
    for (int r = 0; r < n_rows; r++) {
        const int b = rows[4 * r + 2], e = rows[4 * r + 3];
        if (seq < b || seq >= e) continue; /* :137-142 */
        const int tokens = rows[4 * r + 1];
        if (tokens <= 0) continue;
        const float* k = kpool + rows[4 * r] * chunk_elems + (size_t)h * c * d;
        const float* v = vpool + rows[4 * r] * chunk_elems + (size_t)h * c * d;
        gemm_nt(1, tokens, d, q, d * H, k, d, w, tokens); /* :153-167 */
        float m = wmax;
        for (int j = 0; j < tokens; j++) m = fmaxf(m, w[j]);
        for (int j = 0; j < tokens; j++) w[j] = (w[j] - m) / d_sqrt;
        vexp(tokens, w);
        const float scale2 = expf((wmax - m) / d_sqrt);      /* :182 */
        gemm_nn(1, d, tokens, w, tokens, v, d, scale2, o, d * H); /* :185-199 */
        float s = 0.f;
        for (int j = 0; j < tokens; j++) s += w[j];
        wsum = s + scale2 * wsum;
        wmax = m;
    }
    for (int e = 0; e < d; e++) o[e] /= wsum; /* :209-211 */
    free(w);
}

/* kernel_cpu_mkl.cpp:215-242 */
int ca_oracle_seq_first(const float* q, const float* kpool, const float* vpool, const int* rows,
                        int n_rows, int n_seqs, int H, int d, int c, float* out, int n_threads) {
    const float d_sqrt = sqrtf((float)d);
    memset(out, 0, sizeof(float) * (size_t)n_seqs * H * d);
    if (n_threads <= 0) n_threads = omp_get_max_threads();
    omp_set_dynamic(0);
    const int total = n_seqs * H;
#pragma omp parallel for num_threads(n_threads)
    for (int i = 0; i < total; i++) {
        const int h = i / n_seqs, s = i % n_seqs;
        oracle_one_seq(q + (size_t)h * d + (size_t)s * d * H, s, h, kpool, vpool, rows, n_rows,
                       out + (size_t)h * d + (size_t)s * d * H, c, H, d, d_sqrt);
    }
    return 0;
}

/* kernel_cpu_mkl.cpp:364-372 */
int ca_oracle_attention(const float* q, const float* kpool, const float* vpool, const int* rows,
                        int n_rows, int n_seqs, int H, int d, int c, float* out, int partition,
                        int n_threads) {
    if (partition == 0 || partition == 1)
        return ca_oracle_chunk_first(q, kpool, vpool, rows, n_rows, n_seqs, H, d, c, out, n_threads);
    if (partition == 2)
        return ca_oracle_seq_first(q, kpool, vpool, rows, n_rows, n_seqs, H, d, c, out, n_threads);
    return -1; /* "Unsupported partition type" */
}

int ca_oracle_max_threads(void) { return omp_get_max_threads(); }
