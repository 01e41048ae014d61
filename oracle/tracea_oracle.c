/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the arithmetic of Tracea's
 * dense-contraction path.  Nothing in the shipped library links, loads or
 * calls this file; it is the checker the HIP kernels are compared against
 * and the CPU baseline that is timed beside them.
 *
 * Each function names the reference source it follows (paths relative to the
 * reference checkout).  Pinning status of each function:
 *
 *   oracle_gemm_cpu_packed   pinned: closed form A=B=1 (examples/cpu_bench.rs:88-90),
 *                            16^3 known answer (tests/numerical_parity.rs:72-73),
 *                            fp64 naive GEMM, "+=" contract (two calls = 2x).
 *   oracle_gemm_f64          pinned: numpy matmul in float64, closed forms.
 *   oracle_epilogue_apply    pinned: scalar closed forms per functor.
 *   oracle_magic_u32 /
 *   oracle_fast_divmod       pinned: exhaustive equality with / and %.
 *   oracle_conv2d_nhwc       pinned: all-ones interior/border counts, 1x1 == GEMM,
 *                            delta filters == shifts, torch conv2d fp32 fixtures.
 *   oracle_conv_coords       pinned: brute-force nested-loop enumeration.
 *   oracle_conv_transpose2d  pinned: the reference's minimal case and its scatter-form
 *                            statement re-derived as brute force, all-ones tap counts,
 *                            stride 1 == convolution with the flipped filter,
 *                            adjointness <convT(x), y> == <x, conv(y)>, torch
 *                            conv_transpose2d fp32.
 *   oracle_attention         pinned: softmax row-sum invariants, causal row 0,
 *                            Q=0 prefix means, torch SDPA fp32 fixtures.
 *
 * Build: see oracle/Makefile (gcc -O3 -mavx2 -mfma -pthread -shared).
 */
#include <immintrin.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* G3: panel packing (src/kernels/cpu/gemm.rs:208-239)                       */
/* ------------------------------------------------------------------------ */

/* A block (mc x kc, row stride lda) -> panels of mr rows, k-major inside a
 * panel, rows beyond mc zero-filled. */
static void pack_a_panel(const float *src, float *dst, int mc, int kc, int lda, int mr)
{
    size_t d = 0;
    for (int mi = 0; mi < mc; mi += mr)
        for (int l = 0; l < kc; ++l)
            for (int row = 0; row < mr; ++row)
                dst[d++] = (mi + row < mc) ? src[(size_t)(mi + row) * lda + l] : 0.0f;
}

/* B block (kc x nc, row stride ldb) -> panels of 16 columns, k-major inside a
 * panel, columns beyond nc zero-filled. */
static void pack_b_panel(const float *src, float *dst, int kc, int nc, int ldb)
{
    size_t d = 0;
    for (int ni = 0; ni < nc; ni += 16)
        for (int l = 0; l < kc; ++l)
            for (int col = 0; col < 16; ++col)
                dst[d++] = (ni + col < nc) ? src[(size_t)l * ldb + ni + col] : 0.0f;
}

/* ------------------------------------------------------------------------ */
/* G2: register-tile micro kernel (src/kernels/cpu/gemm.rs:12-205)           */
/*                                                                          */
/* mr_tile x 16 accumulators held in YMM registers, per k step: two 8-wide   */
/* loads of the B panel row, one broadcast of each A element, two FMAs per   */
/* row; k ascending.  The tile is then ADDED to C (fp32), rows >= mr skipped.*/
/* valid_cols restricts the write-back to the columns that exist (the        */
/* reference always writes 16 and relies on N being a multiple of 16).       */
/* ------------------------------------------------------------------------ */
static inline void micro_kernel(const float *a, const float *b, float *c, int k, int ldc,
                                int mr, int mr_tile, int valid_cols, int pf_dist)
{
    __m256 acc[6][2];
    for (int r = 0; r < 6; ++r) {
        acc[r][0] = _mm256_setzero_ps();
        acc[r][1] = _mm256_setzero_ps();
    }
    if (mr_tile == 6) {
        for (int l = 0; l < k; ++l) {
            if (pf_dist > 0) _mm_prefetch((const char *)(b + pf_dist), _MM_HINT_T0);
            __m256 b0 = _mm256_loadu_ps(b), b1 = _mm256_loadu_ps(b + 8);
            b += 16;
            for (int r = 0; r < 6; ++r) {
                __m256 av = _mm256_broadcast_ss(a + r);
                acc[r][0] = _mm256_fmadd_ps(av, b0, acc[r][0]);
                acc[r][1] = _mm256_fmadd_ps(av, b1, acc[r][1]);
            }
            a += 6;
        }
    } else {
        for (int l = 0; l < k; ++l) {
            if (pf_dist > 0) _mm_prefetch((const char *)(b + pf_dist), _MM_HINT_T0);
            __m256 b0 = _mm256_loadu_ps(b), b1 = _mm256_loadu_ps(b + 8);
            b += 16;
            for (int r = 0; r < 4; ++r) {
                __m256 av = _mm256_broadcast_ss(a + r);
                acc[r][0] = _mm256_fmadd_ps(av, b0, acc[r][0]);
                acc[r][1] = _mm256_fmadd_ps(av, b1, acc[r][1]);
            }
            a += 4;
        }
    }
    float tmp[16];
    for (int r = 0; r < mr_tile && r < mr; ++r) {
        _mm256_storeu_ps(tmp, acc[r][0]);
        _mm256_storeu_ps(tmp + 8, acc[r][1]);
        float *row = c + (size_t)r * ldc;
        for (int j = 0; j < valid_cols; ++j) row[j] += tmp[j];
    }
}

/* ------------------------------------------------------------------------ */
/* G1: gemm_cpu_packed (src/kernels/cpu/gemm.rs:241-298)                     */
/*                                                                          */
/* C[M,N] += A[M,K] * B[K,N], all row-major fp32.  Loop nest: parallel over  */
/* Mc row blocks; k by Kc; pack A; n by Nc; pack B; mr x 16 micro tiles.     */
/* Deviation, stated: the reference computes the C offset of a micro tile as */
/* mi*n + ni (gemm.rs:280) and omits the Nc block origin, so for N > Nc it   */
/* piles every column block onto the first; its benchmark never reads C      */
/* (examples/cpu_bench.rs:34-72).  The GEMM it means to compute adds nb, and */
/* that is what is restated here.  Flop count and memory traffic are equal.  */
/* ------------------------------------------------------------------------ */
typedef struct {
    int m, n, k, mc, nc, kc, mr, pf;
    const float *a, *b;
    float *c;
    int nblocks;
    volatile int *next; /* shared block counter (work stealing, as rayon) */
} packed_job;

static void packed_block(const packed_job *j, int mb)
{
    const int m = j->m, n = j->n, k = j->k, mc = j->mc, nc = j->nc, kc = j->kc, mr = j->mr;
    const int m_start = mb * mc;
    const int actual_mc = mc < m - m_start ? mc : m - m_start;
    float *packed_a = (float *)aligned_alloc(64, sizeof(float) * (size_t)((mc + mr - 1) / mr * mr) * kc);
    float *packed_b = (float *)aligned_alloc(64, sizeof(float) * (size_t)((nc + 15) / 16 * 16) * kc + 64);
    float *c_block = j->c + (size_t)m_start * n;
    for (int k_idx = 0; k_idx < k; k_idx += kc) {
        const int cur_kc = kc < k - k_idx ? kc : k - k_idx;
        pack_a_panel(j->a + (size_t)m_start * k + k_idx, packed_a, actual_mc, cur_kc, k, mr);
        for (int nb = 0; nb < n; nb += nc) {
            const int actual_nc = nc < n - nb ? nc : n - nb;
            pack_b_panel(j->b + (size_t)k_idx * n + nb, packed_b, cur_kc, actual_nc, n);
            for (int mi = 0; mi < actual_mc; mi += mr) {
                const int cur_mr = mr < actual_mc - mi ? mr : actual_mc - mi;
                const float *a_panel = packed_a + (size_t)(mi / mr) * cur_kc * mr;
                for (int ni = 0; ni < actual_nc; ni += 16) {
                    const float *b_panel = packed_b + (size_t)(ni / 16) * cur_kc * 16;
                    const int cols = 16 < actual_nc - ni ? 16 : actual_nc - ni;
                    micro_kernel(a_panel, b_panel, c_block + (size_t)mi * n + nb + ni, cur_kc, n,
                                 cur_mr, mr, cols, j->pf);
                }
            }
        }
    }
    free(packed_a);
    free(packed_b);
}

static void *packed_worker(void *arg)
{
    const packed_job *j = (const packed_job *)arg;
    for (;;) {
        int mb = __sync_fetch_and_add(j->next, 1);
        if (mb >= j->nblocks) break;
        packed_block(j, mb);
    }
    return NULL;
}

/* mr must be 4 or 6 (the two register tiles the reference dispatches,
 * gemm.rs:193-205); k_unroll only changes loop unrolling in the reference and
 * not the order of additions, so it is accepted and ignored.  Returns 0, or
 * -1 on a bad argument. */
ORACLE_API int oracle_gemm_cpu_packed(int m, int n, int k, int mc, int nc, int kc, int mr,
                                      int k_unroll, int prefetch_distance, const float *a,
                                      const float *b, float *c, int nthreads)
{
    (void)k_unroll;
    if (m <= 0 || n <= 0 || k <= 0 || mc <= 0 || nc <= 0 || kc <= 0 || (mr != 4 && mr != 6))
        return -1;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    volatile int next = 0;
    packed_job j = {m, n, k, mc, nc, kc, mr, prefetch_distance, a, b, c, (m + mc - 1) / mc, &next};
    if (nthreads == 1) {
        packed_worker(&j);
        return 0;
    }
    pthread_t th[256];
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t)
        if (pthread_create(&th[started], NULL, packed_worker, &j) == 0) ++started;
    packed_worker(&j);
    for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Plain GEMM in double precision: C[m,n] = sum_k A(m,k) * B(k,n).           */
/* Element strides let one routine cover row-major B ([K,N]) and the         */
/* column-major B of the fp16 configuration ([N,K] storage).                 */
/* Role of matrixmultiply::sgemm in tests/numerical_parity.rs:76-83.         */
/* ------------------------------------------------------------------------ */
typedef struct {
    int m, n, k;
    const float *a, *b;
    int64_t sam, sak, sbk, sbn;
    double *c;
    volatile int *next;
} f64_job;

static void *f64_worker(void *arg)
{
    const f64_job *j = (const f64_job *)arg;
    double *bt = NULL;
    for (;;) {
        int i = __sync_fetch_and_add(j->next, 1);
        if (i >= j->m) break;
        const float *arow = j->a + (size_t)i * j->sam;
        double *crow = j->c + (size_t)i * j->n;
        if (j->sbn == 1) { /* B rows contiguous in n: axpy form */
            for (int x = 0; x < j->n; ++x) crow[x] = 0.0;
            for (int l = 0; l < j->k; ++l) {
                const double av = arow[(size_t)l * j->sak];
                const float *brow = j->b + (size_t)l * j->sbk;
                for (int x = 0; x < j->n; ++x) crow[x] += av * (double)brow[x];
            }
        } else { /* dot-product form */
            for (int x = 0; x < j->n; ++x) {
                const float *bcol = j->b + (size_t)x * j->sbn;
                double s = 0.0;
                for (int l = 0; l < j->k; ++l)
                    s += (double)arow[(size_t)l * j->sak] * (double)bcol[(size_t)l * j->sbk];
                crow[x] = s;
            }
        }
    }
    free(bt);
    return NULL;
}

ORACLE_API int oracle_gemm_f64(int m, int n, int k, const float *a, int64_t sam, int64_t sak,
                               const float *b, int64_t sbk, int64_t sbn, double *c, int nthreads)
{
    if (m <= 0 || n <= 0 || k <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    volatile int next = 0;
    f64_job j = {m, n, k, a, b, sam, sak, sbk, sbn, c, &next};
    pthread_t th[256];
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t)
        if (pthread_create(&th[started], NULL, f64_worker, &j) == 0) ++started;
    f64_worker(&j);
    for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* E1/E2: epilogue chain on the fp32 accumulator                             */
/* functors: src/kernels/gpu/epilogue.cuh:12-63; op vocabulary:              */
/* src/core/op.rs:70-90; applied in vector order (src/emitter/cuda/          */
/* gemm.rs:35-60, conv.rs:91-116); BatchNorm formula:                        */
/* src/emitter/metal/utils.rs:56-73.                                         */
/* ------------------------------------------------------------------------ */
enum {
    ORACLE_EPI_NONE = 0,
    ORACLE_EPI_BIAS_ADD = 1,
    ORACLE_EPI_RELU = 2,
    ORACLE_EPI_GELU = 3,
    ORACLE_EPI_SILU = 4,
    ORACLE_EPI_RESIDUAL_ADD = 5,
    ORACLE_EPI_BIAS_ADD_SILU = 6,
    ORACLE_EPI_BATCHNORM = 7, /* (v-mean)*rsqrt(var+eps)*gamma+beta */
    ORACLE_EPI_SCALE_SHIFT = 8 /* folded BatchNorm: v*scale+shift */
};

typedef struct {
    int32_t kind;
    float epsilon;
    const float *p0; /* bias | residual | gamma | scale */
    const float *p1; /* beta | shift */
    const float *p2; /* mean */
    const float *p3; /* var */
} oracle_epilogue_op;

/* x is [rows, cols] row-major; channel = column index; residual index =
 * row*cols+col. */
ORACLE_API int oracle_epilogue_apply(float *x, int64_t rows, int64_t cols,
                                     const oracle_epilogue_op *ops, int nops)
{
    for (int o = 0; o < nops; ++o) {
        const oracle_epilogue_op *op = &ops[o];
        for (int64_t r = 0; r < rows; ++r) {
            float *row = x + r * cols;
            for (int64_t c = 0; c < cols; ++c) {
                float v = row[c];
                switch (op->kind) {
                case ORACLE_EPI_NONE: break;
                case ORACLE_EPI_BIAS_ADD: v = v + op->p0[c]; break;
                case ORACLE_EPI_RELU: v = fmaxf(0.0f, v); break;
                case ORACLE_EPI_GELU:
                    v = 0.5f * v * (1.0f + tanhf(0.79788456f * (v + 0.044715f * v * v * v)));
                    break;
                case ORACLE_EPI_SILU: v = v / (1.0f + expf(-v)); break;
                case ORACLE_EPI_RESIDUAL_ADD: v = v + op->p0[r * cols + c]; break;
                case ORACLE_EPI_BIAS_ADD_SILU:
                    v = v + op->p0[c];
                    v = v / (1.0f + expf(-v));
                    break;
                case ORACLE_EPI_BATCHNORM:
                    v = (v - op->p2[c]) * (1.0f / sqrtf(op->p3[c] + op->epsilon)) * op->p0[c] +
                        op->p1[c];
                    break;
                case ORACLE_EPI_SCALE_SHIFT: v = v * op->p0[c] + op->p1[c]; break;
                default: return -1;
                }
                row[c] = v;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* C1: magic_u32 (src/emitter/cuda/conv.rs:6-16)                             */
/* n<=1 -> (0,0); power of two -> (0, log2 n); else the smallest p in        */
/* [32,64) with m = ceil(2^p / n) < 2^32 -> (m, p).                          */
/* ------------------------------------------------------------------------ */
ORACLE_API void oracle_magic_u32(uint32_t n, uint32_t *m_out, uint32_t *p_out)
{
    *m_out = 0;
    *p_out = 0;
    if (n <= 1) return;
    if ((n & (n - 1)) == 0) {
        *p_out = (uint32_t)__builtin_ctz(n);
        return;
    }
    for (uint32_t p = 32; p < 64; ++p) {
        uint64_t m = (((uint64_t)1 << p) + n - 1) / n;
        if (m < ((uint64_t)1 << 32)) {
            *m_out = (uint32_t)m;
            *p_out = p;
            return;
        }
    }
}

/* C1b: device fast_divmod (src/emitter/cuda/conv.rs:144-151) with the
 * self-consistent shift convention of examples/jit_conv_verify.py:6-13:
 * s is the shift beyond 32, i.e. s = p - 32 for the (m,p) of magic_u32. */
ORACLE_API void oracle_fast_divmod(int32_t n, uint32_t m, int32_t s, int32_t d, int32_t *q,
                                   int32_t *r)
{
    if (d == 1) {
        *q = n;
        *r = 0;
    } else if (m == 0) {
        *q = n >> s;
        *r = n & (d - 1);
    } else {
        *q = (int32_t)(((uint64_t)(uint32_t)n * m) >> (32 + s));
        *r = n - *q * d;
    }
}

/* (magic, shift) in the form fast_divmod consumes. */
static void magic_for_divmod(uint32_t d, uint32_t *m, int32_t *s)
{
    uint32_t mm, p;
    oracle_magic_u32(d, &mm, &p);
    *m = mm;
    *s = (mm == 0) ? (int32_t)p : (int32_t)p - 32;
}

/* Checks fast_divmod == (/ , %) for every n in [0, n_max); returns the first
 * n that disagrees, or -1 when all agree. */
ORACLE_API int64_t oracle_divmod_check(uint32_t d, uint32_t n_max)
{
    uint32_t m;
    int32_t s;
    magic_for_divmod(d, &m, &s);
    for (uint32_t n = 0; n < n_max; ++n) {
        int32_t q, r;
        oracle_fast_divmod((int32_t)n, m, s, (int32_t)d, &q, &r);
        if ((uint32_t)q != n / d || (uint32_t)r != n % d) return (int64_t)n;
    }
    return -1;
}

/* ------------------------------------------------------------------------ */
/* C2: ConvParams, 12 x i32 + 8 x u32 = 80 bytes                             */
/* (src/emitter/cuda/conv.rs:134-142; packing src/interface/python.rs:423-435)*/
/* ------------------------------------------------------------------------ */
typedef struct {
    int32_t batch, h_in, w_in, c_in, k_out;
    int32_t h_out, w_out, r_sz, s_sz;
    int32_t stride, pad, dilation;
    uint32_t hw_m, hw_s, w_m, w_s, sic_m, sic_s, c_m, c_s;
} oracle_conv_params;

ORACLE_API int oracle_conv_params_pack(int n, int h, int w, int c, int k, int r, int s, int stride,
                                       int pad, int dilation, oracle_conv_params *p)
{
    if (n <= 0 || h <= 0 || w <= 0 || c <= 0 || k <= 0 || r <= 0 || s <= 0 || stride <= 0 ||
        pad < 0 || dilation <= 0)
        return -1;
    p->batch = n; p->h_in = h; p->w_in = w; p->c_in = c; p->k_out = k;
    p->h_out = (h + 2 * pad - dilation * (r - 1) - 1) / stride + 1;
    p->w_out = (w + 2 * pad - dilation * (s - 1) - 1) / stride + 1;
    p->r_sz = r; p->s_sz = s; p->stride = stride; p->pad = pad; p->dilation = dilation;
    int32_t sh;
    magic_for_divmod((uint32_t)(p->h_out * p->w_out), &p->hw_m, &sh); p->hw_s = (uint32_t)sh;
    magic_for_divmod((uint32_t)p->w_out, &p->w_m, &sh);               p->w_s = (uint32_t)sh;
    magic_for_divmod((uint32_t)(s * c), &p->sic_m, &sh);              p->sic_s = (uint32_t)sh;
    magic_for_divmod((uint32_t)c, &p->c_m, &sh);                      p->c_s = (uint32_t)sh;
    return 0;
}

/* C3/C4 coordinate tables (src/emitter/cuda/conv.rs:176-191, 208-226).
 * rows[m] = {bn, ho, wo} and base_off[m] = bn*H*W*C for every GEMM row;
 * cols[k] = {r, s, ci} for every GEMM k; both through fast_divmod. */
ORACLE_API void oracle_conv_coords(const oracle_conv_params *p, int32_t *rows /*[M,3]*/,
                                   int64_t *base_off /*[M]*/, int32_t *cols /*[K,3]*/)
{
    const int m_gemm = p->batch * p->h_out * p->w_out;
    const int k_gemm = p->r_sz * p->s_sz * p->c_in;
    for (int m = 0; m < m_gemm; ++m) {
        int32_t bn, rem, ho, wo;
        oracle_fast_divmod(m, p->hw_m, (int32_t)p->hw_s, p->h_out * p->w_out, &bn, &rem);
        oracle_fast_divmod(rem, p->w_m, (int32_t)p->w_s, p->w_out, &ho, &wo);
        rows[3 * m] = bn; rows[3 * m + 1] = ho; rows[3 * m + 2] = wo;
        base_off[m] = (int64_t)bn * p->h_in * p->w_in * p->c_in;
    }
    for (int k = 0; k < k_gemm; ++k) {
        int32_t rf, rem, sf, ci;
        oracle_fast_divmod(k, p->sic_m, (int32_t)p->sic_s, p->s_sz * p->c_in, &rf, &rem);
        oracle_fast_divmod(rem, p->c_m, (int32_t)p->c_s, p->c_in, &sf, &ci);
        cols[3 * k] = rf; cols[3 * k + 1] = sf; cols[3 * k + 2] = ci;
    }
}

/* ------------------------------------------------------------------------ */
/* C3 value oracle: direct convolution, NHWC input, [R,S,C,K] weights, NHWK  */
/* output (examples/verify_conv2d.rs:8-44; index formulas conv.rs:214-226,   */
/* 253, 316).  Accumulates in double so the result is the correctly rounded  */
/* target the fp32-accumulating kernels are measured against.                */
/* ------------------------------------------------------------------------ */
typedef struct {
    const float *x, *w;
    float *y;
    int n, h, wd, c, k, r, s, stride, pad, dil, ho, wo;
    volatile int *next;
} conv_job;

static void *conv_worker(void *arg)
{
    const conv_job *j = (const conv_job *)arg;
    const int rows = j->n * j->ho;
    double *acc = (double *)malloc(sizeof(double) * (size_t)j->k);
    for (;;) {
        int row = __sync_fetch_and_add(j->next, 1);
        if (row >= rows) break;
        const int bi = row / j->ho, hi = row % j->ho;
        for (int wi = 0; wi < j->wo; ++wi) {
            for (int ki = 0; ki < j->k; ++ki) acc[ki] = 0.0;
            for (int ri = 0; ri < j->r; ++ri) {
                const int cur_h = hi * j->stride - j->pad + ri * j->dil;
                if (cur_h < 0 || cur_h >= j->h) continue;
                for (int si = 0; si < j->s; ++si) {
                    const int cur_w = wi * j->stride - j->pad + si * j->dil;
                    if (cur_w < 0 || cur_w >= j->wd) continue;
                    const float *xin = j->x + (((size_t)bi * j->h + cur_h) * j->wd + cur_w) * j->c;
                    const float *wf = j->w + ((size_t)(ri * j->s + si) * j->c) * j->k;
                    for (int ci = 0; ci < j->c; ++ci) {
                        const double xv = xin[ci];
                        const float *wrow = wf + (size_t)ci * j->k;
                        for (int ki = 0; ki < j->k; ++ki) acc[ki] += xv * (double)wrow[ki];
                    }
                }
            }
            float *out = j->y + (((size_t)bi * j->ho + hi) * j->wo + wi) * j->k;
            for (int ki = 0; ki < j->k; ++ki) out[ki] = (float)acc[ki];
        }
    }
    free(acc);
    return NULL;
}

ORACLE_API int oracle_conv2d_nhwc(const float *x, const float *w, float *y, int n, int h, int wd,
                                  int c, int k, int r, int s, int stride, int pad, int dilation,
                                  int nthreads)
{
    if (n <= 0 || h <= 0 || wd <= 0 || c <= 0 || k <= 0 || r <= 0 || s <= 0 || stride <= 0 ||
        pad < 0 || dilation <= 0)
        return -1;
    const int ho = (h + 2 * pad - dilation * (r - 1) - 1) / stride + 1;
    const int wo = (wd + 2 * pad - dilation * (s - 1) - 1) / stride + 1;
    if (ho <= 0 || wo <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    volatile int next = 0;
    conv_job j = {x, w, y, n, h, wd, c, k, r, s, stride, pad, dilation, ho, wo, &next};
    pthread_t th[256];
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t)
        if (pthread_create(&th[started], NULL, conv_worker, &j) == 0) ++started;
    conv_worker(&j);
    for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Transposed convolution, NHWC input, weights [C*R*S, K] (row c*R*S + r*S + s */
/* as the reference kernel indexes them, src/emitter/conv_transpose.rs:207-   */
/* 225, 236), NHWK output.  The value is that of the reference's own CPU     */
/* statement (examples/verify_conv_transpose.rs:12-54: ho = hi*stride - pad  */
/* + r), written as the gather the kernel performs (hi = (ho + pad - r) /    */
/* stride where that division is exact).  Accumulates in double.             */
/* ------------------------------------------------------------------------ */
typedef struct {
    const float *x, *w;
    float *y;
    int n, h, wd, c, k, r, s, sh, sw, ph, pw, ho, wo;
    volatile int *next;
} convt_job;

static void *convt_worker(void *arg)
{
    const convt_job *j = (const convt_job *)arg;
    const int rows = j->n * j->ho;
    double *acc = (double *)malloc(sizeof(double) * (size_t)j->k);
    for (;;) {
        int row = __sync_fetch_and_add(j->next, 1);
        if (row >= rows) break;
        const int bi = row / j->ho, oh = row % j->ho;
        for (int ow = 0; ow < j->wo; ++ow) {
            for (int ki = 0; ki < j->k; ++ki) acc[ki] = 0.0;
            for (int ri = 0; ri < j->r; ++ri) {
                const int th = oh + j->ph - ri;
                if (th < 0 || th % j->sh != 0 || th / j->sh >= j->h) continue;
                for (int si = 0; si < j->s; ++si) {
                    const int tw = ow + j->pw - si;
                    if (tw < 0 || tw % j->sw != 0 || tw / j->sw >= j->wd) continue;
                    const float *xin =
                        j->x + (((size_t)bi * j->h + th / j->sh) * j->wd + tw / j->sw) * j->c;
                    for (int ci = 0; ci < j->c; ++ci) {
                        const double xv = xin[ci];
                        const float *wrow = j->w + ((size_t)(ci * j->r + ri) * j->s + si) * j->k;
                        for (int ki = 0; ki < j->k; ++ki) acc[ki] += xv * (double)wrow[ki];
                    }
                }
            }
            float *out = j->y + (((size_t)bi * j->ho + oh) * j->wo + ow) * j->k;
            for (int ki = 0; ki < j->k; ++ki) out[ki] = (float)acc[ki];
        }
    }
    free(acc);
    return NULL;
}

ORACLE_API int oracle_conv_transpose2d_nhwc(const float *x, const float *w, float *y, int n, int h,
                                            int wd, int c, int k, int r, int s, int stride_h,
                                            int stride_w, int pad_h, int pad_w, int opad_h,
                                            int opad_w, int nthreads)
{
    if (n <= 0 || h <= 0 || wd <= 0 || c <= 0 || k <= 0 || r <= 0 || s <= 0 || stride_h <= 0 ||
        stride_w <= 0 || pad_h < 0 || pad_w < 0 || opad_h < 0 || opad_w < 0)
        return -1;
    /* H_out = (H_in - 1) * stride - 2 * pad + kernel + output_padding (conv_transpose.rs:36-37) */
    const int ho = (h - 1) * stride_h - 2 * pad_h + r + opad_h;
    const int wo = (wd - 1) * stride_w - 2 * pad_w + s + opad_w;
    if (ho <= 0 || wo <= 0) return -1;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    volatile int next = 0;
    convt_job j = {x, w, y, n, h, wd, c, k, r, s, stride_h, stride_w, pad_h, pad_w, ho, wo, &next};
    pthread_t th[256];
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t)
        if (pthread_create(&th[started], NULL, convt_worker, &j) == 0) ++started;
    convt_worker(&j);
    for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* A2 value oracle: O = softmax(scale * Q K^T [causal: j > i masked]) V      */
/* for ONE (batch, head) slice, Q/K/V/O row-major [S, D]                     */
/* (examples/verify_fa2_numeric.rs:22-93; causal mask = strictly future      */
/* keys, cuda_emitter.rs.tmp:217-218).  Only the query rows listed in        */
/* row_idx are evaluated, so a sampled check of a long sequence stays cheap; */
/* out is [nrows, D].  Scores and sums are held in double.                   */
/* ------------------------------------------------------------------------ */
typedef struct {
    const float *q, *k, *v;
    float *o;
    int s, d, causal;
    float scale;
    const int32_t *rows;
    int nrows;
    volatile int *next;
} attn_job;

static void *attn_worker(void *arg)
{
    const attn_job *j = (const attn_job *)arg;
    double *p = (double *)malloc(sizeof(double) * (size_t)j->s);
    double *acc = (double *)malloc(sizeof(double) * (size_t)j->d);
    for (;;) {
        int t = __sync_fetch_and_add(j->next, 1);
        if (t >= j->nrows) break;
        const int i = j->rows[t];
        const int jmax = j->causal ? i + 1 : j->s;
        const float *qi = j->q + (size_t)i * j->d;
        double mx = -INFINITY;
        for (int c = 0; c < jmax; ++c) {
            const float *kc = j->k + (size_t)c * j->d;
            double dot = 0.0;
            for (int dd = 0; dd < j->d; ++dd) dot += (double)qi[dd] * (double)kc[dd];
            p[c] = dot * (double)j->scale;
            if (p[c] > mx) mx = p[c];
        }
        double sum = 0.0;
        for (int c = 0; c < jmax; ++c) {
            p[c] = exp(p[c] - mx);
            sum += p[c];
        }
        for (int dd = 0; dd < j->d; ++dd) acc[dd] = 0.0;
        for (int c = 0; c < jmax; ++c) {
            const float *vc = j->v + (size_t)c * j->d;
            const double pc = p[c];
            for (int dd = 0; dd < j->d; ++dd) acc[dd] += pc * (double)vc[dd];
        }
        float *out = j->o + (size_t)t * j->d;
        for (int dd = 0; dd < j->d; ++dd) out[dd] = (float)(acc[dd] / sum);
    }
    free(p);
    free(acc);
    return NULL;
}

ORACLE_API int oracle_attention(const float *q, const float *k, const float *v, float *o, int s,
                                int d, float scale, int causal, const int32_t *row_idx, int nrows,
                                int nthreads)
{
    if (s <= 0 || d <= 0 || nrows < 0) return -1;
    for (int t = 0; t < nrows; ++t)
        if (row_idx[t] < 0 || row_idx[t] >= s) return -1;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    volatile int next = 0;
    attn_job j = {q, k, v, o, s, d, causal, scale, row_idx, nrows, &next};
    pthread_t th[256];
    int started = 0;
    for (int t = 0; t < nthreads - 1; ++t)
        if (pthread_create(&th[started], NULL, attn_worker, &j) == 0) ++started;
    attn_worker(&j);
    for (int t = 0; t < started; ++t) pthread_join(th[t], NULL);
    return 0;
}
