/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of incin's CPU attention op.
 *
 * Nothing in the shipped library may link, load or call this file.  It exists so
 * that tests, the smoke check and the benchmark's CPU-baseline leg have an
 * independent statement of what the reference CPU backend computes for
 * `scaled_dot_product_attention`.
 *
 * The reference (a Rust workspace) cannot be compiled in this environment, so
 * this is a restatement of its algorithm, step for step, in plain C:
 *
 *   composition          crates/incin-backends/src/cpu/ops/shape_ops.rs:1245-1269
 *   batched matmul       crates/incin-backends/src/cpu/ops/matmul.rs:170-255
 *   kernel choice        crates/incin-backends/src/cpu/ops/matmul.rs:316-329, 395-420
 *   f64-accumulate arm   crates/incin-backends/src/cpu/ops/matmul.rs:516-527
 *   FMA row-stream arm   crates/incin-backends/src/cpu/ops/matmul.rs:532-573
 *   mul-then-add arm     crates/incin-backends/src/cpu/ops/matmul.rs:502-515
 *   scalar multiply      crates/incin-backends/src/cpu/ops/elementwise_kernel.rs:87
 *   mask add             crates/incin-backends/src/cpu/ops/elementwise.rs:242-262
 *   softmax              crates/incin-backends/src/cpu/ops/elementwise.rs:971-980, 1062-1077
 *   row max              crates/incin-backends/src/cpu/ops/reduce.rs:160-185
 *   row sum              crates/incin-backends/src/cpu/ops/reduce.rs:87-121
 *   triu (causal mask)   crates/incin-backends/src/cpu/ops/shape_ops.rs:808-830
 *
 * Parity status.  No test in the reference asserts a value produced by its
 * attention operator (the single caller checks the output shape only), so at
 * operator level the reference leaves parity unpinned bitwise.  What pins this
 * file is: the reference's own known-answer vectors for hand-composed
 * attention, matmul and softmax (tests/golden/reference_vectors.json), an
 * independent float64 numpy evaluation, and closed-form invariants
 * (tests/test_oracle_*.py).  Those pin every function below to well inside the
 * 1e-5 tolerance; the exact rounding sequence (f64->f32 narrowing, sequential
 * f32 row sum, the double expf, FMA arm selection) is restated from source
 * but "parity unpinned" at the bit level.
 *
 * Build: see oracle/Makefile (-O2 -ffp-contract=off: the compiler must not fuse
 * or reassociate; FMA appears only where the reference calls it explicitly).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_MAX_BATCH_DIMS 6

/* One attention problem.  All strides are in elements; a stride of 0 states a
 * broadcast axis.  Batch axes are already right-aligned by the caller to the
 * broadcast batch shape `bshape` (rule: cpu/stride.rs:86-106). */
typedef struct {
    int32_t nb;                                   /* number of batch axes */
    int64_t bshape[ORACLE_MAX_BATCH_DIMS];        /* broadcast batch shape */
    int64_t q_bs[ORACLE_MAX_BATCH_DIMS];
    int64_t k_bs[ORACLE_MAX_BATCH_DIMS];
    int64_t v_bs[ORACLE_MAX_BATCH_DIMS];
    int64_t m_bs[ORACLE_MAX_BATCH_DIMS];
    int64_t Sq, Skv, D, Dv;
    int64_t q_rs, q_cs;                           /* q[i,d]   */
    int64_t k_rs, k_cs;                           /* k[j,d]   */
    int64_t v_rs, v_cs;                           /* v[j,c]   */
    int64_t m_rs, m_cs;                           /* mask[i,j] */
    const float *q, *k, *v;
    const float *mask;                            /* nullable dense additive mask */
    /* Synthesised additive mask, used when `mask` is NULL and one of these is
     * set; it takes exactly the values the dense tensor built with the
     * reference's own ops would hold: 0 where attended, -inf where not
     * (`full(-inf).triu(1)`: entries with col >= row + 1 keep -inf, others 0). */
    int32_t causal;                               /* key j masked when j > i + (Skv - Sq) */
    const int32_t *kv_lens;                       /* nullable, one per flattened batch index of k: key j masked when j >= len */
    int64_t kv_lens_bs[ORACLE_MAX_BATCH_DIMS];    /* strides of kv_lens over the batch axes */
    int32_t has_scale;
    double scale;                                 /* used when has_scale != 0 */
    int32_t host_has_fma;                         /* 1: AVX2+FMA host (FMA arm); 0: mul-then-add arm */
} oracle_sdpa_t;

/* ---- matmul arms ------------------------------------------------------- */

/* cpu/ops/matmul.rs:516-527 -- operand read as f64, separate multiply and add,
 * one narrowing to f32 per output element. */
void oracle_gemm_f64acc(int64_t m, int64_t k, int64_t n,
                        const float *lhs, int64_t lrs, int64_t lcs,
                        const float *rhs, int64_t rrs, int64_t rcs,
                        float *out)
{
    for (int64_t row = 0; row < m; ++row) {
        for (int64_t col = 0; col < n; ++col) {
            double acc = 0.0;
            for (int64_t depth = 0; depth < k; ++depth) {
                double a = (double)lhs[row * lrs + depth * lcs];
                double b = (double)rhs[depth * rrs + col * rcs];
                double prod = a * b;
                acc = acc + prod;
            }
            out[row * n + col] = (float)acc;
        }
    }
}

/* cpu/ops/matmul.rs:532-573 -- output row streamed over depth; lanes below
 * n - n%8 use a fused multiply-add, the tail multiplies then adds.
 * `out` must be zero on entry (matmul.rs:234). */
void oracle_gemm_fma_rows(int64_t m, int64_t k, int64_t n,
                          const float *lhs, int64_t lrs, int64_t lcs,
                          const float *rhs, int64_t rrs,
                          float *out)
{
    int64_t n_vec = n - (n % 8);
    for (int64_t row = 0; row < m; ++row) {
        float *o = out + row * n;
        for (int64_t depth = 0; depth < k; ++depth) {
            float s = lhs[row * lrs + depth * lcs];
            const float *r = rhs + depth * rrs;
            for (int64_t col = 0; col < n_vec; ++col) o[col] = fmaf(s, r[col], o[col]);
            for (int64_t col = n_vec; col < n; ++col) {
                float prod = s * r[col];
                o[col] = o[col] + prod;
            }
        }
    }
}

/* cpu/ops/matmul.rs:502-515 -- hosts without AVX2+FMA: multiply, then add. */
void oracle_gemm_muladd_rows(int64_t m, int64_t k, int64_t n,
                             const float *lhs, int64_t lrs, int64_t lcs,
                             const float *rhs, int64_t rrs,
                             float *out)
{
    for (int64_t row = 0; row < m; ++row) {
        float *o = out + row * n;
        for (int64_t depth = 0; depth < k; ++depth) {
            float s = lhs[row * lrs + depth * lcs];
            const float *r = rhs + depth * rrs;
            for (int64_t col = 0; col < n; ++col) {
                float prod = s * r[col];
                o[col] = o[col] + prod;
            }
        }
    }
}

/* cpu/ops/matmul.rs:316-329 with 395-420: the row-streaming arms apply only
 * when the right operand's column stride is 1. */
void oracle_gemm(int64_t m, int64_t k, int64_t n,
                 const float *lhs, int64_t lrs, int64_t lcs,
                 const float *rhs, int64_t rrs, int64_t rcs,
                 float *out, int host_has_fma)
{
    memset(out, 0, (size_t)(m * n) * sizeof(float));
    if (rcs == 1) {
        if (host_has_fma) oracle_gemm_fma_rows(m, k, n, lhs, lrs, lcs, rhs, rrs, out);
        else oracle_gemm_muladd_rows(m, k, n, lhs, lrs, lcs, rhs, rrs, out);
    } else {
        oracle_gemm_f64acc(m, k, n, lhs, lrs, lcs, rhs, rrs, rcs, out);
    }
}

/* ---- softmax over one contiguous row ------------------------------------ */

/* elementwise.rs:971-980 (softmax = exp(log_softmax)), :1062-1077
 * (max_keepdim, sub, exp, sum_keepdim, log, sub), reduce.rs:160-185 (max is
 * tracked in f64 from -inf with a strict '>' so NaN never wins), reduce.rs:87-121
 * (sum is a sequential f32 '+=' from 0).  `tmp` holds n floats. */
void oracle_softmax_row(const float *x, int64_t n, float *p, float *tmp)
{
    double best = -INFINITY;
    for (int64_t j = 0; j < n; ++j) {
        double v = (double)x[j];
        if (v > best) best = v;
    }
    float mx = (float)best;
    for (int64_t j = 0; j < n; ++j) tmp[j] = x[j] - mx;          /* diff */
    float sum = 0.0f;
    for (int64_t j = 0; j < n; ++j) {
        float e = expf(tmp[j]);                                    /* exp_diff */
        sum = sum + e;
    }
    float lse = logf(sum);
    for (int64_t j = 0; j < n; ++j) p[j] = expf(tmp[j] - lse);
}

/* log_softmax alone (elementwise.rs:1062-1077), exposed for the reference's
 * own known-answer vector on it. */
void oracle_log_softmax_row(const float *x, int64_t n, float *out)
{
    double best = -INFINITY;
    for (int64_t j = 0; j < n; ++j) {
        double v = (double)x[j];
        if (v > best) best = v;
    }
    float mx = (float)best;
    float sum = 0.0f;
    for (int64_t j = 0; j < n; ++j) {
        out[j] = x[j] - mx;
        sum = sum + expf(out[j]);
    }
    float lse = logf(sum);
    for (int64_t j = 0; j < n; ++j) out[j] = out[j] - lse;
}

/* ---- helpers ---------------------------------------------------------------- */

static void unflatten(const oracle_sdpa_t *p, int64_t flat, int64_t *idx)
{
    for (int a = p->nb - 1; a >= 0; --a) {
        idx[a] = flat % p->bshape[a];
        flat /= p->bshape[a];
    }
}

static int64_t dot_idx(const int64_t *idx, const int64_t *strides, int nb)
{
    int64_t off = 0;
    for (int a = 0; a < nb; ++a) off += idx[a] * strides[a];
    return off;
}

int64_t oracle_batch_count(const oracle_sdpa_t *p)
{
    int64_t n = 1;
    for (int a = 0; a < p->nb; ++a) n *= p->bshape[a];
    return n;
}

static float scale_as_f32(const oracle_sdpa_t *p)
{
    /* shape_ops.rs:1258-1260: d_k is q's last dim; elementwise_kernel.rs:87: cast to f32 */
    double s = p->has_scale ? p->scale : 1.0 / sqrt((double)p->D);
    return (float)s;
}

static float synth_mask(const oracle_sdpa_t *p, const int64_t *bidx, int64_t i, int64_t j)
{
    int masked = 0;
    if (p->causal && j > i + (p->Skv - p->Sq)) masked = 1;
    if (p->kv_lens) {
        int32_t len = p->kv_lens[dot_idx(bidx, p->kv_lens_bs, p->nb)];
        if (j >= (int64_t)len) masked = 1;
    }
    return masked ? -INFINITY : 0.0f;
}

/* One query row of one batch element, in exactly the arithmetic of the
 * composition.  Every value of the reference's result depends on its own
 * score row only, so this row-at-a-time form gives the same bits as the
 * materialising form below while needing O(Skv) memory.
 * work: 3*Skv floats. */
static void sdpa_one_row(const oracle_sdpa_t *p, int64_t bflat, int64_t i, float *out_row, float *work)
{
    int64_t bidx[ORACLE_MAX_BATCH_DIMS];
    unflatten(p, bflat, bidx);
    const float *q = p->q + dot_idx(bidx, p->q_bs, p->nb);
    const float *k = p->k + dot_idx(bidx, p->k_bs, p->nb);
    const float *v = p->v + dot_idx(bidx, p->v_bs, p->nb);
    float *x = work, *pr = work + p->Skv, *tmp = work + 2 * p->Skv;
    float sc = scale_as_f32(p);

    /* scores = q @ transpose(k): the transposed view has row stride k_cs and
     * column stride k_rs (storage.rs:308-325). */
    const float *qrow = q + i * p->q_rs;
    if (p->k_rs == 1) {
        memset(x, 0, (size_t)p->Skv * sizeof(float));
        if (p->host_has_fma) oracle_gemm_fma_rows(1, p->D, p->Skv, qrow, 0, p->q_cs, k, p->k_cs, x);
        else oracle_gemm_muladd_rows(1, p->D, p->Skv, qrow, 0, p->q_cs, k, p->k_cs, x);
    } else {
        oracle_gemm_f64acc(1, p->D, p->Skv, qrow, 0, p->q_cs, k, p->k_cs, p->k_rs, x);
    }
    for (int64_t j = 0; j < p->Skv; ++j) x[j] = x[j] * sc;
    if (p->mask) {
        const float *m = p->mask + dot_idx(bidx, p->m_bs, p->nb) + i * p->m_rs;
        for (int64_t j = 0; j < p->Skv; ++j) x[j] = x[j] + m[j * p->m_cs];
    } else if (p->causal || p->kv_lens) {
        for (int64_t j = 0; j < p->Skv; ++j) x[j] = x[j] + synth_mask(p, bidx, i, j);
    }
    oracle_softmax_row(x, p->Skv, pr, tmp);
    memset(out_row, 0, (size_t)p->Dv * sizeof(float));
    if (p->v_cs == 1) {
        if (p->host_has_fma) oracle_gemm_fma_rows(1, p->Skv, p->Dv, pr, 0, 1, v, p->v_rs, out_row);
        else oracle_gemm_muladd_rows(1, p->Skv, p->Dv, pr, 0, 1, v, p->v_rs, out_row);
    } else {
        oracle_gemm_f64acc(1, p->Skv, p->Dv, pr, 0, 1, v, p->v_rs, p->v_cs, out_row);
    }
}

/* Selected rows: out is [n_rows, Dv].  Rows are independent; OpenMP only
 * distributes them, it does not change any row's arithmetic. */
int oracle_sdpa_rows(const oracle_sdpa_t *p, int64_t n_rows,
                     const int64_t *row_batch, const int64_t *row_i, float *out)
{
    int fail = 0;
#pragma omp parallel
    {
        float *work = (float *)malloc((size_t)(3 * p->Skv + 8) * sizeof(float));
        if (!work) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for schedule(dynamic, 4)
        for (int64_t r = 0; r < n_rows; ++r) {
            if (work) sdpa_one_row(p, row_batch[r], row_i[r], out + r * p->Dv, work);
        }
        free(work);
    }
    return fail;
}

/* Full output [batch..., Sq, Dv] contiguous, row-streaming form. */
int oracle_sdpa(const oracle_sdpa_t *p, float *out)
{
    int64_t nbatch = oracle_batch_count(p);
    int64_t total = nbatch * p->Sq;
    int fail = 0;
#pragma omp parallel
    {
        float *work = (float *)malloc((size_t)(3 * p->Skv + 8) * sizeof(float));
        if (!work) {
#pragma omp atomic write
            fail = 1;
        }
#pragma omp for schedule(dynamic, 4)
        for (int64_t r = 0; r < total; ++r) {
            if (work) sdpa_one_row(p, r / p->Sq, r % p->Sq, out + r * p->Dv, work);
        }
        free(work);
    }
    return fail;
}

/* ---- materialising form (CPU-baseline timing) ---------------------------------
 * Same arithmetic, but laid out as the reference executes it: every step of
 * the composition writes a whole new buffer; both matmuls and both reductions
 * run on the calling thread; dense elementwise maps of >= 2M elements are
 * spread over threads (elementwise_kernel.rs:25-29, 563-568 -- rayon there,
 * OpenMP here).  Returns 0, or 1 when memory runs out. */
#define PAR_THRESHOLD (2 * 1024 * 1024)

int oracle_sdpa_materialised(const oracle_sdpa_t *p, float *out)
{
    int64_t nbatch = oracle_batch_count(p);
    int64_t Sq = p->Sq, Skv = p->Skv, Dv = p->Dv;
    int64_t tile = Sq * Skv, total = nbatch * tile, rows = nbatch * Sq;
    float sc = scale_as_f32(p);
    float *scores = malloc((size_t)total * 4), *scaled = malloc((size_t)total * 4);
    float *masked = NULL;
    float *mx = malloc((size_t)rows * 4), *diff = malloc((size_t)total * 4);
    float *ex = malloc((size_t)total * 4), *sm = malloc((size_t)rows * 4), *lg = malloc((size_t)rows * 4);
    float *lsm = malloc((size_t)total * 4), *attn = malloc((size_t)total * 4);
    int has_mask = p->mask || p->causal || p->kv_lens;
    if (has_mask) masked = malloc((size_t)total * 4);
    int rc = 1;
    if (!scores || !scaled || !mx || !diff || !ex || !sm || !lg || !lsm || !attn || (has_mask && !masked)) goto done;

    int64_t bidx[ORACLE_MAX_BATCH_DIMS];
    for (int64_t b = 0; b < nbatch; ++b) {                         /* matmul #1, serial */
        unflatten(p, b, bidx);
        const float *q = p->q + dot_idx(bidx, p->q_bs, p->nb);
        const float *k = p->k + dot_idx(bidx, p->k_bs, p->nb);
        oracle_gemm(Sq, p->D, Skv, q, p->q_rs, p->q_cs, k, p->k_cs, p->k_rs, scores + b * tile, p->host_has_fma);
    }
#pragma omp parallel for if (total >= PAR_THRESHOLD)
    for (int64_t e = 0; e < total; ++e) scaled[e] = scores[e] * sc;
    const float *xin = scaled;
    if (has_mask) {
#pragma omp parallel for if (total >= PAR_THRESHOLD)
        for (int64_t b = 0; b < nbatch; ++b) {
            int64_t bi[ORACLE_MAX_BATCH_DIMS];
            unflatten(p, b, bi);
            const float *m = p->mask ? p->mask + dot_idx(bi, p->m_bs, p->nb) : NULL;
            for (int64_t i = 0; i < Sq; ++i)
                for (int64_t j = 0; j < Skv; ++j) {
                    float mv = m ? m[i * p->m_rs + j * p->m_cs] : synth_mask(p, bi, i, j);
                    masked[b * tile + i * Skv + j] = scaled[b * tile + i * Skv + j] + mv;
                }
        }
        xin = masked;
    }
    for (int64_t r = 0; r < rows; ++r) {                           /* max_keepdim, serial */
        double best = -INFINITY;
        for (int64_t j = 0; j < Skv; ++j) {
            double vv = (double)xin[r * Skv + j];
            if (vv > best) best = vv;
        }
        mx[r] = (float)best;
    }
#pragma omp parallel for if (total >= PAR_THRESHOLD)
    for (int64_t e = 0; e < total; ++e) diff[e] = xin[e] - mx[e / Skv];
#pragma omp parallel for if (total >= PAR_THRESHOLD)
    for (int64_t e = 0; e < total; ++e) ex[e] = expf(diff[e]);
    for (int64_t r = 0; r < rows; ++r) {                           /* sum_keepdim, serial */
        float s = 0.0f;
        for (int64_t j = 0; j < Skv; ++j) s = s + ex[r * Skv + j];
        sm[r] = s;
    }
    for (int64_t r = 0; r < rows; ++r) lg[r] = logf(sm[r]);
#pragma omp parallel for if (total >= PAR_THRESHOLD)
    for (int64_t e = 0; e < total; ++e) lsm[e] = diff[e] - lg[e / Skv];
#pragma omp parallel for if (total >= PAR_THRESHOLD)
    for (int64_t e = 0; e < total; ++e) attn[e] = expf(lsm[e]);
    for (int64_t b = 0; b < nbatch; ++b) {                         /* matmul #2, serial */
        unflatten(p, b, bidx);
        const float *v = p->v + dot_idx(bidx, p->v_bs, p->nb);
        oracle_gemm(Sq, Skv, Dv, attn + b * tile, Skv, 1, v, p->v_rs, p->v_cs, out + b * Sq * Dv, p->host_has_fma);
    }
    rc = 0;
done:
    free(scores); free(scaled); free(masked); free(mx); free(diff);
    free(ex); free(sm); free(lg); free(lsm); free(attn);
    return rc;
}

/* triu as the reference's CPU backend evaluates it on a [rows, cols] matrix
 * (shape_ops.rs:808-830): keep entries with col >= row + k, write 0 elsewhere. */
void oracle_triu(const float *in, int64_t rows, int64_t cols, int64_t k, float *out)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c)
            out[r * cols + c] = (c >= r + k) ? in[r * cols + c] : 0.0f;
}

size_t oracle_struct_size(void) { return sizeof(oracle_sdpa_t); }
