/*
 * CPU oracle for the sparse-MLP decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference
 * (NimbleEdge/sparse_transformers) for the one path this repository
 * accelerates.  It exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg have something to compare the HIP kernels against.  The
 * product path (sparse_transformers_amd/) never imports, links or calls it.
 *
 * What each function follows (paths relative to the reference checkout):
 *   orc_cache_create          sparse_transformers/csrc/weight_cache.h:155-227
 *   orc_cache_update          sparse_transformers/csrc/weight_cache.h:84-110,229-359
 *   orc_cache_rebuild (static) sparse_transformers/csrc/weight_cache.h:113-145
 *   orc_mlp_forward           sparse_transformers/csrc/sparse_mlp_op.cpp:89-117,133-191
 *                             (act=RELU is that operator; other activations
 *                              follow src/modeling_skip.py:114-117 and, ungated,
 *                              src/models/opt/modelling_opt_skip.py:116-119)
 *   orc_predictor_scores      src/modeling_skip.py:32-53  (FastLoRAProjection)
 *   orc_mask_threshold        src/modeling_skip.py:206-207,214 (naive, thr = 0, >=)
 *   orc_mask_topk             src/modeling_skip.py:208-211,214
 *   orc_mask_statistical      src/modeling_skip.py:197-202,212-214
 *   orc_approx_topk_threshold sparse_transformers/csrc/approx_topk.h:10-88
 *
 * How the oracle itself is pinned (the reference ships no tests or vectors):
 *   - cache order / layout: against the reference's own C++ compiled from its
 *     sources (oracle/_ref, built by oracle/Makefile) on random mask traces,
 *     and against the golden traces under tests/golden/ written from that
 *     build; plus the invariants  set(indices) == nonzero(mask),
 *     active rows == pool rows (bitwise).
 *   - forward, act=RELU: against the compiled reference operator; all
 *     activations: against float64 closed forms evaluated with numpy/torch.
 *   - predictor / masks: against float64 numpy closed forms, numpy
 *     partition/argsort for top-k, brute force on tiny inputs.
 *   - approx top-k threshold: against the compiled reference operator
 *     (bit-equal: only max, selection and one float multiply are involved) and
 *     the golden vectors written from it.
 *   Floating-point summation order of the reference's BLAS is unspecified, so
 *   floating-point parity is tolerance-based; this oracle accumulates in
 *   double and rounds once.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR_NO_ACTIVE 1 /* reference throws std::runtime_error("No active weights") */
#define ORC_ERR_ARG 2

enum { ORC_ACT_RELU = 0, ORC_ACT_SILU = 1, ORC_ACT_GELU_TANH = 2, ORC_ACT_SIGMOID = 3, ORC_ACT_IDENTITY = 4 };

/* ------------------------------------------------------------------------ */
/* Differential weight cache                                                */
/* ------------------------------------------------------------------------ */

typedef struct orc_cache {
    int64_t I, H;
    int has_gate;
    float *gate_pool, *up_pool, *downT_pool;      /* [I,H] each; downT[i,:] = down[:,i] */
    float *gate_active, *up_active, *down_active; /* [I,H] capacity, first n rows valid */
    int64_t *indices;                             /* ordered active list, length n */
    int64_t *pos;                                 /* index -> position, -1 if inactive
                                                     (the reference's unordered_map) */
    int64_t n;
    uint8_t *mask;                                /* current mask */
    float *concat;                                /* rebuilt [2n,H] (or [n,H]) copy */
    int valid;
} orc_cache;

static void copy_row(float *dst, const float *src, int64_t H) { memcpy(dst, src, (size_t)H * sizeof(float)); }

/* weight_cache.h:113-145: cat([gate_active[:n], up_active[:n]]) is a full copy. */
static int orc_cache_rebuild(orc_cache *c)
{
    if (c->n == 0) return ORC_ERR_NO_ACTIVE;
    size_t blk = (size_t)c->n * (size_t)c->H;
    if (c->has_gate) {
        memcpy(c->concat, c->gate_active, blk * sizeof(float));
        memcpy(c->concat + blk, c->up_active, blk * sizeof(float));
    } else {
        memcpy(c->concat, c->up_active, blk * sizeof(float));
    }
    return ORC_OK;
}

int orc_cache_update(orc_cache *c, const uint8_t *mask);

/* weight_cache.h:155-227.  gate/up are [I,H] row-major, down is [H,I]. */
orc_cache *orc_cache_create(const uint8_t *init_mask, int64_t I, int64_t H, const float *gate, const float *up,
                            const float *down, int has_gate, int *err)
{
    orc_cache *c = (orc_cache *)calloc(1, sizeof(orc_cache));
    size_t tot = (size_t)I * (size_t)H;
    c->I = I;
    c->H = H;
    c->has_gate = has_gate;
    c->up_pool = (float *)malloc(tot * sizeof(float));
    c->downT_pool = (float *)malloc(tot * sizeof(float));
    c->up_active = (float *)malloc(tot * sizeof(float));
    c->down_active = (float *)malloc(tot * sizeof(float));
    if (has_gate) {
        c->gate_pool = (float *)malloc(tot * sizeof(float));
        c->gate_active = (float *)malloc(tot * sizeof(float));
        memcpy(c->gate_pool, gate, tot * sizeof(float));
    }
    c->concat = (float *)malloc((has_gate ? 2 : 1) * tot * sizeof(float));
    memcpy(c->up_pool, up, tot * sizeof(float));
    for (int64_t i = 0; i < I; ++i)
        for (int64_t j = 0; j < H; ++j) c->downT_pool[i * H + j] = down[j * I + i];
    c->indices = (int64_t *)malloc((size_t)I * sizeof(int64_t));
    c->pos = (int64_t *)malloc((size_t)I * sizeof(int64_t));
    for (int64_t i = 0; i < I; ++i) c->pos[i] = -1;
    c->mask = (uint8_t *)calloc((size_t)I, 1); /* current_mask = zeros */
    c->n = 0;
    c->valid = 0;
    int e = orc_cache_update(c, init_mask); /* weight_cache.h:226 */
    if (err) *err = e;
    return c;
}

void orc_cache_destroy(orc_cache *c)
{
    if (!c) return;
    free(c->gate_pool); free(c->up_pool); free(c->downT_pool);
    free(c->gate_active); free(c->up_active); free(c->down_active);
    free(c->indices); free(c->pos); free(c->mask); free(c->concat);
    free(c);
}

static void load_rows(orc_cache *c, int64_t pos, int64_t idx)
{
    int64_t H = c->H;
    if (c->has_gate) copy_row(c->gate_active + pos * H, c->gate_pool + idx * H, H);
    copy_row(c->up_active + pos * H, c->up_pool + idx * H, H);
    copy_row(c->down_active + pos * H, c->downT_pool + idx * H, H);
}

static void move_rows(orc_cache *c, int64_t dst, int64_t src)
{
    int64_t H = c->H;
    if (c->has_gate) copy_row(c->gate_active + dst * H, c->gate_active + src * H, H);
    copy_row(c->up_active + dst * H, c->up_active + src * H, H);
    copy_row(c->down_active + dst * H, c->down_active + src * H, H);
}

/* weight_cache.h:229-359.  Returns ORC_ERR_NO_ACTIVE when the update leaves
 * the cache empty; as in the reference the bookkeeping has then already been
 * changed but the remembered mask has not. */
int orc_cache_update(orc_cache *c, const uint8_t *mask)
{
    int64_t I = c->I;
    int64_t *added = (int64_t *)malloc((size_t)I * sizeof(int64_t));
    int64_t *removed = (int64_t *)malloc((size_t)I * sizeof(int64_t));
    int64_t na = 0, nr = 0;
    /* weight_cache.h:84-110: nonzero() yields ascending indices. */
    for (int64_t i = 0; i < I; ++i) {
        int nw = mask[i] != 0, od = c->mask[i] != 0;
        if (nw && !od) added[na++] = i;
        if (od && !nw) removed[nr++] = i;
    }
    if (na == 0 && nr == 0) { /* :237-240 early return, nothing touched */
        free(added); free(removed);
        return ORC_OK;
    }
    int64_t pairs = na < nr ? na : nr;
    /* phase 1 (:248-277): i-th removed position receives the i-th added index */
    for (int64_t i = 0; i < pairs; ++i) {
        int64_t p = c->pos[removed[i]];
        if (p < 0) continue;
        load_rows(c, p, added[i]);
        c->pos[removed[i]] = -1;
        c->indices[p] = added[i];
        c->pos[added[i]] = p;
    }
    /* phase 2 (:280-307): surplus additions appended in ascending order */
    for (int64_t i = pairs; i < na; ++i) {
        if (c->n >= I) continue; /* buffer full: max_active_indices == I */
        load_rows(c, c->n, added[i]);
        c->indices[c->n] = added[i];
        c->pos[added[i]] = c->n;
        c->n += 1;
    }
    /* phase 3 (:310-353): surplus removals, ascending index order, hole is
     * filled with the element that is last at that moment */
    for (int64_t i = pairs; i < nr; ++i) {
        int64_t p = c->pos[removed[i]];
        if (p < 0) continue;
        if (c->n <= 0) break; /* min_active_indices == 0 */
        int64_t last = c->n - 1;
        if (p != last) {
            int64_t last_idx = c->indices[last];
            move_rows(c, p, last);
            c->indices[p] = last_idx;
            c->pos[last_idx] = p;
        }
        c->n -= 1;
        c->pos[removed[i]] = -1;
    }
    free(added); free(removed);
    int e = orc_cache_rebuild(c); /* :356 */
    if (e != ORC_OK) return e;   /* exception: valid / current_mask not updated */
    c->valid = 1;
    memcpy(c->mask, mask, (size_t)I);
    return ORC_OK;
}

int64_t orc_cache_num_active(const orc_cache *c) { return c->n; }
int orc_cache_valid(const orc_cache *c) { return c->valid; }
void orc_cache_indices(const orc_cache *c, int64_t *out) { memcpy(out, c->indices, (size_t)c->n * sizeof(int64_t)); }
/* [2n,H] (gate rows then up rows), or [n,H] when ungated: get_concat_weight() */
const float *orc_cache_concat(const orc_cache *c) { return c->concat; }
/* packed [n,H]; the reference hands out its transpose view [H,n], strides (1,H) */
const float *orc_cache_down_active(const orc_cache *c) { return c->down_active; }
const float *orc_cache_gate_active(const orc_cache *c) { return c->gate_active; }
const float *orc_cache_up_active(const orc_cache *c) { return c->up_active; }

/* ------------------------------------------------------------------------ */
/* Sparse MLP forward                                                       */
/* ------------------------------------------------------------------------ */

static double act_apply(double v, int act)
{
    switch (act) {
    case ORC_ACT_RELU: return v > 0.0 ? v : 0.0;
    case ORC_ACT_SILU: return v / (1.0 + exp(-v));
    case ORC_ACT_GELU_TANH: {
        const double k = 0.79788456080286535588; /* sqrt(2/pi) */
        return 0.5 * v * (1.0 + tanh(k * (v + 0.044715 * v * v * v)));
    }
    case ORC_ACT_SIGMOID: return 1.0 / (1.0 + exp(-v));
    default: return v;
    }
}

static double dot_d(const float *a, const float *b, int64_t n)
{
    double acc = 0.0;
#pragma omp simd reduction(+ : acc)
    for (int64_t i = 0; i < n; ++i) acc += (double)a[i] * (double)b[i];
    return acc;
}

/*
 * x [B,H]; concat [2n,H] (gate rows, then up rows) or [n,H] when !has_gate;
 * down_active [n,H] packed (row j = column idx_j of the original down matrix);
 * out [B,H]; combined [B, 2n] (or [B,n]): on return its first n columns hold
 * act(gate)*up (act(up-projection) when ungated) and, when gated, columns
 * n..2n hold the raw up projection, exactly what the in-place operator leaves
 * behind (sparse_mlp_op.cpp:151-161,181-186).
 */
void orc_mlp_forward(const float *x, int64_t B, int64_t H, const float *concat, int64_t n, const float *down_active,
                     float *out, float *combined, int act, int has_gate)
{
    int64_t ld = has_gate ? 2 * n : n;
    double *h = (double *)malloc((size_t)B * (size_t)n * sizeof(double));
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; ++j) {
        for (int64_t b = 0; b < B; ++b) {
            const float *xb = x + b * H;
            if (has_gate) {
                double g = dot_d(xb, concat + j * H, H);
                double u = dot_d(xb, concat + (n + j) * H, H);
                /* the operator rounds both projections to float before activation */
                float gf = (float)g, uf = (float)u;
                double hv = act_apply((double)gf, act) * (double)uf;
                h[b * n + j] = hv;
                combined[b * ld + j] = (float)hv;
                combined[b * ld + n + j] = uf;
            } else {
                float uf = (float)dot_d(xb, concat + j * H, H);
                double hv = act_apply((double)uf, act);
                h[b * n + j] = hv;
                combined[b * ld + j] = (float)hv;
            }
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t c0 = 0; c0 < H; c0 += 64) {
        int64_t c1 = c0 + 64 < H ? c0 + 64 : H;
        for (int64_t b = 0; b < B; ++b) {
            double acc[64];
            for (int k = 0; k < 64; ++k) acc[k] = 0.0;
            for (int64_t j = 0; j < n; ++j) {
                double hv = h[b * n + j];
                const float *row = down_active + j * H + c0;
                for (int64_t k = 0; k < c1 - c0; ++k) acc[k] += hv * (double)row[k];
            }
            for (int64_t k = 0; k < c1 - c0; ++k) out[b * H + c0 + k] = (float)acc[k];
        }
    }
    free(h);
}

/* ------------------------------------------------------------------------ */
/* LoRA predictor and masks                                                 */
/* ------------------------------------------------------------------------ */

/* scores[B,I] = (x[B,H] . A[r,H]^T) . Bm[I,r]^T ; the intermediate t[B,r] is
 * rounded to float like the output of the first nn.Linear. */
void orc_predictor_scores(const float *x, int64_t B, int64_t H, const float *A, int64_t r, const float *Bm, int64_t I,
                          float *scores)
{
    float *t = (float *)malloc((size_t)B * (size_t)r * sizeof(float));
    for (int64_t b = 0; b < B; ++b)
        for (int64_t k = 0; k < r; ++k) t[b * r + k] = (float)dot_d(x + b * H, A + k * H, H);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < I; ++i)
        for (int64_t b = 0; b < B; ++b) scores[b * I + i] = (float)dot_d(t + b * r, Bm + i * r, r);
    free(t);
}

/* mask[i] = any_b( scores[b,i] >= thr )  (strict > when !ge) */
void orc_mask_threshold(const float *scores, int64_t B, int64_t I, float thr, int ge, uint8_t *mask)
{
    for (int64_t i = 0; i < I; ++i) {
        int any = 0;
        for (int64_t b = 0; b < B; ++b) {
            float s = scores[b * I + i];
            any |= ge ? (s >= thr) : (s > thr);
        }
        mask[i] = (uint8_t)any;
    }
}

typedef struct { float v; int64_t i; } orc_vi;
static int cmp_desc(const void *a, const void *b)
{
    const orc_vi *x = (const orc_vi *)a, *y = (const orc_vi *)b;
    if (x->v > y->v) return -1;
    if (x->v < y->v) return 1;
    return x->i < y->i ? -1 : (x->i > y->i ? 1 : 0); /* ties: lower index first */
}

/* per row the k largest scores are active, then union over rows */
void orc_mask_topk(const float *scores, int64_t B, int64_t I, int64_t k, uint8_t *mask)
{
    orc_vi *tmp = (orc_vi *)malloc((size_t)I * sizeof(orc_vi));
    memset(mask, 0, (size_t)I);
    if (k > I) k = I;
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t i = 0; i < I; ++i) { tmp[i].v = scores[b * I + i]; tmp[i].i = i; }
        qsort(tmp, (size_t)I, sizeof(orc_vi), cmp_desc);
        for (int64_t j = 0; j < k; ++j) mask[tmp[j].i] = 1;
    }
    free(tmp);
}

/* per row: active iff score > mean + std_pop * z  (population std, strict >),
 * then union over rows.  cutoff[b] (optional) receives the per-row cutoff. */
void orc_mask_statistical(const float *scores, int64_t B, int64_t I, float z, uint8_t *mask, float *cutoff)
{
    memset(mask, 0, (size_t)I);
    for (int64_t b = 0; b < B; ++b) {
        const float *s = scores + b * I;
        double sum = 0.0;
        for (int64_t i = 0; i < I; ++i) sum += s[i];
        double mean = sum / (double)I, ss = 0.0;
        for (int64_t i = 0; i < I; ++i) { double d = s[i] - mean; ss += d * d; }
        float cut = (float)mean + (float)sqrt(ss / (double)I) * z;
        if (cutoff) cutoff[b] = cut;
        for (int64_t i = 0; i < I; ++i) if (s[i] > cut) mask[i] = 1;
    }
}

/* Count-min-style sketch threshold per row.  libstdc++'s std::hash<int64_t> is the identity, so cell
 * (s, p) of the four sketches holds the largest score of the features f with (s*F + f) % W == p,
 * W = min(1024, F/4).  Cells still at -inf are dropped; the result is the sketch_k-th largest of the
 * rest times 0.9f, sketch_k = clamp(k * cells / F, 1, cells); 0 when no cell is left.  F >= 4. */
static int cmp_float_desc(const void *a, const void *b)
{
    const float x = *(const float *)a, y = *(const float *)b;
    return x > y ? -1 : (x < y ? 1 : 0);
}

void orc_approx_topk_threshold(const float *scores, int64_t B, int64_t F, int64_t k, float *threshold)
{
    const int64_t W = F / 4 < 1024 ? F / 4 : 1024;
    float *cell = (float *)malloc((size_t)(4 * W) * sizeof(float));
    for (int64_t b = 0; b < B; ++b) {
        const float *s = scores + b * F;
        for (int64_t i = 0; i < 4 * W; ++i) cell[i] = -INFINITY;
        for (int64_t t = 0; t < 4; ++t)
            for (int64_t f = 0; f < F; ++f) {
                float *c = cell + t * W + (t * F + f) % W;
                if (s[f] > *c) *c = s[f];
            }
        int64_t cells = 0;
        for (int64_t i = 0; i < 4 * W; ++i)
            if (cell[i] != -INFINITY) cell[cells++] = cell[i];
        if (cells == 0) { threshold[b] = 0.f; continue; }
        int64_t sk = k * cells / F;
        if (sk < 1) sk = 1;
        if (sk > cells) sk = cells;
        qsort(cell, (size_t)cells, sizeof(float), cmp_float_desc);
        threshold[b] = cell[sk - 1] * 0.9f;
    }
    free(cell);
}

/* The same for double scores (the reference dispatches on every floating type, approx_topk.h:33); its
 * adjustment factor is then the double 0.9. */
static int cmp_double_desc(const void *a, const void *b)
{
    const double x = *(const double *)a, y = *(const double *)b;
    return (x < y) - (x > y);
}

void orc_approx_topk_threshold_f64(const double *scores, int64_t B, int64_t F, int64_t k, double *threshold)
{
    const int64_t W = F / 4 < 1024 ? F / 4 : 1024;
    double *cell = (double *)malloc((size_t)(4 * W) * sizeof(double));
    for (int64_t b = 0; b < B; ++b) {
        const double *s = scores + b * F;
        for (int64_t i = 0; i < 4 * W; ++i) cell[i] = -INFINITY;
        for (int64_t t = 0; t < 4; ++t)
            for (int64_t f = 0; f < F; ++f) {
                double *c = cell + t * W + (t * F + f) % W;
                if (s[f] > *c) *c = s[f];
            }
        int64_t cells = 0;
        for (int64_t i = 0; i < 4 * W; ++i)
            if (cell[i] != -INFINITY) cell[cells++] = cell[i];
        if (cells == 0) { threshold[b] = 0.0; continue; }
        int64_t sk = k * cells / F;
        if (sk < 1) sk = 1;
        if (sk > cells) sk = cells;
        qsort(cell, (size_t)cells, sizeof(double), cmp_double_desc);
        threshold[b] = cell[sk - 1] * 0.9;
    }
    free(cell);
}
