/*
 * CPU oracle for the MicroAdam step.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the reference's per-tensor MicroAdam
 * update (ista_daslab_optimizers/micro_adam/micro_adam.py:61-94 and :146-328,
 * block_split from ista_daslab_optimizers/tools.py:85-92).  It exists to check
 * the HIP kernels; nothing in the shipped package may link, import or call it.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it.
 *
 * The arithmetic of the reference's device ops lives in the un-vendored package
 * ista-daslab-optimizers-cuda (pyproject.toml:21, unpinned) and is only known by
 * its call sites, so "parity unpinned" applies at that boundary: the numerical
 * choices below (rounding, clamping, nibble order, beta^age table) are frozen by
 * this build.  What pins each function here, without the reference:
 *   ora_block_split / ora_geometry    closed-form integer tables, invariants
 *   ora_block_topk                    brute-force stable sort on the same data
 *   ora_copy_values / ora_zerorize    numpy gather / index_fill
 *   ora_block_minmax                  numpy min / max over the same views
 *   ora_asymm_block_quant(_inv)       closed form of utils/quantizers.py:18-41,
 *                                     min->0, max->15, |Qinv(Q(x))-x| <= u/2
 *   ora_compute_microadam_update      dense Adam (k_init = 1) and a float64
 *                                     sliding-window sum
 *   ora_param_update / weight decay   torch add_/mul_ on CPU
 *
 * Element types: dtype 0 = fp32, dtype 1 = bf16 (stored as uint16_t).  All
 * arithmetic is fp32, no FMA contraction (build with -ffp-contract=off); results
 * are rounded to the destination type round-to-nearest-even.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORA_F32 0
#define ORA_BF16 1

/* ---- scalar helpers --------------------------------------------------- */

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, what torch's .to(torch.bfloat16) does */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float ld(const void *x, int64_t i, int dtype) {
    return dtype == ORA_BF16 ? bf16_to_f32(((const uint16_t *)x)[i]) : ((const float *)x)[i];
}

static inline void st(void *x, int64_t i, int dtype, float v) {
    if (dtype == ORA_BF16) ((uint16_t *)x)[i] = f32_to_bf16(v);
    else ((float *)x)[i] = v;
}

static inline uint32_t abs_key(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    return u & 0x7fffffffu;
}

void ora_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int ora_get_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* exported for the tests' conversion checks */
uint16_t ora_f32_to_bf16(float f) { return f32_to_bf16(f); }
float ora_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* ---- geometry ---------------------------------------------------------- */

/* tools.py:85-92.  n < b gives (1, n); otherwise int(n / b) uses a float
 * division followed by truncation, restated here with a double. */
void ora_block_split(int64_t n, int64_t b, int64_t *count, int64_t *start_last) {
    if (n < b) {
        *count = 1;
        *start_last = n;
        return;
    }
    *count = (int64_t)((double)n / (double)b);
    *start_last = n - n % b;
}

typedef struct {
    int64_t d;
    int64_t d_block_size;           /* micro_adam.py:77 */
    int64_t topk_full_blocks_count; /* :78 */
    int64_t d_index_topk;           /* :78 */
    int64_t k_block_size_many;      /* :79 */
    int64_t k_block_size_few;       /* :80 */
    int64_t k_index;                /* :81 */
    int64_t k;                      /* :82 */
    int64_t quant_full_blocks_count; /* :91 */
    int64_t d_index_quant;           /* :91 */
    int64_t error_bytes;             /* :92 */
    int64_t stats_len;               /* :93-94 */
} ora_geom;

/* micro_adam.py:72-94 */
void ora_geometry(int64_t d, int64_t max_d_block_size, double k_init, int64_t q, ora_geom *g) {
    g->d = d;
    g->d_block_size = d < max_d_block_size ? d : max_d_block_size;
    ora_block_split(d, g->d_block_size, &g->topk_full_blocks_count, &g->d_index_topk);
    g->k_block_size_many = (int64_t)ceil((double)g->d_block_size * k_init);
    g->k_block_size_few = (int64_t)ceil((double)(d - g->d_index_topk) * k_init);
    g->k_index = g->topk_full_blocks_count * g->k_block_size_many;
    g->k = g->k_block_size_many * g->topk_full_blocks_count + g->k_block_size_few;
    ora_block_split(d, q, &g->quant_full_blocks_count, &g->d_index_quant);
    g->error_bytes = (int64_t)ceil((double)d / 2.0);
    g->stats_len = g->quant_full_blocks_count + 1;
}

/* ---- 4-bit error feedback ---------------------------------------------- */

/* Byte j of xq holds element 2j in the high nibble and 2j+1 in the low nibble
 * (utils/quantizers.py:24-27). */
static inline int get_code(const uint8_t *xq, int64_t i) {
    uint8_t b = xq[i >> 1];
    return (i & 1) ? (b & 0x0f) : (b >> 4);
}

/* micro_adam.py:190 (also :267, :298, :313, :322): x += alpha * Qinv(xq).
 * Qinv follows utils/quantizers.py:31-40: code * u + min, u = (max - min) / 15. */
void ora_asymm_block_quant_inv(int64_t d, int64_t q, const uint8_t *xq, const uint16_t *xmin,
                               const uint16_t *xmax, void *x, float alpha, int dtype) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < d; ++i) {
        int64_t b = i / q;
        float mn = bf16_to_f32(xmin[b]);
        float mx = bf16_to_f32(xmax[b]);
        float u = (mx - mn) / 15.0f;
        float deq = (float)get_code(xq, i) * u;
        deq = deq + mn;
        float add = alpha * deq;
        st(x, i, dtype, ld(x, i, dtype) + add);
    }
}

/* micro_adam.py:231 (also :316): xq = Q(x; min, max), utils/quantizers.py:23-24:
 * floor((x - min) / u + 0.5), clamped to [0, 15]; a zero or non-finite range
 * gives code 0. */
void ora_asymm_block_quant(int64_t d, int64_t q, uint8_t *xq, const uint16_t *xmin,
                           const uint16_t *xmax, const void *x, int dtype) {
    int64_t nbytes = (d + 1) / 2;
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < nbytes; ++j) {
        int codes[2] = {0, 0};
        for (int h = 0; h < 2; ++h) {
            int64_t i = 2 * j + h;
            if (i >= d) break;
            int64_t b = i / q;
            float mn = bf16_to_f32(xmin[b]);
            float mx = bf16_to_f32(xmax[b]);
            float u = (mx - mn) / 15.0f;
            int c = 0;
            if (u != 0.0f && isfinite(u)) {
                float v = (ld(x, i, dtype) - mn) / u;
                v = floorf(v + 0.5f);
                v = fmaxf(v, 0.0f);
                v = fminf(v, 15.0f);
                c = (int)v;
            }
            codes[h] = c;
        }
        xq[j] = (uint8_t)((codes[0] << 4) | codes[1]);
    }
}

/* micro_adam.py:217-228: per quantisation block min and max of x, stored bf16.
 * Block b covers [b*q, min((b+1)*q, d)); when d < q block_split gives one block
 * covering everything, which the same indexing reproduces. */
void ora_block_minmax(int64_t d, int64_t q, const void *x, int dtype, uint16_t *xmin,
                      uint16_t *xmax) {
    int64_t nb = (d + q - 1) / q;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b) {
        int64_t lo = b * q, hi = lo + q < d ? lo + q : d;
        float mn = ld(x, lo, dtype), mx = mn;
        for (int64_t i = lo + 1; i < hi; ++i) {
            float v = ld(x, i, dtype);
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        xmin[b] = f32_to_bf16(mn);
        xmax[b] = f32_to_bf16(mx);
    }
}

/* ---- block top-k -------------------------------------------------------- */

/* The kb entries of x[0..n) with the largest |x|; exact ties at the threshold
 * go to the lowest indices.  Output: block-relative indices in ascending order.
 * MSD radix select on the 31 magnitude bits, 8/8/8/7 bits per pass. */
static void block_topk(const void *x, int64_t base, int n, int kb, int dtype, int16_t *out) {
    static const int shifts[4] = {23, 15, 7, 0};
    static const uint32_t dmask[4] = {0xffu, 0xffu, 0xffu, 0x7fu};
    uint32_t prefix = 0, pmask = 0;
    int need = kb;
    if (kb <= 0) return;
    for (int pass = 0; pass < 4; ++pass) {
        int hist[256];
        memset(hist, 0, sizeof hist);
        int sh = shifts[pass];
        uint32_t dm = dmask[pass];
        for (int i = 0; i < n; ++i) {
            uint32_t key = abs_key(ld(x, base + i, dtype));
            if ((key & pmask) == prefix) hist[(key >> sh) & dm]++;
        }
        int above = 0, bin = (int)dm;
        for (; bin > 0; --bin) {
            if (above + hist[bin] >= need) break;
            above += hist[bin];
        }
        need -= above;
        prefix |= (uint32_t)bin << sh;
        pmask |= dm << sh;
    }
    /* prefix is now the threshold key T; `need` of the entries equal to T are taken */
    int w = 0;
    for (int i = 0; i < n && w < kb; ++i) {
        uint32_t key = abs_key(ld(x, base + i, dtype));
        if (key > prefix) out[w++] = (int16_t)i;
        else if (key == prefix && need > 0) {
            out[w++] = (int16_t)i;
            --need;
        }
    }
}

/* micro_adam.py:193-200: I_row[:k_index] and I_row[k_index:]; replaces
 * torch.topk(|x|, sorted=False).indices.to(int16) with a defined tie rule. */
void ora_block_topk(int64_t d, int64_t d_block_size, int64_t k_many, int64_t k_few, const void *x,
                    int dtype, int16_t *I_row) {
    int64_t full = d / d_block_size;
#pragma omp parallel for schedule(dynamic, 8)
    for (int64_t b = 0; b < full; ++b)
        block_topk(x, b * d_block_size, (int)d_block_size, (int)k_many, dtype, I_row + b * k_many);
    if (k_few > 0)
        block_topk(x, full * d_block_size, (int)(d - full * d_block_size), (int)k_few, dtype,
                   I_row + full * k_many);
}

/* micro_adam.py:202-209, direction d2k: out[j] = bf16(inp[blk(j)*DB + I[j]]);
 * direction k2d (sparse_core_mfac_w_ef.py:117-124): out[blk(j)*DB + I[j]] = inp[j]. */
void ora_copy_values(int64_t d, int64_t k, int64_t d_block_size, int64_t k_block_size,
                     const int16_t *indices, const void *inp, void *out, int direction,
                     int dtype) {
    (void)d;
    for (int64_t j = 0; j < k; ++j) {
        int64_t pos = (j / k_block_size) * d_block_size + indices[j];
        if (direction == 1) ((uint16_t *)out)[j] = f32_to_bf16(ld(inp, pos, dtype));
        else st(out, pos, dtype, bf16_to_f32(((const uint16_t *)inp)[j]));
    }
}

/* micro_adam.py:214: vector[blk(j)*DB + I[j]] = 0 */
void ora_zerorize_block_components(void *vector, const int16_t *indices, int64_t d, int64_t k,
                                   int64_t d_block_size, int64_t k_block_size, int dtype) {
    (void)d;
    for (int64_t j = 0; j < k; ++j)
        st(vector, (j / k_block_size) * d_block_size + indices[j], dtype, 0.0f);
}

/* ---- Adam statistics from the window ------------------------------------ */

/* micro_adam.py:277-291.  Row i of the m x k window has age (t-1-i) mod m; rows
 * i < min(t, m) are live.  Per coordinate z1 = sum w1[age] v, z2 = sum w2[age] v*v
 * over live rows in increasing row order, then
 *   out = rne( (z1 * s1) / (eps + sqrtf(z2 * s2)) ),
 *   s1 = (1-beta1)/(1-beta1^t), s2 = (1-beta2)/(1-beta2^t) (double -> fp32),
 *   w[age] = (float)pow(beta, age).
 * Coordinates that no live row names with a non-zero value are left untouched (the caller
 * zeroed out, micro_adam.py:276, so they read as a zero update either way). */
void ora_compute_microadam_update(int64_t t, double beta1, double beta2, double eps,
                                  int64_t d_block_size, int64_t k_block_size, int64_t d,
                                  int64_t m, int64_t k, const int16_t *indices,
                                  const uint16_t *values, void *out, int dtype) {
    int64_t rows = t < m ? t : m;
    float *w1 = (float *)malloc(sizeof(float) * (size_t)m);
    float *w2 = (float *)malloc(sizeof(float) * (size_t)m);
    for (int64_t i = 0; i < m; ++i) {
        int64_t age = ((t - 1 - i) % m + m) % m;
        w1[i] = (float)pow(beta1, (double)age);
        w2[i] = (float)pow(beta2, (double)age);
    }
    float s1 = (float)((1.0 - beta1) / (1.0 - pow(beta1, (double)t)));
    float s2 = (float)((1.0 - beta2) / (1.0 - pow(beta2, (double)t)));
    float epsf = (float)eps;
    int64_t nblocks = (k + k_block_size - 1) / k_block_size;
#pragma omp parallel
    {
        float *z1 = (float *)malloc(sizeof(float) * (size_t)d_block_size);
        float *z2 = (float *)malloc(sizeof(float) * (size_t)d_block_size);
        uint8_t *hit = (uint8_t *)malloc((size_t)d_block_size);
#pragma omp for schedule(dynamic, 8)
        for (int64_t b = 0; b < nblocks; ++b) {
            int64_t j0 = b * k_block_size;
            int64_t j1 = j0 + k_block_size < k ? j0 + k_block_size : k;
            int64_t base = b * d_block_size;
            int64_t n = base + d_block_size <= d ? d_block_size : d - base;
            memset(z1, 0, sizeof(float) * (size_t)n);
            memset(z2, 0, sizeof(float) * (size_t)n);
            memset(hit, 0, (size_t)n);
            for (int64_t r = 0; r < rows; ++r) {
                const int16_t *ir = indices + r * k;
                const uint16_t *vr = values + r * k;
                for (int64_t j = j0; j < j1; ++j) {
                    int idx = ir[j];
                    /* a +-0 value adds nothing and does not mark its coordinate (rows of a
                     * fresh window are all (index 0, value 0)) */
                    if ((vr[j] & 0x7fffu) == 0) continue;
                    float v = bf16_to_f32(vr[j]);
                    float a1 = w1[r] * v;
                    float vv = v * v;
                    float a2 = w2[r] * vv;
                    z1[idx] = z1[idx] + a1;
                    z2[idx] = z2[idx] + a2;
                    hit[idx] = 1;
                }
            }
            for (int64_t i = 0; i < n; ++i) {
                if (!hit[i]) continue;
                float mh = z1[i] * s1;
                float vh = z2[i] * s2;
                float den = epsf + sqrtf(vh);
                st(out, base + i, dtype, mh / den);
            }
        }
        free(z1);
        free(z2);
        free(hit);
    }
    free(w1);
    free(w2);
}

/* ---- parameter update ---------------------------------------------------- */

/* micro_adam.py:234-235: p.mul_(1 - lr*wd); the factor is formed in double by
 * the caller and narrowed to fp32 as torch does for a Python scalar. */
void ora_weight_decay(int64_t d, void *p, float factor, int dtype) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < d; ++i) st(p, i, dtype, ld(p, i, dtype) * factor);
}

/* micro_adam.py:304: p.add_(u, alpha=-lr): fp32 p + (-lr)*u, rounded to p's type. */
void ora_param_update(int64_t d, void *p, const void *u, float neg_lr, int p_dtype, int u_dtype) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < d; ++i) {
        float prod = neg_lr * ld(u, i, u_dtype);
        st(p, i, p_dtype, ld(p, i, p_dtype) + prod);
    }
}

/* ---- the per-tensor step -------------------------------------------------- */

typedef struct {
    int64_t t;      /* global step counter, micro_adam.py:98, :280 */
    int64_t m;
    int64_t q;      /* quant_block_size */
    int64_t max_d_block_size;
    double k_init;
    double alpha;
    double beta1, beta2, eps;
    double lr, wd;
} ora_hyper;

/* micro_adam.py:146-328 for alpha in [0, 1) and alpha == -2.  `grad` is consumed as scratch, as in
 * the reference (:153).  `index` is the ring position (:180, :211) and is
 * advanced.  Returns 0, or -1 for any other alpha. */
static double sum_squares(const void *x, int64_t d, int dtype) {
    double s = 0;
    for (int64_t i = 0; i < d; ++i) {
        const double v = ld(x, i, dtype);
        s += v * v;
    }
    return s;
}

static double count_zeros(const void *x, int64_t d, int dtype) {
    int64_t n = 0;
    for (int64_t i = 0; i < d; ++i) n += ld(x, i, dtype) == 0.0f;
    return (double)n;
}

static void clear(void *x, int64_t d, int dtype) {
    memset(x, 0, (size_t)d * (dtype == ORA_BF16 ? 2 : 4));
}

/* mt: NULL, or the six sums a logging step adds up over the tensors (micro_adam.py:148, :328):
 * [0] |quant_err|^2 (:271), [1] |g|^2 (:155-156), [2] |u|^2 (:307), [3] |Qinv(e)|^2 (:320-324),
 * [4] zeros of u (:308), [5] zeros of quant_err (:272); each += this tensor's share, taken in
 * double from the values as the buffer holds them (rounded to the gradient's type). */
static int update_step_impl(const ora_hyper *h, void *p, void *grad, int dtype, int64_t d,
                            int64_t *index, int16_t *I, uint16_t *V, uint8_t *error,
                            uint16_t *min_vals, uint16_t *max_vals, double *mt, void *quant_err) {
    ora_geom g;
    if (h->alpha < 0 && h->alpha != -2.0) return -1;
    ora_geometry(d, h->max_d_block_size, h->k_init, h->q, &g);
    if (mt) mt[1] += sum_squares(grad, d, dtype);
    int64_t row = *index;
    int16_t *I_row = I + row * g.k;
    uint16_t *V_row = V + row * g.k;

    /* STEP 4, :190 */
    ora_asymm_block_quant_inv(d, h->q, error, min_vals, max_vals, grad, 1.0f, dtype);
    /* STEP 5, :193-200 */
    ora_block_topk(d, g.d_block_size, g.k_block_size_many, g.k_block_size_few, grad, dtype, I_row);
    /* STEP 9, :202-209 */
    ora_copy_values(d, g.k, g.d_block_size, g.k_block_size_many, I_row, grad, V_row, 1, dtype);
    /* :211 */
    *index = (row + 1) % h->m;
    /* STEP 6, :214 */
    ora_zerorize_block_components(grad, I_row, d, g.k, g.d_block_size, g.k_block_size_many, dtype);
    /* STEP 7, :217-228 */
    ora_block_minmax(d, h->q, grad, dtype, min_vals, max_vals);
    /* STEP 8, :231 */
    ora_asymm_block_quant(d, h->q, error, min_vals, max_vals, grad, dtype);
    /* :234-235 */
    if (h->wd > 0) ora_weight_decay(d, p, (float)(1.0 - h->lr * h->wd), dtype);
    /* :238-273, alpha == -2: p = p - a + Qinv(e_new).  The quant_err vector of :259-261, :271
     * (st['quant_err'], rewritten by every step) is kept in the caller's buffer if there is one. */
    if (h->alpha == -2.0) {
        void *qe = quant_err;
        if (mt && !qe) {
            qe = malloc((size_t)d * 4);
            if (!qe) return -2;
        }
        /* :259-261: quant_err = a (it has the parameter's type) */
        if (qe) memcpy(qe, grad, (size_t)d * (dtype == ORA_BF16 ? 2 : 4));
        ora_param_update(d, p, grad, -1.0f, dtype, dtype);                       /* STEP A, :264 */
        clear(grad, d, dtype);                                                   /* :267 */
        ora_asymm_block_quant_inv(d, h->q, error, min_vals, max_vals, grad, 1.0f, dtype);
        ora_param_update(d, p, grad, 1.0f, dtype, dtype);                        /* STEP B, :269 */
        if (qe) /* :271: quant_err -= Qinv(e_new), rounded to its type */
            for (int64_t i = 0; i < d; ++i) st(qe, i, dtype, ld(qe, i, dtype) - ld(grad, i, dtype));
        if (mt) { /* :272-273 */
            mt[0] += sum_squares(qe, d, dtype);
            mt[5] += count_zeros(qe, d, dtype);
        }
        if (qe != quant_err) free(qe);
    }
    /* STEPS 10-11, :276-291 */
    clear(grad, d, dtype);
    ora_compute_microadam_update(h->t, h->beta1, h->beta2, h->eps, g.d_block_size,
                                 g.k_block_size_many, d, h->m, g.k, I, V, grad, dtype);
    /* :296-298 */
    if (h->alpha > 0)
        ora_asymm_block_quant_inv(d, h->q, error, min_vals, max_vals, grad, (float)h->alpha, dtype);
    /* STEP 12, :304 */
    ora_param_update(d, p, grad, (float)(-h->lr), dtype, dtype);
    if (mt) { /* :306-308 */
        mt[2] += sum_squares(grad, d, dtype);
        mt[4] += count_zeros(grad, d, dtype);
    }
    /* :311-316 */
    if (h->alpha > 0) {
        clear(grad, d, dtype);
        ora_asymm_block_quant_inv(d, h->q, error, min_vals, max_vals, grad,
                                  (float)(1.0 - h->alpha), dtype);
        ora_block_minmax(d, h->q, grad, dtype, min_vals, max_vals);
        ora_asymm_block_quant(d, h->q, error, min_vals, max_vals, grad, dtype);
    }
    if (mt) { /* :320-324 */
        clear(grad, d, dtype);
        ora_asymm_block_quant_inv(d, h->q, error, min_vals, max_vals, grad, 1.0f, dtype);
        mt[3] += sum_squares(grad, d, dtype);
    }
    return 0;
}

int ora_update_step(const ora_hyper *h, void *p, void *grad, int dtype, int64_t d, int64_t *index,
                    int16_t *I, uint16_t *V, uint8_t *error, uint16_t *min_vals,
                    uint16_t *max_vals) {
    return update_step_impl(h, p, grad, dtype, d, index, I, V, error, min_vals, max_vals, NULL,
                            NULL);
}

/* ora_update_step / ora_step_metrics (metrics != NULL) that also keep st['quant_err']
 * (micro_adam.py:67-68, :258-271; d elements of the parameter's type) when alpha == -2. */
int ora_update_step_state(const ora_hyper *h, void *p, void *grad, int dtype, int64_t d,
                          int64_t *index, int16_t *I, uint16_t *V, uint8_t *error,
                          uint16_t *min_vals, uint16_t *max_vals, double *metrics,
                          void *quant_err) {
    return update_step_impl(h, p, grad, dtype, d, index, I, V, error, min_vals, max_vals, metrics,
                            quant_err);
}

/* A logging step (micro_adam.py:155-156, :271-272, :306-308, :320-324): ora_update_step, and
 * the tensor's shares added to metrics[0..5] = norm_qe, norm_g, norm_u, norm_e, sp_u, sp_qe
 * (the order of the reference's return value, :328; squared norms, counts of zeros). */
int ora_step_metrics(const ora_hyper *h, void *p, void *grad, int dtype, int64_t d, int64_t *index,
                     int16_t *I, uint16_t *V, uint8_t *error, uint16_t *min_vals,
                     uint16_t *max_vals, double *metrics) {
    if (!metrics) return -1;
    return update_step_impl(h, p, grad, dtype, d, index, I, V, error, min_vals, max_vals, metrics,
                            NULL);
}

/* ---- Sparse M-FAC's two window kernels (same I / V layout) ---------------- */

/* ista_daslab_cuda_sparse_mfac.SP, sparse_mfac/sparse_core_mfac_w_ef.py:185-203: the scalar
 * product of every live window row with the dense vector g,
 *   out[i] += sum_j V[i][j] * g[blk(j)*DB + I[i][j]],   i < m_rows (= min(m, steps), :192).
 * The caller zeroes out first (:186).  The order of the sum is not part of the contract (the
 * device adds per-block partial sums); the oracle accumulates in double so that an fp32
 * result can be checked against it with a bound on the rounding of the sum alone. */
void ora_sparse_scalar_products(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                                int64_t k_block_size, const void *g, int g_dtype,
                                const int16_t *indices, const void *values, int v_dtype,
                                double *out) {
    (void)d;
    for (int64_t i = 0; i < m_rows; ++i) {
        double s = 0.0;
        for (int64_t j = 0; j < k; ++j) {
            int64_t pos = (j / k_block_size) * d_block_size + indices[i * k + j];
            /* the product of two fp32 values is exact in double */
            s += (double)ld(values, i * k + j, v_dtype) * (double)ld(g, pos, g_dtype);
        }
        out[i] += s;
    }
}

/* ista_daslab_cuda_sparse_mfac.LCG, sparse_core_mfac_w_ef.py:205-221: the linear combination
 * of the live window rows with coefficients c (fp32, :167 `M`),
 *   out[blk(j)*DB + I[i][j]] += c[i] * V[i][j],   i < m_rows.
 * The caller zeroes out first (:206).  Frozen here: per coordinate the terms fl(c[i] * v) are
 * added in fp32 in increasing row order (no fused multiply-add), and the sum is added to out
 * with one rounding into out's type. */
void ora_sparse_linear_combination(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                                   int64_t k_block_size, const float *coef,
                                   const int16_t *indices, const void *values, int v_dtype,
                                   void *out, int out_dtype) {
    float *acc = (float *)calloc((size_t)d, sizeof(float));
    for (int64_t i = 0; i < m_rows; ++i)
        for (int64_t j = 0; j < k; ++j) {
            int64_t pos = (j / k_block_size) * d_block_size + indices[i * k + j];
            float term = coef[i] * ld(values, i * k + j, v_dtype);
            acc[pos] = acc[pos] + term;
        }
    for (int64_t i = 0; i < d; ++i) st(out, i, out_dtype, ld(out, i, out_dtype) + acc[i]);
    free(acc);
}
