/*
 * C ABI of libmicroadam_hip.so: the MicroAdam optimizer step as gfx950 HIP kernels.
 *
 * The reference (IST-DASLab/ISTA-DASLab-Optimizers) reaches its device code through two
 * pybind extension modules of the separate package ista-daslab-optimizers-cuda
 * (pyproject.toml:21): ista_daslab_cuda_tools and ista_daslab_cuda_micro_adam.  Every
 * function those modules export on the MicroAdam path has one entry point here with the
 * same argument order and meaning; the call sites cited below are in
 * ista_daslab_optimizers/micro_adam/micro_adam.py (MA) and ista_daslab_optimizers/tools.py.
 *
 * Conventions
 *  - All pointers are DEVICE pointers unless a comment says "host".
 *  - dtype: MA_F32 (0) = float, MA_BF16 (1) = bfloat16 bit patterns (uint16_t).  It is the
 *    type of the dense vectors (gradient / accumulator / update / parameter).  Window values,
 *    and the per-block min / max statistics, are always bf16; window indices int16; error
 *    feedback is packed 4-bit codes, element 2j in the high nibble of byte j.
 *  - stream: a hipStream_t passed as void* (NULL = the default stream).  Work is enqueued and
 *    the call returns; nothing here synchronises, allocates or frees device memory.
 *  - Return value: 0 on success; a positive hipError_t if the runtime refused a launch; a
 *    negative MA_ERR_* code if the arguments are rejected before anything is launched.
 *  - Arithmetic: fp32, no fused multiply-add, round-to-nearest-even into the destination type.
 */
#ifndef MICROADAM_HIP_H
#define MICROADAM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MA_F32 0
#define MA_BF16 1

#define MA_ERR_ARG (-1)         /* null pointer, non-positive size, unknown dtype / direction */
#define MA_ERR_BLOCK_SIZE (-2)  /* top-k block longer than 32768 (int16 indices) */
#define MA_ERR_WINDOW (-3)      /* m larger than MA_MAX_WINDOW */
#define MA_ERR_GEOMETRY (-4)    /* k / k_block_size inconsistent with d and d_block_size */
#define MA_ERR_NOT_FUSABLE (-5) /* tensor does not meet ma_fused_step's layout conditions */
#define MA_ERR_LDS (-6)         /* the launch would need more than 160 KB of LDS */
#define MA_ERR_WORKSPACE (-7)   /* the list needs more than MA_STATIC_WORKSPACE_BYTES of scratch */

#define MA_MAX_WINDOW 64 /* largest window length m the kernels take */
#define MA_MAX_D_BLOCK 32768
#define MA_STATIC_WORKSPACE_BYTES (16 << 20) /* scratch ma_spanning_step_static holds per GPU */
#define MA_MAX_SPARSE_ROWS 4096 /* most window rows the Sparse M-FAC kernels take */

const char *ma_error_string(int code);

/* ---- ista_daslab_cuda_tools ------------------------------------------------------------ */

/* get_sm_count(), MA:40: compute units of the current device (256 on MI355X). */
int ma_get_sm_count(void);

/* get_max_floats_for_shared_memory_per_thread_block(), MA:43: fp32 slots of LDS one
 * workgroup may use, 160 KB / 4 = 40960 on gfx950; MA:44 halves it into d_block_size. */
int ma_get_max_floats_for_shared_memory_per_thread_block(void);

/* copy_values(d, k, d_block_size, k_block_size, indices, inp, out, direction), MA:202-209.
 * direction 1 (d2k): out[j] = bf16(inp[(j / k_block_size) * d_block_size + indices[j]]),
 *   inp is `dtype` of length d, out is bf16 of length k.
 * direction 0 (k2d, sparse_mfac/sparse_core_mfac_w_ef.py:117-124): the reverse scatter,
 *   inp is bf16 of length k, out is `dtype` of length d. */
int ma_copy_values(int64_t d, int64_t k, int64_t d_block_size, int64_t k_block_size,
                   const int16_t *indices, const void *inp, void *out, int direction, int dtype,
                   void *stream);

/* zerorize_block_components(vector, indices, d, k, d_block_size, k_block_size), MA:214:
 * vector[(j / k_block_size) * d_block_size + indices[j]] = 0. */
int ma_zerorize_block_components(void *vector, const int16_t *indices, int64_t d, int64_t k,
                                 int64_t d_block_size, int64_t k_block_size, int dtype,
                                 void *stream);

/* ---- ista_daslab_cuda_micro_adam --------------------------------------------------------- */

/* asymm_block_quant(d, q_block_size, xq, xmin, xmax, x), MA:231, MA:316:
 * xq = Q(x): code = clamp(floor((x - min_b) / u_b + 0.5), 0, 15), u_b = (max_b - min_b) / 15,
 * b = i / q_block_size; a zero or non-finite range gives code 0. */
int ma_asymm_block_quant(int64_t d, int64_t q_block_size, uint8_t *xq, const uint16_t *xmin,
                         const uint16_t *xmax, const void *x, int dtype, void *stream);

/* asymm_block_quant_inv(d, q_block_size, xq, xmin, xmax, x, alpha), MA:190, :267, :298, :313,
 * :322: x += alpha * (code * u_b + min_b). */
int ma_asymm_block_quant_inv(int64_t d, int64_t q_block_size, const uint8_t *xq,
                             const uint16_t *xmin, const uint16_t *xmax, void *x, float alpha,
                             int dtype, void *stream);

/* compute_microadam_update(blocks, threads, carveout, t, beta1, beta2, eps, d_block_size,
 * k_block_size, d, m, k, indices, values, out), MA:277-291.  For every coordinate named by a
 * live window row (row i < min(t, m), age (t-1-i) mod m): z1 = sum beta1^age v, z2 = sum
 * beta2^age v^2 in increasing row order, out = (z1 s1) / (eps + sqrt(z2 s2)) with
 * s = (1-beta)/(1-beta^t).  Entries whose value is +-0 are skipped; coordinates no other entry
 * names are left as they are (the caller zeroes out first, MA:276).  blocks / threads / carveout are the reference's launch hints; they
 * are accepted and ignored (one workgroup per top-k block is launched). */
int ma_compute_microadam_update(int blocks, int threads, int carveout, int64_t t, double beta1,
                                double beta2, double eps, int64_t d_block_size,
                                int64_t k_block_size, int64_t d, int64_t m, int64_t k,
                                const int16_t *indices, const uint16_t *values, void *out,
                                int dtype, void *stream);

/* ---- stock torch ops of the hot path, as kernels ------------------------------------------ */

/* Replaces torch.abs + torch.topk + .to(int16) + slice assignment, MA:193-200, and optionally
 * MA:202-209 and MA:214 in the same launch.  For every top-k block of x (d_block_size
 * elements, the last one shorter) the k_block entries largest in magnitude are found, exact
 * ties at the threshold going to the lowest indices; I_row receives their block-relative
 * indices in ascending order (k_many per full block, then k_few for the tail block).
 * V_row, if not NULL, receives bf16(x) at those positions; if zero_selected != 0 they are
 * then set to 0 in x. */
int ma_block_topk(int64_t d, int64_t d_block_size, int64_t k_many, int64_t k_few, void *x,
                  int16_t *I_row, uint16_t *V_row, int zero_selected, int dtype, void *stream);

/* Replaces _update_quantization_statistics, MA:217-228: bf16 min and max of every
 * quantisation block [b*q, min((b+1)*q, d)) of x. */
int ma_block_minmax(int64_t d, int64_t q_block_size, const void *x, uint16_t *xmin,
                    uint16_t *xmax, int dtype, void *stream);

/* Replaces p.mul_(1 - lr*wd) (MA:234-235, skipped when apply_decay == 0) followed by
 * p.add_(u, alpha=-lr) (MA:304): p = rne(p * decay); p = rne(p + neg_lr * u). */
int ma_param_update(int64_t d, void *p, const void *u, float neg_lr, int apply_decay,
                    float decay, int dtype, void *stream);

/* ---- the fused step ------------------------------------------------------------------------ */

/* One parameter tensor of a fused step.  Pointers are device pointers; the struct itself is
 * host memory. */
typedef struct ma_tensor {
    void *p;            /* parameter, `dtype`, d elements */
    void *g;            /* gradient, `dtype`, d elements; NOT modified by the fused step */
    uint8_t *error;     /* st['error'],    ceil(d/2) bytes,            MA:92 */
    uint16_t *min_vals; /* st['min_vals'], quant_full_blocks_count+1,  MA:93 */
    uint16_t *max_vals; /* st['max_vals'],                             MA:94 */
    int16_t *I;         /* st['I'], m x k,                             MA:86 */
    uint16_t *V;        /* st['V'], m x k,                             MA:87 */
    int64_t d;          /* st['d'] */
    int64_t k;          /* st['k'], row length of I and V,             MA:82 */
    double lr;          /* group['lr'],                                MA:121 */
    double weight_decay; /* group['weight_decay'],                     MA:122 */
    int32_t index;      /* st['index'], the ring row written by this step, MA:180 */
    int32_t reserved;
    void *quant_err;    /* st['quant_err'], `dtype`, d elements, MA:67-68; written by
                           ma_fused_step_quant_err (and ma_logged_step on that route), 16-byte
                           aligned; the other entry points ignore it (may be NULL) */
    uint16_t *row_cuts; /* optional cache kept by ma_fused_step, no counterpart in the reference:
                           m x ma_fused_step_row_cuts() words, or NULL; see there */
} ma_tensor;

typedef struct ma_hyper {
    int64_t t;          /* self.steps after the increment, MA:98, :280 */
    int32_t m;          /* window length */
    int32_t dtype;      /* MA_F32 or MA_BF16, of p and g */
    int64_t quant_block_size;
    int64_t d_block_size; /* self.d_block_size, MA:44 */
    double k_init;
    double beta1, beta2, eps;
} ma_hyper;

/* The whole of update_step (MA:146-328) for alpha == 0, for a list of tensors, in one pass per
 * top-k block: a = g + Qinv(e); block top-k -> I[index], V[index]; residual -> new min/max
 * and 4-bit codes; window -> Adam direction; p update (with decoupled weight decay).  (Tensors
 * whose window is about as dense as the tensor take two launches, the second for the window and
 * the parameters: see ma_fused_step_row_cuts.)  The
 * caller advances st['index'] (MA:211) itself.  Conditions (else MA_ERR_NOT_FUSABLE, nothing
 * launched): quant_block_size a power of two in [8, 4096] that divides d_block_size (or
 * d <= d_block_size) and does not exceed d; p and g 16-byte aligned, error 4-byte aligned;
 * d_block_size a multiple of 8 unless d <= d_block_size. */
int ma_fused_step(const ma_tensor *tensors /* host */, int n_tensors,
                  const ma_hyper *hyper /* host */, void *stream);

/* 0 if ma_fused_step would accept this tensor under `hyper`, else the MA_ERR_* it would
 * return.  Host-only check, launches nothing. */
int ma_fused_step_check(const ma_tensor *tensor /* host */, const ma_hyper *hyper /* host */);

/* ma_fused_step steps tensors whose window has about as many entries as the tensor has
 * coordinates (more than 2560 entries per top-k block, or more than 16 rows) in two launches; the
 * second walks every window row in stretches of 512 coordinates and must know where each row
 * crosses those boundaries.  With tensor->row_cuts == NULL it finds out by reading all rows at
 * every step.  With a buffer of m x (this function's value) uint16 words, set to 0xffff before
 * its first use and from then on written by nobody else, the first launch files the cuts of
 * the row it writes and the second reads them: row r, block b, cut c (the number of entries of
 * that block's stretch of row r whose coordinate is below 512 c) is word
 * (r * blocks + b) * cuts_per_block + c, cuts_per_block = ceil(min(d, d_block_size) / 512) + 1.
 * A row whose first cut is 0xffff is taken as unknown and read in full.  Whoever else rewrites a
 * window row of the tensor (another entry point, a loaded checkpoint) must set that row's
 * words to 0xffff again.  Returns the words per row, 0 if the tensor's step would not use them,
 * negative MA_ERR_* for bad arguments. */
int64_t ma_fused_step_row_cuts(const ma_tensor *tensor, const ma_hyper *hyper);


/* ma_fused_step for 0 < alpha < 1 (densify_update_using_ef, MA:296-298 and MA:311-316), same
 * conditions, still one pass per top-k block: e1 = Q(residual) stays in registers as codes and
 * statistics; window -> Adam direction, + alpha * Qinv(e1); p update; the error feedback that is
 * stored is Q((1 - alpha) * Qinv(e1)) with statistics of its own. */
int ma_fused_step_densified(const ma_tensor *tensors /* host */, int n_tensors,
                            const ma_hyper *hyper /* host */, double alpha, void *stream);

/* The whole of update_step (MA:146-328) when the quantisation blocks are at least as long as
 * the top-k blocks (the reference's documented setting is quant_block_size = 100000), for
 * alpha == 0 and for 0 < alpha < 1 (densify_update_using_ef, MA:296-298 and MA:311-316).  A
 * quantisation block then covers several top-k blocks, whose workgroups have to exchange the
 * extremes of the residual (through the workspace) before any of them can form codes:
 *   1. a = g + Qinv(e); block top-k -> I[index], V[index]; min / max of the residual r per
 *      top-k block to the workspace;
 *   2. min / max of r per quantisation block from the workspace; e1 = Q(r);
 *      alpha == 0: error = e1, min_vals, max_vals; window -> Adam direction; p update (with
 *      decoupled weight decay);
 *      alpha > 0: Qinv(e1) stays in registers; window -> Adam direction, + alpha * Qinv(e1);
 *      p update; error = Q((1 - alpha) * Qinv(e1)), min_vals, max_vals.
 * With alpha > 0 these are two kernel passes and r travels from the first to the second in g.
 * With alpha == 0 they are one pass: a workgroup publishes its extremes and takes those of its
 * neighbours as they arrive; it waits for them a bounded time only (MA_SPAN_SPIN_LIMIT polls
 * per neighbour, an environment variable, default 256, 0 = no wait), and a block that gives
 * up leaves r in g and is taken through step 2 by a second launch.  Either way g may hold r
 * instead of the gradient afterwards (the reference's step destroys p.grad as well,
 * MA:190-316).
 * The caller advances st['index'] itself.  Conditions (else MA_ERR_NOT_FUSABLE, nothing
 * launched): 0 <= alpha < 1 (MA:18); quant_block_size a multiple of 8, not below
 * min(d, d_block_size), below 2^30 and covering at most 62 top-k blocks; alignment as for
 * ma_fused_step.
 * workspace: device memory, 16-byte aligned, at least ma_spanning_step_workspace() bytes,
 * owned by the caller; its contents need not survive between calls. */
int ma_spanning_step(const ma_tensor *tensors /* host */, int n_tensors,
                      const ma_hyper *hyper /* host */, double alpha, void *workspace,
                      int64_t workspace_bytes, void *stream);

/* Bytes of workspace ma_spanning_step needs for this list (32 per top-k block); -1 on bad
 * arguments.  Host-only. */
int64_t ma_spanning_step_workspace(const ma_tensor *tensors /* host */, int n_tensors,
                                    const ma_hyper *hyper /* host */);

/* 0 if ma_spanning_step would accept this tensor, else the MA_ERR_* it would return. */
int ma_spanning_step_check(const ma_tensor *tensor /* host */, const ma_hyper *hyper /* host */,
                            double alpha);

/* ma_spanning_step for callers that cannot allocate device memory or hand over a workspace
 * (tight serving loops, harnesses that forbid hipMalloc, code under HIP graph capture).  No
 * counterpart in the reference.  Same arguments, conditions and results as ma_spanning_step;
 * the workspace is a fixed array of MA_STATIC_WORKSPACE_BYTES (16 MiB) that the library holds
 * in the memory of every GPU it runs on until the process ends, which is room for 524 288
 * top-k blocks per call (10.7e9 elements at d_block_size 20480; the Llama-3-8B list needs
 * 12.6 MB); a list that needs more is rejected with MA_ERR_WORKSPACE and nothing is launched.
 * The call allocates and frees no device memory (on the host it builds its launch plan in
 * ordinary heap memory, as every step entry point does).  The array's address is looked up at
 * the first call on each device, for the device that is current then: the current device must
 * be the one `stream` belongs to.  All calls on one GPU share that GPU's array: it need not be
 * cleared between calls (a call clears or overwrites what it reads), but calls whose kernels
 * may overlap on one GPU (different streams) race on it.  Under graph capture: the step
 * number, the ring row and the learning rate travel by value in the kernel arguments, so a
 * captured call replays exactly that step; capture it anew (or update the kernel nodes) for
 * every step, and make the first, uncaptured call on the device before capturing (it looks up
 * the array and sets kernel attributes). */
int ma_spanning_step_static(const ma_tensor *tensors /* host */, int n_tensors,
                             const ma_hyper *hyper /* host */, double alpha, void *stream);

/* ma_fused_step for alpha == -2 (densify_update_using_quant_error, MA:238-273), same conditions,
 * still one pass per top-k block: with the residual a and the new error feedback e in
 * registers, p = p * (1 - lr * wd) (MA:234-235), p = p - a (MA:264), p = p + Qinv(e) (MA:269),
 * each rounded to the parameter's type, then the Adam step as for alpha == 0.  Every step
 * rewrites st['quant_err'] = a - Qinv(e), rounded to the parameter's type (MA:258-271); a tensor
 * whose quant_err pointer is NULL or not 16-byte aligned is rejected (MA_ERR_ARG /
 * MA_ERR_NOT_FUSABLE) before anything is launched. */
int ma_fused_step_quant_err(const ma_tensor *tensors /* host */, int n_tensors,
                            const ma_hyper *hyper /* host */, void *stream);

/* ---- logging steps (MA:155-156, :271-272, :306-308, :320-324, summed in _log's order MA:328) */
#define MA_ROUTE_FUSED 0     /* as ma_fused_step */
#define MA_ROUTE_DENSIFIED 1 /* as ma_fused_step_densified */
#define MA_ROUTE_SPANNING 2  /* as ma_spanning_step */
#define MA_ROUTE_QUANT_ERR 3 /* as ma_fused_step_quant_err */

/* One step as the entry point named by `route` takes it (same arguments, conditions and
 * results; alpha, workspace and workspace_bytes as that entry point has them, else ignored),
 * that also forms the sums the reference logs every log_interval steps, as side reductions of
 * the same kernels: every top-k block leaves 8 floats in `partials`, a last kernel adds them
 * in double, in a fixed order, and ADDS the totals to sums[0..5] (sums[6..7] unused):
 *   sums[0] |quant_err|^2 (MA:271; route QUANT_ERR only, else 0)   sums[1] |g|^2 (MA:155-156)
 *   sums[2] |u|^2 (MA:307)      sums[3] |Qinv(error)|^2 after the step (MA:320-324)
 *   sums[4] zeros of u (MA:308) sums[5] zeros of quant_err (MA:272)
 * taken from the values as the reference's buffers hold them (rounded to the gradient's
 * type).  Equal inputs give equal bits.
 * partials: device, at least ma_logged_step_partials() floats, contents need not survive the
 * call.  sums: device, 8 doubles, cleared by the caller before the first call of the step. */
int ma_logged_step(int route, const ma_tensor *tensors /* host */, int n_tensors,
                   const ma_hyper *hyper /* host */, double alpha, void *workspace,
                   int64_t workspace_bytes, float *partials, int64_t n_partials, double *sums,
                   void *stream);

/* Floats of `partials` ma_logged_step needs for this list (8 per top-k block); -1 on bad
 * arguments.  Host-only. */
int64_t ma_logged_step_partials(const ma_tensor *tensors /* host */, int n_tensors,
                                const ma_hyper *hyper /* host */);

/* ---- ista_daslab_cuda_sparse_mfac: the kernels that share the window layout -------------- */
/* Sparse M-FAC (sparse_mfac/sparse_core_mfac_w_ef.py, SC below) keeps its m gradients in the
 * same I (int16, block-relative) / V layout as MicroAdam's window; its values are bf16 or, with
 * use_bf16 = False, fp32 (SC:53-58), hence the values_dtype tag.  m_rows is the number of live
 * rows the caller passes (min(m, steps), SC:192, :212); rows are k entries apart. */

/* SP(blocks, threads, version, d, m, k, d_block_size, k_block_size, g, I, V, out, use_bf16),
 * SC:188-201: out[i] += sum_j V[i][j] * g[(j / k_block_size) * d_block_size + I[i][j]] for
 * i < m_rows; the caller zeroes out first (SC:186).  Products and sums in fp32; per top-k
 * block a partial sum per row goes to the workspace, a second kernel adds them in a fixed
 * order, so equal inputs give equal bits.  workspace: device memory, 4-byte aligned, at least
 * ma_sparse_scalar_products_workspace() bytes, contents need not survive the call. */
int ma_sparse_scalar_products(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                              int64_t k_block_size, const void *g, int g_dtype,
                              const int16_t *indices, const void *values, int values_dtype,
                              float *out, void *workspace, int64_t workspace_bytes,
                              void *stream);

/* *bytes = 4 * m_rows * number of top-k blocks.  Host-only. */
int ma_sparse_scalar_products_workspace(int64_t d, int64_t m_rows, int64_t k,
                                        int64_t d_block_size, int64_t k_block_size,
                                        int64_t *bytes /* host */);

/* LCG(blocks, threads, version, d, m, k, d_block_size, k_block_size, M, I, V, out, use_bf16),
 * SC:208-221: out[(j / k_block_size) * d_block_size + I[i][j]] += coef[i] * V[i][j] for
 * i < m_rows; the caller zeroes out first (SC:206).  Per coordinate the terms fl(coef[i] * v)
 * are added in fp32 in increasing row order, and the sum is added to out with one rounding
 * into out_dtype. */
int ma_sparse_linear_combination(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                                 int64_t k_block_size, const float *coef,
                                 const int16_t *indices, const void *values, int values_dtype,
                                 void *out, int out_dtype, void *stream);

/* ma_copy_values with the window values in values_dtype (SC:105-124 with use_bf16 = False keeps
 * fp32 values); dtype is the dense vector's type as in ma_copy_values. */
int ma_copy_values_typed(int64_t d, int64_t k, int64_t d_block_size, int64_t k_block_size,
                         const int16_t *indices, const void *inp, void *out, int direction,
                         int dtype, int values_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif
