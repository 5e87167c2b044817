// libmicroadam_hip.so: kernels, launchers and the C ABI declared in include/microadam_hip.h.
// gfx950 only.  Built by csrc/Makefile with -ffp-contract=off so that the fp32 arithmetic is
// the unfused sequence the header describes.
#include "ma_block.hpp"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>


namespace ma {

// =============================================================================================
// Elementwise kernels: the reference's extension ops taken one at a time
// =============================================================================================

__device__ __forceinline__ uint32_t nibble(uint32_t byte, int64_t i) {
    return (i & 1) ? (byte & 0x0fu) : (byte >> 4);
}

template <typename T>
__device__ __forceinline__ float ldf(const T *x, int64_t i);
template <>
__device__ __forceinline__ float ldf<float>(const float *x, int64_t i) { return x[i]; }
template <>
__device__ __forceinline__ float ldf<uint16_t>(const uint16_t *x, int64_t i) { return bf2f(x[i]); }
__device__ __forceinline__ void stf(float *x, int64_t i, float v) { x[i] = v; }
__device__ __forceinline__ void stf(uint16_t *x, int64_t i, float v) { x[i] = (uint16_t)f2bf(v); }

// x += alpha * (code * u + min); one thread per 8 elements
template <typename T>
__global__ __launch_bounds__(kWG) void quant_inv_kernel(int64_t d, int64_t q, const uint8_t *xq,
                                                        const uint16_t *xmin,
                                                        const uint16_t *xmax, T *x, float alpha) {
    const int64_t i0 = ((int64_t)blockIdx.x * kWG + threadIdx.x) * kChunk;
    if (i0 >= d) return;
    const int n = (int)((d - i0) < kChunk ? (d - i0) : kChunk);
    const bool vec = ((uintptr_t)(x + i0) & 15) == 0;
    float v[8];
    load8(x + i0, 0, n, vec, v);
    int64_t b = i0 / q;
    int64_t rem = i0 - b * q;
    float mn = bf2f(xmin[b]), mx = bf2f(xmax[b]);
    float u = (mx - mn) / 15.0f;
#pragma unroll
    for (int e = 0; e < kChunk; ++e) {
        if (e < n) {
            if (rem == q) {
                rem = 0;
                ++b;
                mn = bf2f(xmin[b]);
                mx = bf2f(xmax[b]);
                u = (mx - mn) / 15.0f;
            }
            const uint32_t code = nibble(xq[(i0 + e) >> 1], i0 + e);
            float deq = (float)code * u;
            deq = deq + mn;
            const float add = alpha * deq;
            v[e] = v[e] + add;
            ++rem;
        }
    }
    store8(x + i0, 0, n, vec, v);
}

__device__ __forceinline__ uint32_t quant_code(float x, float mn, float u, bool ok) {
    float v = (x - mn) / u;
    v = floorf(v + 0.5f);
    v = fmaxf(v, 0.0f);
    v = fminf(v, 15.0f);
    return ok ? (uint32_t)(int)v : 0u;
}

// xq = Q(x); one thread per 8 elements = 4 bytes of codes
template <typename T>
__global__ __launch_bounds__(kWG) void quant_kernel(int64_t d, int64_t q, uint8_t *xq,
                                                    const uint16_t *xmin, const uint16_t *xmax,
                                                    const T *x) {
    const int64_t i0 = ((int64_t)blockIdx.x * kWG + threadIdx.x) * kChunk;
    if (i0 >= d) return;
    const int n = (int)((d - i0) < kChunk ? (d - i0) : kChunk);
    const bool vec = ((uintptr_t)(x + i0) & 15) == 0;
    float v[8];
    load8(x + i0, 0, n, vec, v);
    int64_t b = i0 / q;
    int64_t rem = i0 - b * q;
    float mn = bf2f(xmin[b]), mx = bf2f(xmax[b]);
    float u = (mx - mn) / 15.0f;
    bool ok = u != 0.0f && isfinite(u);
    uint32_t codes[8];
#pragma unroll
    for (int e = 0; e < kChunk; ++e) {
        codes[e] = 0;
        if (e < n) {
            if (rem == q) {
                rem = 0;
                ++b;
                mn = bf2f(xmin[b]);
                mx = bf2f(xmax[b]);
                u = (mx - mn) / 15.0f;
                ok = u != 0.0f && isfinite(u);
            }
            codes[e] = quant_code(v[e], mn, u, ok);
            ++rem;
        }
    }
    uint8_t *dst = xq + (i0 >> 1);
    const int nbytes = (n + 1) >> 1;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (j < nbytes) dst[j] = (uint8_t)((codes[2 * j] << 4) | codes[2 * j + 1]);
}

// bf16 min / max per quantisation block.  per_wave != 0: each wave takes whole blocks in turn
// (small q); else one workgroup per block.
template <typename T>
__global__ __launch_bounds__(kWG) void minmax_kernel(int64_t d, int64_t q, int64_t nblocks,
                                                     const T *x, uint16_t *xmin, uint16_t *xmax,
                                                     int per_wave) {
    __shared__ float smn[kWaves], smx[kWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (per_wave) {
        for (int64_t b = (int64_t)blockIdx.x * kWaves + wave; b < nblocks;
             b += (int64_t)gridDim.x * kWaves) {
            const int64_t lo = b * q, hi = (lo + q < d) ? lo + q : d;
            float mn = INFINITY, mx = -INFINITY;
            for (int64_t i = lo + lane; i < hi; i += kWave) {
                const float v = ldf(x, i);
                mn = v < mn ? v : mn;
                mx = v > mx ? v : mx;
            }
#pragma unroll
            for (int s = 32; s > 0; s >>= 1) {
                const float a = __shfl_xor(mn, s, kWave), c = __shfl_xor(mx, s, kWave);
                mn = a < mn ? a : mn;
                mx = c > mx ? c : mx;
            }
            if (lane == 0) {
                xmin[b] = (uint16_t)f2bf(mn);
                xmax[b] = (uint16_t)f2bf(mx);
            }
        }
    } else {
        for (int64_t b = blockIdx.x; b < nblocks; b += gridDim.x) {
            const int64_t lo = b * q, hi = (lo + q < d) ? lo + q : d;
            float mn = INFINITY, mx = -INFINITY;
            for (int64_t i = lo + tid; i < hi; i += kWG) {
                const float v = ldf(x, i);
                mn = v < mn ? v : mn;
                mx = v > mx ? v : mx;
            }
#pragma unroll
            for (int s = 32; s > 0; s >>= 1) {
                const float a = __shfl_xor(mn, s, kWave), c = __shfl_xor(mx, s, kWave);
                mn = a < mn ? a : mn;
                mx = c > mx ? c : mx;
            }
            if (lane == 0) {
                smn[wave] = mn;
                smx[wave] = mx;
            }
            __syncthreads();
            if (tid == 0) {
#pragma unroll
                for (int w = 1; w < kWaves; ++w) {
                    mn = smn[w] < mn ? smn[w] : mn;
                    mx = smx[w] > mx ? smx[w] : mx;
                }
                xmin[b] = (uint16_t)f2bf(mn);
                xmax[b] = (uint16_t)f2bf(mx);
            }
            __syncthreads();
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kWG) void copy_values_kernel(int64_t k, int64_t dbs, int64_t kbs,
                                                          const int16_t *idx, const void *inp,
                                                          void *out, int direction) {
    const int64_t j = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (j >= k) return;
    const int64_t pos = (j / kbs) * dbs + idx[j];
    if (direction == 1)
        ((uint16_t *)out)[j] = (uint16_t)f2bf(ldf((const T *)inp, pos));
    else
        stf((T *)out, pos, bf2f(((const uint16_t *)inp)[j]));
}

template <typename T>
__global__ __launch_bounds__(kWG) void zerorize_kernel(T *vec, const int16_t *idx, int64_t k,
                                                       int64_t dbs, int64_t kbs) {
    const int64_t j = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (j >= k) return;
    vec[(j / kbs) * dbs + idx[j]] = (T)0;
}

// p = rne(p * decay) (optional); p = rne(p + neg_lr * u); one thread per 8 elements
template <typename T>
__global__ __launch_bounds__(kWG) void param_update_kernel(int64_t d, T *p, const T *u,
                                                           float neg_lr, int apply_decay,
                                                           float decay) {
    const int64_t i0 = ((int64_t)blockIdx.x * kWG + threadIdx.x) * kChunk;
    if (i0 >= d) return;
    const int n = (int)((d - i0) < kChunk ? (d - i0) : kChunk);
    const bool vec = (((uintptr_t)(p + i0) | (uintptr_t)(u + i0)) & 15) == 0;
    float pv[8], uv[8];
    load8(p + i0, 0, n, vec, pv);
    load8(u + i0, 0, n, vec, uv);
#pragma unroll
    for (int e = 0; e < kChunk; ++e) {
        float x = pv[e];
        if (apply_decay) {
            x = x * decay;
            if (sizeof(T) == 2) x = bf2f(f2bf(x));
        }
        const float prod = neg_lr * uv[e];
        pv[e] = x + prod;
    }
    store8(p + i0, 0, n, vec, pv);
}

// Start state of the workspace of a call of the one-pass form: per block (two uint4) the four
// extremes as all-ones words ("not published"), then zeros (flags, counts).
__global__ __launch_bounds__(kWG) void span_clear_kernel(uint4 *ws, int64_t n16) {
    for (int64_t i = (int64_t)blockIdx.x * kWG + threadIdx.x; i < n16; i += (int64_t)gridDim.x * kWG) {
        const uint32_t w = (i & 1) ? 0u : 0xffffffffu;
        ws[i] = make_uint4(w, w, w, w);
    }
}

// ---- standalone top-k (+ gather + zero) ---------------------------------------------------------

template <class R>
__global__ __launch_bounds__(kWG) void block_topk_kernel(int64_t d, int dbs, int k_many,
                                                         int k_few, typename R::elem_t *x,
                                                         int16_t *I_row, uint16_t *V_row,
                                                         int zero_selected, LdsMap L) {
    extern __shared__ __align__(16) unsigned char lds[];
    uint32_t *sh = reinterpret_cast<uint32_t *>(lds);
    uint16_t *sel_idx = reinterpret_cast<uint16_t *>(lds + L.off_sel_idx);
    uint16_t *sel_val = reinterpret_cast<uint16_t *>(lds + L.off_sel_val);
    uint32_t *hist = reinterpret_cast<uint32_t *>(lds + L.off_union);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t b = blockIdx.x;
    const int64_t n_full = d / dbs;
    const int64_t e0 = b * dbs;
    const int n = (int)((d - e0) < dbs ? (d - e0) : dbs);
    const int kb = b < n_full ? k_many : k_few;
    const int64_t col0 = b * k_many;
    typename R::elem_t *xb = x + e0;
    const bool vec = ((uintptr_t)xb & 15) == 0;

    R r;
    load_block(r, xb, n, vec, wave, lane);
    uint32_t T;
    int take_eq;
    select_threshold(r, kb, hist, sh, T, take_eq, L.hist_log2);
    compact_selected(r, T, take_eq, kb, sel_idx, sel_val, sh);
    for (int j = tid; j < kb; j += kWG) {
        const int idx = sel_idx[j];
        I_row[col0 + j] = (int16_t)idx;
        if (V_row) V_row[col0 + j] = sel_val[j];
        if (zero_selected) xb[idx] = (typename R::elem_t)0;
    }
}

// ---- standalone Adam direction from the window ---------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kWG) void window_update_kernel(int64_t d, int dbs, int kbs,
                                                            int64_t k, const int16_t *I,
                                                            const uint16_t *V, T *out,
                                                            WindowWeights W, LdsMap L) {
    extern __shared__ __align__(16) unsigned char lds[];
    float *z1 = reinterpret_cast<float *>(lds + L.off_union);
    float *z2 = z1 + L.z_cap;
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    const int64_t e0 = b * dbs;
    const int n = (int)((d - e0) < dbs ? (d - e0) : dbs);
    const int64_t col0 = b * kbs;
    const int kb = (int)((k - col0) < kbs ? (k - col0) : kbs);

    WindowView wv;
    wv.I = I + col0;
    wv.V = V + col0;
    wv.k = k;
    wv.rows = W.rows;
    wv.cur_row = -1;
    wv.cur_idx = nullptr;
    wv.cur_val = nullptr;
    wv.w1 = W.w1;
    wv.w2 = W.w2;
    for (int lo = 0; lo < n; lo += L.sub_len) {
        const int hi = lo + L.sub_len < n ? lo + L.sub_len : n;
        window_accumulate(wv, kb, lo, hi, z1, z2);
        for (int c = tid; c < hi - lo; c += kWG)
            if (z1[c] != 0.0f || z2[c] != 0.0f)
                stf(out, e0 + lo + c,
                    adam_update<sizeof(T) == 2>(z1[c], z2[c], W.s1, W.s2, W.eps));
        __syncthreads();
    }
}

// =============================================================================================
// Host side
// =============================================================================================


static inline int align16(int x) { return (x + 15) & ~15; }

// LDS plan for a block kernel: longest block `dbs_max`, most entries per block row `kb_max`,
// window length m, bytes per element of the data.
static LdsMap plan_lds(int dbs_max, int kb_max, int m, int elem_bytes, bool one_pass = true,
                       bool ranges_update = false) {
    LdsMap L;
    L.off_sel_idx = kMiscBytes;
    L.off_sel_val = L.off_sel_idx + align16(kb_max * 2);
    L.off_slot = L.off_sel_val + align16(kb_max * 2);
    L.slot_cells = (dbs_max + 7) & ~7;
    // one-pass window stage: two floats and four 16-bit words per entry; otherwise the block is
    // walked in coordinate ranges of at most 4096 with two dense fp32 arrays
    const int64_t entries = (int64_t)m * kb_max;
    const bool fast = one_pass && entries <= kEnt * kWG && m <= kFastRows;
    L.cell_bytes = (elem_bytes == 2 || fast) ? 2 : 4;
    if (!fast && ranges_update) L.cell_bytes = 0;
    L.off_union = L.off_slot + align16(L.slot_cells * (L.cell_bytes ? L.cell_bytes : 2));
    L.fast_cap = 0;
    L.hist_log2 = 5;
    L.compact = 0;
    if (fast && elem_bytes == 2 && m < kFastRows) {
        // bf16: coordinates named by several rows get a slot (two sums and the index, 10
        // bytes) each, at most half as many as there are entries; together with the small
        // histograms of the fast selection that lets three workgroups share a CU
        L.compact = 1;
        L.fast_cap = (int)(entries < 8 ? 8 : entries);
        L.z_cap = (L.fast_cap + 1) / 2;
        L.sub_len = L.slot_cells;
        const int zb = align16(L.z_cap * 10);
        int u = zb > kFastTopkBytes ? zb : kFastTopkBytes;
        L.hist_log2 = 0;
        while ((257 << (L.hist_log2 + 1)) * 4 <= u && L.hist_log2 < 5) ++L.hist_log2;
        L.total = L.off_union + align16(u);
        return L;
    }
    if (fast) {
        L.fast_cap = L.z_cap = (int)(entries < 8 ? 8 : entries);
        L.sub_len = L.slot_cells;
    } else if (L.cell_bytes == 0) {
        // the sums take the place of the cells and of the selection's histograms: as many
        // coordinates per range as fit beside a second workgroup on the CU, in units of 512
        const int room = kLdsLimit / 2 - L.off_slot;
        const int have = L.off_union + kHistBytes - L.off_slot;
        int sub = (room > have ? room : have) / 8 / 512 * 512;
        const int passes = (L.slot_cells + sub - 1) / sub;
        sub = ((L.slot_cells + passes - 1) / passes + 511) / 512 * 512;  // even them out
        L.sub_len = L.z_cap = sub;
        const int zb = 8 * sub;
        L.total = L.off_slot + align16(zb > have ? zb : have);
        return L;
    } else {
        L.sub_len = L.slot_cells < 4096 ? L.slot_cells : 4096;
        L.z_cap = L.sub_len;
    }
    const int zbytes = L.z_cap * (L.fast_cap ? 16 : 8);
    L.total = L.off_union + align16(zbytes > kHistBytes ? zbytes : kHistBytes);
    return L;
}

// LDS plan of a block kernel that ends with the quantisation: the selection's needs only (the
// cells are where the fast selection parks the block; longer block rows take the general
// selection, which leaves the block in registers).
static LdsMap plan_lds_select_only(int dbs_max, int kb_max, int elem_bytes) {
    LdsMap L;
    memset(&L, 0, sizeof L);
    L.off_sel_idx = kMiscBytes;
    L.off_sel_val = L.off_sel_idx + align16(kb_max * 2);
    L.off_slot = L.off_sel_val + align16(kb_max * 2);
    L.slot_cells = (dbs_max + 7) & ~7;
    L.cell_bytes = 2;
    if (kb_max <= kWG) {
        L.off_union = L.off_slot + align16(L.slot_cells * 2);
        L.hist_log2 = 5;
        L.total = L.off_union + kHistBytes;
    } else if (elem_bytes == 2 && kb_max <= kHintLongRow) {
        // the hinted ordered selection parks the block too; the general selection, which is
        // then the exception, makes do with 4 copies of its histogram, and the whole stays
        // within a third of the LDS
        L.off_union = L.off_slot + align16(L.slot_cells * 2);
        L.hist_log2 = 2;
        L.total = L.off_union + ((257 << L.hist_log2) * 4);
    } else {
        L.slot_cells = 0;
        L.off_union = L.off_slot;
        L.hist_log2 = 5;
        L.total = L.off_union + kHistBytes;
    }
    return L;
}

// LDS plan of window_param_kernel: the chunk table of every row, then 8192 floats of sums.
static LdsMap plan_lds_window_param(int dbs_max, int m) {
    LdsMap L;
    memset(&L, 0, sizeof L);
    L.off_slot = kMiscBytes;
    L.slot_cells = (dbs_max + kWinChunk - 1) / kWinChunk + 1;
    // (the row batches read up to kWindowPad table rows past the last one: kept empty)
    L.off_union = L.off_slot + align16((m + kWindowPad) * L.slot_cells * 4);
    L.total = L.off_union + kWaves * (kWinChunk + 8) * 8;  // (above the general form's 32 KiB)
    return L;
}

static void window_weights(int64_t t, int m, double beta1, double beta2, double eps,
                           WindowWeights *W) {
    memset(W, 0, sizeof *W);
    for (int i = 0; i < m; ++i) {
        const int64_t age = ((t - 1 - i) % m + m) % m;
        W->w1[i] = (float)pow(beta1, (double)age);
        W->w2[i] = (float)pow(beta2, (double)age);
    }
    W->s1 = (float)((1.0 - beta1) / (1.0 - pow(beta1, (double)t)));
    W->s2 = (float)((1.0 - beta2) / (1.0 - pow(beta2, (double)t)));
    W->eps = (float)eps;
    W->rows = (int)(t < m ? t : m);
    W->rows_total = m;
}

static inline unsigned grid_for(int64_t work_items) {
    return (unsigned)((work_items + kWG - 1) / kWG);
}

// chunks per thread that cover a block of `dbs` elements; 0 if none does
static int chunks_for(int64_t dbs) {
    if (dbs <= kRound * kClass0) return kClass0;
    if (dbs <= kRound * kClass1) return kClass1;
    if (dbs <= kRound * kClass2) return kClass2;
    if (dbs <= kRound * kClass3) return kClass3;
    return 0;
}

template <template <int> class RT>
static int launch_topk(int C, unsigned grid, int lds_bytes, hipStream_t s, int64_t d, int dbs,
                       int k_many, int k_few, void *x, int16_t *I_row, uint16_t *V_row,
                       int zero_selected, const LdsMap &L) {
#define MA_TOPK_CASE(CC)                                                                     \
    case CC: {                                                                               \
        int rc = allow_big_lds(block_topk_kernel<RT<CC>>, lds_bytes);                        \
        if (rc) return rc;                                                                   \
        return launch_kernel(block_topk_kernel<RT<CC>>, dim3(grid), kWG, lds_bytes, s, d,    \
                             dbs, k_many, k_few, (typename RT<CC>::elem_t *)x, I_row, V_row, \
                             zero_selected, L);                                              \
    }
    switch (C) {
        MA_TOPK_CASE(kClass0)
        MA_TOPK_CASE(kClass1)
        MA_TOPK_CASE(kClass2)
        MA_TOPK_CASE(kClass3)
    }
#undef MA_TOPK_CASE
    return MA_ERR_BLOCK_SIZE;
}

// geometry of one tensor, micro_adam.py:77-82
struct Geometry {
    int64_t dbs, n_full, tail, k_many, k_few, k;
};
static Geometry geometry(int64_t d, int64_t d_block_size, double k_init) {
    Geometry g;
    g.dbs = d < d_block_size ? d : d_block_size;
    g.n_full = d / g.dbs;
    g.tail = d - g.n_full * g.dbs;
    g.k_many = (int64_t)ceil((double)g.dbs * k_init);
    g.k_few = (int64_t)ceil((double)g.tail * k_init);
    g.k = g.n_full * g.k_many + g.k_few;
    return g;
}

// what every fused route asks of a tensor and the hyper-parameters
static int common_check(const ma_tensor *t, const ma_hyper *h, Geometry *g) {
    if (!t || !h) return MA_ERR_ARG;
    if (!t->p || !t->g || !t->error || !t->min_vals || !t->max_vals || !t->I || !t->V)
        return MA_ERR_ARG;
    if (t->d <= 0 || h->t < 1 || h->m < 1 || (h->dtype != MA_F32 && h->dtype != MA_BF16))
        return MA_ERR_ARG;
    if (h->m > MA_MAX_WINDOW) return MA_ERR_WINDOW;
    if (h->d_block_size < 1 || h->quant_block_size < 1) return MA_ERR_ARG;
    if (!(h->k_init > 0.0 && h->k_init <= 1.0)) return MA_ERR_ARG;
    if (t->index < 0 || t->index >= h->m) return MA_ERR_ARG;
    *g = geometry(t->d, h->d_block_size, h->k_init);
    if (g->dbs > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    if (g->k != t->k) return MA_ERR_GEOMETRY;
    if ((((uintptr_t)t->p | (uintptr_t)t->g) & 15) != 0 || ((uintptr_t)t->error & 3) != 0)
        return MA_ERR_NOT_FUSABLE;
    return 0;
}

// dense: with 0 < alpha < 1
static int fused_check(const ma_tensor *t, const ma_hyper *h, bool dense = false) {
    Geometry g;
    const int rc = common_check(t, h, &g);
    if (rc) return rc;
    const int64_t q = h->quant_block_size;
    (void)dense;
    if (q < 8 || q > 4096 || (q & (q - 1)) != 0) return MA_ERR_NOT_FUSABLE;
    if (t->d < q) return MA_ERR_NOT_FUSABLE;
    const bool single = t->d <= h->d_block_size;
    if (!single && (g.dbs % q != 0 || g.dbs % 8 != 0)) return MA_ERR_NOT_FUSABLE;
    // the block kernels' LDS plans (with and without densification) must fit the hardware
    const int eb = h->dtype == MA_BF16 ? 2 : 4;
    if (plan_lds((int)g.dbs, (int)g.k_many, h->m, eb, true, true).total > kLdsLimit ||
        plan_lds((int)g.dbs, (int)g.k_many, h->m, eb, true, false).total > kLdsLimit)
        return MA_ERR_LDS;
    return 0;
}

constexpr int kSpanMaxBlocks = 64;  // top-k blocks one quantisation block may touch
constexpr unsigned kSweepGroups = 256;  // workgroups of the sweep behind a one-pass launch

// Polls a workgroup of the one-pass form spends at most on one neighbour's flag (each a sleep
// of some 500 cycles and a load from device memory, say 2 us).  MA_SPAN_SPIN_LIMIT overrides
// it: 0 makes every block give up at once and take the second pass, which is how the tests
// reach that path.
static int span_spin_limit() {
    const char *e = getenv("MA_SPAN_SPIN_LIMIT");
    if (e && *e) {
        const long v = strtol(e, nullptr, 10);
        return v < 0 ? 0 : v > 1000000 ? 1000000 : (int)v;
    }
    return 256;
}

// the two-pass route: 0 <= alpha < 1, quantisation blocks a multiple of 8 and at least as long
// as the top-k blocks
static int span_check(const ma_tensor *t, const ma_hyper *h, double alpha) {
    Geometry g;
    const int rc = common_check(t, h, &g);
    if (rc) return rc;
    if (!(alpha >= 0.0) || !(alpha < 1.0)) return MA_ERR_NOT_FUSABLE;
    const int64_t q = h->quant_block_size;
    if (q % 8 != 0 || q < g.dbs || q >= (1LL << 30)) return MA_ERR_NOT_FUSABLE;
    if ((q + g.dbs - 1) / g.dbs + 1 > kSpanMaxBlocks) return MA_ERR_NOT_FUSABLE;
    const bool single = t->d <= h->d_block_size;
    if (!single && g.dbs % 8 != 0) return MA_ERR_NOT_FUSABLE;
    if (plan_lds((int)g.dbs, (int)g.k_many, h->m, h->dtype == MA_BF16 ? 2 : 4, true, false).total >
        kLdsLimit)
        return MA_ERR_LDS;
    return 0;
}

static inline int64_t span_ws_bytes(const ma_tensor *t, const ma_hyper *h) {
    const Geometry g = geometry(t->d, h->d_block_size, h->k_init);
    return (g.n_full + (g.tail > 0 ? 1 : 0)) * kSpanWords * 4;
}

}  // namespace ma

using namespace ma;

extern "C" {

const char *ma_error_string(int code) {
    switch (code) {
        case 0: return "ok";
        case MA_ERR_ARG: return "bad argument (null pointer, size, dtype or direction)";
        case MA_ERR_BLOCK_SIZE: return "top-k block longer than 32768 elements";
        case MA_ERR_WINDOW: return "window length m exceeds MA_MAX_WINDOW";
        case MA_ERR_GEOMETRY: return "k / k_block_size inconsistent with d and d_block_size";
        case MA_ERR_NOT_FUSABLE: return "tensor does not meet the fused step's layout conditions";
        case MA_ERR_LDS: return "launch would need more than 160 KB of LDS";
        case MA_ERR_WORKSPACE:
            return "list needs more workspace than ma_spanning_step_static holds "
                   "(32 bytes per top-k block, MA_STATIC_WORKSPACE_BYTES in all)";
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

int ma_get_sm_count(void) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return -1;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return -1;
    return n;
}

int ma_get_max_floats_for_shared_memory_per_thread_block(void) {
    return kLdsLimit / 4;  // gfx950: 160 KB of LDS per workgroup
}

#define MA_DISPATCH_DTYPE(dtype, CALL_F32, CALL_BF16) \
    if ((dtype) == MA_F32) return CALL_F32;           \
    if ((dtype) == MA_BF16) return CALL_BF16;         \
    return MA_ERR_ARG;

int ma_copy_values(int64_t d, int64_t k, int64_t d_block_size, int64_t k_block_size,
                   const int16_t *indices, const void *inp, void *out, int direction, int dtype,
                   void *stream) {
    if (!indices || !inp || !out || d <= 0 || k < 0 || d_block_size <= 0 || k_block_size <= 0)
        return MA_ERR_ARG;
    if (direction != 0 && direction != 1) return MA_ERR_ARG;
    if (d_block_size > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    // every j must land inside d: the last block row may not reach past the tensor
    if (((k + k_block_size - 1) / k_block_size - 1) * d_block_size >= d && k > 0)
        return MA_ERR_GEOMETRY;
    if (k == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(copy_values_kernel<float>, dim3(grid_for(k)), kWG, 0, s, k, d_block_size,
                      k_block_size, indices, inp, out, direction),
        launch_kernel(copy_values_kernel<uint16_t>, dim3(grid_for(k)), kWG, 0, s, k, d_block_size,
                      k_block_size, indices, inp, out, direction))
}

int ma_zerorize_block_components(void *vector, const int16_t *indices, int64_t d, int64_t k,
                                 int64_t d_block_size, int64_t k_block_size, int dtype,
                                 void *stream) {
    if (!vector || !indices || d <= 0 || k < 0 || d_block_size <= 0 || k_block_size <= 0)
        return MA_ERR_ARG;
    if (d_block_size > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    if (k > 0 && ((k + k_block_size - 1) / k_block_size - 1) * d_block_size >= d)
        return MA_ERR_GEOMETRY;
    if (k == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(zerorize_kernel<float>, dim3(grid_for(k)), kWG, 0, s, (float *)vector,
                      indices, k, d_block_size, k_block_size),
        launch_kernel(zerorize_kernel<uint16_t>, dim3(grid_for(k)), kWG, 0, s, (uint16_t *)vector,
                      indices, k, d_block_size, k_block_size))
}

int ma_asymm_block_quant(int64_t d, int64_t q, uint8_t *xq, const uint16_t *xmin,
                         const uint16_t *xmax, const void *x, int dtype, void *stream) {
    if (!xq || !xmin || !xmax || !x || d <= 0 || q <= 0) return MA_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const unsigned grid = grid_for((d + kChunk - 1) / kChunk);
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(quant_kernel<float>, dim3(grid), kWG, 0, s, d, q, xq, xmin, xmax,
                      (const float *)x),
        launch_kernel(quant_kernel<uint16_t>, dim3(grid), kWG, 0, s, d, q, xq, xmin, xmax,
                      (const uint16_t *)x))
}

int ma_asymm_block_quant_inv(int64_t d, int64_t q, const uint8_t *xq, const uint16_t *xmin,
                             const uint16_t *xmax, void *x, float alpha, int dtype,
                             void *stream) {
    if (!xq || !xmin || !xmax || !x || d <= 0 || q <= 0) return MA_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const unsigned grid = grid_for((d + kChunk - 1) / kChunk);
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(quant_inv_kernel<float>, dim3(grid), kWG, 0, s, d, q, xq, xmin, xmax,
                      (float *)x, alpha),
        launch_kernel(quant_inv_kernel<uint16_t>, dim3(grid), kWG, 0, s, d, q, xq, xmin, xmax,
                      (uint16_t *)x, alpha))
}

int ma_block_minmax(int64_t d, int64_t q, const void *x, uint16_t *xmin, uint16_t *xmax,
                    int dtype, void *stream) {
    if (!x || !xmin || !xmax || d <= 0 || q <= 0) return MA_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const int64_t nblocks = (d + q - 1) / q;
    const int per_wave = q <= 1024;
    int64_t wgs = per_wave ? (nblocks + kWaves - 1) / kWaves : nblocks;
    if (wgs > 65536 * 16) wgs = 65536 * 16;
    const unsigned grid = (unsigned)wgs;
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(minmax_kernel<float>, dim3(grid), kWG, 0, s, d, q, nblocks,
                      (const float *)x, xmin, xmax, per_wave),
        launch_kernel(minmax_kernel<uint16_t>, dim3(grid), kWG, 0, s, d, q, nblocks,
                      (const uint16_t *)x, xmin, xmax, per_wave))
}

int ma_param_update(int64_t d, void *p, const void *u, float neg_lr, int apply_decay, float decay,
                    int dtype, void *stream) {
    if (!p || !u || d <= 0) return MA_ERR_ARG;
    hipStream_t s = (hipStream_t)stream;
    const unsigned grid = grid_for((d + kChunk - 1) / kChunk);
    MA_DISPATCH_DTYPE(dtype,
        launch_kernel(param_update_kernel<float>, dim3(grid), kWG, 0, s, d, (float *)p,
                      (const float *)u, neg_lr, apply_decay, decay),
        launch_kernel(param_update_kernel<uint16_t>, dim3(grid), kWG, 0, s, d, (uint16_t *)p,
                      (const uint16_t *)u, neg_lr, apply_decay, decay))
}

int ma_block_topk(int64_t d, int64_t d_block_size, int64_t k_many, int64_t k_few, void *x,
                  int16_t *I_row, uint16_t *V_row, int zero_selected, int dtype, void *stream) {
    if (!x || !I_row || d <= 0 || d_block_size <= 0 || d_block_size > d) return MA_ERR_ARG;
    if (dtype != MA_F32 && dtype != MA_BF16) return MA_ERR_ARG;
    if (d_block_size > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    const int64_t n_full = d / d_block_size, tail = d - n_full * d_block_size;
    if (k_many < 1 || k_many > d_block_size || k_few < 0 || k_few > tail || (tail > 0) != (k_few > 0))
        return MA_ERR_GEOMETRY;
    const int C = chunks_for(d_block_size);
    if (!C) return MA_ERR_BLOCK_SIZE;
    const LdsMap L = plan_lds((int)d_block_size, (int)k_many, 1, 2);
    if (L.total > kLdsLimit) return MA_ERR_LDS;
    const unsigned grid = (unsigned)(n_full + (tail > 0 ? 1 : 0));
    hipStream_t s = (hipStream_t)stream;
    if (dtype == MA_F32)
        return launch_topk<RegsF32>(C, grid, L.total, s, d, (int)d_block_size, (int)k_many,
                                    (int)k_few, x, I_row, V_row, zero_selected, L);
    return launch_topk<RegsBF16>(C, grid, L.total, s, d, (int)d_block_size, (int)k_many,
                                 (int)k_few, x, I_row, V_row, zero_selected, L);
}

int ma_compute_microadam_update(int blocks, int threads, int carveout, int64_t t, double beta1,
                                double beta2, double eps, int64_t d_block_size,
                                int64_t k_block_size, int64_t d, int64_t m, int64_t k,
                                const int16_t *indices, const uint16_t *values, void *out,
                                int dtype, void *stream) {
    (void)blocks; (void)threads; (void)carveout;
    if (!indices || !values || !out || d <= 0 || k <= 0 || t < 1 || m < 1) return MA_ERR_ARG;
    if (d_block_size <= 0 || k_block_size <= 0 || k_block_size > d_block_size) return MA_ERR_ARG;
    if (dtype != MA_F32 && dtype != MA_BF16) return MA_ERR_ARG;
    if (m > MA_MAX_WINDOW) return MA_ERR_WINDOW;
    if (d_block_size > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    const int64_t nblocks = (k + k_block_size - 1) / k_block_size;
    // every block row must start inside the tensor
    if ((nblocks - 1) * d_block_size >= d) return MA_ERR_GEOMETRY;
    WindowWeights W;
    window_weights(t, (int)m, beta1, beta2, eps, &W);
    const LdsMap L = plan_lds((int)d_block_size, (int)k_block_size, (int)m, 2, false);
    if (L.total > kLdsLimit) return MA_ERR_LDS;
    hipStream_t s = (hipStream_t)stream;
    int rc;
    if (dtype == MA_F32) {
        if ((rc = allow_big_lds(window_update_kernel<float>, L.total))) return rc;
        return launch_kernel(window_update_kernel<float>, dim3((unsigned)nblocks), kWG, L.total, s,
                             d, (int)d_block_size, (int)k_block_size, k, indices, values,
                             (float *)out, W, L);
    }
    if ((rc = allow_big_lds(window_update_kernel<uint16_t>, L.total))) return rc;
    return launch_kernel(window_update_kernel<uint16_t>, dim3((unsigned)nblocks), kWG, L.total, s,
                         d, (int)d_block_size, (int)k_block_size, k, indices, values,
                         (uint16_t *)out, W, L);
}

int ma_fused_step_check(const ma_tensor *tensor, const ma_hyper *hyper) {
    return fused_check(tensor, hyper);
}

// Does ma_fused_step (alpha == 0, no logging) step a tensor of d elements in two launches?  Its
// window does not fit the one-pass stage of the block kernel then.
static bool window_apart(int64_t d, const ma_hyper *h, int elem_bytes) {
    const Geometry g = geometry(d, h->d_block_size, h->k_init);
    return plan_lds((int)g.dbs, (int)g.k_many, h->m, elem_bytes, true, true).cell_bytes == 0;
}

// words per window row of the cache of chunk cuts, see the header
static int64_t row_cut_words(int64_t d, const ma_hyper *h) {
    const Geometry g = geometry(d, h->d_block_size, h->k_init);
    const int64_t blocks = g.n_full + (g.tail > 0 ? 1 : 0);
    return blocks * ((g.dbs + kWinChunk - 1) / kWinChunk + 1);
}

int64_t ma_fused_step_row_cuts(const ma_tensor *tensor, const ma_hyper *hyper) {
    if (!tensor || !hyper) return MA_ERR_ARG;
    const int rc = fused_check(tensor, hyper);
    if (rc) return rc;
    const Geometry g = geometry(tensor->d, hyper->d_block_size, hyper->k_init);
    // only rows of more than 512 entries per block are written in coordinate order, which is
    // what the cuts describe
    if (!window_apart(tensor->d, hyper, hyper->dtype == MA_BF16 ? 2 : 4) || g.k_many <= kWG)
        return 0;
    return row_cut_words(tensor->d, hyper);
}

// One planned launch of a step: the kernel's parameters and the register-tile class it runs in.
struct PlannedLaunch {
    FusedParams P;
    int C;
    int kind;  // kWholeStep, or the two launches that share a step: kBlockPart, kWindowPart
};
enum { kWholeStep = 0, kBlockPart = 1, kWindowPart = 2 };

// Short tensors (one block of up to 4096 / 12288 elements) have kernels of their own, so that
// they do not occupy a workgroup sized for the hardware block; but when a call holds few of
// them next to longer tensors, a launch of their own costs more than that: up to this many
// blocks of a smaller class ride along in the call's largest class instead.
constexpr int64_t kMergeBlocks = 768;

// Blocks (work items) a list of tensors makes; -1 for a tensor without elements.
static int64_t count_blocks(const ma_tensor *tensors, int n_tensors, const ma_hyper *h) {
    int64_t blocks = 0;
    for (int i = 0; i < n_tensors; ++i) {
        if (tensors[i].d <= 0 || h->d_block_size < 1) return -1;
        const Geometry g = geometry(tensors[i].d, h->d_block_size, h->k_init);
        blocks += g.n_full + (g.tail > 0 ? 1 : 0);
    }
    return blocks;
}

// Second stage of a logging step's sums: one workgroup adds the blocks' slots in a fixed order,
// in double, and adds the totals to sums[0..7].
constexpr int kReduceThreads = 1024;
__global__ __launch_bounds__(kReduceThreads) void metrics_reduce_kernel(const float *partials,
                                                                         int64_t blocks,
                                                                         double *sums) {
    __shared__ double part[kReduceThreads];
    // thread t adds component t % 8 of the blocks t / 8, t / 8 + 128, ...
    const int comp = threadIdx.x % kMetricSlots, first = threadIdx.x / kMetricSlots;
    double acc = 0.0;
    for (int64_t b = first; b < blocks; b += kReduceThreads / kMetricSlots)
        acc += (double)partials[b * kMetricSlots + comp];
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int half = kReduceThreads / 2; half >= kMetricSlots; half >>= 1) {
        if ((int)threadIdx.x < half) part[threadIdx.x] += part[threadIdx.x + half];
        __syncthreads();
    }
    if (threadIdx.x < kMetricSlots) sums[threadIdx.x] += part[threadIdx.x];
}

// aux: kAux* bits.  With kAuxLog, metrics holds kMetricSlots floats per block of the call.
static int step_impl(const ma_tensor *tensors, int n_tensors, const ma_hyper *h, void *stream,
                     bool span, double alpha, void *ws, int64_t ws_bytes, int aux = 0,
                     float *metrics = nullptr) {
    const bool dense = !span && alpha > 0.0;
    if (!tensors || !h || n_tensors < 0) return MA_ERR_ARG;
    if ((aux & kAuxQuantErr) && (span || dense)) return MA_ERR_NOT_FUSABLE;
    if ((aux & kAuxLog) && !metrics) return MA_ERR_ARG;
    for (int i = 0; i < n_tensors; ++i) {
        const int rc =
            span ? span_check(&tensors[i], h, alpha) : fused_check(&tensors[i], h, alpha > 0.0);
        if (rc) return rc;
        if (aux & kAuxQuantErr) {  // st['quant_err'] is written with 16-byte stores
            if (!tensors[i].quant_err) return MA_ERR_ARG;
            if (((uintptr_t)tensors[i].quant_err & 15) != 0) return MA_ERR_NOT_FUSABLE;
        }
    }
    if (n_tensors == 0) return 0;
    int64_t ws_need = 0;
    if (span) {
        for (int i = 0; i < n_tensors; ++i) ws_need += span_ws_bytes(&tensors[i], h);
        if (!ws || ws_bytes < ws_need || ((uintptr_t)ws & 15) != 0) return MA_ERR_ARG;
    }
    hipStream_t s = (hipStream_t)stream;
    int q_shift = 0;
    while (!span && (1LL << q_shift) < h->quant_block_size) ++q_shift;
    WindowWeights W;
    window_weights(h->t, h->m, h->beta1, h->beta2, h->eps, &W);
    const int elem_bytes = h->dtype == MA_BF16 ? 2 : 4;
    const int d_block_size =
        (int)(h->d_block_size > MA_MAX_D_BLOCK ? MA_MAX_D_BLOCK : h->d_block_size);

    // ---- which class every tensor runs in
    static const int classes[4] = {kClass0, kClass1, kClass2, kClass3};
    std::vector<int> cls(n_tensors);
    int64_t blocks_in[4] = {0, 0, 0, 0};
    int largest = 0;
    for (int i = 0; i < n_tensors; ++i) {
        const Geometry g = geometry(tensors[i].d, h->d_block_size, h->k_init);
        const int C = chunks_for(g.dbs);
        int ci = 0;
        while (classes[ci] != C) ++ci;
        cls[i] = ci;
        blocks_in[ci] += g.n_full + (g.tail > 0 ? 1 : 0);
        if (ci > largest) largest = ci;
    }
    for (int i = 0; i < n_tensors; ++i)
        if (cls[i] < largest && blocks_in[cls[i]] <= kMergeBlocks) cls[i] = largest;

    // ---- all launches are laid out and checked before the first one starts, so that a call
    //      either steps every tensor or none
    std::vector<PlannedLaunch> plan;
    int64_t items_before = 0;  // work items of the launches laid out so far
    // the two-pass route's workspace is handed out in the order the tensors are laid out, so the
    // slots of a launch's tensors follow each other from those of its first tensor
    int64_t ws_off = 0;
    // tensors whose window is too large for the one-pass stage are stepped in two launches
    // (block part, window part) of their own, whatever else the call holds: which form a tensor
    // takes depends on its sizes alone
    std::vector<char> apart(n_tensors, 0);
    if (!span && !dense && !aux)
        for (int i = 0; i < n_tensors; ++i)
            apart[i] = window_apart(tensors[i].d, h, elem_bytes) ? 1 : 0;
    std::vector<int> order;
    for (int ci = 0; ci < 4; ++ci)
    for (int form = 0; form < 2; ++form) {
        // the class's tensors of this form in list order, those shorter than a top-k block (one
        // partial block each: they finish early) behind the others
        order.clear();
        for (int pass = 0; pass < 2; ++pass)
            for (int i = 0; i < n_tensors; ++i) {
                if (cls[i] != ci || apart[i] != form) continue;
                const bool is_short = tensors[i].d < h->d_block_size;
                if (is_short == (pass == 1)) order.push_back(i);
            }
        const int in_class = (int)order.size();
        if (in_class == 0) continue;
        // the class's tensors are spread evenly over as few launches as hold them (the
        // descriptors travel by value, kTensorsPerLaunch at most)
        const int launches = (in_class + kTensorsPerLaunch - 1) / kTensorsPerLaunch;
        const int per_launch = (in_class + launches - 1) / launches;
        int count = 0, short_items = 0;
        int64_t items = 0;
        int dbs_max = 0, kb_max = 0;
        auto close = [&]() -> int {
            if (count == 0) return 0;
            FusedParams &P = plan.back().P;
            P.n_tensors = count;
            P.W = W;
            P.L = plan_lds(dbs_max, kb_max, h->m, elem_bytes, true, !span && !dense);
            P.d_block_size = d_block_size;
            P.q_shift = q_shift;
            P.total_items = (int32_t)items;
            P.short_items = short_items;
            P.q_span = span ? (int32_t)h->quant_block_size : 0;
            P.alpha = (float)alpha;
            P.keep = (float)(1.0 - alpha);
            P.metrics = (aux & kAuxLog) ? metrics + items_before * kMetricSlots : nullptr;
            P.win_apart = 0;
            P.spin_limit = span_spin_limit();
            plan.back().kind = kWholeStep;
            int rc = P.L.total > kLdsLimit ? MA_ERR_LDS : 0;
            if (!span && !dense && !aux && P.L.cell_bytes == 0) {
                // a window too large for the one-pass stage: the block kernel ends with the
                // quantisation, a second launch over the same blocks forms the update
                P.win_apart = 1;
                P.L = plan_lds_select_only(dbs_max, kb_max, elem_bytes);
                plan.back().kind = kBlockPart;
                PlannedLaunch second = plan.back();
                second.kind = kWindowPart;
                second.P.L = plan_lds_window_param(dbs_max, h->m);
                if (second.P.L.total > kLdsLimit || P.L.total > kLdsLimit) rc = MA_ERR_LDS;
                plan.push_back(second);
            }
            items_before += items;
            count = short_items = 0;
            items = 0;
            dbs_max = kb_max = 0;
            return rc;
        };
        for (const int i : order) {
            const ma_tensor &t = tensors[i];
            const Geometry g = geometry(t.d, h->d_block_size, h->k_init);
            const int64_t ws_here = ws_off;
            if (span) ws_off += span_ws_bytes(&t, h);
            const int64_t nb = g.n_full + (g.tail > 0 ? 1 : 0);
            if (count == per_launch || items + nb > 0x7fffffff) {
                const int rc = close();
                if (rc) return rc;
            }
            if (count == 0) {
                plan.emplace_back();
                plan.back().C = classes[ci];
            }
            TensorDesc &D = plan.back().P.t[count];
            D.p = t.p;
            D.g = t.g;
            D.err = t.error;
            D.mn = t.min_vals;
            D.mx = t.max_vals;
            D.I = t.I;
            D.V = t.V;
            D.d = t.d;
            D.k = t.k;
            D.row = t.index;
            D.k_many = (int32_t)g.k_many;
            D.k_few = (int32_t)g.k_few;
            D.first_block = (int32_t)items;
            D.neg_lr = (float)(-t.lr);
            D.apply_decay = t.weight_decay > 0.0 ? 1 : 0;
            D.decay = (float)(1.0 - t.lr * t.weight_decay);
            D.blk0 = 0;
            D.ws = span ? reinterpret_cast<float *>(static_cast<char *>(ws) + ws_here)
                   : (aux & kAuxQuantErr) ? static_cast<float *>(t.quant_err)
                   : apart[i] ? reinterpret_cast<float *>(t.row_cuts)
                              : nullptr;
            items += nb;
            if (t.d < h->d_block_size) ++short_items;  // (nb == 1, and only short ones follow)
            if (g.dbs > dbs_max) dbs_max = (int)g.dbs;
            if (g.k_many > kb_max) kb_max = (int)g.k_many;
            ++count;
        }
        const int rc = close();
        if (rc) return rc;
    }

    // Two rounds over the plan: the first prepares every launch (kernel attributes: all that
    // can fail apart from a launch itself), the second launches.
    // the one-pass form of the two-pass route (every step but a logging one) starts from a
    // cleared workspace: its flags and counts are set as the blocks go
    const bool one_pass = span && !aux && !(alpha > 0.0);
    for (int round = 0; round < 2; ++round)
    for (const PlannedLaunch &L : plan) {
        if (one_pass && round == 1 && &L == &plan.front()) {
            const int64_t n16 = ws_need / 16;
            const unsigned cg = (unsigned)((n16 + kWG - 1) / kWG < 4096 ? (n16 + kWG - 1) / kWG : 4096);
            const int rc0 = launch_kernel(span_clear_kernel, dim3(cg), kWG, 0, s,
                                          reinterpret_cast<uint4 *>(ws), n16);
            if (rc0) return rc0;
        }
        const FusedParams &P = L.P;
        const unsigned grid = round == 0 ? 0u : (unsigned)P.total_items;
        const bool bf16 = h->dtype == MA_BF16;
        int rc = 0;
        if (dense && aux) {
            rc = bf16 ? launch_fused_dense_log_bf16(L.C, grid, P.L.total, s, P)
                      : launch_fused_dense_log_f32(L.C, grid, P.L.total, s, P);
        } else if (dense) {
            rc = bf16 ? launch_fused_dense_bf16(L.C, grid, P.L.total, s, P)
                      : launch_fused_dense_f32(L.C, grid, P.L.total, s, P);
        } else if (!span && aux) {
            rc = bf16 ? launch_fused_aux_bf16(L.C, aux, grid, P.L.total, s, P)
                      : launch_fused_aux_f32(L.C, aux, grid, P.L.total, s, P);
        } else if (L.kind == kWindowPart) {
            rc = bf16 ? launch_window_param_bf16(grid, P.L.total, s, P)
                      : launch_window_param_f32(grid, P.L.total, s, P);
        } else if (L.kind == kBlockPart) {
            rc = bf16 ? launch_fused_apart_bf16(L.C, grid, P.L.total, s, P)
                      : launch_fused_apart_f32(L.C, grid, P.L.total, s, P);
        } else if (!span) {
            rc = bf16 ? launch_fused_bf16(L.C, grid, P.L.total, s, P)
                      : launch_fused_f32(L.C, grid, P.L.total, s, P);
        } else {
            // alpha > 0 and logging steps: two passes; else one pass and the sweep over the
            // blocks it deferred
            const int passes[2] = {alpha > 0.0 ? 1 : one_pass ? 6 : 4,
                                   alpha > 0.0 ? 2 : one_pass ? 8 : 3};
            for (int i = 0; i < 2 && rc == 0; ++i) {
                unsigned g2 = grid;
                if (one_pass && i == 1 && grid > kSweepGroups) g2 = kSweepGroups;
                if (aux)
                    rc = bf16 ? launch_span_log_bf16(L.C, passes[i], g2, P.L.total, s, P)
                              : launch_span_log_f32(L.C, passes[i], g2, P.L.total, s, P);
                else
                    rc = bf16 ? launch_span_bf16(L.C, passes[i], g2, P.L.total, s, P)
                              : launch_span_f32(L.C, passes[i], g2, P.L.total, s, P);
            }
        }
        // A launch the runtime refuses after an earlier one of the same call has started leaves
        // the step applied to some tensors only: such an error is not one to retry after.
        if (rc) return rc;
    }
    return 0;
}

int ma_fused_step(const ma_tensor *tensors, int n_tensors, const ma_hyper *h, void *stream) {
    return step_impl(tensors, n_tensors, h, stream, false, 0.0, nullptr, 0);
}

int ma_fused_step_densified(const ma_tensor *tensors, int n_tensors, const ma_hyper *h,
                            double alpha, void *stream) {
    if (!(alpha > 0.0) || !(alpha < 1.0)) return MA_ERR_NOT_FUSABLE;
    return step_impl(tensors, n_tensors, h, stream, false, alpha, nullptr, 0);
}

int ma_fused_step_quant_err(const ma_tensor *tensors, int n_tensors, const ma_hyper *h,
                            void *stream) {
    return step_impl(tensors, n_tensors, h, stream, false, 0.0, nullptr, 0, kAuxQuantErr);
}

int64_t ma_logged_step_partials(const ma_tensor *tensors, int n_tensors, const ma_hyper *h) {
    if (!tensors || !h || n_tensors < 0) return -1;
    const int64_t blocks = count_blocks(tensors, n_tensors, h);
    return blocks < 0 ? -1 : blocks * kMetricSlots;
}

int ma_logged_step(int route, const ma_tensor *tensors, int n_tensors, const ma_hyper *h,
                   double alpha, void *workspace, int64_t workspace_bytes, float *partials,
                   int64_t n_partials, double *sums, void *stream) {
    if (!tensors || !h || n_tensors < 0 || !sums) return MA_ERR_ARG;
    const int64_t blocks = count_blocks(tensors, n_tensors, h);
    if (blocks < 0) return MA_ERR_ARG;
    if (blocks > 0 && (!partials || n_partials < blocks * kMetricSlots ||
                       ((uintptr_t)partials & 3) != 0))
        return MA_ERR_ARG;
    int rc;
    switch (route) {
        case MA_ROUTE_FUSED:
            rc = step_impl(tensors, n_tensors, h, stream, false, 0.0, nullptr, 0, kAuxLog, partials);
            break;
        case MA_ROUTE_DENSIFIED:
            if (!(alpha > 0.0) || !(alpha < 1.0)) return MA_ERR_NOT_FUSABLE;
            rc = step_impl(tensors, n_tensors, h, stream, false, alpha, nullptr, 0, kAuxLog,
                           partials);
            break;
        case MA_ROUTE_SPANNING:
            rc = step_impl(tensors, n_tensors, h, stream, true, alpha, workspace, workspace_bytes,
                           kAuxLog, partials);
            break;
        case MA_ROUTE_QUANT_ERR:
            rc = step_impl(tensors, n_tensors, h, stream, false, 0.0, nullptr, 0,
                           kAuxLog | kAuxQuantErr, partials);
            break;
        default:
            return MA_ERR_ARG;
    }
    if (rc || blocks == 0) return rc;
    return launch_kernel(metrics_reduce_kernel, dim3(1), kReduceThreads, 0, (hipStream_t)stream,
                         partials, blocks, sums);
}

int ma_spanning_step_check(const ma_tensor *tensor, const ma_hyper *hyper, double alpha) {
    return span_check(tensor, hyper, alpha);
}

int64_t ma_spanning_step_workspace(const ma_tensor *tensors, int n_tensors, const ma_hyper *h) {
    if (!tensors || !h || n_tensors < 0) return -1;
    int64_t need = 0;
    for (int i = 0; i < n_tensors; ++i) {
        if (tensors[i].d <= 0 || h->d_block_size < 1) return -1;
        need += span_ws_bytes(&tensors[i], h);
    }
    return need;
}

int ma_spanning_step(const ma_tensor *tensors, int n_tensors, const ma_hyper *h, double alpha,
                      void *workspace, int64_t workspace_bytes, void *stream) {
    return step_impl(tensors, n_tensors, h, stream, true, alpha, workspace, workspace_bytes);
}

// ---- ma_spanning_step without a caller workspace and without any allocation -----------------
// The per-block extremes of the residual go to a fixed array in device memory.  Every GPU the
// library runs on holds its own copy of the array at its own address; the address is looked
// up once per device, with that device current, and only that pointer is handed to kernels.
constexpr int64_t kStaticScratchBytes = MA_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];  // per device, null until looked up
static std::mutex g_scratch_mutex;

static int static_scratch(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return MA_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return MA_ERR_ARG;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

int ma_spanning_step_static(const ma_tensor *tensors, int n_tensors, const ma_hyper *h,
                             double alpha, void *stream) {
    if (!tensors || !h || n_tensors < 0) return MA_ERR_ARG;
    int64_t need = 0;
    for (int i = 0; i < n_tensors; ++i) {
        if (tensors[i].d <= 0 || h->d_block_size < 1) return MA_ERR_ARG;
        need += span_ws_bytes(&tensors[i], h);
    }
    if (need > kStaticScratchBytes) return MA_ERR_WORKSPACE;
    void *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc) return rc;
    return step_impl(tensors, n_tensors, h, stream, true, alpha, ws, kStaticScratchBytes);
}

}  // extern "C"
