// Sparse M-FAC's kernels over the window of MicroAdam's layout (m rows of k block-relative int16
// indices and k values, k_block_size entries per top-k block of d_block_size coordinates):
//   scalar products of the rows with a dense vector
//     (ista_daslab_cuda_sparse_mfac.SP, sparse_mfac/sparse_core_mfac_w_ef.py:185-203),
//   linear combination of the rows into a dense vector
//     (ista_daslab_cuda_sparse_mfac.LCG, sparse_core_mfac_w_ef.py:205-221),
//   copy_values with fp32 window values (sparse_core_mfac_w_ef.py:105-124, use_bf16 = False).
// One 512-thread workgroup per top-k block: the block of the dense vector lives in LDS, the
// window entries of the block stream past it once.  Part of libmicroadam_hip.so.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/microadam_hip.h"
#include "ma_device.hpp"

namespace ma {
namespace {

constexpr int kLdsBytes = 160 * 1024;
constexpr int kBatchRows = 16;         // rows the linear combination requests ahead
constexpr int kDotUnroll = 4;          // entries a lane requests ahead in the scalar products

__device__ __forceinline__ float widen(float x) { return x; }
__device__ __forceinline__ float widen(uint16_t x) { return bf2f(x); }
__device__ __forceinline__ void narrow(float *p, float v) { *p = v; }
__device__ __forceinline__ void narrow(uint16_t *p, float v) { *p = (uint16_t)f2bf(v); }

struct BlockSpan {
    int64_t e0;    // first coordinate of the top-k block
    int64_t col0;  // first window column of the block
    int len;       // coordinates in the block
    int kb;        // window entries per row in the block
};

__device__ __forceinline__ BlockSpan block_span(int64_t d, int dbs, int kbs, int64_t k) {
    BlockSpan s;
    const int64_t b = blockIdx.x;
    s.e0 = b * dbs;
    s.col0 = b * kbs;
    const int64_t len = d - s.e0, kb = k - s.col0;
    s.len = (int)(len < dbs ? len : dbs);
    s.kb = (int)(kb < kbs ? kb : kbs);
    return s;
}

// ---- scalar products ------------------------------------------------------------------------
// partial[b][r] = sum over the entries of row r in block b of V * g; a wave per row, the lanes'
// sums folded by a butterfly.  The second kernel adds the blocks' partial sums in a fixed order.
template <typename TG, typename TV>
__global__ __launch_bounds__(kWG) void sparse_dot_kernel(int64_t d, int dbs, int kbs, int64_t k,
                                                         int m_rows, const TG *g,
                                                         const int16_t *I, const TV *V,
                                                         float *partial) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const BlockSpan S = block_span(d, dbs, kbs, k);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    TG *gl = (TG *)lds_raw;

    const TG *src = g + S.e0;
    constexpr int kPer16 = 16 / sizeof(TG);
    int staged = 0;
    if ((((uintptr_t)src) & 15) == 0) {
        const int n16 = S.len / kPer16;
        for (int i = tid; i < n16; i += kWG) ((uint4 *)gl)[i] = ((const uint4 *)src)[i];
        staged = n16 * kPer16;
    }
    for (int i = staged + tid; i < S.len; i += kWG) gl[i] = src[i];
    __syncthreads();

    // the workgroups of one block (gridDim.y of them) share its rows; a wave takes two rows at
    // a time so that both rows' entries are in flight together
    constexpr int kWaves = kWG / 64;
    const int per = (m_rows + (int)gridDim.y - 1) / (int)gridDim.y;
    const int row_lo = (int)blockIdx.y * per;
    const int row_hi = row_lo + per < m_rows ? row_lo + per : m_rows;
    for (int r = row_lo + wave; r < row_hi; r += 2 * kWaves) {
        const int r2 = r + kWaves;
        const bool two = r2 < row_hi;
        const int64_t atA = (int64_t)r * k + S.col0, atB = (int64_t)(two ? r2 : r) * k + S.col0;
        float accA = 0.0f, accB = 0.0f;
        for (int j0 = 0; j0 < S.kb; j0 += 64 * kDotUnroll) {
            int ixA[kDotUnroll], ixB[kDotUnroll];
            TV vA[kDotUnroll], vB[kDotUnroll];
#pragma unroll
            for (int u = 0; u < kDotUnroll; ++u) {
                const int j = j0 + u * 64 + lane;
                ixA[u] = ixB[u] = -1;
                vA[u] = vB[u] = (TV)0;
                if (j < S.kb) {
                    ixA[u] = I[atA + j];
                    vA[u] = V[atA + j];
                    if (two) {
                        ixB[u] = I[atB + j];
                        vB[u] = V[atB + j];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < kDotUnroll; ++u) {
                if ((unsigned)ixA[u] < (unsigned)S.len) accA += widen(vA[u]) * widen(gl[ixA[u]]);
                if ((unsigned)ixB[u] < (unsigned)S.len) accB += widen(vB[u]) * widen(gl[ixB[u]]);
            }
        }
#pragma unroll
        for (int s = 32; s > 0; s >>= 1) {
            accA += __shfl_xor(accA, s, 64);
            accB += __shfl_xor(accB, s, 64);
        }
        // straight to the workspace: LDS holds the block of g and nothing else, so that four
        // workgroups with a 20480-element bf16 block share a CU
        if (lane == 0) {
            float *dst = partial + (int64_t)blockIdx.x * m_rows;
            dst[r] = accA;
            if (two) dst[r2] = accB;
        }
    }
}

// out[r] += sum over blocks of partial[b][r]: a wave per row, lane l adds blocks l, l + 64, ...
// in increasing order, then the butterfly
__global__ __launch_bounds__(kWG) void sparse_dot_reduce_kernel(const float *partial,
                                                                int64_t nblocks, int m_rows,
                                                                float *out) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * (kWG / 64) + (threadIdx.x >> 6);
    if (r >= m_rows) return;
    float acc = 0.0f;
    for (int64_t b = lane; b < nblocks; b += 64) acc += partial[b * m_rows + r];
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) acc += __shfl_xor(acc, s, 64);
    if (lane == 0) out[r] = out[r] + acc;
}

// ---- linear combination ---------------------------------------------------------------------
// acc[c] (fp32, LDS) takes the terms coef[r] * V[r][j] of the block's coordinates row by row in
// increasing r: the entries of one row name distinct coordinates, so a row is applied without
// atomics, and a barrier separates rows.  With at most 512 entries per row a thread holds one
// column of kBatchRows rows, the next batch requested before the current one is applied.
template <typename TO, typename TV, int WG>
__global__ __launch_bounds__(WG) void sparse_combine_kernel(int64_t d, int dbs, int kbs,
                                                             int64_t k, int m_rows,
                                                             const float *coef, const int16_t *I,
                                                             const TV *V, TO *out) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    float *acc = (float *)lds_raw;
    const BlockSpan S = block_span(d, dbs, kbs, k);
    const int tid = threadIdx.x;
    for (int i = tid; i < S.len; i += WG) acc[i] = 0.0f;
    __syncthreads();

    if (S.kb <= WG) {
        // thread tid holds column tid of kBatchRows consecutive rows.  Requests are
        // unconditional (row and column clamped into the window) and their results stay as
        // loaded until they are applied, so that all of a batch is in flight at once.
        const bool mine = tid < S.kb;
        const int16_t *Ic = I + S.col0 + (mine ? tid : 0);
        const TV *Vc = V + S.col0 + (mine ? tid : 0);
        int nix[kBatchRows];
        TV nraw[kBatchRows];
        float ncoef[kBatchRows];
        auto request = [&](int r0) {
#pragma unroll
            for (int u = 0; u < kBatchRows; ++u) {
                const int row = r0 + u < m_rows ? r0 + u : m_rows - 1;
                nix[u] = Ic[(int64_t)row * k];
                nraw[u] = Vc[(int64_t)row * k];
                ncoef[u] = coef[row];
            }
        };
        request(0);
        for (int r0 = 0; r0 < m_rows; r0 += kBatchRows) {
            int ix[kBatchRows];
            float term[kBatchRows];
#pragma unroll
            for (int u = 0; u < kBatchRows; ++u) {
                ix[u] = (mine && (unsigned)nix[u] < (unsigned)S.len) ? nix[u] : -1;
                term[u] = ncoef[u] * widen(nraw[u]);
            }
            if (r0 + kBatchRows < m_rows) request(r0 + kBatchRows);
#pragma unroll
            for (int u = 0; u < kBatchRows; ++u) {
                if (r0 + u < m_rows) {
                    if (ix[u] >= 0) acc[ix[u]] = acc[ix[u]] + term[u];
                    __syncthreads();
                }
            }
        }
    } else {
        for (int r = 0; r < m_rows; ++r) {
            const float c = coef[r];
            const int64_t at = (int64_t)r * k + S.col0;
            for (int j = tid; j < S.kb; j += WG) {
                const int ix = I[at + j];
                const float term = c * widen(V[at + j]);
                if ((unsigned)ix < (unsigned)S.len) acc[ix] = acc[ix] + term;
            }
            __syncthreads();
        }
    }

    TO *dst = out + S.e0;
    for (int i = tid; i < S.len; i += WG) narrow(dst + i, widen(dst[i]) + acc[i]);
}

// ---- copy_values with typed window values ---------------------------------------------------
template <typename TD, typename TV>
__global__ __launch_bounds__(kWG) void copy_values_typed_kernel(int64_t k, int64_t dbs,
                                                                int64_t kbs, const int16_t *idx,
                                                                const void *inp, void *out,
                                                                int direction) {
    const int64_t j = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (j >= k) return;
    const int64_t pos = (j / kbs) * dbs + idx[j];
    if (direction == 1)
        narrow((TV *)out + j, widen(((const TD *)inp)[pos]));
    else
        narrow((TD *)out + pos, widen(((const TV *)inp)[j]));
}

template <typename K>
int allow_lds(K kernel, int bytes) {
    if (bytes <= 64 * 1024) return 0;
    return (int)hipFuncSetAttribute((const void *)kernel,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

int window_check(int64_t d, int64_t m_rows, int64_t k, int64_t dbs, int64_t kbs,
                 int64_t *nblocks) {
    if (d <= 0 || k <= 0 || m_rows < 0 || dbs <= 0 || kbs <= 0 || kbs > dbs) return MA_ERR_ARG;
    if (dbs > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    if (m_rows > MA_MAX_SPARSE_ROWS) return MA_ERR_WINDOW;
    *nblocks = (k + kbs - 1) / kbs;
    // every block row must start inside the vector
    if ((*nblocks - 1) * dbs >= d || *nblocks >= (int64_t)1 << 31) return MA_ERR_GEOMETRY;
    return 0;
}

bool known(int dtype) { return dtype == MA_F32 || dtype == MA_BF16; }

}  // namespace
}  // namespace ma

using namespace ma;

#define MA_DISPATCH2(A, B, CALL)                                      \
    if ((A) == MA_F32 && (B) == MA_F32) { CALL(float, float) }        \
    else if ((A) == MA_F32) { CALL(float, uint16_t) }                 \
    else if ((B) == MA_F32) { CALL(uint16_t, float) }                 \
    else { CALL(uint16_t, uint16_t) }

extern "C" {

int ma_sparse_scalar_products_workspace(int64_t d, int64_t m_rows, int64_t k,
                                        int64_t d_block_size, int64_t k_block_size,
                                        int64_t *bytes) {
    int64_t nblocks = 0;
    if (!bytes) return MA_ERR_ARG;
    const int rc = window_check(d, m_rows, k, d_block_size, k_block_size, &nblocks);
    if (rc) return rc;
    *bytes = nblocks * m_rows * (int64_t)sizeof(float);
    return 0;
}

int ma_sparse_scalar_products(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                              int64_t k_block_size, const void *g, int g_dtype,
                              const int16_t *indices, const void *values, int values_dtype,
                              float *out, void *workspace, int64_t workspace_bytes,
                              void *stream) {
    int64_t nblocks = 0;
    if (!g || !indices || !values || !out || !known(g_dtype) || !known(values_dtype))
        return MA_ERR_ARG;
    int rc = window_check(d, m_rows, k, d_block_size, k_block_size, &nblocks);
    if (rc) return rc;
    if (m_rows == 0) return 0;
    if (!workspace || ((uintptr_t)workspace & 3) ||
        workspace_bytes < nblocks * m_rows * (int64_t)sizeof(float))
        return MA_ERR_ARG;
    const int esize = g_dtype == MA_F32 ? 4 : 2;
    const int lds = (int)((d_block_size * esize + 15) & ~(int64_t)15);
    if (lds > kLdsBytes) return MA_ERR_LDS;
    hipStream_t s = (hipStream_t)stream;
    float *partial = (float *)workspace;
    // enough workgroups to fill the CUs several times over, at least 64 rows each
    int64_t gy = (4096 + nblocks - 1) / nblocks, gy_max = m_rows / 64;
    gy = gy > gy_max ? gy_max : gy;
    gy = gy < 1 ? 1 : gy;
#define CALL(TG, TV)                                                                            \
    if ((rc = allow_lds(sparse_dot_kernel<TG, TV>, lds))) return rc;                            \
    rc = launch_kernel(sparse_dot_kernel<TG, TV>, dim3((unsigned)nblocks, (unsigned)gy), kWG,   \
                       lds, s, d, (int)d_block_size, (int)k_block_size, k, (int)m_rows,         \
                       (const TG *)g, indices, (const TV *)values, partial);
    MA_DISPATCH2(g_dtype, values_dtype, CALL)
#undef CALL
    if (rc) return rc;
    const unsigned rgrid = (unsigned)((m_rows + kWG / 64 - 1) / (kWG / 64));
    return launch_kernel(sparse_dot_reduce_kernel, dim3(rgrid), kWG, 0, s, partial, nblocks,
                         (int)m_rows, out);
}

int ma_sparse_linear_combination(int64_t d, int64_t m_rows, int64_t k, int64_t d_block_size,
                                 int64_t k_block_size, const float *coef,
                                 const int16_t *indices, const void *values, int values_dtype,
                                 void *out, int out_dtype, void *stream) {
    int64_t nblocks = 0;
    if (!coef || !indices || !values || !out || !known(out_dtype) || !known(values_dtype))
        return MA_ERR_ARG;
    int rc = window_check(d, m_rows, k, d_block_size, k_block_size, &nblocks);
    if (rc) return rc;
    if (m_rows == 0) return 0;
    const int lds = (int)(d_block_size * 4);
    if (lds > kLdsBytes) return MA_ERR_LDS;
    hipStream_t s = (hipStream_t)stream;
    // rows of at most 256 entries go to 256-thread workgroups: a row's barrier then joins four
    // waves instead of eight
#define CALL_WG(TO, TV, WG)                                                                     \
    if ((rc = allow_lds(sparse_combine_kernel<TO, TV, WG>, lds))) return rc;                    \
    rc = launch_kernel(sparse_combine_kernel<TO, TV, WG>, dim3((unsigned)nblocks), WG, lds, s,  \
                       d, (int)d_block_size, (int)k_block_size, k, (int)m_rows, coef, indices,  \
                       (const TV *)values, (TO *)out);
#define CALL(TO, TV)                                                                            \
    if (k_block_size <= 256) { CALL_WG(TO, TV, 256) } else { CALL_WG(TO, TV, kWG) }
    MA_DISPATCH2(out_dtype, values_dtype, CALL)
#undef CALL
#undef CALL_WG
    return rc;
}

int ma_copy_values_typed(int64_t d, int64_t k, int64_t d_block_size, int64_t k_block_size,
                         const int16_t *indices, const void *inp, void *out, int direction,
                         int dtype, int values_dtype, void *stream) {
    if (!indices || !inp || !out || d <= 0 || k < 0 || d_block_size <= 0 || k_block_size <= 0)
        return MA_ERR_ARG;
    if ((direction != 0 && direction != 1) || !known(dtype) || !known(values_dtype))
        return MA_ERR_ARG;
    if (d_block_size > MA_MAX_D_BLOCK) return MA_ERR_BLOCK_SIZE;
    if (k > 0 && ((k + k_block_size - 1) / k_block_size - 1) * d_block_size >= d)
        return MA_ERR_GEOMETRY;
    if (k == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned grid = (unsigned)((k + kWG - 1) / kWG);
#define CALL(TD, TV)                                                                   \
    rc = launch_kernel(copy_values_typed_kernel<TD, TV>, dim3(grid), kWG, 0, s, k,     \
                       d_block_size, k_block_size, indices, inp, out, direction);
    int rc = 0;
    MA_DISPATCH2(dtype, values_dtype, CALL)
#undef CALL
    return rc;
}

}  // extern "C"
