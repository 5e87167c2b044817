// The block kernels of the MicroAdam step: one 512-thread workgroup per top-k block, the block
// held in registers.  Shared by the translation units that instantiate them (one per data type
// and route, so that they compile side by side); gfx950 only.
#pragma once
#include "ma_device.hpp"

#include "../../include/microadam_hip.h"

namespace ma {


// LDS map shared by the block kernels (byte offsets from the start of dynamic LDS)
struct LdsMap {
    int off_sel_idx;  // uint16[kb_max]
    int off_sel_val;  // uint16[kb_max]
    int off_slot;     // slot_cells cells of cell_bytes
    int off_union;    // histograms and candidate lists during selection, then the window stage's arrays
    int slot_cells;   // multiple of 8, >= longest block
    int z_cap;        // entries the window stage's arrays hold
    int sub_len;      // coordinates handled per window pass
    int fast_cap;     // entries the one-pass window stage has room for, 0: none
    int hist_log2;    // log2 of the histogram copies the general selection has room for
    int compact;      // bf16 one-pass window stage with slots per coordinate instead of lists
    int cell_bytes;   // width of a slot cell: 2, or 4 for fp32 data in the general window stage;
                      // 0: no cells, the general window stage updates the parameters range by range
    int total;        // bytes
};
constexpr int kMiscBytes = 256;  // the kSh* words at the very start
constexpr int kFastTopkBytes = (2 * kSmallHistWords + 512) * 4;
constexpr int kHistBytes =
    257 * kHistCopies * 4 > kFastTopkBytes ? 257 * kHistCopies * 4 : kFastTopkBytes;

constexpr int kWindowPad = 16;  // zero weights behind the last row, for code that reads rows in batches
struct WindowWeights {
    float w1[kMaxWindow + kWindowPad];
    float w2[kMaxWindow + kWindowPad];
    float s1, s2, eps;
    int rows;        // live rows: min(t, m)
    int rows_total;  // m
};

// ---- the fused step -----------------------------------------------------------------------------------

struct TensorDesc {
    void *p;
    const void *g;
    uint8_t *err;
    uint16_t *mn;
    uint16_t *mx;
    int16_t *I;
    uint16_t *V;
    int64_t d;
    int64_t k;
    int32_t row;
    int32_t k_many;
    int32_t k_few;
    int32_t first_block;  // first work item of this tensor inside the launch
    float neg_lr;
    float decay;
    int32_t apply_decay;
    int32_t blk0;         // block of the tensor that its first work item stands for
    float *ws;            // two-pass route: per-block extremes of the residual;
                          // alpha == -2: st['quant_err'] (elements of the data's type);
                          // two-launch form of dense windows: the cache of row cuts (uint16
                          // words) or null; else unused
};
// The descriptors travel by value in the kernel arguments (112 bytes each; the runtime passes
// arguments of this size intact).  Fewer, longer launches: each launch ends with a partly
// filled round of workgroups, and small tensors would otherwise queue up behind each other.
constexpr int kTensorsPerLaunch = 160;

struct FusedParams {
    TensorDesc t[kTensorsPerLaunch];
    WindowWeights W;
    LdsMap L;
    int32_t n_tensors;
    int32_t d_block_size;
    int32_t q_shift;  // log2(quant_block_size)
    int32_t total_items;  // work items (blocks) of the launch
    int32_t short_items;  // of them, at the end: tensors shorter than a top-k block, one item each
    // two-pass route (quantisation blocks at least as long as the top-k blocks)
    int32_t q_span;   // quantisation block length, a multiple of 8
    float alpha;      // share of the dequantised error feedback added to the update
    float keep;       // (float)(1 - alpha): share that stays in the error feedback
    // logging steps (kernels compiled with kAuxLog): kMetricSlots floats per work item
    float *metrics;
    // the block kernel ends with the quantisation; window_param_kernel does the rest
    int32_t win_apart;
    // one-pass form of the two-pass route: polls a workgroup spends at most on waiting for the
    // extremes of the blocks that share its quantisation blocks (0: it does not wait at all)
    int32_t spin_limit;
};

// Extras of a block kernel (template parameter AUX, a set of bits).  Kernels with extras run
// rarely or on request, and are compiled for any quantisation group with the register budget
// of two workgroups per CU.
//   kAuxLog: a logging step (MA:155-156, :271-272, :306-308, :320-324): every block leaves the
//            sums of its elements in its metrics slot, in the order of the reference's return
//            value (MA:328): |quant_err|^2, |g|^2, |u|^2, |Qinv(e)|^2, zeros of u, zeros of
//            quant_err (the counts as floats; two unused floats pad the slot to 32 bytes).
//            The values are summed as the reference's buffers hold them (rounded to the
//            gradient's type), in fp32 and in a fixed order.
//   kAuxQuantErr: alpha == -2 (MA:238-273): what the quantisation of the residual loses goes
//            straight into the parameters, p = p - a, then p = p + Qinv(e) (each rounded to
//            the parameter's type) before the Adam step.
constexpr int kAuxLog = 1, kAuxQuantErr = 2;
constexpr int kSpanWords = 8;  // workspace words per top-k block of the two-pass route
constexpr int kRowCutStep = 512;  // coordinates between two cuts of a window row
constexpr int kHintLongRow = 4 * 512;  // longest block row whose previous threshold is looked up

// Layout of a tensor's cache of row cuts: (row, block, cut) -> word
struct RowCuts {
    int64_t blocks;
    int per_block;
    __host__ __device__ RowCuts(int64_t d, int64_t d_block_size) {
        const int64_t dbs = d < d_block_size ? d : d_block_size;
        blocks = (d + dbs - 1) / dbs;
        per_block = (int)((dbs + kRowCutStep - 1) / kRowCutStep) + 1;
    }
    __host__ __device__ int64_t at(int64_t row, int64_t block) const {
        return (row * blocks + block) * per_block;
    }
};
constexpr int kMetricSlots = 8;
enum { kMtQuantErr = 0, kMtGrad = 1, kMtUpdate = 2, kMtError = 3, kMtUpdateZeros = 4, kMtQuantErrZeros = 5 };

template <class R>
struct RawChunk;
template <int C>
struct RawChunk<RegsBF16<C>> {
    uint4 q;
    __device__ __forceinline__ void load(const uint16_t *base, int off, int n, bool full) {
        if (full || off + kChunk <= n) {
            // read once: streamed past the caches (1 % on the 7B step)
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            const u4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(base + off));
            q = make_uint4(t.x, t.y, t.z, t.w);
        } else {
            uint32_t r[4] = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (off + i < n) r[i >> 1] |= (uint32_t)base[off + i] << (16 * (i & 1));
            q = make_uint4(r[0], r[1], r[2], r[3]);
        }
    }
    __device__ __forceinline__ void to_float(float (&v)[8]) const {
        const uint32_t r[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(r[i] << 16);
            v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ void from_float(const float (&v)[8]) {
        q = make_uint4(f2bf_pair(v[0], v[1]), f2bf_pair(v[2], v[3]), f2bf_pair(v[4], v[5]),
                       f2bf_pair(v[6], v[7]));
    }
};
template <int C>
struct RawChunk<RegsF32<C>> {
    float v_[8];
    __device__ __forceinline__ void load(const float *base, int off, int n, bool full) {
        if (full) {
            const float4 a = *reinterpret_cast<const float4 *>(base + off);
            const float4 b = *reinterpret_cast<const float4 *>(base + off + 4);
            v_[0] = a.x; v_[1] = a.y; v_[2] = a.z; v_[3] = a.w;
            v_[4] = b.x; v_[5] = b.y; v_[6] = b.z; v_[7] = b.w;
        } else {
            load8(base, off, n, true, v_);
        }
    }
    __device__ __forceinline__ void to_float(float (&v)[8]) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = v_[i];
    }
    __device__ __forceinline__ void from_float(const float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v_[i] = v[i];
    }
};

// One-pass window stage: the rows * kb entries of a block are dealt out over the workgroup,
// entry e to thread e % kWG, and requested at the start of the block.
constexpr int kEnt = 5;        // entries per thread at most
constexpr int kFastRows = 16;  // window rows at most: a coordinate's rows are a 16-bit mask

// Where one top-k block lives: everything a stage needs to address it, copied out of the
// launch parameters.  Wave-uniform (lives in scalar registers).
struct BlockGeo {
    TensorDesc D;
    int64_t e0;    // first element
    int64_t col0;  // first window column
    int n;         // elements in the block
    int kb;        // entries selected from it
};

__device__ __forceinline__ BlockGeo make_geo(const FusedParams &P, int ti, int64_t b) {
    BlockGeo G;
    G.D = P.t[ti];
    const int64_t d = G.D.d;
    const int dbs = (int)(d < P.d_block_size ? d : P.d_block_size);
    const int64_t n_full = d / dbs;
    G.e0 = b * dbs;
    G.n = (int)((d - G.e0) < dbs ? (d - G.e0) : dbs);
    G.kb = b < n_full ? G.D.k_many : G.D.k_few;
    G.col0 = b * G.D.k_many;
    return G;
}

// The step of one block, cut into stages.  The register arrays are members; the stages say
// which of them they fill and which they consume.
//   FULL: the block has exactly kRound*C elements, so no chunk needs a bounds check.
//   QL:   lanes per quantisation block fixed at compile time (4: q = 32, 8: q = 64), 0: any.
template <class R, bool FULL, int QL, int AUX = 0>
struct FusedBlock {
    typedef typename R::elem_t elem_t;
    static constexpr int C = R::kC;
    static constexpr bool LOG = (AUX & kAuxLog) != 0, QE = (AUX & kAuxQuantErr) != 0;

    // ---- the sums of a logging step: per thread, then per workgroup in log_flush
    float mt[LOG ? 6 : 1];

    __device__ __forceinline__ void log_square(int which, float v) {
        if constexpr (LOG) {
            const float sq = v * v;
            mt[which] = mt[which] + sq;
        }
    }
    __device__ __forceinline__ void log_zero(int which, float v) {
        if constexpr (LOG) mt[which] = mt[which] + (v == 0.0f ? 1.0f : 0.0f);
    }
    // the update of 8 coordinates of which the first `valid` belong to the block
    __device__ __forceinline__ void log_update(const float (&uv)[8], int valid) {
        if constexpr (LOG) {
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                if (e < valid) {
                    log_square(kMtUpdate, uv[e]);
                    log_zero(kMtUpdateZeros, uv[e]);
                }
            }
        }
    }

    // the error feedback just formed: codes (as floats) of 8 elements against (mn, u)
    __device__ __forceinline__ void log_error(const float (&cf)[8], float mnf, float u, int valid) {
        if constexpr (LOG) {
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                float deq = cf[e] * u;
                deq = deq + mnf;
                if (e < valid) log_square(kMtError, to_elem(0.0f + deq));
            }
        }
    }

    // The workgroup's sums of the components in `mask` go to the block's slot (the other
    // components belong to another pass over the same blocks): lanes, then waves, in a fixed
    // order.  Every thread calls it, at the end of the kernel.
    __device__ __forceinline__ void log_flush(int item, unsigned mask) {
        if constexpr (LOG) {
            __syncthreads();  // the kSh* words are free from here on
            float *part = reinterpret_cast<float *>(sh);
#pragma unroll
            for (int j = 0; j < 6; ++j) {
                float v = mt[j];
#pragma unroll
                for (int o = 32; o >= 1; o >>= 1) v = v + __shfl_xor(v, o, kWave);
                if (lane == 0) part[wave * 6 + j] = v;
            }
            __syncthreads();
            if (tid < kMetricSlots && ((mask >> tid) & 1u)) {
                float v = 0.0f;
                if (tid < 6)
                    for (int w = 0; w < kWG / kWave; ++w) v = v + part[w * 6 + tid];
                P.metrics[(int64_t)item * kMetricSlots + tid] = v;
            }
        }
    }

    const FusedParams &P;
    uint32_t *sh, *counter, *hist;
    uint16_t *sel_idx, *sel_val, *coord;
    // One LDS cell per coordinate of the block.  16 bits wide for bf16 data (window bookkeeping,
    // then the update's bf16 bits) and in the one-pass window stage for fp32 data (bookkeeping,
    // then 1 + the record that holds the update); 32 bits (the update's bits) for fp32 data in
    // the general window stage.
    uint16_t *cell16;
    uint32_t *cell32;
    float *z1, *z2;
    int tid, lane, wave, q_shift, ql;
    bool slot_clear;  // the slot cells are already zero when the update stage begins
    bool row_in_lds;  // the window row of this step is taken from sel_idx / sel_val, not from HBM
    Divisor d15;

    RawChunk<R> praw[C];          // parameters              load_params_window -> update
    uint32_t entI[kEnt];          // entries of the older window rows, kept as loaded so that
    uint32_t entV[kEnt];          // nothing waits for them    load_params_window -> update
    RawChunk<R> graw[C];          // gradient                load_grad_inputs   -> dequant
    // 4-bit codes and statistics                            load_grad_inputs   -> dequant
    // With a full block and a compile-time quantisation group the wave's statistics are
    // fetched once, 64 per register (kCoStats registers per array), and handed to the lanes
    // by cross-lane reads in dequant; otherwise every chunk loads its own pair.
    static constexpr bool kCoop = FULL && QL > 0;
    static constexpr int kWaveStats = kCoop ? C * kWave / (QL > 0 ? QL : 1) : 0;
    static constexpr int kCoStats = kCoop ? (kWaveStats + kWave - 1) / kWave : 1;
    uint32_t cw[C], smn[kCoop ? kCoStats : C], smx[kCoop ? kCoStats : C];
    R r;                          // accumulator             dequant            -> quantize

    __device__ __forceinline__ FusedBlock(const FusedParams &P_, unsigned char *lds) : P(P_) {
        sh = reinterpret_cast<uint32_t *>(lds);
        counter = sh + kShCounter;
        sel_idx = reinterpret_cast<uint16_t *>(lds + P.L.off_sel_idx);
        sel_val = reinterpret_cast<uint16_t *>(lds + P.L.off_sel_val);
        cell16 = reinterpret_cast<uint16_t *>(lds + P.L.off_slot);
        cell32 = reinterpret_cast<uint32_t *>(lds + P.L.off_slot);
        hist = reinterpret_cast<uint32_t *>(lds + P.L.off_union);
        // without cells the sums of a coordinate range take everything from the cells' place on
        z1 = reinterpret_cast<float *>(lds + (P.L.cell_bytes == 0 ? P.L.off_slot : P.L.off_union));
        z2 = z1 + P.L.z_cap;
        coord = reinterpret_cast<uint16_t *>(z2 + P.L.z_cap);
        tid = threadIdx.x;
        lane = tid & 63;
        wave = tid >> 6;
        q_shift = QL > 0 ? (QL == 4 ? 5 : 6) : P.q_shift;
        ql = 1 << (q_shift - 3);
        // 1/15 rounded to nearest; div_shared is exact for a reciprocal within one ulp
        d15.u = 15.0f;
        d15.r = 0x1.111112p-4f;
        slot_clear = false;
        row_in_lds = true;
        wide = false;
        if constexpr (LOG) {
#pragma unroll
            for (int j = 0; j < 6; ++j) mt[j] = 0.0f;
        }
    }

    __device__ __forceinline__ bool fast_window(const BlockGeo &G) const {
        return P.W.rows * G.kb <= P.L.fast_cap && P.W.rows <= kFastRows && P.L.sub_len >= G.n;
    }

    // ---- parameters and the older window rows: requested early, consumed last
    __device__ __forceinline__ void load_params_window(const BlockGeo &G) {
        load_params(G);
        wide = wide_window(G);
        if (wide)
            load_window_wide(G);
        else
            load_window(G);
    }

    __device__ __forceinline__ void load_params(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const elem_t *p = reinterpret_cast<const elem_t *>(G.D.p) + G.e0;
#pragma unroll
        for (int c = 0; c < C; ++c) praw[c].load(p, chunk_off<C>(wave, c, lane), n, FULL);
    }

    __device__ __forceinline__ void load_window(const BlockGeo &G) {
        const bool fw = fast_window(G);
        const int entries = fw ? P.W.rows * G.kb : 0;
        const float rkb = __builtin_amdgcn_rcpf((float)G.kb);
#pragma unroll
        for (int i = 0; i < kEnt; ++i) {
            entI[i] = entV[i] = 0;
            if (__builtin_amdgcn_readfirstlane(wave) * kWave + i * kWG < entries) {
                const int e = tid + i * kWG;
                const int row = entry_row(e, rkb);
                if (e < entries && (row != G.D.row || !row_in_lds)) {
                    const int64_t at = (int64_t)row * G.D.k + G.col0 + (e - row * G.kb);
                    entI[i] = reinterpret_cast<const uint16_t *>(G.D.I)[at];
                    entV[i] = G.D.V[at];
                }
            }
        }
    }

    // row of window entry e when a row has 1 / rkb entries: (e + 0.5) / kb is at least 0.5 / kb
    // away from an integer, far more than the rounding of the two operations
    static __device__ __forceinline__ int entry_row(int e, float rkb) {
        return (int)(((float)e + 0.5f) * rkb);
    }

    // ---- a lower bound for this step's selection threshold: the magnitudes of the entries the
    //      previous step took from this block (hint_topk_bf16 tries the smallest, lowered a little)
    uint32_t hint;

    __device__ __forceinline__ void load_hint(const BlockGeo &G) {
        hint = 0x7fffu;
        if constexpr (FULL && R::kBF16) {
            const int prev = (G.D.row == 0 ? P.W.rows_total : G.D.row) - 1;
            const uint16_t *Vp = G.D.V + ((int64_t)prev * G.D.k + G.col0);
            if (G.kb <= kWG) {
                if (tid < G.kb) hint = Vp[tid] & 0x7fffu;
            } else if (G.kb <= kHintLongRow) {
                for (int j = tid; j < G.kb; j += kWG) hint = min(hint, Vp[j] & 0x7fffu);
            }
        }
    }

    // ---- gradient, 4-bit error feedback and its statistics
    __device__ __forceinline__ void load_grad_inputs(const BlockGeo &G) {
        load_hint(G);
        const int n = FULL ? C * kRound : G.n;
        const elem_t *g = reinterpret_cast<const elem_t *>(G.D.g) + G.e0;
        const uint8_t *err = G.D.err + (G.e0 >> 1);
        const uint16_t *mnp = G.D.mn + (G.e0 >> q_shift);
        const uint16_t *mxp = G.D.mx + (G.e0 >> q_shift);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            graw[c].load(g, off, n, FULL);
            cw[c] = 0;
            if constexpr (kCoop) {
                cw[c] = *reinterpret_cast<const uint32_t *>(err + ((unsigned)off >> 1));
                continue;
            } else {
                smn[c] = smx[c] = 0;
            }
            if (FULL || off < n) {
                if (FULL || off + kChunk <= n) {
                    cw[c] = *reinterpret_cast<const uint32_t *>(err + ((unsigned)off >> 1));
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        cw[c] |= (uint32_t)err[(off >> 1) + j] << (8 * j);
                }
                const unsigned qb = (unsigned)off >> q_shift;
                smn[c] = mnp[qb];
                smx[c] = mxp[qb];
            }
        }
        if constexpr (kCoop) {
            const unsigned wave_first = (unsigned)(wave * C * kWave) / (unsigned)QL;
#pragma unroll
            for (int i = 0; i < kCoStats; ++i) {
                const unsigned j = (unsigned)(i * kWave + lane);
                smn[i] = smx[i] = 0;
                if (j < (unsigned)kWaveStats) {
                    smn[i] = mnp[wave_first + j];
                    smx[i] = mxp[wave_first + j];
                }
            }
        }
    }

    // ---- a = g + Qinv(e), rounded to the element type (MA:190)
    __device__ __forceinline__ void dequant(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        // with the wave's statistics spread over the lanes, each lane forms the step of the
        // quantisation blocks it holds once, and the chunks fetch (min, step)
        float su[kCoStats];
        if constexpr (kCoop) {
#pragma unroll
            for (int i = 0; i < kCoStats; ++i) su[i] = div15(bf2f(smx[i]) - bf2f(smn[i]), d15);
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            float v[8];
            graw[c].to_float(v);
            if constexpr (LOG) {  // (elements past the block's end were loaded as zeros)
#pragma unroll
                for (int e = 0; e < kChunk; ++e) log_square(kMtGrad, v[e]);
            }
            float mn, u;
            if constexpr (kCoop) {
                const int j0 = c * (kWave / QL);  // first statistic of this chunk in the wave
                const int src = (j0 & (kWave - 1)) + lane / QL;
                mn = bf2f((uint32_t)__shfl((int)smn[j0 >> 6], src, kWave));
                u = __int_as_float(__shfl(__float_as_int(su[j0 >> 6]), src, kWave));
            } else {
                mn = bf2f(smn[c]);
                u = div15(bf2f(smx[c]) - mn, d15);
            }
            // the nibbles as bytes of two words (even elements high), one conversion each
            uint32_t odd = cw[c] & 0x0f0f0f0fu, even = (cw[c] >> 4) & 0x0f0f0f0fu;
            // (hidden from the optimiser, which would turn the byte reads back into bit-field
            // extracts of cw, one more instruction per element)
            asm volatile("" : "+v"(odd), "+v"(even));
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                const uint32_t code = (((e & 1) ? odd : even) >> (8 * (e >> 1))) & 0xffu;
                float deq = (float)code * u;
                deq = deq + mn;
                v[e] = v[e] + deq;
            }
            if (!FULL && off + kChunk > n) {
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (off + e >= n) v[e] = 0.0f;
            }
            r.set_chunk(c, v);
            __builtin_amdgcn_sched_barrier(0);
        }
        launder(r);
    }

    // ---- block top-k (MA:193-200), gather (MA:202-209), zero (MA:214), window row write
    __device__ __forceinline__ void topk_and_row(const BlockGeo &G) {
        const int kb = G.kb;
        bool topk_done = false;
        if constexpr (FULL && R::kBF16) {
            if (kb <= kWG) {
                topk_done = hint_topk_bf16(r, kb, hint, cell16, hist, sh, sel_idx, sel_val);
                if (!topk_done)
                    topk_done = fast_topk_bf16(r, kb, cell16, hist, sh, sel_idx, sel_val);
                launder(r);
                // the block was parked in the slot cells and every thread cleared its own
                slot_clear = topk_done && P.L.slot_cells == C * kRound;
            }
        }
        row_sorted = !topk_done;  // the selections below list their entries by coordinate
        if constexpr (FULL && R::kBF16) {
            // block rows too long for the candidate lists, where the LDS plan has the cells to
            // park the block in: threshold and ordered selection from the hint
            if (kb > kWG && kb <= kHintLongRow && P.L.cell_bytes == 2 &&
                P.L.slot_cells >= C * kRound) {
                topk_done = hint_sorted_topk_bf16(r, kb, hint, cell16, hist, sh, sel_idx, sel_val);
                launder(r);
            }
        }
        if (!topk_done) {
            uint32_t T;
            int take_eq;
            bool have = false;
            if constexpr (FULL && R::kBF16) {
                // (without the cells: the hint gives the threshold at least)
                if (kb > kWG && kb <= kHintLongRow)
                    have = hint_threshold_bf16(r, kb, hint, hist, sh, T, take_eq);
            }
            if (!have) select_threshold(r, kb, hist, sh, T, take_eq, P.L.hist_log2);
            launder(r);
            compact_selected(r, T, take_eq, kb, sel_idx, sel_val, sh);
            launder(r);
        }
        int16_t *Irow = G.D.I + ((int64_t)G.D.row * G.D.k + G.col0);
        uint16_t *Vrow = G.D.V + ((int64_t)G.D.row * G.D.k + G.col0);
        for (int j = tid; j < kb; j += kWG) {
            Irow[(unsigned)j] = (int16_t)sel_idx[j];
            Vrow[(unsigned)j] = sel_val[j];
        }
    }

    // Two-launch form: where the row just written (still in sel_idx) crosses the multiples of
    // kRowCutStep coordinates goes to the tensor's cache of row cuts, if it keeps one, for
    // window_param_kernel: cut c = number of entries with coordinate < c * kRowCutStep.  A row
    // that is not listed by coordinate is marked unknown.
    bool row_sorted;
    __device__ __forceinline__ void file_row_cuts(const BlockGeo &G) {
        uint16_t *cuts = reinterpret_cast<uint16_t *>(G.D.ws);
        if (cuts == nullptr) return;
        const RowCuts where(G.D.d, P.d_block_size);
        uint16_t *mine = cuts + where.at(G.D.row, block_id(G));
        const int nch = (G.n + kRowCutStep - 1) / kRowCutStep;
        if (!row_sorted) {
            if (tid == 0) mine[0] = 0xffffu;
            return;
        }
        if (tid <= nch) {
            const int bound = tid * kRowCutStep;
            int lo = 0, hi = G.kb;  // first entry whose coordinate is not below `bound`
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if ((int)sel_idx[mid] < bound) lo = mid + 1; else hi = mid;
            }
            mine[tid] = (uint16_t)lo;
        }
    }

    // ---- residual statistics (MA:217-228) and 4-bit codes (MA:231)
    __device__ __forceinline__ void quantize(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        uint8_t *err = G.D.err + (G.e0 >> 1);
        uint16_t *mnp = G.D.mn + (G.e0 >> q_shift);
        uint16_t *mxp = G.D.mx + (G.e0 >> q_shift);
        // Quantisation blocks of 1024, 2048 or 4096 elements cover 2, 4 or 8 of the 512-element
        // stretches a wave holds per chunk: every (wave, chunk) leaves its extremes in LDS
        // (where the selection's histograms were), and each takes those of its block's stretches.
        const bool long_q = QL == 0 && ql > kWave;
        float *stretch = reinterpret_cast<float *>(hist);  // [wave * C + chunk][min, max]
        if (long_q) {
            __syncthreads();  // the selection may still be reading its lists there
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int off = chunk_off<C>(wave, c, lane);
                float mn = INFINITY, mx = -INFINITY;
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    if (FULL || off + e < n) {
                        mn = fmin_raw(mn, r.val(c, e));
                        mx = fmax_raw(mx, r.val(c, e));
                    }
                }
                group_minmax<0>(mn, mx, kWave);
                if (lane == 0) {
                    stretch[(wave * C + c) * 2] = mn;
                    stretch[(wave * C + c) * 2 + 1] = mx;
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            float x[8];
            float mn = INFINITY, mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
            if (FULL) {
                minmax8(x, mn, mx);
            } else {
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    if (off + e < n) {
                        mn = fmin_raw(mn, x[e]);
                        mx = fmax_raw(mx, x[e]);
                    }
                }
            }
            if (long_q) {
                const int per = ql / kWave;  // stretches per quantisation block
                const int first = (wave * C + c) / per * per;
                mn = INFINITY;
                mx = -INFINITY;
                for (int j = 0; j < per; ++j) {
                    mn = fmin_raw(mn, stretch[(first + j) * 2]);
                    mx = fmax_raw(mx, stretch[(first + j) * 2 + 1]);
                }
            } else {
                group_minmax<QL>(mn, mx, ql);
            }
            const uint32_t mnb = f2bf(mn), mxb = f2bf(mx);
            if (FULL || off < n) {
                if ((lane & (ql - 1)) == 0) {
                    const unsigned qb = (unsigned)off >> q_shift;
                    mnp[qb] = (uint16_t)mnb;
                    mxp[qb] = (uint16_t)mxb;
                }
                const float mnf = bf2f(mnb), mxf = bf2f(mxb);
                const float u = div15(mxf - mnf, d15);
                float cf[8];
                codes8(x, mnf, u, cf);
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (!FULL && off + e >= n) cf[e] = 0.0f;
                const uint32_t codes = pack_codes(cf);
                if (FULL || off + kChunk <= n) {
                    *reinterpret_cast<uint32_t *>(err + ((unsigned)off >> 1)) = codes;
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        err[(off >> 1) + j] = (uint8_t)(codes >> (8 * j));
                }
                if constexpr (LOG || QE) quant_err_chunk(G, c, off, n, x, cf, mnf, u);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // What the new error feedback stands for, d = Qinv(e) as a cleared buffer of the
    // gradient's type receives it (MA:267-268, :321-322): its squares for a logging step, and
    // with alpha == -2 the parameter steps p = p * decay (MA:234-235), p = p - a (MA:264),
    // p = p + d (MA:269) on the parameters held in praw, and quant_err = a - d (MA:259-270).
    __device__ __forceinline__ void quant_err_chunk(const BlockGeo &G, int c, int off, int n,
                                                    const float (&x)[8], const float (&cf)[8],
                                                    float mnf, float u) {
        float pv[8], lost[8];
        if constexpr (QE) praw[c].to_float(pv);
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            float deq = cf[e] * u;
            deq = deq + mnf;
            const float d = to_elem(0.0f + deq);
            const bool valid = FULL || off + e < n;
            if (valid) log_square(kMtError, d);
            lost[e] = 0.0f;
            if constexpr (QE) {
                if (G.D.apply_decay != 0) pv[e] = to_elem(pv[e] * G.D.decay);
                pv[e] = to_elem(pv[e] + (-1.0f) * x[e]);
                pv[e] = to_elem(pv[e] + d);
                if (valid) {
                    lost[e] = to_elem(x[e] - d);
                    log_square(kMtQuantErr, lost[e]);
                    log_zero(kMtQuantErrZeros, lost[e]);
                }
            }
        }
        if constexpr (QE) {
            praw[c].from_float(pv);
            // st['quant_err'] = a - Qinv(e) (MA:259-271)
            store8(reinterpret_cast<elem_t *>(G.D.ws) + G.e0, off, FULL ? 0x7fffffff : n, true,
                   lost);
        }
    }

    // the weight decay of the update stages: with alpha == -2 it has been applied already
    __device__ __forceinline__ bool decay_pending(const BlockGeo &G) const {
        return !QE && G.D.apply_decay != 0;
    }

    // ---- Adam direction from the window (MA:277-291), then p = p * (1 - lr*wd) (MA:234-235)
    //      and p += -lr * u (MA:304).  The slot cells end up holding the update's bits, 0
    //      where no window row names the coordinate.
    __device__ __forceinline__ void update(const BlockGeo &G) {
        if (P.L.cell_bytes == 0) {
            update_by_ranges(G);
        } else if (wide) {
            update_wide(G);
        } else {
            window_stage(G);
            param_stage(G);
        }
    }

    // =========================================================================================
    // Window and parameter stage of a full bf16 block whose window fits one pass (the usual
    // case: m = 10 rows of 1 %).  Against window_stage + param_stage:
    //  * the older rows are fetched four entries per 8-byte load: thread t takes the entries
    //    4w - a .. 4w - a + 3 of older row t / W (w = t % W, W loads per row, a = 1 if the
    //    block's stretch of that row starts on an odd entry, so that every load is 4-byte
    //    aligned), and entry t of the row this step selected, which is still in LDS;
    //  * coordinates named by several rows are summed through lists: the entry of the lowest
    //    row reserves one cell per row of the coordinate, every entry files its two terms at
    //    its row's rank, the owner adds them in that order (the order of the rows, as in
    //    compute_microadam_update): four barriers, no loop over rows;
    //  * without weight decay only the coordinates the window names change, so the
    //    parameters are parked in the coordinate cells, the owners of the updates change
    //    their cells, and the block goes back to memory as it lies there: a few dozen
    //    vector instructions instead of four per element.
    // =========================================================================================
    bool wide;                  // this block takes the stage below
    uint32_t wI[2], wV[2];      // four entries of an older row: indices, values (bf16 bits)
    int w_first, w_row;         // number of the first of the four in the block's stretch of
                                // the row (-1 .. kb-1); the row, -1: none

    __device__ __forceinline__ bool wide_window(const BlockGeo &G) const {
        if constexpr (!(R::kBF16 && FULL) || LOG) {
            return false;  // (a logging step needs the update of every coordinate)
        } else {
            if (!P.L.compact || !row_in_lds || !fast_window(G)) return false;
            if ((((uintptr_t)G.D.I | (uintptr_t)G.D.V) & 3) != 0) return false;
            const int W = G.kb / 4 + 1;
            return older_rows(G) * W <= kWG && G.kb <= kWG && P.W.rows <= 15;
        }
    }

    // live rows that come from memory: all but the row this step writes (which is live unless
    // the caller's ring position and step count disagree; it is then written and not read)
    __device__ __forceinline__ int older_rows(const BlockGeo &G) const {
        return P.W.rows - (G.D.row < P.W.rows ? 1 : 0);
    }

    __device__ __forceinline__ void load_window_wide(const BlockGeo &G) {
        struct __attribute__((aligned(4))) Pair32 {
            uint32_t x, y;
        };
        const int W = G.kb / 4 + 1;
        const int older = older_rows(G);
        const int ro = (int)(((float)tid + 0.5f) * __builtin_amdgcn_rcpf((float)W));
        const int w = tid - ro * W;
        w_row = -1;
        w_first = 0;
        wI[0] = wI[1] = wV[0] = wV[1] = 0;
        if (ro < older) {
            const int row = (ro < G.D.row || G.D.row >= P.W.rows) ? ro : ro + 1;
            const int64_t e_first = (int64_t)row * G.D.k + G.col0;
            const int a = (int)(e_first & 1);
            const int64_t e_base = e_first - a + 4 * w;
            w_first = 4 * w - a;
            w_row = row;
            const uint16_t *Ip = reinterpret_cast<const uint16_t *>(G.D.I) + e_base;
            const uint16_t *Vp = G.D.V + e_base;
            if (e_base + 4 <= (int64_t)P.W.rows_total * G.D.k) {
                const Pair32 qi = *reinterpret_cast<const Pair32 *>(Ip);
                const Pair32 qv = *reinterpret_cast<const Pair32 *>(Vp);
                wI[0] = qi.x; wI[1] = qi.y; wV[0] = qv.x; wV[1] = qv.y;
            } else {  // the last load of the last row may not reach past the arrays
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (e_base + j < (int64_t)P.W.rows_total * G.D.k) {
                        wI[j >> 1] |= (uint32_t)Ip[j] << (16 * (j & 1));
                        wV[j >> 1] |= (uint32_t)Vp[j] << (16 * (j & 1));
                    }
                }
            }
        }
    }

    __device__ __forceinline__ void update_wide(const BlockGeo &G) {
        if constexpr (R::kBF16 && FULL) update_wide_bf16<false>(G);
    }

    // The window stage alone: the slot cells end up holding the update's bits (0 where no
    // window row names the coordinate), for a parameter stage of the caller's.  Ends with a
    // barrier.
    __device__ __forceinline__ void window_cells(const BlockGeo &G) {
        if constexpr (R::kBF16 && FULL) {
            if (wide) {
                update_wide_bf16<true>(G);
                return;
            }
        }
        window_stage(G);
    }

    // CELLS_ONLY: stop once the cells hold the updates (window_cells)
    template <bool CELLS_ONLY>
    __device__ __forceinline__ void update_wide_bf16(const BlockGeo &G) {
        constexpr int n = C * kRound;
        constexpr int kSlots = 5;  // four entries of an older row, one of this step's row
        const TensorDesc &D = G.D;
        const int kb = G.kb;
        // entries of coordinates that several rows name wait in a queue: key, two terms and a
        // link cell each, at most one per thread
        uint32_t *lcount = sh + kShLinks, *qcount = sh + kShCounter;
        constexpr int kQueue = kWG;
        uint32_t *qkey = hist;
        float *qa1 = reinterpret_cast<float *>(hist + kQueue), *qa2 = qa1 + kQueue;
        uint16_t *link = reinterpret_cast<uint16_t *>(qa2 + kQueue);
        const bool queue_fits = P.L.total - P.L.off_union >= kQueue * 14;
        if (!slot_clear) {
            __syncthreads();  // the LDS of the selection is reused below
            for (int i = tid; i < n / 8; i += kWG)
                reinterpret_cast<uint4 *>(cell16)[i] = make_uint4(0, 0, 0, 0);
        }
        if (tid < kFastRows) {
            sh[kShW1 + tid] = __float_as_uint(P.W.w1[tid]);
            sh[kShW2 + tid] = __float_as_uint(P.W.w2[tid]);
        }
        if (tid == 0) *lcount = *qcount = 0;
        __syncthreads();
        // ---- every entry marks its row in the cell of its coordinate
        uint32_t tag[kSlots];  // index | value << 16; all ones: no entry
        int myrow[kSlots];
#pragma unroll
        for (int j = 0; j < kSlots; ++j) {
            uint32_t idx, vb;
            bool have;
            if (j < 4) {
                idx = (wI[j >> 1] >> (16 * (j & 1))) & 0xffffu;
                vb = (wV[j >> 1] >> (16 * (j & 1))) & 0xffffu;
                have = w_row >= 0 && (unsigned)(w_first + j) < (unsigned)kb;
                myrow[j] = w_row;
            } else {
                have = tid < kb && D.row < P.W.rows;
                idx = have ? sel_idx[tid] : 0u;
                vb = have ? sel_val[tid] : 0u;
                myrow[j] = D.row;
            }
            // +-0 values add nothing and are skipped; idx < n keeps a corrupt index inside
            have = have && idx < (uint32_t)n && (vb & 0x7fffu) != 0;
            tag[j] = have ? (idx | vb << 16) : 0xffffffffu;
            if (have) atomicOr(cell32 + (idx >> 1), (1u << myrow[j]) << ((idx & 1u) * 16));
        }
        __syncthreads();
        // ---- a coordinate named by one row has its sums from that entry; the entries of the
        //      others queue up with their rank among the coordinate's rows
        const float w1_old = w_row >= 0 ? __uint_as_float(sh[kShW1 + w_row]) : 0.0f;
        const float w2_old = w_row >= 0 ? __uint_as_float(sh[kShW2 + w_row]) : 0.0f;
        const float w1_cur = __uint_as_float(sh[kShW1 + D.row]);
        const float w2_cur = __uint_as_float(sh[kShW2 + D.row]);
        constexpr int kOwned = kSlots + 1;  // the last: a queued coordinate this thread sums
        float z1[kOwned], z2[kOwned];       // sums of the coordinates this thread updates
        uint32_t own[kOwned];               // their indices; all ones: none
#pragma unroll
        for (int j = 0; j < kSlots; ++j) {
            own[j] = 0xffffffffu;
            z1[j] = z2[j] = 0.0f;
            if (tag[j] != 0xffffffffu) {
                const uint32_t idx = tag[j] & 0xffffu, row = (uint32_t)myrow[j];
                const uint32_t mask = cell16[idx];
                const float v = bf2f(tag[j] >> 16);
                const float vv = v * v;
                const float a1 = (j < 4 ? w1_old : w1_cur) * v;
                const float a2 = (j < 4 ? w2_old : w2_cur) * vv;
                if (mask == 1u << row) {
                    z1[j] = 0.0f + a1;
                    z2[j] = 0.0f + a2;
                    own[j] = idx;
                } else {
                    const uint32_t at = atomicAdd(qcount, 1u);
                    if (at < (uint32_t)kQueue) {
                        const uint32_t rank = (uint32_t)__popc(mask & ((1u << row) - 1u));
                        qkey[at] = idx | rank << 15 | (uint32_t)__popc(mask) << 19;
                        qa1[at] = a1;
                        qa2[at] = a2;
                    }
                }
            }
        }
        own[kSlots] = 0xffffffffu;
        z1[kSlots] = z2[kSlots] = 0.0f;
        __syncthreads();
        const uint32_t queued = *qcount;
        if (queued > (uint32_t)kQueue || !queue_fits) {
            // more entries share coordinates than the queue holds: the general stage, which
            // takes its entries in its own order and serves shared coordinates row by row
            slot_clear = false;
            load_window(G);
            window_stage(G);
            if (!CELLS_ONLY) param_stage(G);
            return;
        }
        if (queued != 0) {
            // queued entry t belongs to thread t.  The lowest row of a coordinate reserves one
            // link cell per row and leaves the first cell's number in the coordinate's cell
            // (the marks are not needed any more); every entry files its queue position at its
            // rank; the lowest row adds the terms in that order, the order of the rows.
            uint32_t key = 0;
            const bool mine = (uint32_t)tid < queued;
            if (mine) {
                key = qkey[tid];
                if (((key >> 15) & 15u) == 0)
                    cell16[key & 0x7fffu] = (uint16_t)atomicAdd(lcount, key >> 19);
            }
            __syncthreads();
            uint32_t base = 0;
            if (mine) {
                base = cell16[key & 0x7fffu];  // the cells are not read again after this
                uint32_t at = base + ((key >> 15) & 15u);
                at = at < (uint32_t)kQueue ? at : (uint32_t)kQueue - 1u;
                link[at] = (uint16_t)tid;
            }
            __syncthreads();
            if (mine && ((key >> 15) & 15u) == 0) {
                const int terms = (int)(key >> 19);
                float s1 = 0.0f, s2 = 0.0f;
                for (int r = 0; r < terms; ++r) {
                    uint32_t at = base + (uint32_t)r;
                    at = at < (uint32_t)kQueue ? at : (uint32_t)kQueue - 1u;
                    uint32_t q = link[at];
                    q = q < (uint32_t)kQueue ? q : (uint32_t)kQueue - 1u;
                    s1 = s1 + qa1[q];
                    s2 = s2 + qa2[q];
                }
                z1[kSlots] = s1;
                z2[kSlots] = s2;
                own[kSlots] = key & 0x7fffu;
            }
        }
        uint32_t upd[kOwned];  // index | update's bf16 bits << 16; all ones: none
#pragma unroll
        for (int j = 0; j < kOwned; ++j) {
            upd[j] = 0xffffffffu;
            if (own[j] != 0xffffffffu) {
                const float u = adam_update<R::kBF16>(z1[j], z2[j], P.W.s1, P.W.s2, P.W.eps);
                upd[j] = own[j] | f2bf(u) << 16;
            }
        }
        // nobody reads the cells' marks any more: the last readers passed a barrier above
        const float neg_lr = D.neg_lr;
        if (CELLS_ONLY || decay_pending(G)) {
            // every parameter changes: the updates go to the cells, the dense stage does the rest
#pragma unroll
            for (int j = 0; j < kOwned; ++j)
                if (upd[j] != 0xffffffffu) cell16[upd[j] & 0xffffu] = (uint16_t)(upd[j] >> 16);
            __syncthreads();
            if (!CELLS_ONLY) param_stage(G);
            return;
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
            *reinterpret_cast<uint4 *>(cell16 + chunk_off<C>(wave, c, lane)) = praw[c].q;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kOwned; ++j) {
            if (upd[j] != 0xffffffffu) {
                const uint32_t idx = upd[j] & 0xffffu;
                const float prod = neg_lr * bf2f(upd[j] >> 16);
                cell16[idx] = (uint16_t)f2bf(bf2f(cell16[idx]) + prod);
            }
        }
        __syncthreads();
        elem_t *p = reinterpret_cast<elem_t *>(D.p) + G.e0;
        const int tid2 = opaque_tid(), lane2 = tid2 & 63, wave2 = tid2 >> 6;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave2, c, lane2);
            const uint4 q = *reinterpret_cast<const uint4 *>(cell16 + off);
            typedef uint32_t u4 __attribute__((ext_vector_type(4)));
            const u4 t = {q.x, q.y, q.z, q.w};
            __builtin_nontemporal_store(t, reinterpret_cast<u4 *>(p + off));
        }
    }

    // General window stage without coordinate cells: for each coordinate range (a multiple of
    // 512, so a chunk lies inside one range) the sums, then the Adam direction in place of
    // z1, then the parameter update of the chunks in the range.
    __device__ __forceinline__ void update_by_ranges(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const TensorDesc &D = G.D;
        elem_t *p = reinterpret_cast<elem_t *>(D.p) + G.e0;
        const float neg_lr = D.neg_lr, decay = D.decay;
        const bool apply_decay = decay_pending(G);
        WindowView wv;
        wv.I = D.I + G.col0;
        wv.V = D.V + G.col0;
        wv.k = D.k;
        wv.rows = P.W.rows;
        wv.cur_row = row_in_lds ? D.row : -1;
        wv.cur_idx = sel_idx;
        wv.cur_val = sel_val;
        wv.w1 = P.W.w1;
        wv.w2 = P.W.w2;
        __syncthreads();  // the LDS of the selection is reused below
        for (int lo = 0; lo < n; lo += P.L.sub_len) {
            const int hi = lo + P.L.sub_len < n ? lo + P.L.sub_len : n;
            window_accumulate(wv, G.kb, lo, hi, z1, z2);
            for (int c = tid; c < hi - lo; c += kWG) {
                float u = 0.0f;
                if (z1[c] != 0.0f || z2[c] != 0.0f)
                    u = adam_update<R::kBF16>(z1[c], z2[c], P.W.s1, P.W.s2, P.W.eps);
                z1[c] = R::kBF16 ? bf2f(f2bf(u)) : u;
            }
            __syncthreads();
            // store addresses formed afresh, as in param_stage
            const int tid2 = opaque_tid(), lane2 = tid2 & 63, wave2 = tid2 >> 6;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int off = chunk_off<C>(wave2, c, lane2);
                if (off >= lo && off < hi && (FULL || off < n)) {
                    float pv[8];
                    praw[c].to_float(pv);
#pragma unroll
                    for (int e = 0; e < kChunk; ++e) {
                        // the range may end inside the chunk only at the end of the block
                        const float u = (FULL || off + e < n) ? z1[off - lo + e] : 0.0f;
                        if (apply_decay) pv[e] = to_elem(pv[e] * decay);
                        const float prod = neg_lr * u;
                        pv[e] = pv[e] + prod;
                        if (FULL || off + e < n) {
                            log_square(kMtUpdate, u);
                            log_zero(kMtUpdateZeros, u);
                        }
                    }
                    store8(p, off, FULL ? 0x7fffffff : n, true, pv);
                }
            }
            __syncthreads();
        }
    }

    // The slot cells end up holding the update's bits, 0 where no window row names the
    // coordinate.  Ends with a barrier.
    __device__ __forceinline__ void window_stage(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const int kb = G.kb;
        const int rows = P.W.rows;
        const TensorDesc &D = G.D;
        if (!slot_clear) {
            __syncthreads();  // the LDS of the selection is reused below
            for (int i = tid; i < P.L.slot_cells * P.L.cell_bytes / 16; i += kWG)
                reinterpret_cast<uint4 *>(cell16)[i] = make_uint4(0, 0, 0, 0);
        }
        if (fast_window(G)) {
            // Every entry of the window is handled once, kEnt per thread.  The rows that name
            // a coordinate are first gathered as a bit mask in its slot cell.  A coordinate
            // named by one row gets its update from that entry alone.  The entries of the
            // others go to a list; the entry of the lowest row owns the coordinate, hands out
            // one link cell per later row, the later rows file their list position there by
            // rank, and the owner adds them up in that order, which is the order of the rows.
            uint32_t *mcount = sh + kShCounter, *lcount = sh + kShLinks, *scount = sh + kShTies;
            float *f1 = z1, *f2 = z2;
            const int cap = P.L.z_cap;
            uint16_t *mI = coord, *mR = mI + cap, *mM = mR + cap, *link = mM + cap;
            if (tid < kFastRows) {
                sh[kShW1 + tid] = __float_as_uint(P.W.w1[tid]);
                sh[kShW2 + tid] = __float_as_uint(P.W.w2[tid]);
            }
            if (tid == 0) *mcount = *lcount = *scount = 0;
            const int wave_first = __builtin_amdgcn_readfirstlane(wave) * kWave;
            const int entries = rows * kb;
            const float rkb = __builtin_amdgcn_rcpf((float)kb);
            __syncthreads();
#pragma unroll
            for (int i = 0; i < kEnt; ++i) {
                uint32_t tag = 0xffffffffu;  // index | row << 16, all ones: nothing to add
                if (wave_first + i * kWG < entries) {
                    const int e = tid + i * kWG;
                    const int row = entry_row(e, rkb);
                    if (e < entries) {
                        uint32_t idx = entI[i], vb = entV[i];
                        if (row == D.row && row_in_lds) {
                            idx = sel_idx[e - row * kb];
                            vb = sel_val[e - row * kb];
                            entV[i] = vb;
                        }
                        // +-0 values add nothing and are skipped (the rows of a fresh window
                        // are all (index 0, value 0)); idx < n keeps a corrupt index inside
                        if (idx < (uint32_t)n && (vb & 0x7fffu) != 0) {
                            tag = idx | (uint32_t)row << 16;
                            atomicOr(cell32 + (idx >> 1), (1u << row) << ((idx & 1u) * 16));
                        }
                    }
                }
                entI[i] = tag;
            }
            __syncthreads();
            if (R::kBF16 && P.L.compact) {
                // Slots instead of lists.  A coordinate named by one row gets its update from
                // that entry.  The others are served row by row, rows separated by barriers:
                // the first row to come (the lowest) takes a slot for the coordinate and marks
                // the cell with bit 15 and the slot, later rows add into the slot's sums, so
                // these are formed in row order.  At most half as many slots as entries.
                float *s1 = z1, *s2 = z2;
                uint16_t *scoord = coord;
                uint32_t multi = 0;  // bit i: entry i shares its coordinate
#pragma unroll
                for (int i = 0; i < kEnt; ++i) {
                    const uint32_t tag = entI[i];
                    if (tag != 0xffffffffu) {
                        const uint32_t idx = tag & 0xffffu, row = tag >> 16;
                        // a cell that a lower row has already marked is not a single either
                        if (cell16[idx] == 1u << row) {
                            const float v = bf2f(entV[i]);
                            const float a1 = __uint_as_float(sh[kShW1 + row]) * v;
                            const float vv = v * v;
                            const float a2 = __uint_as_float(sh[kShW2 + row]) * vv;
                            const float u =
                                adam_update<R::kBF16>(0.0f + a1, 0.0f + a2, P.W.s1, P.W.s2, P.W.eps);
                            cell16[idx] = (uint16_t)f2bf(u);
                        } else {
                            multi |= 1u << i;
                        }
                    }
                }
                for (int r = 0; r < rows; ++r) {
#pragma unroll
                    for (int i = 0; i < kEnt; ++i) {
                        const uint32_t tag = entI[i];
                        if (((multi >> i) & 1u) != 0 && (tag >> 16) == (uint32_t)r) {
                            const uint32_t idx = tag & 0xffffu;
                            const float v = bf2f(entV[i]);
                            const float a1 = __uint_as_float(sh[kShW1 + r]) * v;
                            const float vv = v * v;
                            const float a2 = __uint_as_float(sh[kShW2 + r]) * vv;
                            const uint32_t c = cell16[idx];
                            if ((c & 0x8000u) == 0) {
                                const uint32_t slot = atomicAdd(mcount, 1u);
                                if (slot < (uint32_t)cap) {
                                    cell16[idx] = (uint16_t)(0x8000u | slot);
                                    s1[slot] = 0.0f + a1;
                                    s2[slot] = 0.0f + a2;
                                    scoord[slot] = (uint16_t)idx;
                                }
                            } else {
                                const uint32_t slot = c & 0x7fffu;
                                s1[slot] = s1[slot] + a1;
                                s2[slot] = s2[slot] + a2;
                            }
                        }
                    }
                    __syncthreads();
                }
                const int used = (int)(*mcount < (uint32_t)cap ? *mcount : (uint32_t)cap);
                for (int sl = tid; sl < used; sl += kWG) {
                    const float u = adam_update<R::kBF16>(s1[sl], s2[sl], P.W.s1, P.W.s2, P.W.eps);
                    cell16[scoord[sl]] = (uint16_t)f2bf(u);
                }
                __syncthreads();
                return;
            }
#pragma unroll
            for (int i = 0; i < kEnt; ++i) {
                const uint32_t tag = entI[i];
                if (tag != 0xffffffffu) {
                    const uint32_t idx = tag & 0xffffu, row = tag >> 16;
                    const uint32_t mask = cell16[idx];
                    const float v = bf2f(entV[i]);
                    const float a1 = __uint_as_float(sh[kShW1 + row]) * v;
                    const float vv = v * v;
                    const float a2 = __uint_as_float(sh[kShW2 + row]) * vv;
                    if (mask == 1u << row) {
                        const float u =
                            adam_update<R::kBF16>(0.0f + a1, 0.0f + a2, P.W.s1, P.W.s2, P.W.eps);
                        if (R::kBF16) {
                            cell16[idx] = (uint16_t)f2bf(u);
                        } else {  // fp32: the update keeps its bits in a record of its own,
                                  // handed out from the top of the list arrays
                            const uint32_t s = (uint32_t)cap - 1u - atomicAdd(scount, 1u);
                            f1[s] = u;
                            cell16[idx] = (uint16_t)(s + 1u);
                        }
                    } else {
                        const uint32_t s = atomicAdd(mcount, 1u);
                        f1[s] = a1;
                        f2[s] = a2;
                        mI[s] = (uint16_t)idx;
                        mR[s] = (uint16_t)row;
                        mM[s] = (uint16_t)mask;
                    }
                }
            }
            __syncthreads();
            const int listed = (int)(*mcount < (uint32_t)cap ? *mcount : (uint32_t)cap);
            for (int s = tid; s < listed; s += kWG) {
                const uint32_t mask = mM[s], below = mask & ((1u << mR[s]) - 1u);
                if (below == 0)
                    cell16[mI[s]] = (uint16_t)atomicAdd(lcount, (uint32_t)__popc(mask) - 1u);
            }
            __syncthreads();
            for (int s = tid; s < listed; s += kWG) {
                const uint32_t mask = mM[s], below = mask & ((1u << mR[s]) - 1u);
                if (below != 0) {
                    const uint32_t at = (uint32_t)cell16[mI[s]] + (uint32_t)__popc(below) - 1u;
                    if (at < (uint32_t)cap) link[at] = (uint16_t)s;
                }
            }
            __syncthreads();
            for (int s = tid; s < listed; s += kWG) {
                const uint32_t mask = mM[s], below = mask & ((1u << mR[s]) - 1u);
                if (below == 0) {
                    const uint32_t idx = mI[s], base = cell16[idx];
                    float s1 = 0.0f + f1[s], s2 = 0.0f + f2[s];
                    const int later = __popc(mask) - 1;
                    for (int r = 0; r < later; ++r) {
                        // a valid window keeps base + r and the link inside the list
                        uint32_t at = base + (uint32_t)r;
                        at = at < (uint32_t)cap ? at : (uint32_t)cap - 1u;
                        uint32_t o = link[at];
                        o = o < (uint32_t)cap ? o : (uint32_t)cap - 1u;
                        s1 = s1 + f1[o];
                        s2 = s2 + f2[o];
                    }
                    const float u = adam_update<R::kBF16>(s1, s2, P.W.s1, P.W.s2, P.W.eps);
                    if (R::kBF16) {
                        cell16[idx] = (uint16_t)f2bf(u);
                    } else {  // the owner's record has given its sums and takes the update
                        f1[s] = u;
                        cell16[idx] = (uint16_t)(s + 1);
                    }
                }
            }
            __syncthreads();
        } else {
            WindowView wv;
            wv.I = D.I + G.col0;
            wv.V = D.V + G.col0;
            wv.k = D.k;
            wv.rows = rows;
            wv.cur_row = row_in_lds ? D.row : -1;
            wv.cur_idx = sel_idx;
            wv.cur_val = sel_val;
            wv.w1 = P.W.w1;
            wv.w2 = P.W.w2;
            for (int lo = 0; lo < n; lo += P.L.sub_len) {
                const int hi = lo + P.L.sub_len < n ? lo + P.L.sub_len : n;
                window_accumulate(wv, kb, lo, hi, z1, z2);
                for (int c = tid; c < hi - lo; c += kWG) {
                    if (z1[c] != 0.0f || z2[c] != 0.0f) {
                        const float u = adam_update<R::kBF16>(z1[c], z2[c], P.W.s1, P.W.s2, P.W.eps);
                        if (R::kBF16) cell16[lo + c] = (uint16_t)f2bf(u);
                        else cell32[lo + c] = __float_as_uint(u);
                    }
                }
                __syncthreads();
            }
        }
    }

    // the Adam direction of the 8 coordinates at `off`, as the window stage left it in the cells
    __device__ __forceinline__ void update8(int off, float (&uv)[8]) const {
        if (R::kBF16 || P.L.cell_bytes == 2) {
            const uint4 q = *reinterpret_cast<const uint4 *>(cell16 + off);
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
            if (R::kBF16) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uv[2 * i] = __uint_as_float(w[i] << 16);
                    uv[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
                }
            } else {
                const float *rec = z1;  // record s holds the update of the coordinate with cell s + 1
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t c = (i & 1) ? (w[i >> 1] >> 16) : (w[i >> 1] & 0xffffu);
                    uv[i] = 0.0f;
                    if (c != 0) uv[i] = rec[c - 1];
                }
            }
        } else {
            const uint4 a = *reinterpret_cast<const uint4 *>(cell32 + off);
            const uint4 b2 = *reinterpret_cast<const uint4 *>(cell32 + off + 4);
            uv[0] = __uint_as_float(a.x); uv[1] = __uint_as_float(a.y);
            uv[2] = __uint_as_float(a.z); uv[3] = __uint_as_float(a.w);
            uv[4] = __uint_as_float(b2.x); uv[5] = __uint_as_float(b2.y);
            uv[6] = __uint_as_float(b2.z); uv[7] = __uint_as_float(b2.w);
        }
    }

    __device__ __forceinline__ void param_stage(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const TensorDesc &D = G.D;
        elem_t *p = reinterpret_cast<elem_t *>(D.p) + G.e0;
        const float neg_lr = D.neg_lr, decay = D.decay;
        const bool apply_decay = decay_pending(G);
        // the store addresses are formed afresh: kept from the loads, they would sit in
        // registers (or in scratch) through the whole window stage
        const int tid2 = opaque_tid(), lane2 = tid2 & 63, wave2 = tid2 >> 6;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave2, c, lane2);
            if (FULL || off < n) {
                float pv[8], uv[8];
                praw[c].to_float(pv);
                update8(off, uv);
                log_update(uv, FULL ? kChunk : n - off);
                if (apply_decay) {
#pragma unroll
                    for (int e = 0; e < kChunk; ++e) {
                        pv[e] = pv[e] * decay;
                        if (R::kBF16) pv[e] = bf2f(f2bf(pv[e]));
                    }
                }
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    const float prod = neg_lr * uv[e];
                    pv[e] = pv[e] + prod;
                }
                store8(p, off, FULL ? 0x7fffffff : n, true, pv);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- alpha > 0 with quantisation blocks inside the block (MA:296-298, 311-316) -------------
    // quantize_dense replaces quantize: e1 = Q(r) is kept as packed codes with its statistics
    // (for the update, which adds alpha * Qinv(e1)), and the error feedback that is stored is
    // Q of r2 = (1 - alpha) * Qinv(e1) with statistics of its own.
    uint32_t dcodes[C], dstat[C];  // e1 of the chunk; its min | max << 16 (bf16 bits)

    __device__ __forceinline__ void quantize_dense(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        uint8_t *err = G.D.err + (G.e0 >> 1);
        uint16_t *mnp = G.D.mn + (G.e0 >> q_shift);
        uint16_t *mxp = G.D.mx + (G.e0 >> q_shift);
        // quantisation blocks of 1024 to 4096 elements: the extremes of the 512-element
        // stretches meet in LDS, as in quantize
        const bool long_q = QL == 0 && ql > kWave;
        float *stretch = reinterpret_cast<float *>(hist);  // [wave * C + chunk][min, max]
        if (long_q) {
            __syncthreads();  // the selection may still be reading its lists there
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const int off = chunk_off<C>(wave, c, lane);
                float mn = INFINITY, mx = -INFINITY;
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    if (FULL || off + e < n) {
                        mn = fmin_raw(mn, r.val(c, e));
                        mx = fmax_raw(mx, r.val(c, e));
                    }
                }
                group_minmax<0>(mn, mx, kWave);
                if (lane == 0) {
                    stretch[(wave * C + c) * 2] = mn;
                    stretch[(wave * C + c) * 2 + 1] = mx;
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            float x[8];
            float mn = INFINITY, mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
            if (FULL) {
                minmax8(x, mn, mx);
            } else {
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    if (off + e < n) {
                        mn = fmin_raw(mn, x[e]);
                        mx = fmax_raw(mx, x[e]);
                    }
                }
            }
            if (long_q) {
                const int per = ql / kWave;  // stretches per quantisation block
                const int first = (wave * C + c) / per * per;
                mn = INFINITY;
                mx = -INFINITY;
                for (int j = 0; j < per; ++j) {
                    mn = fmin_raw(mn, stretch[(first + j) * 2]);
                    mx = fmax_raw(mx, stretch[(first + j) * 2 + 1]);
                }
            } else {
                group_minmax<QL>(mn, mx, ql);
            }
            const uint32_t mnb = f2bf(mn), mxb = f2bf(mx);
            dstat[c] = mnb | mxb << 16;
            dcodes[c] = 0;
            float r2[8];
            float mn2 = INFINITY, mx2 = -INFINITY;
            const float mnf = bf2f(mnb);
            const float u = div15(bf2f(mxb) - mnf, d15);
            if (FULL || off < n) {
                float cf[8];
                codes8(x, mnf, u, cf);
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (!FULL && off + e >= n) cf[e] = 0.0f;
                dcodes[c] = pack_codes(cf);
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    float deq = cf[e] * u;
                    deq = deq + mnf;
                    const float keep = P.keep * deq;
                    r2[e] = to_elem(0.0f + keep);
                    if (FULL || off + e < n) {
                        mn2 = fmin_raw(mn2, r2[e]);
                        mx2 = fmax_raw(mx2, r2[e]);
                    }
                }
            }
            if (long_q) {
                // r2 does not decrease with the code, nor the code with the element: the
                // extremes of r2 over the quantisation block are r2 at the codes of the
                // extremes of r, which every chunk of the block knows
                float ext[8], ce[8];
#pragma unroll
                for (int e = 0; e < kChunk; ++e) ext[e] = (e & 1) ? mx : mn;
                codes8(ext, mnf, u, ce);
                float lo = ce[0] * u, hi = ce[1] * u;
                lo = lo + mnf;
                hi = hi + mnf;
                lo = P.keep * lo;
                hi = P.keep * hi;
                mn2 = to_elem(0.0f + lo);
                mx2 = to_elem(0.0f + hi);
            } else {
                group_minmax<QL>(mn2, mx2, ql);
            }
            const uint32_t mn2b = f2bf(mn2), mx2b = f2bf(mx2);
            if (FULL || off < n) {
                if ((lane & (ql - 1)) == 0) {
                    const unsigned qb = (unsigned)off >> q_shift;
                    mnp[qb] = (uint16_t)mn2b;
                    mxp[qb] = (uint16_t)mx2b;
                }
                const float m2f = bf2f(mn2b);
                const float u2 = div15(bf2f(mx2b) - m2f, d15);
                float cf[8];
                codes8(r2, m2f, u2, cf);
                log_error(cf, m2f, u2, FULL ? kChunk : n - off);
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (!FULL && off + e >= n) cf[e] = 0.0f;
                const uint32_t codes = pack_codes(cf);
                if (FULL || off + kChunk <= n) {
                    *reinterpret_cast<uint32_t *>(err + ((unsigned)off >> 1)) = codes;
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        err[(off >> 1) + j] = (uint8_t)(codes >> (8 * j));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // p = p * decay; u = rne(Adam + alpha * Qinv(e1)); p += -lr * u.  After window_stage.
    __device__ __forceinline__ void param_stage_dense(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const TensorDesc &D = G.D;
        elem_t *p = reinterpret_cast<elem_t *>(D.p) + G.e0;
        const float neg_lr = D.neg_lr, decay = D.decay;
        const bool apply_decay = decay_pending(G);
        // the store addresses are formed afresh: kept from the loads, they would sit in
        // registers (or in scratch) through the whole window stage
        const int tid2 = opaque_tid(), lane2 = tid2 & 63, wave2 = tid2 >> 6;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave2, c, lane2);
            if (FULL || off < n) {
                float pv[8], uv[8];
                praw[c].to_float(pv);
                update8(off, uv);
                const float mnf = bf2f(dstat[c] & 0xffffu);
                const float u = div15(bf2f(dstat[c] >> 16) - mnf, d15);
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    if (apply_decay) pv[e] = to_elem(pv[e] * decay);
                    const uint32_t code = (dcodes[c] >> (8 * (e >> 1) + ((e & 1) ? 0 : 4))) & 15u;
                    float deq = (float)code * u;
                    deq = deq + mnf;
                    const float add = P.alpha * deq;
                    const float ud = to_elem(uv[e] + add);
                    const float prod = neg_lr * ud;
                    pv[e] = pv[e] + prod;
                    if (FULL || off + e < n) {
                        log_square(kMtUpdate, ud);
                        log_zero(kMtUpdateZeros, ud);
                    }
                }
                store8(p, off, FULL ? 0x7fffffff : n, true, pv);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // =========================================================================================
    // Two-pass route: quantisation blocks of q_span >= block length elements (q_span a
    // multiple of 8), so a top-k block meets at most two of them and their statistics need
    // every top-k block they cover.  0 <= alpha < 1 (alpha > 0: MA:296-298, 311-316).
    //   pass 1: a = g + Qinv(e), top-k, window row; the residual r goes to the gradient
    //           buffer, its exact min / max per (block, segment) to the workspace
    //   pass 2: statistics of r from the workspace; e1 = Q(r), d1 = Qinv(e1) in registers;
    //           u = Adam(window) + alpha * d1; p update; r2 = (1 - alpha) * d1; e = Q(r2)
    //           (alpha == 0: e = e1, u = Adam(window))
    // r2 is a non-decreasing function of the code, and the code of the element, so the
    // statistics of r2 over a quantisation block are r2 at the codes of r's extremes: pass 2
    // needs no second reduction across blocks.
    // Segment 0 of a block is its part in the quantisation block of its first element,
    // segment 1 the rest.  Workspace: a slot of 8 words per block: min0, max0, min1, max1
    // (floats), then four words the one-pass form uses for its list of deferred blocks.
    //
    // One-pass form (the same arithmetic, the residual never leaves the registers; the
    // workspace starts with the four floats of every block as all-ones words and the rest
    // zero): a workgroup publishes the extremes of its block right after the selection, goes
    // on with what does not need the statistics, and then takes the extremes of the blocks
    // that share its quantisation blocks as they are published.  Blocks that share a quantisation block are
    // neighbours, neighbouring blocks are dispatched together, and every workgroup publishes
    // before it waits, so the wait is short; it is bounded all the same (spin_limit polls), and
    // a workgroup that gives up stores its residual in the gradient buffer and lists its block:
    // a second launch takes the listed blocks through the second pass of the two-pass form.
    // The old statistics of a quantisation block are overwritten by the block that holds its
    // first element only after that block has seen all blocks of the quantisation block
    // published, i.e. after all of them have read the old statistics.
    // =========================================================================================
    struct Span {
        int64_t qb0;  // quantisation block of the block's first element
        int bnd;      // offset inside the block where the next one starts, INT_MAX if it does not
    };

    __device__ __forceinline__ Span make_span(const BlockGeo &G) const {
        const int n = FULL ? C * kRound : G.n;
        Span S;
        const int64_t q = P.q_span;
        S.qb0 = G.e0 / q;
        const int64_t rel = (S.qb0 + 1) * q - G.e0;
        S.bnd = rel < n ? (int)rel : 0x7fffffff;
        return S;
    }

    __device__ __forceinline__ int64_t block_id(const BlockGeo &G) const {
        const int64_t dbs = G.D.d < P.d_block_size ? G.D.d : P.d_block_size;
        return G.e0 / dbs;
    }

    // min / max over the workgroup of two pairs; every thread gets the result.  Uses the 32
    // words at kShW1 and three barriers.
    __device__ __forceinline__ void wg_minmax2(float (&mn)[2], float (&mx)[2]) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) group_minmax<0>(mn[s2], mx[s2], kWave);
        __syncthreads();
        if (lane == 0) {
            sh[kShW1 + wave * 4 + 0] = __float_as_uint(mn[0]);
            sh[kShW1 + wave * 4 + 1] = __float_as_uint(mx[0]);
            sh[kShW1 + wave * 4 + 2] = __float_as_uint(mn[1]);
            sh[kShW1 + wave * 4 + 3] = __float_as_uint(mx[1]);
        }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            mn[0] = fmin_raw(mn[0], __uint_as_float(sh[kShW1 + w * 4 + 0]));
            mx[0] = fmax_raw(mx[0], __uint_as_float(sh[kShW1 + w * 4 + 1]));
            mn[1] = fmin_raw(mn[1], __uint_as_float(sh[kShW1 + w * 4 + 2]));
            mx[1] = fmax_raw(mx[1], __uint_as_float(sh[kShW1 + w * 4 + 3]));
        }
        __syncthreads();  // the words are free again
    }

    __device__ __forceinline__ void store_partials(const BlockGeo &G, float (&mn)[2],
                                                   float (&mx)[2]) {
        wg_minmax2(mn, mx);
        if (tid == 0)
            *reinterpret_cast<float4 *>(G.D.ws + block_id(G) * kSpanWords) =
                make_float4(mn[0], mx[0], mn[1], mx[1]);
    }

    // exact min / max of r over the two quantisation blocks this top-k block meets, from the
    // partials of all top-k blocks that cover them (at most 64 each: lane i takes one)
    __device__ __forceinline__ void gather_extremes(const BlockGeo &G, const Span &S,
                                                    float (&mnx)[2], float (&mxx)[2]) const {
        const int64_t q = P.q_span;
        const int64_t dbs = G.D.d < P.d_block_size ? G.D.d : P.d_block_size;
        const int64_t nblk = (G.D.d + dbs - 1) / dbs;
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            float mn = INFINITY, mx = -INFINITY;
            if (s2 == 0 || S.bnd != 0x7fffffff) {
                const int64_t Q = S.qb0 + s2;
                const int64_t first = Q * q;
                const int64_t b_lo = first / dbs;
                int64_t b_hi = (first + q - 1) / dbs;
                b_hi = b_hi < nblk - 1 ? b_hi : nblk - 1;
                const int64_t b = b_lo + lane;
                if (b <= b_hi) {
                    const int seg = b * dbs >= first ? 0 : 1;
                    const float *w = G.D.ws + b * kSpanWords + seg * 2;
                    mn = w[0];
                    mx = w[1];
                }
                group_minmax<0>(mn, mx, kWave);
            }
            mnx[s2] = mn;
            mxx[s2] = mx;
        }
    }

    // Statistics of r (sp_mn / sp_mx) and of r2 (sp2_mn / sp2_mx) for both segments, from the
    // exact extremes of r.
    template <bool DENSE>
    __device__ __forceinline__ void span_statistics(const BlockGeo &G, const Span &S) {
        float mnx[2], mxx[2];
        gather_extremes(G, S, mnx, mxx);
        statistics_from_extremes<DENSE>(mnx, mxx);
    }

    template <bool DENSE>
    __device__ __forceinline__ void statistics_from_extremes(const float (&mnx)[2],
                                                             const float (&mxx)[2]) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            sp_mn[s2] = f2bf(mnx[s2]);
            sp_mx[s2] = f2bf(mxx[s2]);
            if (!DENSE) {  // alpha == 0: e = Q(r), the statistics kept are r's
                sp2_mn[s2] = sp_mn[s2];
                sp2_mx[s2] = sp_mx[s2];
                continue;
            }
            const float mnf = bf2f(sp_mn[s2]);
            const float u = div15(bf2f(sp_mx[s2]) - mnf, d15);
            float x[8], cf[8];
#pragma unroll
            for (int e = 0; e < kChunk; ++e) x[e] = (e & 1) ? mxx[s2] : mnx[s2];
            codes8(x, mnf, u, cf);
            float lo = cf[0] * u, hi = cf[1] * u;
            lo = lo + mnf;
            hi = hi + mnf;
            lo = P.keep * lo;
            hi = P.keep * hi;
            sp2_mn[s2] = f2bf(to_elem(0.0f + lo));
            sp2_mx[s2] = f2bf(to_elem(0.0f + hi));
        }
        // (the same in every lane: kept in scalar registers from here on)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            sp_mn[s2] = (uint32_t)__builtin_amdgcn_readfirstlane((int)sp_mn[s2]);
            sp_mx[s2] = (uint32_t)__builtin_amdgcn_readfirstlane((int)sp_mx[s2]);
            sp2_mn[s2] = (uint32_t)__builtin_amdgcn_readfirstlane((int)sp2_mn[s2]);
            sp2_mx[s2] = (uint32_t)__builtin_amdgcn_readfirstlane((int)sp2_mx[s2]);
        }
    }

    // 4-bit codes of 8 values against (mn, u) as small exact floats: floor((x - mn)/u + 0.5)
    // clamped to [0, 15]; all zero when the range is zero or not finite.  Same arithmetic as
    // the quantize stage.
    __device__ __forceinline__ void codes8(const float (&x)[8], float mnf, float u,
                                           float (&cf)[8]) const {
        const float lim = 32.0f * u;
        float y[8];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            y[e] = x[e] - mnf;
            // fp32 data may leave the bf16-rounded range; anything beyond +-32 u clamps to an
            // end code either way
            if (!R::kBF16) y[e] = __builtin_amdgcn_fmed3f(y[e], -lim, lim);
        }
        if (divisor_is_plain(u)) {
            const Divisor dv = make_divisor(u);
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                const float v = floorf(div_shared(y[e], dv) + 0.5f);
                // bf16 data lies inside its exact statistics: no clamp needed
                cf[e] = R::kBF16 ? v : __builtin_amdgcn_fmed3f(v, 0.0f, 15.0f);
            }
        } else {
            // a step that is zero, not finite, tiny, huge or has an all-ones significand: the
            // compiler's division; with so coarse a step even bf16 data can leave [0, 15]
            const bool ok = u != 0.0f && isfinite(u);
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                const float v = floorf(y[e] / u + 0.5f);
                cf[e] = ok ? __builtin_amdgcn_fmed3f(v, 0.0f, 15.0f) : 0.0f;
            }
        }
    }

    // two 16-bit halves, nibble order (e0 e1)(e2 e3) | (e4 e5)(e6 e7), even element high
    static __device__ __forceinline__ uint32_t pack_codes(const float (&cf)[8]) {
        float lo = cf[2];
        lo = __builtin_fmaf(lo, 16.0f, cf[3]);
        lo = __builtin_fmaf(lo, 16.0f, cf[0]);
        lo = __builtin_fmaf(lo, 16.0f, cf[1]);
        float hi = cf[6];
        hi = __builtin_fmaf(hi, 16.0f, cf[7]);
        hi = __builtin_fmaf(hi, 16.0f, cf[4]);
        hi = __builtin_fmaf(hi, 16.0f, cf[5]);
        return (uint32_t)lo | ((uint32_t)hi << 16);
    }

    static __device__ __forceinline__ float to_elem(float v) {
        return R::kBF16 ? bf2f(f2bf(v)) : v;
    }

    // ---- pass 1 ------------------------------------------------------------------------------
    uint32_t sp_mn[2], sp_mx[2];    // statistics of r in the two segments (bf16 bits)
    uint32_t sp2_mn[2], sp2_mx[2];  // statistics of r2

    __device__ __forceinline__ void span_load_grad_inputs(const BlockGeo &G, const Span &S) {
        load_hint(G);
        const int n = FULL ? C * kRound : G.n;
        const elem_t *g = reinterpret_cast<const elem_t *>(G.D.g) + G.e0;
        const uint8_t *err = G.D.err + (G.e0 >> 1);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            graw[c].load(g, off, n, FULL);
            cw[c] = 0;
            if (FULL || off < n) {
                if (FULL || off + kChunk <= n) {
                    cw[c] = *reinterpret_cast<const uint32_t *>(err + ((unsigned)off >> 1));
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        cw[c] |= (uint32_t)err[(off >> 1) + j] << (8 * j);
                }
            }
        }
        sp_mn[0] = G.D.mn[S.qb0];
        sp_mx[0] = G.D.mx[S.qb0];
        sp_mn[1] = sp_mx[1] = 0;
        if (S.bnd != 0x7fffffff) {
            sp_mn[1] = G.D.mn[S.qb0 + 1];
            sp_mx[1] = G.D.mx[S.qb0 + 1];
        }
    }

    __device__ __forceinline__ void span_dequant(const BlockGeo &G, const Span &S) {
        const int n = FULL ? C * kRound : G.n;
        const float mn0 = bf2f(sp_mn[0]), mn1 = bf2f(sp_mn[1]);
        const float u0 = div15(bf2f(sp_mx[0]) - mn0, d15), u1 = div15(bf2f(sp_mx[1]) - mn1, d15);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            float v[8];
            graw[c].to_float(v);
            if constexpr (LOG) {
#pragma unroll
                for (int e = 0; e < kChunk; ++e) log_square(kMtGrad, v[e]);
            }
            const bool second = off >= S.bnd;
            const float mn = second ? mn1 : mn0, u = second ? u1 : u0;
            // the nibbles as bytes of two words (even elements high), one conversion each, as
            // in dequant
            uint32_t odd = cw[c] & 0x0f0f0f0fu, even = (cw[c] >> 4) & 0x0f0f0f0fu;
            asm volatile("" : "+v"(odd), "+v"(even));
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                const uint32_t code = (((e & 1) ? odd : even) >> (8 * (e >> 1))) & 0xffu;
                float deq = (float)code * u;
                deq = deq + mn;
                v[e] = v[e] + deq;
            }
            if (!FULL && off + kChunk > n) {
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (off + e >= n) v[e] = 0.0f;
            }
            r.set_chunk(c, v);
            __builtin_amdgcn_sched_barrier(0);
        }
        launder(r);
    }

    // the residual goes to the gradient buffer (which the step may destroy, MA:190-214 does)
    __device__ __forceinline__ void span_store_residual(const BlockGeo &G, const Span &S) {
        const int n = FULL ? C * kRound : G.n;
        elem_t *out = reinterpret_cast<elem_t *>(const_cast<void *>(G.D.g)) + G.e0;
        float mn[2] = {INFINITY, INFINITY}, mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            if (FULL || off < n) {
                float x[8];
                float lmn = INFINITY, lmx = -INFINITY;
#pragma unroll
                for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
                if (FULL) {
                    minmax8(x, lmn, lmx);
                } else {
#pragma unroll
                    for (int e = 0; e < kChunk; ++e) {
                        if (off + e < n) {
                            lmn = fmin_raw(lmn, x[e]);
                            lmx = fmax_raw(lmx, x[e]);
                        }
                    }
                }
                const bool second = off >= S.bnd;
                mn[0] = fmin_raw(mn[0], second ? INFINITY : lmn);
                mx[0] = fmax_raw(mx[0], second ? -INFINITY : lmx);
                mn[1] = fmin_raw(mn[1], second ? lmn : INFINITY);
                mx[1] = fmax_raw(mx[1], second ? lmx : -INFINITY);
                store8(out, off, FULL ? 0x7fffffff : n, true, x);
            }
        }
        store_partials(G, mn, mx);
    }

    // ---- one-pass form ---------------------------------------------------------------------
    // extremes of the residual (in the registers) per segment, to the workspace, then the flag
    __device__ __forceinline__ void span_publish(const BlockGeo &G, const Span &S) {
        const int n = FULL ? C * kRound : G.n;
        float mn[2] = {INFINITY, INFINITY}, mx[2] = {-INFINITY, -INFINITY};
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            if (FULL || off < n) {
                float x[8];
                float lmn = INFINITY, lmx = -INFINITY;
#pragma unroll
                for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
                if (FULL) {
                    minmax8(x, lmn, lmx);
                } else {
#pragma unroll
                    for (int e = 0; e < kChunk; ++e) {
                        if (off + e < n) {
                            lmn = fmin_raw(lmn, x[e]);
                            lmx = fmax_raw(lmx, x[e]);
                        }
                    }
                }
                const bool second = off >= S.bnd;
                mn[0] = fmin_raw(mn[0], second ? INFINITY : lmn);
                mx[0] = fmax_raw(mx[0], second ? -INFINITY : lmx);
                mn[1] = fmin_raw(mn[1], second ? lmn : INFINITY);
                mx[1] = fmax_raw(mx[1], second ? lmx : -INFINITY);
            }
        }
        wg_minmax2(mn, mx);
        if (tid == 0) {
            // One 64-bit store per segment, past this XCD's L2 (device scope) and without any
            // fence: the pair is all that is handed over, it arrives whole, and a pair that
            // has not arrived reads as the all-ones words the workspace was cleared to (a
            // published minimum is never that NaN; a block whose extremes are NaN looks
            // unpublished, and its neighbours give up and take the second pass).
            uint64_t *w = reinterpret_cast<uint64_t *>(G.D.ws + block_id(G) * kSpanWords);
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2)
                __hip_atomic_store(w + s2,
                                   (uint64_t)__float_as_uint(mn[s2]) |
                                       (uint64_t)__float_as_uint(mx[s2]) << 32,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // Waits (wave 0 polls, at most P.spin_limit times per flag) until all blocks that share
    // this block's quantisation blocks have published, then forms the statistics as
    // span_statistics does.  False, for every thread, if some block did not publish in time.
    // Uses sh[kShTies] and the 4 words at sh[kShSel]; two barriers.
    template <bool DENSE>
    __device__ __forceinline__ bool span_await(const BlockGeo &G, const Span &S) {
        const int64_t q = P.q_span;
        const int64_t dbs = G.D.d < P.d_block_size ? G.D.d : P.d_block_size;
        const int64_t nblk = (G.D.d + dbs - 1) / dbs;
        if (wave == 0) {
            bool ok = true;
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                float mn = INFINITY, mx = -INFINITY;
                if (s2 == 0 || S.bnd != 0x7fffffff) {
                    const int64_t Q = S.qb0 + s2;
                    const int64_t first = Q * q;
                    const int64_t b_lo = first / dbs;
                    int64_t b_hi = (first + q - 1) / dbs;
                    b_hi = b_hi < nblk - 1 ? b_hi : nblk - 1;
                    const int64_t b = b_lo + lane;
                    if (b <= b_hi) {
                        const int seg = b * dbs >= first ? 0 : 1;
                        uint64_t *w =
                            reinterpret_cast<uint64_t *>(G.D.ws + b * kSpanWords) + seg;
                        int left = P.spin_limit;
                        uint64_t pair =
                            __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        while ((uint32_t)pair == 0xffffffffu && left > 0) {
                            __builtin_amdgcn_s_sleep(8);
                            --left;
                            pair = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                        ok = ok && (uint32_t)pair != 0xffffffffu;
                        mn = __uint_as_float((uint32_t)pair);
                        mx = __uint_as_float((uint32_t)(pair >> 32));
                    }
                    group_minmax<0>(mn, mx, kWave);
                }
                if (lane == 0) {
                    sh[kShSel + 2 * s2] = __float_as_uint(mn);
                    sh[kShSel + 2 * s2 + 1] = __float_as_uint(mx);
                }
            }
            const bool all_ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
            if (lane == 0) sh[kShTies] = all_ok ? 1u : 0u;
        }
        __syncthreads();
        const bool all_ok = sh[kShTies] != 0;
        float mnx[2], mxx[2];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            mnx[s2] = __uint_as_float(sh[kShSel + 2 * s2]);
            mxx[s2] = __uint_as_float(sh[kShSel + 2 * s2 + 1]);
        }
        __syncthreads();  // the words are free again
        if (all_ok) statistics_from_extremes<DENSE>(mnx, mxx);
        return all_ok;
    }

    // Gives up on the one-pass form for this block: the residual goes to the gradient buffer,
    // where the second pass of the two-pass form expects it.
    __device__ __forceinline__ void span_defer(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        elem_t *out = reinterpret_cast<elem_t *>(const_cast<void *>(G.D.g)) + G.e0;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            if (FULL || off < n) {
                float x[8];
#pragma unroll
                for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
                store8(out, off, FULL ? 0x7fffffff : n, true, x);
            }
        }
    }

    // the residual of chunk c as fp32: from the registers of the one-pass form, or as the
    // second pass loaded it
    template <bool FROM_R>
    __device__ __forceinline__ void residual8(int c, float (&x)[8]) const {
        if (FROM_R) {
#pragma unroll
            for (int e = 0; e < kChunk; ++e) x[e] = r.val(c, e);
        } else {
            graw[c].to_float(x);
        }
    }

    // ---- pass 2 -----------------------------------------------------------------------
    // The window row the first pass wrote comes back into sel_idx / sel_val, where the window
    // stages expect the row of this step: requested first, stored once the other requests
    // are out.
    uint32_t row_i, row_v;

    __device__ __forceinline__ void span_load_row(const BlockGeo &G) {
        row_i = row_v = 0;
        if (tid < G.kb) {
            const int64_t at = (int64_t)G.D.row * G.D.k + G.col0 + tid;
            row_i = reinterpret_cast<const uint16_t *>(G.D.I)[at];
            row_v = G.D.V[at];
        }
        row_in_lds = true;
    }

    __device__ __forceinline__ void span_row_to_lds(const BlockGeo &G) {
        if (tid < G.kb) {
            sel_idx[tid] = (uint16_t)row_i;
            sel_val[tid] = (uint16_t)row_v;
        }
        for (int j = tid + kWG; j < G.kb; j += kWG) {
            const int64_t at = (int64_t)G.D.row * G.D.k + G.col0 + j;
            sel_idx[j] = reinterpret_cast<const uint16_t *>(G.D.I)[at];
            sel_val[j] = G.D.V[at];
        }
    }

    __device__ __forceinline__ void span_load_residual(const BlockGeo &G) {
        const int n = FULL ? C * kRound : G.n;
        const elem_t *g = reinterpret_cast<const elem_t *>(G.D.g) + G.e0;
#pragma unroll
        for (int c = 0; c < C; ++c) graw[c].load(g, chunk_off<C>(wave, c, lane), n, FULL);
    }

    // alpha == 0, second pass: e = Q(r) against the statistics of r, and the statistics arrays
    template <bool FROM_R = false>
    __device__ __forceinline__ void span_codes_stage(const BlockGeo &G, const Span &S) {
        const int n = FULL ? C * kRound : G.n;
        const TensorDesc &D = G.D;
        uint8_t *err = D.err + (G.e0 >> 1);
        const float mn0 = bf2f(sp_mn[0]), mn1 = bf2f(sp_mn[1]);
        const float u0 = div15(bf2f(sp_mx[0]) - mn0, d15), u1 = div15(bf2f(sp_mx[1]) - mn1, d15);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            if (FULL || off < n) {
                const bool second = off >= S.bnd;
                float x[8], cf[8];
                residual8<FROM_R>(c, x);
                codes8(x, second ? mn1 : mn0, second ? u1 : u0, cf);
                log_error(cf, second ? mn1 : mn0, second ? u1 : u0, FULL ? kChunk : n - off);
#pragma unroll
                for (int e = 0; e < kChunk; ++e)
                    if (!FULL && off + e >= n) cf[e] = 0.0f;
                const uint32_t codes = pack_codes(cf);
                if (FULL || off + kChunk <= n) {
                    *reinterpret_cast<uint32_t *>(err + ((unsigned)off >> 1)) = codes;
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        err[(off >> 1) + j] = (uint8_t)(codes >> (8 * j));
                }
            }
        }
        span_store_statistics(G, S);
    }

    // the block that holds the first element of a quantisation block writes its statistics
    __device__ __forceinline__ void span_store_statistics(const BlockGeo &G, const Span &S) {
        if (tid == 0) {
            if (G.e0 == S.qb0 * (int64_t)P.q_span) {
                G.D.mn[S.qb0] = (uint16_t)sp2_mn[0];
                G.D.mx[S.qb0] = (uint16_t)sp2_mx[0];
            }
            if (S.bnd != 0x7fffffff) {
                G.D.mn[S.qb0 + 1] = (uint16_t)sp2_mn[1];
                G.D.mx[S.qb0 + 1] = (uint16_t)sp2_mx[1];
            }
        }
    }

    // alpha > 0, second pass: p = p * decay; u = rne(Adam + alpha * d1); p += -lr * u;
    // r2 = rne(0 + keep * d1); e = Q(r2); the statistics arrays.  After window_cells.
    // d1 = Qinv(e1) takes 16 values per segment, and alpha * d1 and the code of r2 with them:
    // both come from a table of 2 x 16 entries that 32 threads fill first, so that an element
    // costs one quantisation, not two.
    template <bool FROM_R = false>
    __device__ __forceinline__ void span_param_stage(const BlockGeo &G, const Span &S) {
        const int n = FULL ? C * kRound : G.n;
        const TensorDesc &D = G.D;
        elem_t *p = reinterpret_cast<elem_t *>(D.p) + G.e0;
        uint8_t *err = D.err + (G.e0 >> 1);
        const float neg_lr = D.neg_lr, decay = D.decay;
        const bool apply_decay = decay_pending(G);
        const float mn0 = bf2f(sp_mn[0]), mn1 = bf2f(sp_mn[1]);
        const float u0 = div15(bf2f(sp_mx[0]) - mn0, d15), u1 = div15(bf2f(sp_mx[1]) - mn1, d15);
        const float m20 = bf2f(sp2_mn[0]), m21 = bf2f(sp2_mn[1]);
        const float v0 = div15(bf2f(sp2_mx[0]) - m20, d15), v1 = div15(bf2f(sp2_mx[1]) - m21, d15);
        // [segment][code]: alpha * d1, code of r2; in the kSh* words, which the window stage
        // has finished with (the fp32 window stage leaves the updates in its own arrays)
        static_assert(kMiscBytes >= 32 * 8, "the table takes the kSh* words");
        uint2 *table = reinterpret_cast<uint2 *>(sh);
        if (tid < 32) {
            const bool second = tid >= 16;
            const float mnf = second ? mn1 : mn0, u = second ? u1 : u0;
            float deq = (float)(tid & 15) * u;
            const float d1 = deq + mnf;
            const float add = P.alpha * d1;
            const float keep = P.keep * d1;
            float r2[8], c2[8];
#pragma unroll
            for (int e = 0; e < kChunk; ++e) r2[e] = to_elem(0.0f + keep);
            codes8(r2, second ? m21 : m20, second ? v1 : v0, c2);
            table[tid] = make_uint2(__float_as_uint(add), (uint32_t)c2[0]);
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int off = chunk_off<C>(wave, c, lane);
            if (FULL || off < n) {
                const bool second = off >= S.bnd;
                float x[8], cf[8];
                residual8<FROM_R>(c, x);
                codes8(x, second ? mn1 : mn0, second ? u1 : u0, cf);
                const uint2 *mine = table + (second ? 16 : 0);
                float pv[8], uv[8];
                praw[c].to_float(pv);
                update8(off, uv);
                uint32_t codes = 0;
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    const uint2 t = mine[(uint32_t)cf[e]];
                    if (apply_decay) pv[e] = to_elem(pv[e] * decay);
                    const float ud = to_elem(uv[e] + __uint_as_float(t.x));
                    const float prod = neg_lr * ud;
                    pv[e] = pv[e] + prod;
                    const bool valid = FULL || off + e < n;
                    // nibble order (e0 e1)(e2 e3) | (e4 e5)(e6 e7), even element high
                    constexpr int kShift[8] = {4, 0, 12, 8, 20, 16, 28, 24};
                    if (valid) codes |= t.y << kShift[e];
                    if constexpr (LOG) {
                        if (valid) {
                            log_square(kMtUpdate, ud);
                            log_zero(kMtUpdateZeros, ud);
                            float deq = (float)t.y * (second ? v1 : v0);
                            deq = deq + (second ? m21 : m20);
                            log_square(kMtError, to_elem(0.0f + deq));
                        }
                    }
                }
                store8(p, off, FULL ? 0x7fffffff : n, true, pv);
                if (FULL || off + kChunk <= n) {
                    *reinterpret_cast<uint32_t *>(err + ((unsigned)off >> 1)) = codes;
                } else {
                    const int nbytes = (n - off + 1) >> 1;
                    for (int j = 0; j < nbytes; ++j)
                        err[(off >> 1) + j] = (uint8_t)(codes >> (8 * j));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        span_store_statistics(G, S);
    }
};

// Work item of this workgroup.  The hardware hands consecutive workgroups of a launch to the
// chip's 8 XCDs in turn (workgroup i runs on XCD i % 8, each with its own L2); the items are
// dealt out so that every XCD walks one contiguous eighth of the launch's blocks, which the
// memory system serves measurably faster than eight interleaved walks (stores most of all).
// The launch's last `short_items` items (tensors shorter than a block, which finish early) are
// dealt out apart, an eighth to every XCD behind its share of the others: the workgroups that
// start last are then short ones, and the launch does not end on a round of full blocks.
__device__ __forceinline__ int xcd_contiguous_item(int total_items, int short_items) {
    constexpr int kXcds = 8;
    const int bid = (int)blockIdx.x;
    const int x = bid % kXcds, j = bid / kXcds;
    const int q = total_items / kXcds, r = total_items % kXcds;
    const int qs = short_items / kXcds, rs = short_items % kXcds;
    // XCD x runs all_here workgroups; items before its own, of either kind
    const int all_here = q + (x < r ? 1 : 0), short_here = qs + (x < rs ? 1 : 0);
    const int all_before = x * q + (x < r ? x : r), short_before = x * qs + (x < rs ? x : rs);
    const int long_here = all_here - short_here, long_before = all_before - short_before;
    return j < long_here ? long_before + j
                         : (total_items - short_items) + short_before + (j - long_here);
}

// which tensor owns workgroup / work item `w` of the launch (first_block is ascending)
__device__ __forceinline__ int find_tensor(const FusedParams &P, int w) {
    // the last tensor whose first work item is not beyond w
    int lo = 0, hi = P.n_tensors - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (w >= P.t[mid].first_block) lo = mid; else hi = mid - 1;
    }
    return lo;
}

// One workgroup per block: any block shape.  Tensor i contributes its blocks
// blk0 .. blk0 + (first_block[i+1] - first_block[i]) - 1.
//   WIN: what becomes of the window and the parameters.  kWinFused: everything in this kernel.
//        kWinApart: nothing; the kernel ends with the quantisation, and window_param_kernel,
//        launched behind it, forms the update and steps the parameters.
constexpr int kWinFused = 0, kWinApart = 2;

template <class R, int MIN_WAVES, int QL, bool DENSE = false, int WIN = kWinFused, int AUX = 0>
__global__ __launch_bounds__(kWG, MIN_WAVES) void fused_step_kernel(FusedParams P) {
    extern __shared__ __align__(16) unsigned char lds[];
    const int item = xcd_contiguous_item(P.total_items, P.short_items);
    const int ti = find_tensor(P, item);
    const BlockGeo G = make_geo(P, ti, P.t[ti].blk0 + (item - P.t[ti].first_block));
    auto run = [&](auto &fb) {
        fb.load_grad_inputs(G);
        fb.dequant(G);
        fb.topk_and_row(G);
        if constexpr (WIN == kWinApart) fb.file_row_cuts(G);
        if constexpr (DENSE) {
            fb.quantize_dense(G);
            fb.load_params(G);
            fb.load_window(G);
            fb.window_stage(G);
            fb.param_stage_dense(G);
        } else {
            // parameters and window entries are asked for before the quantisation, which
            // hides their latency (the selection runs with more registers free without them)
            if constexpr (WIN != kWinApart) fb.load_params_window(G);
            fb.quantize(G);
            if constexpr (WIN != kWinApart) fb.update(G);
        }
        fb.log_flush(item, 0xffu);
    };
    if (G.n == R::kC * kRound) {
        FusedBlock<R, true, QL, AUX> fb(P, lds);
        run(fb);
    } else {
        FusedBlock<R, false, QL, AUX> fb(P, lds);
        run(fb);
    }
}

// Two-pass route, see FusedBlock; one workgroup per block.
//   alpha > 0:  PASS 1 (residual and its extremes), PASS 2 (everything else)
//   alpha == 0: PASS 4 (PASS 1 and the parameter update, which does not wait for the
//               statistics), PASS 3 (codes of the residual)
//   Logging steps: the first pass leaves |g|^2 (and, as PASS 4, the update's sums) and clears
//   the components no pass forms; the second leaves the rest.
// One-pass form of the same route, alpha == 0, no logging: PASS 6 does the whole step of a block,
// exchanging the extremes of the residual through the workspace; PASS 8 is PASS 3 for the blocks
// PASS 6 deferred, launched behind it with a fixed number of workgroups.  The deferred blocks are
// listed: their count is word kSpanDeferCount of the first block slot of the launch's workspace
// (the slot of block 0 of the launch's first tensor), the i-th deferred work item is word
// kSpanDeferItem of the i-th slot from there (the launch has at most as many work items as
// there are slots from its first to the end of the workspace).
// (With alpha > 0 the one-pass form was built as well and measured slower than the two passes:
// its second half needs the registers of the second pass on top of the residual, which costs
// the third workgroup per CU or spills, and neither pass is short of memory bandwidth by
// enough to pay for that.)
constexpr int kSpanDeferItem = 4, kSpanDeferCount = 6;

template <class R, int MIN_WAVES, int PASS, int AUX = 0>
__global__ __launch_bounds__(kWG, MIN_WAVES) void span_step_kernel(FusedParams P) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr bool kSweep = PASS == 8;
    uint32_t *slots = reinterpret_cast<uint32_t *>(P.t[0].ws);
    uint32_t *defer_count = slots + kSpanDeferCount;
    // (PASS 6) this block gives up: listed for the sweep
    auto list_deferred = [&](int item) {
        if (threadIdx.x == 0) {
            const uint32_t at = atomicAdd(defer_count, 1u);
            slots[(int64_t)at * kSpanWords + kSpanDeferItem] = (uint32_t)item;
        }
    };
    auto run = [&](auto &fb, const BlockGeo &G, int item) {
        const auto S = fb.make_span(G);
        if constexpr (PASS == 1 || PASS == 4) {
            fb.span_load_grad_inputs(G, S);
            fb.span_dequant(G, S);
            fb.topk_and_row(G);
            fb.span_store_residual(G, S);
            if constexpr (PASS == 4) {
                fb.load_params_window(G);
                fb.update(G);
            }
        } else if constexpr (PASS == 2) {
            fb.span_load_row(G);
            fb.wide = fb.wide_window(G);
            if (fb.wide) fb.load_window_wide(G); else fb.load_window(G);
            fb.span_load_residual(G);
            fb.span_row_to_lds(G);
            fb.template span_statistics<true>(G, S);
            fb.window_cells(G);
            // (asked for only now: the residual and the parameters both held through the
            // window stage cost the registers that stage needs; the parameters are wanted
            // last in the stage below, so they are the ones that wait)
            fb.load_params(G);
            fb.span_param_stage(G, S);
        } else if constexpr (PASS == 3 || PASS == 8) {
            fb.span_load_residual(G);
            fb.template span_statistics<false>(G, S);
            fb.span_codes_stage(G, S);
        } else {  // PASS 6
            fb.span_load_grad_inputs(G, S);
            fb.span_dequant(G, S);
            fb.topk_and_row(G);
            fb.span_publish(G, S);
            // (the parameters are asked for once the residual has left the registers: both
            // held through the wait and the codes would not fit the register budget of three
            // workgroups per CU)
            if (fb.template span_await<false>(G, S)) {
                fb.template span_codes_stage<true>(G, S);
            } else {
                fb.span_defer(G);
                list_deferred(item);
            }
            fb.load_params_window(G);
            fb.update(G);
        }
        constexpr unsigned kUnused = 1u << kMtQuantErr | 1u << kMtQuantErrZeros | 3u << 6;
        constexpr unsigned kUpdate = 1u << kMtUpdate | 1u << kMtUpdateZeros;
        fb.log_flush(item, PASS == 1   ? kUnused | 1u << kMtGrad
                           : PASS == 4 ? kUnused | 1u << kMtGrad | kUpdate
                           : PASS == 2 ? kUpdate | 1u << kMtError
                                       : 1u << kMtError);
    };
    auto one = [&](int item) {
        const int ti = find_tensor(P, item);
        const BlockGeo G = make_geo(P, ti, P.t[ti].blk0 + (item - P.t[ti].first_block));
        if (G.n == R::kC * kRound) {
            FusedBlock<R, true, 0, AUX> fb(P, lds);
            run(fb, G, item);
        } else {
            FusedBlock<R, false, 0, AUX> fb(P, lds);
            run(fb, G, item);
        }
    };
    if constexpr (kSweep) {
        const uint32_t listed = *defer_count < (uint32_t)P.total_items ? *defer_count
                                                                       : (uint32_t)P.total_items;
        for (uint32_t i = blockIdx.x; i < listed; i += gridDim.x) {
            const uint32_t item = slots[(int64_t)i * kSpanWords + kSpanDeferItem];
            if (item < (uint32_t)P.total_items) one((int)item);
            __syncthreads();
        }
    } else {
        one(xcd_contiguous_item(P.total_items, P.short_items));
    }
}

// =============================================================================================
// Window and parameters apart from the block kernel (kWinApart): Adam direction from the window
// (MA:277-291), p = p * (1 - lr*wd) (MA:234-235), p += -lr * u (MA:304), for windows with about
// as many entries as the block has coordinates (m = 20 rows of 5 %), where the sums of all
// coordinates do not fit the LDS at once and the block kernel's own window stage is a chain of
// barrier-separated row steps.  One workgroup per top-k block; it reads the window rows
// (including the one the block kernel has just written) and the parameters, nothing else.
//
// Rows that list their entries by increasing coordinate (as every kernel of this library writes
// them when a block row has more than 512 entries) are cut at the multiples of 1024
// coordinates: chunk ch of a row is the stretch table[row][ch] .. table[row][ch + 1] of its
// entries.  A wave then owns a chunk: its 1024 pairs of sums live in the wave's own 8 KiB of
// LDS, it adds the rows' stretches in row order (the LDS operations of one wave execute in
// program order and a row names a coordinate once, so no barrier is needed and every sum is
// formed in row order, as compute_microadam_update forms it), and lane l steps the 16
// parameters at 16 l of the chunk.
// A block in which some row is not in increasing order, or holds an index outside the block,
// takes the general form instead: coordinate ranges of 4096 with a barrier after every row.
//   LDS: the kSh* words | table: rows x (chunks + 1) int32 at L.off_slot, row stride
//   L.slot_cells | sums: 8 x (kWinChunk + 8) pairs of floats at L.off_union (per wave one
//   cell (z1, z2) per coordinate of a chunk and a spare one; the general form uses the same
//   memory as 2 x 4096 floats).
// =============================================================================================
constexpr int kWinShift = 9;
constexpr int kWinChunk = 1 << kWinShift;  // coordinates per chunk: 8 for each of 64 lanes
static_assert(kWinChunk == kRowCutStep, "the cached row cuts are the chunk boundaries");
constexpr int kWinRowBatch = 10;    // rows whose stretches are requested together

// two window entries as they lie in memory, from any 2-byte boundary (the hardware takes
// unaligned loads)
struct __attribute__((packed, aligned(2))) EntryPair {
    uint32_t w;
};

// value of the lane below (lane 0 and lanes without a source get `first`)
__device__ __forceinline__ uint32_t lane_below(uint32_t v, uint32_t first) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)first, (int)v, 0x138 /* wave_shr:1 */, 0xF,
                                                 0xF, false);
}

template <class R, int MIN_WAVES>
__global__ __launch_bounds__(kWG, MIN_WAVES) void window_param_kernel(FusedParams P) {
    typedef typename R::elem_t elem_t;
    extern __shared__ __align__(16) unsigned char lds[];
    uint32_t *sh = reinterpret_cast<uint32_t *>(lds);
    int *table = reinterpret_cast<int *>(lds + P.L.off_slot);
    float *sums = reinterpret_cast<float *>(lds + P.L.off_union);
    const int item = xcd_contiguous_item(P.total_items, P.short_items);
    const int ti = find_tensor(P, item);
    const BlockGeo G = make_geo(P, ti, P.t[ti].blk0 + (item - P.t[ti].first_block));
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = G.n, kb = G.kb, rows = P.W.rows;
    const int nch = (n + kWinChunk - 1) / kWinChunk;
    const int stride = nch + 1;
    const int64_t k = G.D.k;
    const uint16_t *Ib = reinterpret_cast<const uint16_t *>(G.D.I) + G.col0;
    const uint16_t *Vb = G.D.V + G.col0;
    elem_t *p = reinterpret_cast<elem_t *>(G.D.p) + G.e0;
    const float neg_lr = G.D.neg_lr, decay = G.D.decay;
    const bool apply_decay = G.D.apply_decay != 0;

    // ---- where every row crosses the chunk boundaries, and whether all rows are in order.
    //      Thread t takes the entries 2t and 2t + 1 of every row (one load), the entry before
    //      them comes from the lane below, for lane 0 from memory.
    if (tid == 0) sh[0] = 0;
    __syncthreads();
    // from the tensor's cache of row cuts, when it keeps one and knows every live row
    // (fused_step_kernel files a row's cuts when it writes the row in coordinate order)
    const uint16_t *cuts = reinterpret_cast<const uint16_t *>(G.D.ws);
    bool cached = cuts != nullptr;
    if (cached) {
        const RowCuts where(G.D.d, P.d_block_size);
        const int64_t block = G.e0 / (G.D.d < P.d_block_size ? G.D.d : P.d_block_size);
        bool unknown = false;
        for (int i = tid; i < rows * stride; i += kWG) {
            const int r = i / stride, ch = i - r * stride;
            const uint32_t cut = cuts[where.at(r, block) + ch];
            table[i] = 2 * (int)cut;
            if (ch == 0 && cut != 0) unknown = true;
        }
        if (unknown) atomicOr(&sh[0], 2u);
        __syncthreads();
        cached = sh[0] == 0;
        __syncthreads();
        if (tid == 0) sh[0] = 0;
    }
    bool bad = false;
    if (!cached) {
    for (int i = tid; i < rows * stride; i += kWG) table[i] = 2 * kb;
    __syncthreads();
    for (int j0 = 0; j0 < kb; j0 += 2 * kWG) {
        const int j = j0 + 2 * tid;
        for (int r0 = 0; r0 < rows; r0 += kWinRowBatch) {
            uint32_t pair[kWinRowBatch], before[kWinRowBatch];
#pragma unroll
            for (int i = 0; i < kWinRowBatch; ++i) {
                pair[i] = 0xffffffffu;
                before[i] = 0;
                if (r0 + i < rows) {
                    const uint16_t *Ir = Ib + (int64_t)(r0 + i) * k;
                    if (j + 1 < kb)
                        pair[i] = reinterpret_cast<const EntryPair *>(Ir + (unsigned)j)->w;
                    else if (j < kb)
                        pair[i] = (uint32_t)Ir[(unsigned)j] | 0xffff0000u;
                    if (lane == 0 && j > 0 && j < kb) before[i] = Ir[(unsigned)(j - 1)];
                }
            }
#pragma unroll
            for (int i = 0; i < kWinRowBatch; ++i) {
                if (r0 + i < rows) {
                    // (the lane below holds the two entries before this lane's)
                    const uint32_t below = lane_below(pair[i] >> 16, before[i]);
                    const int c0 = (int)(pair[i] & 0xffffu), c1 = (int)(pair[i] >> 16);
                    const int cb = j > 0 ? (int)below : -1;
                    int *trow = table + (r0 + i) * stride;
                    if (j < kb) {
                        if (c0 <= cb || c0 >= n) {
                            bad = true;
                        } else {
                            for (int ch = (cb >> kWinShift) + 1; ch <= (c0 >> kWinShift); ++ch)
                                trow[ch] = 2 * j;
                        }
                    }
                    if (j + 1 < kb) {
                        if (c1 <= c0 || c1 >= n) {
                            bad = true;
                        } else {
                            for (int ch = (c0 >> kWinShift) + 1; ch <= (c1 >> kWinShift); ++ch)
                                trow[ch] = 2 * (j + 1);
                        }
                    }
                }
            }
        }
    }
    }
    // (the batches below read up to kWindowPad rows past the live ones: empty stretches)
    for (int i = rows * stride + tid; i < (rows + kWindowPad) * stride; i += kWG) table[i] = 0;
    if (bad) atomicOr(&sh[0], 1u);
    __syncthreads();
    // One buffer per array for all rows of the block's stretch of the window, the row chosen by
    // a scalar byte offset: possible while the rows from this block's first entry to its
    // stretch of the last row span less than 4 GiB.
    const uint64_t span_bytes = ((uint64_t)(P.W.rows_total - 1) * (uint64_t)k + (uint64_t)kb) * 2u;
    const bool in_order = sh[0] == 0 && span_bytes <= 0xffffffffull;
    // table[row][ch]: byte offset of the first entry of chunk ch in the row's stretch of the
    // block

    // p = p * decay; p += -lr * u for the 8 parameters at `off`, u from their 8 pairs of sums
    auto step8 = [&](int off, const RawChunk<R> &praw, const float (&a1)[8], const float (&a2)[8]) {
        float pv[8];
        praw.to_float(pv);
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            float u = 0.0f;
            if (a1[e] != 0.0f || a2[e] != 0.0f) {
                u = adam_update<R::kBF16>(a1[e], a2[e], P.W.s1, P.W.s2, P.W.eps);
            }
            if (apply_decay) {
                pv[e] = pv[e] * decay;
                if (R::kBF16) pv[e] = bf2f(f2bf(pv[e]));
            }
            const float prod = neg_lr * u;
            pv[e] = pv[e] + prod;
        }
        store8(p, off, n, true, pv);
    };

    if (in_order) {
        // per wave one cell (z1, z2) per coordinate of a chunk and a spare one that takes what
        // is not for this chunk
        constexpr int kPerLane = kWinChunk / kWave;  // coordinates of a chunk per lane
        float2 *z = reinterpret_cast<float2 *>(sums) + wave * (kWinChunk + 8);
        const uint32_t lane2 = (uint32_t)lane * 2u;
        const __amdgpu_buffer_rsrc_t all_i = byte_buffer(Ib, (uint32_t)span_bytes);
        const __amdgpu_buffer_rsrc_t all_v = byte_buffer(Vb, (uint32_t)span_bytes);
        const int row_stride = (int)(uint32_t)(2 * k);  // bytes from a row to the next
        const int last_row = P.W.rows_total - 1;
        for (int ch = wave; ch < nch; ch += kWaves) {
            const int base = ch * kWinChunk, off = base + lane * kPerLane;
            RawChunk<R> praw[kPerLane / kChunk];
#pragma unroll
            for (int h = 0; h < kPerLane / kChunk; ++h)
                praw[h].load(p, off + h * kChunk, n, base + kWinChunk <= n);
            const float4 zero4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
            for (int i = 0; i < kPerLane / 2; ++i)
                reinterpret_cast<float4 *>(z + lane * kPerLane)[i] = zero4;
            __builtin_amdgcn_wave_barrier();
            // rows with more than 64 entries in this chunk (bit r), found once for the chunk
            uint64_t long_rows = 0;
            {
                int len = 0;
                if (lane < rows) len = table[lane * stride + ch + 1] - table[lane * stride + ch];
                long_rows = __builtin_amdgcn_ballot_w64(len > 2 * kWave);
            }
            for (int r0 = 0; r0 < rows; r0 += kWinRowBatch) {
                // ---- all requests of the batch first: entry s + lane of every row's stretch,
                //      through one buffer per array with the row as a scalar offset.  Lanes
                //      past the stretch's end (their entries belong to later chunks, blocks or
                //      rows) are sorted out when the sums are formed; the rows behind the last
                //      live one have empty stretches and zero weights and are read from the
                //      last row.  Straight-line code: nothing between the requests waits for
                //      an answer.
                uint32_t ei[kWinRowBatch], ev[kWinRowBatch];
                float w1[kWinRowBatch], w2[kWinRowBatch];
                uint32_t at[kWinRowBatch], e2[kWinRowBatch];
                const int *tp = table + r0 * stride + ch;
                static_assert(kWinRowBatch <= kWindowPad, "weights and table rows past the last");
#pragma unroll
                for (int i = 0; i < kWinRowBatch; ++i) {
                    at[i] = (uint32_t)tp[i * stride] + lane2;
                    e2[i] = (uint32_t)tp[i * stride + 1];
                    w1[i] = P.W.w1[r0 + i];  // (zero behind the last row)
                    w2[i] = P.W.w2[r0 + i];
                }
#pragma unroll
                for (int i = 0; i < kWinRowBatch; ++i) {
                    const int r = min(r0 + i, last_row);
                    const int row_bytes = r * row_stride;  // (below 4 GiB, see span_bytes)
                    // (a lane past the stretch may point past the buffer: it reads 0 then)
                    ei[i] = __builtin_amdgcn_raw_buffer_load_b16(all_i, (int)at[i], row_bytes, 0);
                    ev[i] = __builtin_amdgcn_raw_buffer_load_b16(all_v, (int)at[i], row_bytes, 0);
                }
                // ---- then the sums, row after row.  What a lane past its stretch's end has
                //      read goes to the spare cell; +-0 values change nothing anywhere (the rows
                //      of a fresh window are all (0, 0), and a coordinate counts as named when a
                //      sum is not zero).
#pragma unroll
                for (int i = 0; i < kWinRowBatch; ++i) {
                    auto add = [&](uint32_t idx, uint32_t vb, bool mine) {
                        const uint32_t c = mine ? idx - (uint32_t)base : (uint32_t)kWinChunk;
                        const float v = bf2f(vb);
                        const float t1 = w1[i] * v;
                        const float vv = v * v;
                        const float t2 = w2[i] * vv;
                        float2 x = z[c];
                        x.x = x.x + t1;
                        x.y = x.y + t2;
                        z[c] = x;
                    };
                    add(ei[i], ev[i], at[i] < e2[i]);
                    if ((long_rows >> (r0 + i)) & 1u) {  // the rest of the stretch, before the next row
                        const int row_bytes = (r0 + i) * row_stride;
                        const uint32_t end = e2[i];
                        for (uint32_t a2 = at[i] + 2u * kWave; a2 < end; a2 += 2u * kWave) {
                            const uint32_t idx =
                                __builtin_amdgcn_raw_buffer_load_b16(all_i, (int)a2, row_bytes, 0);
                            const uint32_t vb =
                                __builtin_amdgcn_raw_buffer_load_b16(all_v, (int)a2, row_bytes, 0);
                            add(idx, vb, true);
                        }
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int h = 0; h < kPerLane / kChunk; ++h) {
                float a1[8], a2[8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 q =
                        reinterpret_cast<const float4 *>(z + lane * kPerLane + h * kChunk)[i];
                    a1[2 * i] = q.x;
                    a2[2 * i] = q.y;
                    a1[2 * i + 1] = q.z;
                    a2[2 * i + 1] = q.w;
                }
                if (off + h * kChunk < n) step8(off + h * kChunk, praw[h], a1, a2);
            }
            __builtin_amdgcn_wave_barrier();
        }
    } else {
        constexpr int kRange = 4096;
        float *z1 = sums, *z2 = sums + kRange;
        WindowView wv;
        wv.I = G.D.I + G.col0;
        wv.V = Vb;
        wv.k = k;
        wv.rows = rows;
        wv.cur_row = -1;
        wv.cur_idx = nullptr;
        wv.cur_val = nullptr;
        wv.w1 = P.W.w1;
        wv.w2 = P.W.w2;
        for (int lo = 0; lo < n; lo += kRange) {
            const int hi = lo + kRange < n ? lo + kRange : n;
            window_accumulate(wv, kb, lo, hi, z1, z2);
            for (int off = lo + tid * kChunk; off < hi; off += kWG * kChunk) {
                RawChunk<R> praw;
                praw.load(p, off, n, false);
                float a1[8], a2[8];
#pragma unroll
                for (int e = 0; e < kChunk; ++e) {
                    a1[e] = off + e < hi ? z1[off - lo + e] : 0.0f;
                    a2[e] = off + e < hi ? z2[off - lo + e] : 0.0f;
                }
                step8(off, praw, a1, a2);
            }
            __syncthreads();
        }
    }
}

// =============================================================================================
// Launchers
// =============================================================================================

constexpr int kLdsLimit = 160 * 1024;


template <class K>
static int allow_big_lds(K kernel, int bytes) {
    if (bytes <= 64 * 1024) return 0;
    return (int)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

constexpr int kWavesThreeWG = 3 * kWG / 256;  // three workgroups per CU
constexpr int kMinWaves = kWG / 128;  // waves per SIMD the block kernels are compiled for: two workgroups per CU

template <class R, int QL, bool DENSE = false, int WIN = kWinFused, int AUX = 0>
static int launch_fused_one(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    // bf16 blocks of up to 20480 elements fit 80 registers and a third of the LDS: three
    // workgroups per CU; the kernels with extras take the budget of two
    constexpr int kWaves_ =
        (R::kBF16 && R::kC <= kClass2 && AUX == 0) ? kWavesThreeWG : kMinWaves;
    // grid == 0: the preparation of the launch only (whatever may fail apart from the launch
    // itself), so that a call can prepare all its launches before the first one starts
    if (grid == 0) return allow_big_lds(fused_step_kernel<R, kWaves_, QL, DENSE, WIN, AUX>, lds_bytes);
    return launch_kernel(fused_step_kernel<R, kWaves_, QL, DENSE, WIN, AUX>, dim3(grid), kWG,
                         lds_bytes, s, P);
}

// the kernels with extras (logging, alpha == -2): one per class, any quantisation group
template <template <int> class RT, bool DENSE, int AUX>
static int launch_fused_aux(int C, unsigned grid, int lds_bytes, hipStream_t s,
                            const FusedParams &P) {
    switch (C) {
        case kClass0: return launch_fused_one<RT<kClass0>, 0, DENSE, kWinFused, AUX>(grid, lds_bytes, s, P);
        case kClass1: return launch_fused_one<RT<kClass1>, 0, DENSE, kWinFused, AUX>(grid, lds_bytes, s, P);
        case kClass2: return launch_fused_one<RT<kClass2>, 0, DENSE, kWinFused, AUX>(grid, lds_bytes, s, P);
        case kClass3: return launch_fused_one<RT<kClass3>, 0, DENSE, kWinFused, AUX>(grid, lds_bytes, s, P);
    }
    return MA_ERR_BLOCK_SIZE;
}

// alpha > 0
template <template <int> class RT>
static int launch_fused_dense(int C, unsigned grid, int lds_bytes, hipStream_t s,
                              const FusedParams &P) {
    if (C == kClass2 && P.q_shift == 6)
        return launch_fused_one<RT<kClass2>, 8, true>(grid, lds_bytes, s, P);
    if (C == kClass2 && P.q_shift == 5)
        return launch_fused_one<RT<kClass2>, 4, true>(grid, lds_bytes, s, P);
    switch (C) {
        case kClass0: return launch_fused_one<RT<kClass0>, 0, true>(grid, lds_bytes, s, P);
        case kClass1: return launch_fused_one<RT<kClass1>, 0, true>(grid, lds_bytes, s, P);
        case kClass2: return launch_fused_one<RT<kClass2>, 0, true>(grid, lds_bytes, s, P);
        case kClass3: return launch_fused_one<RT<kClass3>, 0, true>(grid, lds_bytes, s, P);
    }
    return MA_ERR_BLOCK_SIZE;
}

// the block kernels that leave window and parameters to window_param_kernel
template <template <int> class RT>
static int launch_fused_apart(int C, unsigned grid, int lds_bytes, hipStream_t s,
                              const FusedParams &P) {
    if (C == kClass2 && P.q_shift == 6)
        return launch_fused_one<RT<kClass2>, 8, false, kWinApart>(grid, lds_bytes, s, P);
    if (C == kClass2 && P.q_shift == 5)
        return launch_fused_one<RT<kClass2>, 4, false, kWinApart>(grid, lds_bytes, s, P);
    switch (C) {
        case kClass0: return launch_fused_one<RT<kClass0>, 0, false, kWinApart>(grid, lds_bytes, s, P);
        case kClass1: return launch_fused_one<RT<kClass1>, 0, false, kWinApart>(grid, lds_bytes, s, P);
        case kClass2: return launch_fused_one<RT<kClass2>, 0, false, kWinApart>(grid, lds_bytes, s, P);
        case kClass3: return launch_fused_one<RT<kClass3>, 0, false, kWinApart>(grid, lds_bytes, s, P);
    }
    return MA_ERR_BLOCK_SIZE;
}

template <class R>
static int launch_window_param(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    if (grid == 0) return allow_big_lds(window_param_kernel<R, kWavesThreeWG>, lds_bytes);
    return launch_kernel(window_param_kernel<R, kWavesThreeWG>, dim3(grid), kWG, lds_bytes, s, P);
}

template <template <int> class RT>
static int launch_fused(int C, unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P) {
    // the hardware-sized block gets kernels with the quantisation group size compiled in
    if (C == kClass2 && P.q_shift == 6) return launch_fused_one<RT<kClass2>, 8>(grid, lds_bytes, s, P);
    if (C == kClass2 && P.q_shift == 5) return launch_fused_one<RT<kClass2>, 4>(grid, lds_bytes, s, P);
    switch (C) {
        case kClass0: return launch_fused_one<RT<kClass0>, 0>(grid, lds_bytes, s, P);
        case kClass1: return launch_fused_one<RT<kClass1>, 0>(grid, lds_bytes, s, P);
        case kClass2: return launch_fused_one<RT<kClass2>, 0>(grid, lds_bytes, s, P);
        case kClass3: return launch_fused_one<RT<kClass3>, 0>(grid, lds_bytes, s, P);
    }
    return MA_ERR_BLOCK_SIZE;
}

template <class R, int AUX = 0>
static int launch_span_one(int pass, unsigned grid, int lds_bytes, hipStream_t s,
                           const FusedParams &P) {
    // the first pass has the register needs of the fused kernel
    constexpr int kFirst =
        (R::kBF16 && R::kC <= kClass2 && AUX == 0) ? kWavesThreeWG : kMinWaves;
    // grid == 0: the preparation only, as in launch_fused_one
#define MA_SPAN_CASE(PASS_, WAVES_, LDS_)                                                      \
    case PASS_:                                                                                \
        if (grid == 0) return allow_big_lds(span_step_kernel<R, WAVES_, PASS_, AUX>, LDS_);    \
        return launch_kernel(span_step_kernel<R, WAVES_, PASS_, AUX>, dim3(grid), kWG, LDS_, s, P);
    switch (pass) {
        MA_SPAN_CASE(1, kFirst, lds_bytes)
        MA_SPAN_CASE(2, kFirst, lds_bytes)
        MA_SPAN_CASE(4, kFirst, lds_bytes)
        MA_SPAN_CASE(3, kMinWaves, kMiscBytes)  // needs the kSh* words only
    }
    if constexpr (AUX == 0) {  // the one-pass form and its sweeps
        switch (pass) {
            MA_SPAN_CASE(6, kFirst, lds_bytes)
            MA_SPAN_CASE(8, kMinWaves, kMiscBytes)
        }
    }
#undef MA_SPAN_CASE
    return MA_ERR_ARG;
}

template <template <int> class RT, int AUX = 0>
static int launch_span(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                       const FusedParams &P) {
    switch (C) {
        case kClass0: return launch_span_one<RT<kClass0>, AUX>(pass, grid, lds_bytes, s, P);
        case kClass1: return launch_span_one<RT<kClass1>, AUX>(pass, grid, lds_bytes, s, P);
        case kClass2: return launch_span_one<RT<kClass2>, AUX>(pass, grid, lds_bytes, s, P);
        case kClass3: return launch_span_one<RT<kClass3>, AUX>(pass, grid, lds_bytes, s, P);
    }
    return MA_ERR_BLOCK_SIZE;
}

// The instantiations, one translation unit each.
int launch_fused_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P);
int launch_fused_f32(int C, unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P);
int launch_fused_apart_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s,
                            const FusedParams &P);
int launch_fused_apart_f32(int C, unsigned grid, int lds_bytes, hipStream_t s,
                           const FusedParams &P);
int launch_window_param_bf16(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P);
int launch_window_param_f32(unsigned grid, int lds_bytes, hipStream_t s, const FusedParams &P);
int launch_fused_dense_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s,
                            const FusedParams &P);
int launch_fused_dense_f32(int C, unsigned grid, int lds_bytes, hipStream_t s,
                           const FusedParams &P);
int launch_span_bf16(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                     const FusedParams &P);
int launch_span_f32(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                    const FusedParams &P);
// with extras: aux is a set of kAux* bits, not 0; dense and two-pass steps take kAuxLog only
int launch_fused_aux_bf16(int C, int aux, unsigned grid, int lds_bytes, hipStream_t s,
                          const FusedParams &P);
int launch_fused_aux_f32(int C, int aux, unsigned grid, int lds_bytes, hipStream_t s,
                         const FusedParams &P);
int launch_fused_dense_log_bf16(int C, unsigned grid, int lds_bytes, hipStream_t s,
                                const FusedParams &P);
int launch_fused_dense_log_f32(int C, unsigned grid, int lds_bytes, hipStream_t s,
                               const FusedParams &P);
int launch_span_log_bf16(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                         const FusedParams &P);
int launch_span_log_f32(int C, int pass, unsigned grid, int lds_bytes, hipStream_t s,
                        const FusedParams &P);

}  // namespace ma
