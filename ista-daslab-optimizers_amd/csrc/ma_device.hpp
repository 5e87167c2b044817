// Device-side building blocks of the MicroAdam step for gfx950 (wave64, 160 KB LDS per CU).
//
// One workgroup of kWG = 512 threads (8 waves, two per SIMD) owns one top-k block of up to
// kRound*C = 4096*C elements and keeps it in VGPRs for the whole step.  Wave w, chunk c, lane l holds
// the 8 consecutive elements starting at ((w*C + c)*64 + l)*8, so every 128-bit load of a
// wave covers one contiguous KiB (bf16) and the block's index order is (wave, chunk, lane,
// element).  Elements past the block's length read as +0.0, which the lowest-index tie rule
// makes harmless for the selection: a padded zero can never rank before a real element.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ma {

// Launches `kernel` and returns what the runtime says about THIS launch (0, or a hipError_t).
// The arguments are converted to the kernel's own parameter types.  (The <<< >>> form reports
// nothing itself, and hipGetLastError() after it returns, and clears, whatever error any earlier
// call of the thread left behind.)
template <class T>
struct launch_arg {
    typedef T type;
};
template <class... P>
static inline int launch_kernel(void (*kernel)(P...), dim3 grid, unsigned block, size_t lds_bytes,
                                hipStream_t stream, typename launch_arg<P>::type... args) {
    void *argv[] = {const_cast<void *>(static_cast<const void *>(&args))...};
    return (int)hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, dim3(block), argv,
                                lds_bytes, stream);
}

constexpr int kWG = 512;  // threads per workgroup of the block kernels
constexpr int kWave = 64;
constexpr int kWaves = kWG / kWave;
constexpr int kChunk = 8;        // elements per lane per chunk
constexpr int kRound = kWG * kChunk;  // elements one chunk of every thread covers together
// register-tile classes: chunks per thread for blocks up to 4096 / ~10-12 K / 20480 / 32768
constexpr int kClass0 = 1;
constexpr int kClass1 = 3;
constexpr int kClass2 = 5;
constexpr int kClass3 = 8;
// words of the small LDS scratch every block kernel has at offset 0
constexpr int kShScan = 0;      // 8 words: per-wave partial sums
constexpr int kShCounter = 8;   // slot allocation counter of the window pass
constexpr int kShPivot = 9;     // radix select: digit of the pivot bin
constexpr int kShNeed = 10;     //               keys still to take inside it
constexpr int kShNEq = 11;      //               keys in the pivot bin
constexpr int kShTies = 12;     // fast top-k: tie list length
constexpr int kShLinks = 13;    // window pass: link cells handed out
constexpr int kShCnts = 16;     // 8 words: candidates per wave
constexpr int kShSel = 24;      // 8 words: (pivot digit, keys still to take) per radix pass of
                                //          the two selections of the fast top-k
constexpr int kShW1 = 32;       // 16 words: beta1^age of the window rows
constexpr int kShW2 = 48;       // 16 words: beta2^age of the window rows
constexpr int kHistCopies = 32;  // LDS histogram replicas, one per bank
constexpr int kMaxWindow = 64;

// The thread id as a value the optimiser cannot see through.  The selection helpers derive
// their lane offsets from this, so that the offsets are rebuilt where they are used instead
// of being computed once and kept in long-lived registers.
__device__ __forceinline__ int opaque_tid() {
    int t = (int)threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

// ---- scalar helpers -----------------------------------------------------------------------

__device__ __forceinline__ float bf2f(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t f2bf(float f) {
    __bf16 b = (__bf16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ uint32_t f2bf_pair(float lo, float hi) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    f2 v = {lo, hi};
    b2 r = __builtin_convertvector(v, b2);
    return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ uint32_t mbcnt(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Value of the DPP source lane, 0 where the pattern has no source or the lane is masked off.
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ uint32_t dpp_or0(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, BANK_MASK, false);
}

// Inclusive prefix sum over the 64 lanes, all in the VALU (no LDS round trips).
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v, int lane) {
    (void)lane;
    v += dpp_or0<0x111>(v);             // row_shr:1
    v += dpp_or0<0x112>(v);             // row_shr:2
    v += dpp_or0<0x114, 0xF, 0xE>(v);   // row_shr:4, lanes 4..15 of each row
    v += dpp_or0<0x118, 0xF, 0xC>(v);   // row_shr:8, lanes 8..15 of each row
    v += dpp_or0<0x142, 0xA>(v);        // row_bcast:15 into rows 1 and 3
    v += dpp_or0<0x143, 0xC>(v);        // row_bcast:31 into rows 2 and 3
    return v;
}

// min / max of two numbers that are not NaN, one instruction each.  (fminf / fmaxf, and the
// median-of-three builtin with an infinity, are lowered with a re-quieting of both operands.)
__device__ __forceinline__ float fmin_raw(float a, float b) {
    float d;
    asm("v_min_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float fmax_raw(float a, float b) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}

// the same of three numbers, still one instruction
__device__ __forceinline__ float fmin3_raw(float a, float b, float c) {
    float d;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
__device__ __forceinline__ float fmax3_raw(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
// min and max of the 8 values of a chunk: four instructions each
__device__ __forceinline__ void minmax8(const float (&x)[8], float &mn, float &mx) {
    mn = fmin_raw(fmin3_raw(fmin3_raw(fmin3_raw(x[0], x[1], x[2]), x[3], x[4]), x[5], x[6]), x[7]);
    mx = fmax_raw(fmax3_raw(fmax3_raw(fmax3_raw(x[0], x[1], x[2]), x[3], x[4]), x[5], x[6]), x[7]);
}

template <int CTRL>
__device__ __forceinline__ float dpp_perm(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// mn = min(mn, mn of the lane the pattern names), mx likewise: one instruction each, the
// cross-lane read folded into the operation.  (A vector write followed by a cross-lane read of
// the same register needs two idle issue slots in between, which the compiler cannot see
// inside an asm statement: the s_nop provides them.)
#define MA_DPP_MINMAX(NAME, PATTERN)                                                       \
    __device__ __forceinline__ void NAME(float &mn, float &mx) {                           \
        asm volatile("s_nop 1\n\t"                                                         \
                     "v_min_f32_dpp %0, %0, %0 " PATTERN " row_mask:0xf bank_mask:0xf\n\t" \
                     "v_max_f32_dpp %1, %1, %1 " PATTERN " row_mask:0xf bank_mask:0xf"      \
                     : "+v"(mn), "+v"(mx));                                                \
    }
MA_DPP_MINMAX(minmax_swap1, "quad_perm:[1,0,3,2]")
MA_DPP_MINMAX(minmax_swap2, "quad_perm:[2,3,0,1]")
MA_DPP_MINMAX(minmax_half_mirror, "row_half_mirror")
MA_DPP_MINMAX(minmax_mirror, "row_mirror")
#undef MA_DPP_MINMAX

// min / max over aligned groups of `ql` lanes (a power of two), result in every lane.
// QL > 0 fixes the group size at compile time; QL == 0 takes it from `ql`.
template <int QL>
__device__ __forceinline__ void group_minmax(float &mn, float &mx, int ql_runtime) {
    const int ql = QL > 0 ? QL : ql_runtime;
    if (ql >= 2) minmax_swap1(mn, mx);
    if (ql >= 4) minmax_swap2(mn, mx);
    if (ql >= 8) minmax_half_mirror(mn, mx);
    if (ql >= 16) minmax_mirror(mn, mx);
    for (int s = 16; s < ql; s <<= 1) {
        mn = fmin_raw(mn, __shfl_xor(mn, s, kWave));
        mx = fmax_raw(mx, __shfl_xor(mx, s, kWave));
    }
}

// Inclusive scan over the workgroup in thread order.  sh4 is kWaves words of LDS.
__device__ __forceinline__ uint32_t wg_incl_scan(uint32_t v, uint32_t *sh4, int lane, int wave) {
    uint32_t s = wave_incl_scan(v, lane);
    if (lane == kWave - 1) sh4[wave] = s;
    __syncthreads();
    uint32_t add = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
        if (w < wave) add += sh4[w];
    __syncthreads();
    return s + add;
}

// ---- a top-k block in registers ------------------------------------------------------------

template <int C>
struct RegsBF16 {
    static constexpr int kC = C;
    static constexpr bool kBF16 = true;
    static constexpr int kElemBytes = 2;
    typedef uint16_t elem_t;
    uint32_t w[C][4];         // two bf16 per register

    __device__ __forceinline__ uint32_t key(int c, int e) const {
        uint32_t x = w[c][e >> 1];
        return (e & 1) ? ((x >> 16) & 0x7fffu) : (x & 0x7fffu);
    }
    __device__ __forceinline__ float val(int c, int e) const {
        uint32_t x = w[c][e >> 1];
        return __uint_as_float((e & 1) ? (x & 0xffff0000u) : (x << 16));
    }
    __device__ __forceinline__ uint32_t bf16_bits(int c, int e) const {
        uint32_t x = w[c][e >> 1];
        return (e & 1) ? (x >> 16) : (x & 0xffffu);
    }
    __device__ __forceinline__ void zero(int c, int e) {
        w[c][e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
    }
    __device__ __forceinline__ void set_chunk(int c, const float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) w[c][i] = f2bf_pair(v[2 * i], v[2 * i + 1]);
    }
};

template <int C>
struct RegsF32 {
    static constexpr int kC = C;
    static constexpr bool kBF16 = false;
    static constexpr int kElemBytes = 4;
    typedef float elem_t;
    float w[C][8];

    __device__ __forceinline__ uint32_t key(int c, int e) const {
        return __float_as_uint(w[c][e]) & 0x7fffffffu;
    }
    __device__ __forceinline__ float val(int c, int e) const { return w[c][e]; }
    __device__ __forceinline__ uint32_t bf16_bits(int c, int e) const { return f2bf(w[c][e]); }
    __device__ __forceinline__ void zero(int c, int e) { w[c][e] = 0.0f; }
    __device__ __forceinline__ void set_chunk(int c, const float (&v)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) w[c][i] = v[i];
    }
};

// element offset of (wave, chunk, lane) inside the block
template <int C>
__device__ __forceinline__ int chunk_off(int wave, int c, int lane) {
    return ((wave * C + c) * kWave + lane) * kChunk;
}

// Load 8 consecutive elements as fp32.  `vec` says the 16-byte path is legal for this block
// (base 16-byte aligned); chunks that cross the block's end go element by element and
// elements past `n` read as +0.0.
__device__ __forceinline__ void load8(const uint16_t *base, int off, int n, bool vec,
                                      float (&v)[8]) {
    if (vec && off + kChunk <= n) {
        uint4 q = *reinterpret_cast<const uint4 *>(base + off);
        uint32_t r[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(r[i] << 16);
            v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (off + i < n) ? bf2f(base[off + i]) : 0.0f;
    }
}

__device__ __forceinline__ void load8(const float *base, int off, int n, bool vec,
                                      float (&v)[8]) {
    if (vec && off + kChunk <= n) {
        float4 a = *reinterpret_cast<const float4 *>(base + off);
        float4 b = *reinterpret_cast<const float4 *>(base + off + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (off + i < n) ? base[off + i] : 0.0f;
    }
}

// Store 8 consecutive elements given as fp32, rounding to the element type.
__device__ __forceinline__ void store8(uint16_t *base, int off, int n, bool vec,
                                       const float (&v)[8]) {
    if (vec && off + kChunk <= n) {
        uint4 q;
        q.x = f2bf_pair(v[0], v[1]);
        q.y = f2bf_pair(v[2], v[3]);
        q.z = f2bf_pair(v[4], v[5]);
        q.w = f2bf_pair(v[6], v[7]);
        // written once, not read again by this kernel: streamed past the caches
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u4 t = {q.x, q.y, q.z, q.w};
        __builtin_nontemporal_store(t, reinterpret_cast<u4 *>(base + off));
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (off + i < n) base[off + i] = (uint16_t)f2bf(v[i]);
    }
}

__device__ __forceinline__ void store8(float *base, int off, int n, bool vec,
                                       const float (&v)[8]) {
    if (vec && off + kChunk <= n) {
        *reinterpret_cast<float4 *>(base + off) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(base + off + 4) = make_float4(v[4], v[5], v[6], v[7]);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (off + i < n) base[off + i] = v[i];
    }
}

template <class R>
__device__ __forceinline__ void load_block(R &r, const typename R::elem_t *base, int n, bool vec,
                                           int wave, int lane) {
#pragma unroll
    for (int c = 0; c < R::kC; ++c) {
        float v[8];
        load8(base, chunk_off<R::kC>(wave, c, lane), n, vec, v);
        r.set_chunk(c, v);
    }
}

// Keeps the compiler from carrying values derived from the block registers (unpacked keys,
// widened floats) from one phase into the next: after this it only knows the registers.
template <class R>
__device__ __forceinline__ void launder(R &r) {
#pragma unroll
    for (int c = 0; c < R::kC; ++c) {
#pragma unroll
        for (int i = 0; i < (R::kBF16 ? 4 : 8); ++i) asm volatile("" : "+v"(r.w[c][i]));
    }
}

// ---- threshold search: MSD radix select over the magnitude bits -----------------------------
//
// Finds the key T of the kb-th largest magnitude and how many entries equal to T belong to
// the top kb (`take_eq` >= 1).  Each pass histograms one digit of the keys that still match
// the prefix into `hist`, 2^copies_log2 replicated copies per bin (32 where the LDS allows it, so
// that every lane adds into its own bank whatever the data look like), then scans the bins
// from the top.
//   hist: 257 << copies_log2 words (bin 256 is a discard bin), sh: 8 words.  Ends with a barrier.
template <class R>
__device__ __forceinline__ void select_threshold(R &r, int kb, uint32_t *hist, uint32_t *sh,
                                                 uint32_t &T, int &take_eq, int copies_log2) {
    const int copies = 1 << copies_log2;
    constexpr int kPasses = R::kBF16 ? 2 : 4;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    uint32_t prefix = 0, pmask = 0;
    int need = kb;
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
        const int bits = (pass == kPasses - 1) ? 7 : 8;
        const int shift = R::kBF16 ? (pass == 0 ? 7 : 0) : (pass == 3 ? 0 : 23 - 8 * pass);
        const int nb = 1 << bits;
        const uint32_t dm = nb - 1;
        for (int i = tid; i < (nb + 1) * copies; i += kWG) hist[i] = 0;
        launder(r);
        __syncthreads();
#pragma unroll
        for (int c = 0; c < R::kC; ++c) {
#pragma unroll
            for (int e = 0; e < kChunk; ++e) {
                const uint32_t key = r.key(c, e);
                // keys off the prefix count into a spare bin: cheaper than branching
                const uint32_t bin = (key & pmask) == prefix ? ((key >> shift) & dm) : 256u;
                atomicAdd(&hist[(bin << copies_log2) + (lane & (copies - 1))], 1u);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        // thread tid owns bin nb-1-tid so that a forward scan walks the bins from the top
        const int bin = nb - 1 - tid;
        uint32_t cnt = 0;
        if (bin >= 0) {
            for (int j = 0; j < copies; ++j)
                cnt += hist[(bin << copies_log2) + ((j + tid) & (copies - 1))];
        }
        uint32_t incl = wg_incl_scan(cnt, sh, lane, wave);
        uint32_t excl = incl - cnt;
        if (bin >= 0 && excl < (uint32_t)need && (uint32_t)need <= incl) {
            sh[kShPivot] = (uint32_t)bin;
            sh[kShNeed] = (uint32_t)need - excl;
        }
        __syncthreads();
        prefix |= sh[kShPivot] << shift;
        pmask |= dm << shift;
        need = (int)sh[kShNeed];
    }
    __syncthreads();
    T = prefix;
    take_eq = need;
}

// ---- top-k through thread maxima (bf16, k much smaller than the block) -------------------------
//
// Every thread keeps the largest key of each of its 8-element chunks, and the largest of those.
// If L is the kb-th largest thread maximum, at least kb threads hold an element >= L, so the
// kb-th largest element T satisfies T >= L: every member of the top-k has key >= L.  For k = 1 %
// of the block about 1.3 k elements pass that test (only chunks whose maximum reaches L are
// looked at again), and the exact top-k (magnitude first, lowest index on ties) is then taken
// among those few candidates.  The block itself waits in LDS meanwhile.

// largest 15-bit magnitude key among the 8 bf16 values of a chunk
__device__ __forceinline__ uint32_t chunk_max_key(const uint32_t (&w)[4]) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    us2 k0 = __builtin_bit_cast(us2, w[0] & 0x7fff7fffu);
    us2 k1 = __builtin_bit_cast(us2, w[1] & 0x7fff7fffu);
    us2 k2 = __builtin_bit_cast(us2, w[2] & 0x7fff7fffu);
    us2 k3 = __builtin_bit_cast(us2, w[3] & 0x7fff7fffu);
    k0 = __builtin_elementwise_max(k0, k1);
    k2 = __builtin_elementwise_max(k2, k3);
    k0 = __builtin_elementwise_max(k0, k2);
    const uint32_t m = __builtin_bit_cast(uint32_t, k0);
    const uint32_t lo = m & 0xffffu, hi = m >> 16;
    return lo > hi ? lo : hi;
}

constexpr int kSmallCopies = 2;
constexpr int kSmallHistWords = 2 * 257 * kSmallCopies;  // one histogram per pass

// kb-th largest of the N * 256 keys (15 bits each) held N per thread; 1 <= kb <= N * 256.
// Two radix passes (8 + 7 bits).  Every thread counts its keys into a replicated LDS
// histogram; wave 0 alone then walks the 256 bins from the top (4 bins per lane, a DPP prefix
// sum across lanes) and publishes the digit that holds the kb-th key, which costs two
// barriers per pass instead of a workgroup-wide scan.
//   hist: kSmallHistWords words, all zero, and all threads past the barrier that says so;
//   shp: 4 words of its own per call.  Ends with the barrier after the second walk: a caller
//   that uses the same hist / shp words again puts a barrier in between.
//   valid: bit i set if v[i] takes part.  take_eq: how many keys equal to the result belong
//   to the top kb; n_eq: how many keys equal it in all.
template <int N>
__device__ __forceinline__ uint32_t select_kth_key15(const uint32_t (&v)[N], uint32_t valid,
                                                     int kb, uint32_t *hist, uint32_t *shp,
                                                     uint32_t *sh_neq, int &take_eq, int &n_eq) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    uint32_t prefix = 0, pmask = 0;
    int need = kb;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int shift = pass == 0 ? 7 : 0;
        const uint32_t dm = pass == 0 ? 255u : 127u;
        uint32_t *h = hist + pass * 257 * kSmallCopies;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const bool in = ((valid >> i) & 1u) != 0 && (v[i] & pmask) == prefix;
            const uint32_t bin = in ? ((v[i] >> shift) & dm) : 256u;
            atomicAdd(&h[bin * kSmallCopies + (lane & (kSmallCopies - 1))], 1u);
        }
        __syncthreads();
        if (wave == 0) {
            // lane l owns bins 255-4l .. 252-4l (bins above dm are empty in the second pass)
            uint32_t c[4], tot = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int bin = 255 - 4 * lane - i;
                c[i] = 0;
#pragma unroll
                for (int k = 0; k < kSmallCopies; ++k) c[i] += h[bin * kSmallCopies + k];
                tot += c[i];
            }
            const uint32_t incl = wave_incl_scan(tot, lane);
            uint32_t above = incl - tot;  // keys in bins above this lane's
            if (above < (uint32_t)need && (uint32_t)need <= incl) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (above < (uint32_t)need && (uint32_t)need <= above + c[i]) {
                        shp[2 * pass] = (uint32_t)(255 - 4 * lane - i);
                        shp[2 * pass + 1] = (uint32_t)need - above;
                        *sh_neq = c[i];
                    }
                    above += c[i];
                }
            }
        }
        __syncthreads();
        prefix |= shp[2 * pass] << shift;
        pmask |= dm << shift;
        need = (int)shp[2 * pass + 1];
    }
    take_eq = need;
    n_eq = (int)*sh_neq;
    return prefix;
}

// The same selection in one pass for keys known to be at least `base`: the digit is
// min(key - base, 255), so every bin below 255 is one key value.  Returns the kb-th largest key
// as select_kth_key15 does, or 0xffffffff if it fell into the bin of the keys base + 255 and
// above (then nothing else is valid either).  hist: 257 * kSmallCopies zero words; shp: 2 words.
__device__ __forceinline__ uint32_t walk_near_bins(int kb, uint32_t base, const uint32_t *hist,
                                                   uint32_t *shp, uint32_t *sh_neq, int &take_eq,
                                                   int &n_eq);

template <int N>
__device__ __forceinline__ uint32_t select_kth_near(const uint32_t (&v)[N], uint32_t valid,
                                                    int kb, uint32_t base, uint32_t *hist,
                                                    uint32_t *shp, uint32_t *sh_neq,
                                                    int &take_eq, int &n_eq) {
    const int tid = opaque_tid(), lane = tid & 63;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const uint32_t off = v[i] - base;
        const uint32_t bin = ((valid >> i) & 1u) != 0 ? (off < 255u ? off : 255u) : 256u;
        atomicAdd(&hist[bin * kSmallCopies + (lane & (kSmallCopies - 1))], 1u);
    }
    __syncthreads();
    return walk_near_bins(kb, base, hist, shp, sh_neq, take_eq, n_eq);
}

// Second half of select_kth_near: the bins are filled (and a barrier has passed); wave 0 walks
// them from the top.  shp[0] must hold 255 beforehand if fewer than kb keys may have been counted.
__device__ __forceinline__ uint32_t walk_near_bins(int kb, uint32_t base, const uint32_t *hist,
                                                   uint32_t *shp, uint32_t *sh_neq, int &take_eq,
                                                   int &n_eq) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    if (wave == 0) {
        uint32_t c[4], tot = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int bin = 255 - 4 * lane - i;
            c[i] = 0;
#pragma unroll
            for (int k = 0; k < kSmallCopies; ++k) c[i] += hist[bin * kSmallCopies + k];
            tot += c[i];
        }
        const uint32_t incl = wave_incl_scan(tot, lane);
        uint32_t above = incl - tot;
        if (above < (uint32_t)kb && (uint32_t)kb <= incl) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (above < (uint32_t)kb && (uint32_t)kb <= above + c[i]) {
                    shp[0] = (uint32_t)(255 - 4 * lane - i);
                    shp[1] = (uint32_t)kb - above;
                    *sh_neq = c[i];
                }
                above += c[i];
            }
        }
    }
    __syncthreads();
    const uint32_t bin = shp[0];
    take_eq = (int)shp[1];
    n_eq = (int)*sh_neq;
    return bin < 255u ? base + bin : 0xffffffffu;
}

constexpr int kCandPerWave = 512 / kWaves;  // candidate slots per wave (a multiple of 16); more falls back

template <int CAP, class R>
__device__ __forceinline__ bool topk_among_candidates(R &r, int kb, uint16_t *park,
                                                      uint32_t *hist, uint32_t *sh,
                                                      uint16_t *sel_idx, uint16_t *sel_val,
                                                      uint32_t filled, uint32_t at_least,
                                                      const uint32_t *lists, uint16_t *ties,
                                                      uint32_t key_base);

// min over the 64 lanes, in lane 63 (DPP only)
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ uint32_t dpp_or_ones(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)v, CTRL, ROW_MASK, BANK_MASK, false);
}
__device__ __forceinline__ uint32_t wave_min_to_last(uint32_t v) {
    v = min(v, dpp_or_ones<0x111>(v));
    v = min(v, dpp_or_ones<0x112>(v));
    v = min(v, dpp_or_ones<0x114, 0xF, 0xE>(v));
    v = min(v, dpp_or_ones<0x118, 0xF, 0xC>(v));
    v = min(v, dpp_or_ones<0x142, 0xA>(v));
    v = min(v, dpp_or_ones<0x143, 0xC>(v));
    return v;
}

// The fast top-k with a lower bound known beforehand.  `hint` is a 15-bit magnitude key held
// by the threads that have one (others pass 0x7fff); the smallest of them, lowered by a
// thirty-second, is tried as the bound L: every element with key >= L becomes a candidate, and if
// at least kb turn up (so the kb-th largest is among them) and they fit the lists, the exact
// top-kb is taken among them as in fast_topk_bf16.  Callers pass the magnitudes of the entries
// the previous step selected from this block: their smallest is that step's threshold, and
// thresholds of successive steps differ by a per cent or so.  Any hint gives the same selection
// or a refusal (false, r unchanged): a hint that is too high finds fewer than kb candidates, one
// that is too low overflows the lists.  Candidates are listed in the order (wave, lane, chunk,
// element).  hist, sh, park as in fast_topk_bf16.
template <class R>
__device__ __forceinline__ bool hint_topk_bf16(R &r, int kb, uint32_t hint, uint16_t *park,
                                               uint32_t *hist, uint32_t *sh, uint16_t *sel_idx,
                                               uint16_t *sel_val) {
    constexpr int C = R::kC;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    const uint32_t wmin = wave_min_to_last(hint);
    if (lane == kWave - 1) sh[kShScan + wave] = wmin;
    // only the second histogram is used here; the candidate lists take the place of the first
    for (int i = tid; i < kSmallHistWords; i += kWG) hist[kSmallHistWords + i] = 0;
    __syncthreads();
    uint32_t hmin = 0x7fffu;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) hmin = min(hmin, sh[kShScan + w]);
    // L = hmin lowered by 1/32, as a key (truncation only lowers it further)
    const float lf = __uint_as_float(hmin << 16) * 0.96875f;
    const uint32_t L = __float_as_uint(lf) >> 16;
    const uint32_t LL = L | L << 16;
    // Flags of the elements with key >= L: bit 15 of (key | 0x8000) - L in each 16-bit half.
    // Byte B of flo holds, for chunk c = 0..3, element B at bit 2c and element 4 + B at bit
    // 2c + 1; fhi the same for the chunks above.
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    static_assert(C <= 8, "two words of flags");
    uint32_t flo = 0, fhi = 0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        uint32_t t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const us2 a = __builtin_bit_cast(us2, (r.w[c][i] & 0x7fff7fffu) | 0x80008000u);
            t[i] = __builtin_bit_cast(uint32_t, (us2)(a - __builtin_bit_cast(us2, LL)));
        }
        // the bytes whose top bits are the flags: elements 0..3 -> x, elements 4..7 -> y
        const uint32_t x = __builtin_amdgcn_perm(t[1], t[0], 0x07050301u) & 0x80808080u;
        const uint32_t y = __builtin_amdgcn_perm(t[3], t[2], 0x07050301u) & 0x80808080u;
        const uint32_t z = (x >> 7) | (y >> 6);
        if (c < 4) flo |= z << (2 * c);
        else fhi |= z << (2 * (c - 4));
        const int off = chunk_off<C>(wave, c, lane);
        *reinterpret_cast<uint4 *>(park + off) =
            make_uint4(r.w[c][0], r.w[c][1], r.w[c][2], r.w[c][3]);
    }
    const uint32_t cnt = (uint32_t)(__popc(flo) + __popc(fhi));
    const uint32_t incl = wave_incl_scan(cnt, lane);
    const uint32_t filled = (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    constexpr int kCap = 128;  // list slots per wave
    static_assert(kCap * kWaves <= kSmallHistWords, "the lists take the first histogram's place");
    uint32_t *mine = hist + wave * kCap;
    if (filled <= (uint32_t)kCap) {
        // one candidate per lane and turn, lowest flag first; its key is read back from the
        // parked block (the lane's own cells)
        uint32_t pos = incl - cnt;
        const int off0 = chunk_off<C>(wave, 0, lane);
        while (__builtin_amdgcn_ballot_w64((flo | fhi) != 0) != 0) {
            const bool low = flo != 0;
            const uint32_t f = low ? flo : fhi;
            if (f != 0) {
                const int b = __ffs(f) - 1;
                if (low) flo &= flo - 1;
                else fhi &= fhi - 1;
                const int c = ((b >> 1) & 3) + (low ? 0 : 4);
                const int e = (b >> 3) + 4 * (b & 1);
                const int off = off0 + c * (kWave * kChunk) + e;
                const uint32_t key = park[off] & 0x7fffu;
                mine[pos] = (key << 15) | (uint32_t)(32767 - off);
                ++pos;
            }
        }
    }
    if (lane == 0) sh[kShCnts + wave] = filled;
    __syncthreads();
    return topk_among_candidates<kCap>(r, kb, park, hist, sh, sel_idx, sel_val, filled,
                                       (uint32_t)kb, hist,
                                       reinterpret_cast<uint16_t *>(hist + 2 * kSmallHistWords),
                                       L);
}

// The threshold of a full bf16 block's kb largest magnitudes from a lower bound known
// beforehand, for selections too long for the candidate lists of hint_topk_bf16 (which then
// take compact_selected).  `hint` as there.  The elements with key >= L are counted by key - L,
// straight from the registers, in the bins of select_kth_near; true with (T, take_eq) as
// select_threshold gives them, false (uniformly) if fewer than kb elements reach L, the kb-th
// largest lies 255 key steps or more above L, or there is no usable hint.  Any hint gives the
// same threshold or a refusal.  hist: 257 * kSmallCopies words; sh: the kSh* words.
template <class R>
__device__ __forceinline__ bool hint_threshold_bf16(const R &r, int kb, uint32_t hint,
                                                    uint32_t *hist, uint32_t *sh, uint32_t &T,
                                                    int &take_eq) {
    constexpr int C = R::kC;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    const uint32_t wmin = wave_min_to_last(hint);
    if (lane == kWave - 1) sh[kShScan + wave] = wmin;
    for (int i = tid; i < 257 * kSmallCopies; i += kWG) hist[i] = 0;
    if (tid == 0) {
        sh[kShSel] = 255u;  // stays if fewer than kb elements are counted
        sh[kShSel + 1] = 0u;
    }
    __syncthreads();
    uint32_t hmin = 0x7fffu;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) hmin = min(hmin, sh[kShScan + w]);
    const float lf = __uint_as_float(hmin << 16) * 0.96875f;
    const uint32_t L = __float_as_uint(lf) >> 16;
    bool usable = L != 0 && hmin != 0x7fffu;  // (a fresh window's rows are all zero)
    if (usable) {
        const uint32_t LL = L | L << 16;
        typedef unsigned short us2 __attribute__((ext_vector_type(2)));
        uint32_t *mine = hist + (lane & (kSmallCopies - 1));
#pragma unroll
        for (int c = 0; c < C; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // per 16-bit half: (key | 0x8000) - L has bit 15 set exactly when key >= L, and
                // then key - L below it
                const us2 a = __builtin_bit_cast(us2, (r.w[c][i] & 0x7fff7fffu) | 0x80008000u);
                const uint32_t t = __builtin_bit_cast(uint32_t, (us2)(a - __builtin_bit_cast(us2, LL)));
                if (t & 0x8000u) atomicAdd(mine + min(t & 0x7fffu, 255u) * kSmallCopies, 1u);
                if (t & 0x80000000u)
                    atomicAdd(mine + min((t >> 16) & 0x7fffu, 255u) * kSmallCopies, 1u);
            }
        }
    }
    __syncthreads();
    int n_eq;
    const uint32_t found =
        walk_near_bins(kb, L, hist, sh + kShSel, sh + kShNEq, take_eq, n_eq);
    T = found;
    return usable && found != 0xffffffffu;
}

// Flags of the elements of a register-resident bf16 block whose key is at least `bound` (a
// 15-bit key, or 0x8000 for "none").  Byte B of `lo` holds, for chunk c = 0..3, element B at bit
// 2c and element 4 + B at bit 2c + 1; `hi` the same for the chunks above.
template <class R>
__device__ __forceinline__ void flags_at_least(const R &r, uint32_t bound, uint32_t &lo,
                                               uint32_t &hi) {
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    static_assert(R::kC <= 8, "two words of flags");
    const uint32_t BB = bound | bound << 16;
    lo = hi = 0;
#pragma unroll
    for (int c = 0; c < R::kC; ++c) {
        uint32_t t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // per 16-bit half: bit 15 of (key | 0x8000) - bound says key >= bound
            const us2 a = __builtin_bit_cast(us2, (r.w[c][i] & 0x7fff7fffu) | 0x80008000u);
            t[i] = __builtin_bit_cast(uint32_t, (us2)(a - __builtin_bit_cast(us2, BB)));
        }
        // the bytes whose top bits are the flags: elements 0..3 -> x, elements 4..7 -> y
        const uint32_t x = __builtin_amdgcn_perm(t[1], t[0], 0x07050301u) & 0x80808080u;
        const uint32_t y = __builtin_amdgcn_perm(t[3], t[2], 0x07050301u) & 0x80808080u;
        const uint32_t z = (x >> 7) | (y >> 6);
        if (c < 4) lo |= z << (2 * c);
        else hi |= z << (2 * (c - 4));
    }
}

// The block top-k of a full bf16 block with a lower bound known beforehand (as hint_topk_bf16
// takes it), for selections too long for candidate lists, and with the entries listed by
// increasing coordinate, which is the order compact_selected gives and window_param_kernel
// relies on.  The block is parked in `park` (kRound * C uint16 cells); the elements with key >= L
// are counted by key - L in the bins of select_kth_near (one turn per flagged element of a
// lane, so a few turns instead of one step per element); with the threshold T known, every
// lane ranks its own elements >= T from the flags alone (counts per chunk, a scan over the
// lanes per chunk, the waves' totals), moves the selected ones to sel_idx / sel_val and clears
// them in the parked block, from which r is read back.  Ties at T go to the lowest coordinates.
// False (uniformly, r unchanged) if fewer than kb elements reach L, the kb-th largest lies 255
// key steps or more above L, or there is no usable hint; any hint gives the same selection or a
// refusal.  hist: 257 * kSmallCopies words; sh: the kSh* words.  Ends with a barrier.
template <class R>
__device__ __forceinline__ bool hint_sorted_topk_bf16(R &r, int kb, uint32_t hint, uint16_t *park,
                                                      uint32_t *hist, uint32_t *sh,
                                                      uint16_t *sel_idx, uint16_t *sel_val) {
    constexpr int C = R::kC;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    const uint32_t wmin = wave_min_to_last(hint);
    if (lane == kWave - 1) sh[kShScan + wave] = wmin;
    for (int i = tid; i < 257 * kSmallCopies; i += kWG) hist[i] = 0;
    if (tid == 0) {
        sh[kShSel] = 255u;  // stays if fewer than kb elements are counted
        sh[kShSel + 1] = 0u;
    }
    __syncthreads();
    uint32_t hmin = 0x7fffu;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) hmin = min(hmin, sh[kShScan + w]);
    const float lf = __uint_as_float(hmin << 16) * 0.96875f;
    const uint32_t L = __float_as_uint(lf) >> 16;
    if (L == 0 || hmin == 0x7fffu) return false;  // (a fresh window's rows are all zero)

    const int off0 = chunk_off<C>(wave, 0, lane);
    // element behind flag bit b of the low / high word: chunk, then offset in the block
    auto offset_of = [&](int b, bool low) {
        const int c = ((b >> 1) & 3) + (low ? 0 : 4);
        const int e = (b >> 3) + 4 * (b & 1);
        return off0 + c * (kWave * kChunk) + e;
    };
#pragma unroll
    for (int c = 0; c < C; ++c)
        *reinterpret_cast<uint4 *>(park + chunk_off<C>(wave, c, lane)) =
            make_uint4(r.w[c][0], r.w[c][1], r.w[c][2], r.w[c][3]);
    uint32_t flo, fhi;
    flags_at_least(r, L, flo, fhi);
    uint32_t *mine = hist + (lane & (kSmallCopies - 1));
    while (__builtin_amdgcn_ballot_w64((flo | fhi) != 0) != 0) {
        const bool low = flo != 0;
        const uint32_t f = low ? flo : fhi;
        if (f != 0) {
            const int b = __ffs(f) - 1;
            if (low) flo &= flo - 1;
            else fhi &= fhi - 1;
            const uint32_t key = park[offset_of(b, low)] & 0x7fffu;  // (the lane's own cell)
            atomicAdd(mine + min(key - L, 255u) * kSmallCopies, 1u);
        }
    }
    __syncthreads();
    int take_eq, n_eq;
    const uint32_t T = walk_near_bins(kb, L, hist, sh + kShSel, sh + kShNEq, take_eq, n_eq);
    if (T == 0xffffffffu) return false;

    // ---- flags of the elements >= T and of those == T; their counts before every lane's chunk
    uint32_t glo, ghi, alo, ahi;
    flags_at_least(r, T, glo, ghi);
    flags_at_least(r, T + 1u, alo, ahi);
    const uint32_t qlo = glo & ~alo, qhi = ghi & ~ahi;  // == T
    uint32_t pre[C];  // low 16: entries >= T before this lane's chunk; high 16: == T
    uint32_t run = 0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const uint32_t m = 0x03030303u << (2 * (c & 3));
        const uint32_t cnt = (uint32_t)__popc((c < 4 ? glo : ghi) & m) +
                             ((uint32_t)__popc((c < 4 ? qlo : qhi) & m) << 16);
        const uint32_t incl = wave_incl_scan(cnt, lane);
        pre[c] = run + incl - cnt;
        run += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    }
    if (lane == 0) sh[kShScan + wave] = run;
    __syncthreads();
    uint32_t base = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
        if (w < wave) base += sh[kShScan + w];

    // ---- one turn per selected candidate of a lane: its rank from the flags below it
    uint32_t tlo = glo, thi = ghi;
    while (__builtin_amdgcn_ballot_w64((tlo | thi) != 0) != 0) {
        const bool low = tlo != 0;
        const uint32_t f = low ? tlo : thi;
        if (f != 0) {
            const int b = __ffs(f) - 1;
            if (low) tlo &= tlo - 1;
            else thi &= thi - 1;
            const int cq = (b >> 1) & 3, c = cq + (low ? 0 : 4), B = b >> 3;
            // flags of the same chunk of this lane with lower coordinates: elements 0..3 sit at
            // bit 2 cq of the bytes, elements 4..7 one bit above
            const uint32_t firsts = 0x01010101u << (2 * cq), seconds = firsts << 1;
            const uint32_t bytes_below = (1u << (8 * B)) - 1u;
            const uint32_t below = (b & 1) ? (firsts | (seconds & bytes_below))
                                           : (firsts & bytes_below);
            uint32_t p = pre[0];
#pragma unroll
            for (int k = 1; k < C; ++k) p = c == k ? pre[k] : p;
            p += base;
            const uint32_t ge_word = low ? glo : ghi, eq_word = low ? qlo : qhi;
            const uint32_t ge_before = (p & 0xffffu) + (uint32_t)__popc(ge_word & below);
            const uint32_t eq_before = (p >> 16) + (uint32_t)__popc(eq_word & below);
            const bool is_eq = ((eq_word >> b) & 1u) != 0;
            const bool sel = !is_eq || eq_before < (uint32_t)take_eq;
            const uint32_t pos = (ge_before - eq_before) + min(eq_before, (uint32_t)take_eq);
            if (sel && pos < (uint32_t)kb) {
                const int off = offset_of(b, low);
                sel_idx[pos] = (uint16_t)off;
                sel_val[pos] = park[off];
                park[off] = 0;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const uint4 q = *reinterpret_cast<const uint4 *>(park + chunk_off<C>(wave, c, lane));
        r.w[c][0] = q.x;
        r.w[c][1] = q.y;
        r.w[c][2] = q.z;
        r.w[c][3] = q.w;
    }
    return true;
}

// The fast top-k of a full bf16 block.  `park` (kRound*C uint16 cells) receives the block;
// on success (returns true, uniformly) sel_idx / sel_val hold the kb selected entries, largest
// magnitude first, the selected cells are zeroed, and r is reloaded from `park`.  On false
// (a wave found more candidates than it has room for: heavy ties) r is reloaded unchanged.
//   hist: 2*kSmallHistWords + kWaves*kCandPerWave words; sh: the kSh* words.  1 <= kb <= 256.
//   On success every thread has also cleared the cells of `park` that hold its own chunks.
// Output order: entries above the threshold key in candidate-list order, then the kept
// entries equal to it by increasing index; deterministic for given data.
template <class R>
__device__ __forceinline__ bool fast_topk_bf16(R &r, int kb, uint16_t *park, uint32_t *hist,
                                               uint32_t *sh, uint16_t *sel_idx,
                                               uint16_t *sel_val) {
    constexpr int C = R::kC;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    uint32_t *cand = hist + 2 * kSmallHistWords;
    // the histograms of both selections are cleared here, under the one barrier that also
    // covers the parked block
    for (int i = tid; i < 2 * kSmallHistWords; i += kWG) hist[i] = 0;
    uint32_t cmax[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int off = chunk_off<C>(wave, c, lane);
        *reinterpret_cast<uint4 *>(park + off) =
            make_uint4(r.w[c][0], r.w[c][1], r.w[c][2], r.w[c][3]);
        cmax[c] = chunk_max_key(r.w[c]);
    }
    __syncthreads();
    int unused_take, unused_eq;
    // one key per thread: the largest of its chunk maxima
    uint32_t tmax[1] = {cmax[0]};
#pragma unroll
    for (int c = 1; c < C; ++c) tmax[0] = cmax[c] > tmax[0] ? cmax[c] : tmax[0];
    const uint32_t L = select_kth_key15<1>(tmax, 1u, kb, hist, sh + kShSel, sh + kShNEq,
                                           unused_take, unused_eq);

    // candidates: every element with key >= L, wave by wave into the wave's own list
    uint32_t todo = 0;
#pragma unroll
    for (int c = 0; c < C; ++c) todo |= (cmax[c] >= L ? 1u : 0u) << c;
    uint32_t *mine = cand + wave * kCandPerWave;
    uint32_t filled = 0;  // wave-uniform
    while (__ballot(todo != 0) != 0) {
        const bool has = todo != 0;
        const int c = has ? __ffs(todo) - 1 : 0;
        todo &= todo - 1;
        const int off = ((wave * C + c) * kWave + lane) * kChunk;
        const uint4 q = *reinterpret_cast<const uint4 *>(park + off);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        uint32_t m8 = 0;
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            const uint32_t key = (e & 1) ? ((w[e >> 1] >> 16) & 0x7fffu) : (w[e >> 1] & 0x7fffu);
            m8 |= (key >= L ? 1u : 0u) << e;
        }
        if (!has) m8 = 0;
        const uint32_t cnt = __popc(m8);
        const uint32_t incl = wave_incl_scan(cnt, lane);
        uint32_t pos = filled + incl - cnt;
        filled += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        while (m8) {
            const int e = __ffs(m8) - 1;
            m8 &= m8 - 1;
            const uint32_t pair = (e >> 1) == 0 ? w[0] : (e >> 1) == 1 ? w[1] : (e >> 1) == 2 ? w[2] : w[3];
            const uint32_t key = (pair >> ((e & 1) * 16)) & 0x7fffu;
            if (pos < (uint32_t)kCandPerWave) mine[pos] = (key << 15) | (uint32_t)(32767 - (off + e));
            ++pos;
        }
    }
    // pad the wave's list to a multiple of 16 with zeros (never greater than a candidate)
    if (lane < 16 && filled + lane < (uint32_t)kCandPerWave) mine[filled + lane] = 0;
    if (lane == 0) sh[kShCnts + wave] = filled;
    __syncthreads();
    // ties are listed in the first histograms, which are free by then
    return topk_among_candidates<kCandPerWave>(r, kb, park, hist, sh, sel_idx, sel_val, filled, 0,
                                               cand, reinterpret_cast<uint16_t *>(hist), 0);
}

// Second half of the fast selections.  Every wave has filed its candidates (composites
// key << 15 | 32767 - index, every element of the top kb among them) in its list and their
// number in sh[kShCnts + wave], the block is parked, and a barrier has passed.  Returns false,
// with r reloaded unchanged, if a wave had more candidates than its list holds, if there are
// fewer than `at_least` candidates in all (then the lists may miss members of the top kb), or
// if too many candidates tie at the threshold.
template <int CAP, class R>
__device__ __forceinline__ bool topk_among_candidates(R &r, int kb, uint16_t *park,
                                                      uint32_t *hist, uint32_t *sh,
                                                      uint16_t *sel_idx, uint16_t *sel_val,
                                                      uint32_t filled, uint32_t at_least,
                                                      const uint32_t *lists, uint16_t *ties,
                                                      uint32_t key_base) {
    constexpr int C = R::kC;
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    const uint32_t *mine = lists + wave * CAP;
    uint32_t cnts[kWaves];
    bool ok = true;
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        cnts[w] = sh[kShCnts + w];
        ok = ok && cnts[w] <= (uint32_t)CAP;
        total += cnts[w];
    }
    ok = ok && total >= at_least;
    if (ok) {
        // Exact top-kb among the candidates (every thread takes those of its own wave's list,
        // one per lane and 64 list slots): a radix select on their keys gives the threshold key
        // T and the number of entries equal to T to keep; entries above T get consecutive
        // output slots by a prefix sum over the threads, entries equal to T are ranked among
        // themselves by index (they are few).
        constexpr int kMine = CAP / kWave;  // candidates per thread
        uint32_t my[kMine], keys[kMine];
        uint32_t have = 0;
#pragma unroll
        for (int s = 0; s < kMine; ++s) {
            const uint32_t i = (uint32_t)(s * kWave + lane);
            const bool got = i < filled;
            my[s] = got ? mine[i] : 0u;
            keys[s] = my[s] >> 15;
            have |= (got ? 1u : 0u) << s;
        }
        if (tid == 0) sh[kShTies] = 0;
        int take_eq, n_eq;
        // candidates known to lie at or above a key (the hinted selection's bound; at least
        // kb of them, so the kb-th exists) are told apart in one pass
        const uint32_t T =
            key_base != 0
                ? select_kth_near<kMine>(keys, have, kb, key_base, hist + kSmallHistWords,
                                         sh + kShSel + 4, sh + kShNEq, take_eq, n_eq)
                : select_kth_key15<kMine>(keys, have, kb, hist + kSmallHistWords,
                                          sh + kShSel + 4, sh + kShNEq, take_eq, n_eq);
        constexpr int kMaxTies = 512;
        ok = n_eq <= kMaxTies && T != 0xffffffffu;
        if (ok) {
            uint32_t n_gt = 0;
#pragma unroll
            for (int s = 0; s < kMine; ++s) n_gt += (((have >> s) & 1u) != 0 && keys[s] > T) ? 1u : 0u;
            const uint32_t incl = wg_incl_scan(n_gt, sh, lane, wave);
            uint32_t pos = incl - n_gt;
            uint32_t tie_idx[kMine];
#pragma unroll
            for (int s = 0; s < kMine; ++s) tie_idx[s] = 0xffffu;
#pragma unroll
            for (int s = 0; s < kMine; ++s) {
                if (((have >> s) & 1u) == 0) continue;
                const uint32_t idx = 32767u - (my[s] & 0x7fffu);
                if (keys[s] > T) {
                    sel_idx[pos] = (uint16_t)idx;
                    sel_val[pos] = park[idx];
                    park[idx] = 0;
                    ++pos;
                } else if (keys[s] == T) {
                    const uint32_t at = atomicAdd(&sh[kShTies], 1u);
                    ties[at] = (uint16_t)idx;
                    tie_idx[s] = idx;
                }
            }
            __syncthreads();
            const int first_eq = kb - take_eq;  // output slots before the ties
#pragma unroll
            for (int s = 0; s < kMine; ++s) {
                if (tie_idx[s] == 0xffffu) continue;
                uint32_t rank = 0;
                for (int j = 0; j < n_eq; ++j) rank += ties[j] < tie_idx[s] ? 1u : 0u;
                if (rank < (uint32_t)take_eq) {
                    sel_idx[first_eq + rank] = (uint16_t)tie_idx[s];
                    sel_val[first_eq + rank] = park[tie_idx[s]];
                    park[tie_idx[s]] = 0;
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const int off = chunk_off<C>(wave, c, lane);
        const uint4 q = *reinterpret_cast<const uint4 *>(park + off);
        r.w[c][0] = q.x;
        r.w[c][1] = q.y;
        r.w[c][2] = q.z;
        r.w[c][3] = q.w;
        if (ok) *reinterpret_cast<uint4 *>(park + off) = make_uint4(0, 0, 0, 0);
    }
    return ok;
}

// ---- ordered compaction ------------------------------------------------------------------------
//
// Selects every entry with key > T plus the first `take_eq` entries (in index order) with
// key == T, writes (block-relative index, bf16 value) to sel_idx / sel_val in ascending index
// order and zeroes the selected entries in the registers.  sh: 8 words.  Ends with a barrier.
template <class R>
__device__ __forceinline__ void compact_selected(R &r, uint32_t T, int take_eq, int kb,
                                                 uint16_t *sel_idx, uint16_t *sel_val,
                                                 uint32_t *sh) {
    const int tid = opaque_tid(), lane = tid & 63, wave = tid >> 6;
    uint32_t pre[R::kC];  // low 16: entries >= T before this lane's chunk; high 16: == T
    uint32_t run = 0;
#pragma unroll
    for (int c = 0; c < R::kC; ++c) {
        uint32_t cnt = 0;
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            uint32_t key = r.key(c, e);
            cnt += (key >= T ? 1u : 0u) + (key == T ? 0x10000u : 0u);
        }
        uint32_t incl = wave_incl_scan(cnt, lane);
        pre[c] = run + incl - cnt;
        run += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (lane == 0) sh[wave] = run;
    launder(r);
    __syncthreads();
    uint32_t base = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
        if (w < wave) base += sh[w];
#pragma unroll
    for (int c = 0; c < R::kC; ++c) {
        uint32_t p = pre[c] + base;
        uint32_t ge_before = p & 0xffffu, eq_before = p >> 16;
        const int off = chunk_off<R::kC>(wave, c, lane);
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
            uint32_t key = r.key(c, e);
            if (key >= T) {
                bool is_eq = key == T;
                bool sel = !is_eq || eq_before < (uint32_t)take_eq;
                uint32_t pos = (ge_before - eq_before) + min(eq_before, (uint32_t)take_eq);
                if (sel && pos < (uint32_t)kb) {
                    sel_idx[pos] = (uint16_t)(off + e);
                    sel_val[pos] = (uint16_t)r.bf16_bits(c, e);
                    r.zero(c, e);
                }
                ge_before += 1;
                eq_before += is_eq ? 1u : 0u;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
}

// ---- Adam statistics of one block from its window rows ---------------------------------------------
//
// General form, for windows too large for the one-pass stage of the fused kernel: the block is
// walked in coordinate ranges [lo, hi) short enough for two dense fp32 arrays z1 / z2 in LDS
// (one cell per coordinate of the range).  Window rows are visited in increasing row order with
// a barrier between rows, and inside a row all indices are distinct, so every coordinate's sums
// are formed in a fixed order.  The entries are fetched kWindowDepth steps ahead of their use.
// On return (after a barrier) z1[c - lo], z2[c - lo] hold the weighted sums of coordinate c, both
// zero where no row names it.
struct WindowView {
    const int16_t *I;   // window indices, row stride k, already offset to this block's columns
    const uint16_t *V;  // window values, same layout
    int64_t k;
    int rows;           // live rows: min(t, m)
    int cur_row;        // row written in this step, taken from LDS instead of memory (-1: none)
    const uint16_t *cur_idx;
    const uint16_t *cur_val;
    const float *w1;    // beta1^age per row
    const float *w2;
};

constexpr int kWindowDepth = 4;

__device__ __forceinline__ void window_accumulate(const WindowView &wv, int kb, int lo, int hi,
                                                  float *z1, float *z2) {
    const int tid = opaque_tid();
    for (int i = tid; i < hi - lo; i += kWG) {
        z1[i] = 0.0f;
        z2[i] = 0.0f;
    }
    __syncthreads();
    const int trips = (kb + kWG - 1) / kWG;
    const int steps = wv.rows * trips;
    // Step s is entry j = it * kWG + tid of window row `row`, (row, it) counting up with `it`
    // the faster digit; the fetch stream runs kWindowDepth steps ahead of the process stream.
    int frow = 0, fit = 0;  // wave-uniform
    auto fetch = [&](uint32_t &idx, uint32_t &vb) {
        idx = 0xffffu;  // never inside a range
        vb = 0;
        if (frow < wv.rows) {
            const int j = fit * kWG + tid;
            if (j < kb) {
                if (frow == wv.cur_row) {
                    idx = wv.cur_idx[j];
                    vb = wv.cur_val[j];
                } else {
                    const int16_t *Ir = wv.I + (int64_t)frow * wv.k;
                    const uint16_t *Vr = wv.V + (int64_t)frow * wv.k;
                    idx = (uint16_t)Ir[j];
                    vb = Vr[j];
                }
            }
            if (++fit == trips) {
                fit = 0;
                ++frow;
            }
        }
    };
    uint32_t nI[kWindowDepth], nV[kWindowDepth];
#pragma unroll
    for (int i = 0; i < kWindowDepth; ++i) fetch(nI[i], nV[i]);
    int prow = 0, pit = 0;
    const uint32_t span = (uint32_t)(hi - lo);
    for (int base = 0; base < steps; base += kWindowDepth) {
        uint32_t cI[kWindowDepth], cV[kWindowDepth];
#pragma unroll
        for (int i = 0; i < kWindowDepth; ++i) {
            cI[i] = nI[i];
            cV[i] = nV[i];
        }
#pragma unroll
        for (int i = 0; i < kWindowDepth; ++i) fetch(nI[i], nV[i]);
#pragma unroll
        for (int i = 0; i < kWindowDepth; ++i) {
            if (prow < wv.rows) {
                const uint32_t c = cI[i] - (uint32_t)lo;
                // the range test also keeps a corrupt index from leaving the block; +-0 values
                // add nothing and are skipped (the rows of a fresh window are all (0, 0))
                if (c < span && (cV[i] & 0x7fffu) != 0) {
                    const float v = bf2f(cV[i]);
                    const float a1 = wv.w1[prow] * v;
                    const float vv = v * v;
                    const float a2 = wv.w2[prow] * vv;
                    z1[c] = z1[c] + a1;
                    z2[c] = z2[c] + a2;
                }
                if (++pit == trips) {
                    pit = 0;
                    ++prow;
                    __syncthreads();
                }
            }
        }
    }
}

// ---- division by a value shared by many numerators ---------------------------------------------
//
// y / u, correctly rounded, with the reciprocal paid once.  r = rcp(u) refined by one Newton
// step is the correctly rounded reciprocal unless u's significand is all ones, and with such
// an r the sequence q = y * r; e = fma(-u, q, y); q + e * r (one rounding) is the correctly
// rounded quotient (Markstein's theorem; checked against IEEE division on 12e9 operand pairs,
// random, at rounding boundaries and on bf16's grid, from every reciprocal seed within one
// ulp: no difference; with an all-ones significand it does fail).  No operand scaling and no
// special-case fix-up, so callers keep u normal with a biased exponent in [32, 222] and its
// significand not all ones (divisor_is_plain; they scale u and y by an exact power of two or
// take the compiler's division otherwise), and |y| within a few multiples of 16 u; a quotient
// too small to be normal is only ever compared with 1/2.
struct Divisor {
    float u, r;
};

__device__ __forceinline__ bool divisor_is_plain(float u) {
    const uint32_t b = __float_as_uint(u);
    return ((b >> 23) & 0xffu) - 32u <= 190u && (b & 0x7fffffu) != 0x7fffffu;
}

__device__ __forceinline__ Divisor make_divisor(float u) {
    Divisor d;
    d.u = u;
    const float r0 = __builtin_amdgcn_rcpf(u);
    const float e = __builtin_fmaf(-u, r0, 1.0f);
    d.r = __builtin_fmaf(e, r0, r0);
    return d;
}

__device__ __forceinline__ float div_shared(float y, const Divisor &d) {
    const float q = y * d.r;
    const float e = __builtin_fmaf(-d.u, q, y);
    return __builtin_fmaf(e, d.r, q);
}

// x / 15 for the quantisation step u = (max - min) / 15: the shared-divisor sequence when the
// range is comfortably normal, the compiler's full division otherwise.
__device__ __forceinline__ float div15(float x, const Divisor &d15) {
    const uint32_t ex = (__float_as_uint(x) >> 23) & 0xffu;
    if (ex - 32u <= 190u) return div_shared(x, d15);
    return x / 15.0f;
}

// (z1 s1) / (eps + sqrt(z2 s2)), square root and quotient correctly rounded.
// Short way: the square root by Goldschmidt's iteration from rsq (g = x y, h = y / 2 refined
// once together, then g + (x - g g) h in one rounding: equal to the correctly rounded root for
// every significand and every seed within two ulp of 1 / sqrt(x), checked exhaustively), the
// quotient by div_shared's sequence.  Both without scaling or special cases, so a wave in which
// some lane's operands are zero, tiny, huge or not finite takes the compiler's expansions.
__device__ __forceinline__ float adam_direction(float z1, float z2, float s1, float s2,
                                                float eps) {
    const float mh = z1 * s1;
    const float vh = z2 * s2;
    const float y = __builtin_amdgcn_rsqf(vh);
    float g = vh * y, h = 0.5f * y;
    const float r = __builtin_fmaf(-h, g, 0.5f);
    g = __builtin_fmaf(g, r, g);
    h = __builtin_fmaf(h, r, h);
    const float d = __builtin_fmaf(-g, g, vh);
    const float root = __builtin_fmaf(d, h, g);
    const float den = eps + root;
    const float u = div_shared(mh, make_divisor(den));
    // vh in [2^-90, 2^90], |mh| in [2^-40, 2^90], den plain: then nothing above leaves the
    // normal range and the quotient is normal
    const uint32_t ev = (__float_as_uint(vh) >> 23) & 0xffu, em = (__float_as_uint(mh) >> 23) & 0xffu;
    const bool fine = ev - 37u <= 180u && em - 87u <= 130u && divisor_is_plain(den);
    if (__builtin_amdgcn_ballot_w64(!fine) == 0) return u;
    return mh / (eps + sqrtf(vh));
}

// The same direction for a bf16 update: only its rounding to bf16 is wanted, so eight bits of
// the quotient decide and an approximation settles almost every case.  q = mh * rcp(eps +
// sqrt(vh)) with the hardware's square root and reciprocal (one ulp each) lies within 3.5 * 2^-23
// (relative; at most 7 ulp) of the correctly rounded quotient of the correctly rounded terms,
// provided nothing on the way is subnormal or overflows: vh >= 2^-100 (then the root and the
// denominator are comfortably normal) and q itself has an exponent in [-100, 100].  Then q and
// the exact quotient round to the same bf16 value unless q lies within 7 ulp of a tie, i.e.
// unless its low 16 bits are that close to 0x8000; 16 is asked.  A wave in which some lane fails
// one of the tests (about one call in thirty at random data) takes the exact way for all lanes.
// Returns the update as bf16 bits.
__device__ __forceinline__ uint32_t adam_direction_bf16(float z1, float z2, float s1, float s2,
                                                        float eps) {
    const float mh = z1 * s1;
    const float vh = z2 * s2;
    const float root = __builtin_amdgcn_sqrtf(vh);
    const float den = eps + root;
    const float q = mh * __builtin_amdgcn_rcpf(den);
    const uint32_t b = __float_as_uint(q);
    // low 16 bits outside [0x8000 - 15, 0x8000 + 15]
    const bool far_from_tie = (b & 0xffffu) - 0x7ff1u > 30u;
    const bool safe = vh >= 0x1p-100f && ((b >> 23) & 0xffu) - 27u <= 200u && far_from_tie;
    if (__builtin_amdgcn_ballot_w64(!safe) == 0) return f2bf(q);
    return f2bf(adam_direction(z1, z2, s1, s2, eps));
}

// The direction as the update buffer of the data's type holds it: rounded to bf16 for bf16 data
// (so that a later conversion to bf16 changes nothing), fp32 otherwise.
template <bool BF16>
__device__ __forceinline__ float adam_update(float z1, float z2, float s1, float s2, float eps) {
    if (BF16) return bf2f(adam_direction_bf16(z1, z2, s1, s2, eps));
    return adam_direction(z1, z2, s1, s2, eps);
}

// A raw buffer over `bytes` bytes at p: loads past the end return 0 instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t byte_buffer(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

}  // namespace ma
