// Streaming kernels of known size, used to calibrate measurements of the MicroAdam step: what
// the HBM counters read per byte, and what rate this device sustains for the step's own access
// shape (512-thread workgroups, each owning one contiguous 40 KiB stretch of every array and
// moving it as five 16-byte accesses per lane, a contiguous KiB per wave and access).  Built
// into a library of its own, libmicroadam_probe.so, which only the benchmark loads; no
// counterpart in the reference.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "stream_probe.h"

namespace ma {
namespace {

constexpr int kProbeErrArg = -1;  // bad argument
constexpr int kThreads = 512;
constexpr int kChunks = 5;
constexpr int kSegBytes = kThreads * kChunks * 16;  // 40 KiB per workgroup and array

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

template <bool NT>
__device__ __forceinline__ u4 ld(const u4 *p) {
    return NT ? __builtin_nontemporal_load(p) : *p;
}
template <bool NT>
__device__ __forceinline__ void st(u4 *p, u4 v) {
    if (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// MODE 0: read a.  1: write c.  2: c = a.  3: b = f(a, b) (two reads, one write: the step's mix).
// 4: the step's three large streams: reads a (2 B per element), b (2 B), e (0.5 B); writes b, e.
// 5: writes c and, once the stores have completed and this CU's L1 is emptied, reads the same
//    stretch back: what the L2 fetches for it tells whether lines just written are served from
//    the L2 (a workgroup handing data to another of its XCD would rely on that).
template <int MODE, bool NT>
__global__ __launch_bounds__(kThreads) void stream_kernel(const u4 *a, u4 *b, u4 *c, uint32_t *e,
                                                          int64_t segments, uint32_t *sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u4 acc = {0, 0, 0, 0};
    for (int64_t s = blockIdx.x; s < segments; s += gridDim.x) {
        const int64_t base = s * (kSegBytes / 16);
        u4 va[kChunks], vb[kChunks];
        uint32_t ve[kChunks];
#pragma unroll
        for (int k = 0; k < kChunks; ++k) {
            const int64_t i = base + (wave * kChunks + k) * 64 + lane;
            if (MODE == 0 || MODE == 2 || MODE == 3 || MODE == 4) va[k] = ld<NT>(a + i);
            if (MODE == 3 || MODE == 4) vb[k] = ld<NT>(b + i);
            if (MODE == 4) ve[k] = e[i];
        }
#pragma unroll
        for (int k = 0; k < kChunks; ++k) {
            const int64_t i = base + (wave * kChunks + k) * 64 + lane;
            if (MODE == 0) acc ^= va[k];
            if (MODE == 1) st<NT>(c + i, u4{(uint32_t)i, 1u, 2u, 3u});
            if (MODE == 2) st<NT>(c + i, va[k]);
            if (MODE == 3) st<NT>(b + i, va[k] + vb[k]);
            if (MODE == 4) {
                st<NT>(b + i, va[k] + vb[k] + ve[k]);
                e[i] = ve[k] ^ va[k].x;
            }
            if (MODE == 5) st<NT>(c + i, u4{(uint32_t)i, 1u, 2u, 3u});
        }
        if (MODE == 5) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            asm volatile("buffer_inv sc0" ::: "memory");
#pragma unroll
            for (int k = 0; k < kChunks; ++k)
                acc ^= ld<false>(c + base + (wave * kChunks + k) * 64 + lane);
        }
    }
    if ((MODE == 0 || MODE == 5) && (acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) *sink = acc.x;
}

template <int MODE>
int launch(bool nt, unsigned grid, hipStream_t s, const void *a, void *b, void *c, void *e,
           int64_t segments, void *sink) {
    const u4 *pa = (const u4 *)a;
    u4 *pb = (u4 *)b, *pc = (u4 *)c;
    uint32_t *pe = (uint32_t *)e, *ps = (uint32_t *)sink;
    void *argv[] = {&pa, &pb, &pc, &pe, &segments, &ps};
    const void *kernel = nt ? reinterpret_cast<const void *>(stream_kernel<MODE, true>)
                            : reinterpret_cast<const void *>(stream_kernel<MODE, false>);
    return (int)hipLaunchKernel(kernel, dim3(grid), dim3(kThreads), argv, 0, s);
}

}  // namespace
}  // namespace ma

extern "C" int ma_stream_probe(int mode, int nontemporal, int64_t bytes, int64_t workgroups,
                               const void *a, void *b, void *c, void *e, void *sink,
                               void *stream) {
    using namespace ma;
    if (bytes <= 0 || bytes % kSegBytes != 0 || !sink) return kProbeErrArg;
    const int64_t segments = bytes / kSegBytes;
    if (segments > 0x7fffffff) return kProbeErrArg;
    const bool need_a = mode == 0 || mode == 2 || mode == 3 || mode == 4;
    const bool need_b = mode == 3 || mode == 4, need_c = mode == 1 || mode == 2 || mode == 5;
    if ((need_a && !a) || (need_b && !b) || (need_c && !c) || (mode == 4 && !e)) return kProbeErrArg;
    const unsigned grid = (unsigned)(workgroups > 0 && workgroups < segments ? workgroups : segments);
    hipStream_t s = (hipStream_t)stream;
    switch (mode) {
        case 0: return launch<0>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
        case 1: return launch<1>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
        case 2: return launch<2>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
        case 3: return launch<3>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
        case 4: return launch<4>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
        case 5: return launch<5>(nontemporal != 0, grid, s, a, b, c, e, segments, sink);
    }
    return kProbeErrArg;
}
