// What this GPU's memory system delivers to plain streaming kernels: the measured
// denominators beside the published 8 TB/s HBM peak.  Read-only, write-only and copy
// kernels (16-byte vectors, 256-lane blocks; the better of a grid-stride shape and a one-pass
// shape, per kind and size), timed with the dispatches' own start/end timestamps, over buffers far
// larger than the 256 MB Infinity Cache; plus the launch-to-launch time of an empty
// kernel, the fixed cost every kernel in a stream pays.  No counterpart in the reference:
// it never measures its device's bandwidth (reports/12_references.md has link figures only).
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <vector>

#include "../../include/tbvcoll.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;

// SHAPE 0: four vectors per lane, grid-stride over a capped grid (the shape of the data path's large kernels)
// SHAPE 1: one vector per lane, one pass, as many blocks as it takes
// Measured on 1 GiB (TB/s): read  plain 4/stride 6.3, plain 1/pass 6.7, non-temporal 4/stride 7.05
//                           write plain 4/stride 5.7, non-temporal 4/stride 5.5, plain 1/pass 6.85
//                           copy  plain 4/stride 5.6, non-temporal both 4/stride 6.0, non-temporal load 1/pass 6.47
// kind 0: read (the xor of what was read is kept so the loads cannot be dropped)   kind 1: write
// kind 2: copy, non-temporal loads   kind 3: copy, plain accesses
template <int KIND, int U, bool NT_LOAD, bool LOOP>
__global__ __launch_bounds__(kBlock) void k_stream(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t nvec, u32x4* sink)
{
    const size_t tile = (size_t)kBlock * U;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t base = (size_t)blockIdx.x * tile; base < nvec; base += (size_t)gridDim.x * tile) {
        u32x4 x[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * kBlock + threadIdx.x;
            if (KIND == 1) { u32x4 v = {(uint32_t)i, 1u, 2u, 3u}; x[u] = v; }
            else if (i < nvec) x[u] = NT_LOAD ? __builtin_nontemporal_load(src + i) : src[i];
            else x[u] = acc;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * kBlock + threadIdx.x;
            if (i >= nvec) continue;
            if (KIND == 0) { acc.x ^= x[u].x; acc.y ^= x[u].y; acc.z ^= x[u].z; acc.w ^= x[u].w; }
            else dst[i] = x[u];
        }
        if (!LOOP) break;
    }
    if (KIND == 0 && acc.x == 0x12345678u && acc.y == 0x9abcdef0u && acc.z == 0x0fedcba9u) *sink = acc;
}

__global__ void k_nothing(u32x4* sink) { if (sink && threadIdx.x == 4096) sink->x = 1; }

struct Bufs {
    char* src = nullptr; char* dst = nullptr; u32x4* sink = nullptr;
    std::vector<hipEvent_t> ev;
    ~Bufs()
    {
        if (src) (void)hipFree(src);
        if (dst) (void)hipFree(dst);
        if (sink) (void)hipFree(sink);
        for (auto e : ev) (void)hipEventDestroy(e);
    }
};

// shape 0: four vectors per lane, grid-stride, at most `cap` blocks; shape 1: one vector per lane, one pass
void launch(int kind, int shape, size_t cap, hipStream_t st, hipEvent_t e0, hipEvent_t e1, const char* src, char* dst, size_t nvec, u32x4* sink)
{
    const u32x4* s = (const u32x4*)src; u32x4* d = (u32x4*)dst;
    if (shape == 1) {
        const dim3 grid((unsigned)((nvec + kBlock - 1) / kBlock));
        switch (kind) {
            case 0: hipExtLaunchKernelGGL((k_stream<0, 1, true, false>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
            case 1: hipExtLaunchKernelGGL((k_stream<1, 1, false, false>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
            case 2: hipExtLaunchKernelGGL((k_stream<2, 1, true, false>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
            default: hipExtLaunchKernelGGL((k_stream<3, 1, false, false>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
        }
        return;
    }
    const size_t tiles = (nvec + (size_t)kBlock * 4 - 1) / ((size_t)kBlock * 4);
    const dim3 grid((unsigned)std::min(tiles, cap));
    switch (kind) {
        case 0: hipExtLaunchKernelGGL((k_stream<0, 4, true, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
        case 1: hipExtLaunchKernelGGL((k_stream<1, 4, false, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
        case 2: hipExtLaunchKernelGGL((k_stream<2, 4, true, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
        default: hipExtLaunchKernelGGL((k_stream<3, 4, false, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink); break;
    }
}

}  // namespace

// Streams `bytes` per launch (kind 0 read, 1 write, 2 copy with non-temporal loads, 3 plain copy) `reps`
// times inside a pool of `pool_bytes` (>= bytes; successive launches take successive windows of the pool, so
// with a pool beyond the Infinity Cache every launch finds its operands in HBM).  Returns the mean and the
// minimum launch duration in microseconds (the dispatches' own timestamps).  Allocates and frees its pool:
// a measurement tool for benches, not part of the data path.
extern "C" int tbv_emu_hbm_probe(int kind, size_t bytes, size_t pool_bytes, int reps, double* mean_us, double* min_us)
{
    if (kind < 0 || kind > 3 || bytes < 4096 || (bytes & 15) || pool_bytes < bytes || reps < 1 || reps > 4096) return -1;
    Bufs b;
    if (kind != 1 && hipMalloc((void**)&b.src, pool_bytes) != hipSuccess) return -1;
    if (kind != 0 && hipMalloc((void**)&b.dst, pool_bytes) != hipSuccess) return -1;
    if (hipMalloc((void**)&b.sink, 64) != hipSuccess) return -1;
    if (b.src && hipMemset(b.src, 0x5a, pool_bytes) != hipSuccess) return -1;
    if (b.dst && hipMemset(b.dst, 0x11, pool_bytes) != hipSuccess) return -1;
    hipStream_t st = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) return -1;
    b.ev.resize(2 * (size_t)reps);
    for (auto& e : b.ev) if (hipEventCreate(&e) != hipSuccess) { (void)hipStreamDestroy(st); return -1; }
    const size_t nvec = bytes >> 4, windows = pool_bytes / bytes;
    if ((nvec + kBlock - 1) / kBlock > 0x7fffffffu) { (void)hipStreamDestroy(st); return -1; }
    const size_t cap = bytes >= ((size_t)256 << 20) ? 16384 : 1024;
    int rc = 0;
    double sum = 0, mn = 1e30;
    // both shapes, the faster one (by its mean) is the figure: which one wins depends on the kind and the size
    for (int shape = 0; shape < 2 && rc == 0; shape++) {
        if (kind == 3 && shape == 1) break;                // the plain copy stays the one plain shape, as a reference
        for (int i = 0; i < 3 + reps && rc == 0; i++) {    // three untimed launches first
            const size_t w = ((size_t)i % windows) * bytes;
            const bool timed = i >= 3;
            launch(kind, shape, cap, st, timed ? b.ev[2 * (size_t)(i - 3)] : nullptr, timed ? b.ev[2 * (size_t)(i - 3) + 1] : nullptr,
                   b.src ? b.src + w : nullptr, b.dst ? b.dst + w : nullptr, nvec, b.sink);
            if (hipGetLastError() != hipSuccess) rc = -1;
        }
        if (hipStreamSynchronize(st) != hipSuccess) rc = -1;
        double s1 = 0, m1 = 1e30;
        for (int i = 0; i < reps && rc == 0; i++) {
            float ms = 0;
            if (hipEventElapsedTime(&ms, b.ev[2 * (size_t)i], b.ev[2 * (size_t)i + 1]) != hipSuccess) { rc = -1; break; }
            s1 += ms * 1e3; m1 = std::min(m1, (double)ms * 1e3);
        }
        if (rc == 0 && (shape == 0 || s1 < sum)) { sum = s1; mn = m1; }
    }
    (void)hipStreamDestroy(st);
    if (rc != 0) return -1;
    if (mean_us) *mean_us = sum / reps;
    if (min_us) *min_us = mn;
    return 0;
}

// Launch-to-launch time of an empty kernel in one stream, in microseconds: `reps` launches bracketed by two
// events.  Every kernel of the data path pays this much stream time before it moves a byte.
extern "C" int tbv_emu_launch_floor(int reps, double* us_per_launch)
{
    if (reps < 1 || reps > 100000 || !us_per_launch) return -1;
    hipStream_t st = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) return -1;
    int rc = -1;
    if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
        for (int i = 0; i < 16; i++) hipLaunchKernelGGL(k_nothing, dim3(1024), dim3(kBlock), 0, st, (u32x4*)nullptr);
        (void)hipStreamSynchronize(st);
        (void)hipEventRecord(e0, st);
        for (int i = 0; i < reps; i++) hipLaunchKernelGGL(k_nothing, dim3(1024), dim3(kBlock), 0, st, (u32x4*)nullptr);
        (void)hipEventRecord(e1, st);
        float ms = 0;
        if (hipStreamSynchronize(st) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) { *us_per_launch = ms * 1e3 / reps; rc = 0; }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipStreamDestroy(st);
    return rc;
}
