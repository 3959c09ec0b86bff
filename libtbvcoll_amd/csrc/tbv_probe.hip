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

#include "../../include/tbvcoll_emu.h"

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
// WT: stores written through the L2 and non-temporal (what the data path's streaming profile does with its output)
__device__ __forceinline__ void store_through(u32x4* p, u32x4 v)
{
    const uint64_t addr = (uint64_t)p;
    // (the builtin returns a signed int: through uint32_t, or a low word with bit 31 set would smear over the high one)
    const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32)) << 32) |
                          (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xffffffff, 0x00020000);
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (uint32_t)(addr - base), 0, 1 | 2 | 16);     // sc0 nt sc1
}
template <int KIND, int U, bool NT_LOAD, bool LOOP, bool WT = false>
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
            else if (WT) store_through(dst + i, x[u]);
            else dst[i] = x[u];
        }
        if (!LOOP) break;
    }
    if (KIND == 0 && acc.x == 0x12345678u && acc.y == 0x9abcdef0u && acc.z == 0x0fedcba9u) *sink = acc;
}

// The four streams of one all-reduce step and nothing else: read the local tensor and the received payload, write
// the bounce and the bf16 sum (with the data path's own cache hints), two vectors per lane, one pass, no block
// counting, no completion word, no gate.  What
// the memory system delivers to this body on cache-cold operands is the floor under every form of the step.
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t add_bf16x2(uint32_t x, uint32_t y)
{
    f32x2 s;
    s.x = __uint_as_float(x << 16) + __uint_as_float(y << 16);
    s.y = __uint_as_float(x & 0xffff0000u) + __uint_as_float(y & 0xffff0000u);
    bf16x2 r = __builtin_convertvector(s, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}
__global__ __launch_bounds__(kBlock) void k_step_floor(const u32x4* a, const u32x4* b, u32x4* bounce, u32x4* out)
{
    // whole tiles only (the host checks), arguments preloaded into registers (this file's compile flags): nothing
    // stands between the start of a wave and its first load
    const size_t base = (size_t)blockIdx.x * kBlock * 2 + threadIdx.x;
    u32x4 x[2], y[2];
#pragma unroll
    for (int u = 0; u < 2; u++) { x[u] = a[base + (size_t)u * kBlock]; y[u] = __builtin_nontemporal_load(b + base + (size_t)u * kBlock); }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const size_t i = base + (size_t)u * kBlock;
        u32x4 r = {add_bf16x2(x[u].x, y[u].x), add_bf16x2(x[u].y, y[u].y), add_bf16x2(x[u].z, y[u].z), add_bf16x2(x[u].w, y[u].w)};
        __builtin_nontemporal_store(x[u], bounce + i);
        store_through(out + i, r);
    }
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

// shape 0: four vectors per lane, grid-stride, at most `cap` blocks; shape 1: one vector per lane, one pass;
// shapes 2 and 3: the same two with stores written through the L2 (write and non-temporal copy only)
void launch(int kind, int shape, size_t cap, hipStream_t st, hipEvent_t e0, hipEvent_t e1, const char* src, char* dst, size_t nvec, u32x4* sink)
{
    const u32x4* s = (const u32x4*)src; u32x4* d = (u32x4*)dst;
    if (shape == 3) {
        const dim3 grid((unsigned)((nvec + kBlock - 1) / kBlock));
        if (kind == 1) hipExtLaunchKernelGGL((k_stream<1, 1, false, false, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink);
        else hipExtLaunchKernelGGL((k_stream<2, 1, true, false, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink);
        return;
    }
    if (shape == 2) {
        const size_t tiles4 = (nvec + (size_t)kBlock * 4 - 1) / ((size_t)kBlock * 4);
        const dim3 grid((unsigned)std::min(tiles4, cap));
        if (kind == 1) hipExtLaunchKernelGGL((k_stream<1, 4, false, true, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink);
        else hipExtLaunchKernelGGL((k_stream<2, 4, true, true, true>), grid, dim3(kBlock), 0, st, e0, e1, 0, s, d, nvec, sink);
        return;
    }
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
    // every shape, the fastest one (by its mean) is the figure: which one wins depends on the kind and the size
    for (int shape = 0; shape < 4 && rc == 0; shape++) {
        if (kind == 3 && shape == 1) break;                // the plain copy stays the one plain shape, as a reference
        if (shape >= 2 && kind != 1 && kind != 2) break;   // only kinds that store have write-through shapes
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

// Device time per launch of k_step_floor on `bytes` of bf16 (a multiple of 16), `reps` launches back to back between
// two events, rotating over 12 local/output tensors and 16 received/bounce buffers (beyond the Infinity Cache for
// 16 MiB).  The bounce buffers are uncached memory, as the library's send ring is; they are kept until the process
// ends (uncached memory is never handed back to the driver here).
extern "C" int tbv_emu_step_floor(size_t bytes, int reps, double* us_per_launch)
{
    constexpr int NA = 12, NB = 16;
    static char* bounce_pool = nullptr;
    static size_t bounce_pool_bytes = 0;
    if (bytes < 8192 || (bytes & 8191) || bytes > ((size_t)64 << 20) || reps < 1 || reps > 100000 || !us_per_launch) return -1;     // whole tiles of 8 KiB
    if (bounce_pool_bytes < NB * bytes) {
        char* p = nullptr;
        if (hipExtMallocWithFlags((void**)&p, NB * bytes, hipDeviceMallocUncached) != hipSuccess) return -1;
        bounce_pool = p; bounce_pool_bytes = NB * bytes;     // a smaller, older pool stays allocated on purpose
    }
    char *a = nullptr, *o = nullptr, *b = nullptr;
    hipStream_t st = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = -1;
    const size_t nvec = bytes >> 4;
    const dim3 grid((unsigned)(nvec / (2 * kBlock)));
    auto run = [&](int i) {
        hipLaunchKernelGGL(k_step_floor, grid, dim3(kBlock), 0, st, (const u32x4*)(a + (size_t)(i % NA) * bytes), (const u32x4*)(b + (size_t)(i % NB) * bytes),
                           (u32x4*)(bounce_pool + (size_t)(i % NB) * bytes), (u32x4*)(o + (size_t)(i % NA) * bytes));
    };
    if (hipMalloc((void**)&a, NA * bytes) == hipSuccess && hipMalloc((void**)&o, NA * bytes) == hipSuccess &&
        hipMalloc((void**)&b, NB * bytes) == hipSuccess && hipMemset(a, 0x3c, NA * bytes) == hipSuccess &&
        hipMemset(b, 0x3d, NB * bytes) == hipSuccess && hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess &&
        hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
        for (int i = 0; i < 96; i++) run(i);
        (void)hipStreamSynchronize(st);
        (void)hipEventRecord(e0, st);
        for (int i = 0; i < reps; i++) run(i);
        (void)hipEventRecord(e1, st);
        float ms = 0;
        if (hipStreamSynchronize(st) == hipSuccess && hipGetLastError() == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) {
            *us_per_launch = ms * 1e3 / reps; rc = 0;
        }
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (st) (void)hipStreamDestroy(st);
    if (a) (void)hipFree(a);
    if (o) (void)hipFree(o);
    if (b) (void)hipFree(b);
    return rc;
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
