// One step of the data path for callers that cannot allocate: pack into a bounce buffer the
// caller owns, raise its completion word, sum into the output, raise a done word.  The
// kernels are the library's own (pack, sum, merged launch); what differs from the entry
// points that go through tbv_ar_init is where their scratch lives: the block-completion
// counters are a file-scope device array instead of a hipMalloc'ed block, so this entry
// point calls no allocator, needs no initialisation and can be used under HIP graph
// capture or from a serving loop that forbids hipMalloc.
//
// No counterpart in the reference, whose only scratch (the `arrive` counters,
// step4/libtbvcoll.cpp:96,323) is allocated in tbv_ar_init.
#include <hip/hip_runtime.h>

#include <stdio.h>

#include <atomic>

#include "../../include/tbvcoll.h"
#include "tbv_kernels.h"

namespace {

// Two counter blocks (pack completion, sum completion), 16 KiB in all.  Each GPU the library
// runs on holds its own copy until the process ends.  Every counter returns to zero when its
// last block has arrived, so a completed call leaves the array clean for the next one.
static __device__ __align__(256) unsigned int scratch[2 * tbv::kCounterWords];

constexpr int kMaxDevices = 64;
// per-device address of `scratch` (the array's name is only a host-side handle for the symbol)
std::atomic<unsigned int*> g_scratch_ptr[kMaxDevices];

// Device address of this device's copy of the counters; looked up once per device with that
// device current.  Returns null after printing why.
unsigned int* scratch_on_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        fprintf(stderr, "[tbvcoll] no-alloc step: no current HIP device (or index beyond %d)\n", kMaxDevices - 1);
        return nullptr;
    }
    unsigned int* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    void* sym = nullptr;
    const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sym) {
        fprintf(stderr, "[tbvcoll] no-alloc step: hipGetSymbolAddress failed on device %d: %s\n", dev, hipGetErrorString(e));
        return nullptr;
    }
    g_scratch_ptr[dev].store((unsigned int*)sym, std::memory_order_release);
    return (unsigned int*)sym;
}

// The address if this device's copy has been looked up already, else null; makes no HIP call beyond hipGetDevice.
unsigned int* bound_scratch_on_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    return g_scratch_ptr[dev].load(std::memory_order_acquire);
}

inline bool al16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

}  // namespace

namespace tbv {
// Called by tbv_ar_init so that the first no-alloc step on this device finds the address already there.
bool noalloc_bind_device() { return scratch_on_current_device() != nullptr; }
}

extern "C" int tbv_step_noalloc(void* out, const void* local, const void* received, void* bounce, int bounce_uncached,
                                size_t nbytes, int dtype, unsigned long long* pack_word, unsigned long long* done_word,
                                unsigned long long seq, void* stream)
{
    if (!out || !local || !received || !bounce) { fprintf(stderr, "[tbvcoll] no-alloc step: null buffer\n"); return -1; }
    if (dtype < 0 || dtype > 2) { fprintf(stderr, "[tbvcoll] no-alloc step: unknown dtype %d\n", dtype); return -1; }
    if (nbytes > (size_t)TBV_NOALLOC_MAX_BYTES) {
        fprintf(stderr, "[tbvcoll] no-alloc step: %zu bytes exceeds the limit of %zu\n", nbytes, (size_t)TBV_NOALLOC_MAX_BYTES);
        return -2;
    }
    if (!(al16(out) && al16(local) && al16(received) && al16(bounce))) {
        fprintf(stderr, "[tbvcoll] no-alloc step: buffers must be 16-byte aligned\n");
        return -1;
    }
    if (nbytes == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    unsigned int* ctr = bound_scratch_on_current_device();
    if (!ctr) {
        // The look-up below can make the runtime load the code object and set the array up, which is not allowed while
        // a stream is being captured: the first call on a device has to come before any capture (or tbv_ar_init has).
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) {
            fprintf(stderr, "[tbvcoll] no-alloc step: first call on this device is inside a stream capture; call it once "
                            "(or tbv_ar_init) on the device before capturing\n");
            return -1;
        }
        (void)hipGetLastError();
        ctr = scratch_on_current_device();
    }
    if (!ctr) return -1;

    tbv::PackArgs pa{};
    pa.dst = bounce; pa.src = local; pa.nbytes = nbytes; pa.seq = seq;
    pa.cflag = pack_word; pa.arrive = ctr;
    pa.sigmode = bounce_uncached ? 0 : 1;            // a cached bounce is written back before it is declared complete
    tbv::SumArgs sa{};
    sa.out = out; sa.a = local; sa.b = received; sa.nbytes = nbytes; sa.dtype = dtype; sa.seq = seq;
    sa.done = done_word; sa.done_arrive = ctr + tbv::kCounterWords;

    // Pack blocks and sum blocks of the one-launch form read `local` independently, so a sum block could store out[i]
    // before the pack block has read local[i]: in place the step takes the fused body (one lane loads local[i] once and
    // does both stores); an output that overlaps `local` in any other way gets two launches, one after the other.
    const uintptr_t lo = (uintptr_t)local, oo = (uintptr_t)out;
    const bool inplace = out == local, overlap = oo < lo + nbytes && lo < oo + nbytes;
    hipError_t e;
    if (bounce_uncached && nbytes > 16384 && !overlap) {
        e = tbv::launch_pack_sum_merged(pa, sa, st);             // pack blocks and sum blocks in one launch
    } else if (bounce_uncached && nbytes > 16384 && inplace) {
        e = tbv::launch_pack_sum(pa, sa, st);                    // one body: load once, store to the bounce and to the output
    } else {
        e = tbv::launch_pack(pa, st);
        if (e == hipSuccess) e = tbv::launch_sum(sa, st);
    }
    if (e != hipSuccess) { fprintf(stderr, "[tbvcoll] no-alloc step: launch failed: %s\n", hipGetErrorString(e)); return -1; }
    return 0;
}
