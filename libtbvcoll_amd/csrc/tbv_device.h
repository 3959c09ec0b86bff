// Device-side building blocks shared by the kernel files: 16-byte vector types, the cache
// hints of the data streams, the element arithmetic of the sum (what the HIP headers'
// operator+ computes, step4/libtbvcoll.cpp:165), grid-wide completion counting
// (replaces the arrive counter of k_copy_sig, step4/libtbvcoll.cpp:135-139) and the
// in-kernel flag gate (k_waitflag, step4/libtbvcoll.cpp:155-160).
#pragma once
#include <hip/hip_runtime.h>

#include "tbv_kernels.h"

namespace tbv {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// Cache hints of the four data streams, two profiles measured on MI355X with the 16 MiB step.
//
// Resident profile (STREAM = false): what a step touches stays in the 256 MB Infinity Cache
// (small rings, the same tensors every step).  The local tensor is read twice (pack, then
// sum) and the receive slots are re-read every NSLOT calls, so both are left to allocate in
// the caches; the output is written once and never read here, so it is stored non-temporally
// and leaves the cache to the operands (sum 7.6 -> 6.6 us); the uncached bounce gets no hint.
// Non-temporal loads of the local tensor or the receive slot cost 1-2 us per step here.
//
// Streaming profile (STREAM = true): the rings are larger than the cache, every operand
// comes from HBM and nothing written is read again soon.  The receive slot is loaded and
// the bounce and the output are stored non-temporally; the local tensor keeps ordinary
// loads because the sum re-reads it a few microseconds after the pack (pack + sum
// 15.98 -> 14.18 us on cache-cold buffers; the same hints cost 0.3 us when everything is
// cache resident, which is why there are two profiles).
// ONCE: this kernel is the only reader of the local tensor (pack and sum fused in one body)
template <bool STREAM, bool ONCE> __device__ __forceinline__ uint32_t __attribute__((ext_vector_type(4))) ld_a(const uint32_t __attribute__((ext_vector_type(4)))* p)
{
    return *p;          // non-temporal here costs about 1 us per 16 MiB even when this kernel is the only reader
}
template <bool STREAM> __device__ __forceinline__ uint32_t __attribute__((ext_vector_type(4))) ld_b(const uint32_t __attribute__((ext_vector_type(4)))* p)
{
    return STREAM ? __builtin_nontemporal_load(p) : *p;
}
// The output in the streaming profile is written THROUGH the L2 (system scope) as well as non-temporally: a line
// that is merely non-temporal still sits dirty in the L2 until it is evicted or the kernel ends, where the
// write-back of what is left stands between this kernel and the next (merged launch, 16 MiB cache-cold, same
// box: non-temporal 12.20 us per launch, write-through + non-temporal 11.89, write-through alone 12.65,
// plain 13.0).  No builtin sets the scope bits of a 16-byte global store; the raw buffer store takes them as its
// cache-policy operand (sc0 = 1, nt = 2, sc1 = 16), so the store goes out as a buffer store whose descriptor is
// built around the wave's lowest address (lanes store to ascending addresses, so the first active lane holds it;
// a wave's stores span far less than the 4 GiB a 32-bit offset reaches).  An inline-asm store is not an option:
// the compiler does not know it for a 16-byte store and leaves out the wait states this GPU needs before the
// next instruction may overwrite the data registers (seen as stale first dwords in some vectors).
__device__ __forceinline__ void st_through(uint32_t __attribute__((ext_vector_type(4)))* p, uint32_t __attribute__((ext_vector_type(4))) v)
{
    const uint64_t addr = (uint64_t)p;
    // (the builtin returns a signed int: through uint32_t, or a low word with bit 31 set would smear over the high one)
    const uint64_t base = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(addr >> 32)) << 32) |
                          (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)addr);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0xffffffff, 0x00020000);
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (uint32_t)(addr - base), 0, 1 | 2 | 16);
}
template <bool STREAM> __device__ __forceinline__ void st_out(uint32_t __attribute__((ext_vector_type(4)))* p, uint32_t __attribute__((ext_vector_type(4))) v)
{
    if (STREAM) st_through(p, v);
    else __builtin_nontemporal_store(v, p);
}
// In place the output's lines are in the L2 already (this kernel has just read them as the local tensor), and writing
// them through costs more than it saves: fused body, 16 MiB cache-cold in place, 13.4 us written through, 12.2
// non-temporal or plain.  `in_place` is uniform over the grid.
// (A merged launch for in-place calls, its pack and sum waves ordered pairwise through a word per wave, was built
// and measured: 12.1 us, no better than the fused body with these stores, so in place keeps the fused body.)
template <bool STREAM> __device__ __forceinline__ void st_out_at(uint32_t __attribute__((ext_vector_type(4)))* p, uint32_t __attribute__((ext_vector_type(4))) v, bool in_place)
{
    if (STREAM && !in_place) st_through(p, v);
    else __builtin_nontemporal_store(v, p);
}
// The same choice at run time (block-uniform), for the kernels that are not compiled once per profile.
__device__ __forceinline__ void st_result(uint32_t __attribute__((ext_vector_type(4)))* p, uint32_t __attribute__((ext_vector_type(4))) v, int through)
{
    if (through) st_through(p, v);
    else __builtin_nontemporal_store(v, p);
}
template <bool STREAM> __device__ __forceinline__ void st_bounce(uint32_t __attribute__((ext_vector_type(4)))* p, uint32_t __attribute__((ext_vector_type(4))) v)
{
    if (STREAM) __builtin_nontemporal_store(v, p); else *p = v;
}

static constexpr int kThreads = 256;        // 4 wavefronts of 64
static constexpr int kMaxSmallThreads = 1024;
static constexpr int kMaxGrid = 256 * 8;     // 256 CUs, up to 8 resident blocks each
// A kernel that waits for the flag inside holds its wave slots while it waits.  Whatever has to
// run for the flag to come up (another stream's copy, another library's kernel) needs slots too,
// so the part of a grid that waits is kept to half of the GPU's 8192 wave slots at most (1024 blocks
// of 4 waves); the blocks loop instead.  Measured with the 16 MiB step and its flag already up
// (pack blocks + gated sum blocks in one launch, cache-cold): 256 blocks x 4 vectors per lane 18.2 us,
// 512 x 4 15.4, 512 x 2 14.4, 1024 x 4 14.2, 1024 x 2 13.0 (ungated merged launch: 12.35).
static constexpr int kGatedMaxGrid = 1024;

// ---------------------------------------------------------------- arithmetic

// bf16: widen both operands to fp32 (exact), add in fp32, round to nearest even.
// The fptrunc of a float pair lowers to v_cvt_pk_bf16_f32 on gfx950.
__device__ __forceinline__ uint32_t add_bf16x2(uint32_t x, uint32_t y)
{
    f32x2 s;
    s.x = __uint_as_float(x << 16) + __uint_as_float(y << 16);
    s.y = __uint_as_float(x & 0xffff0000u) + __uint_as_float(y & 0xffff0000u);
    bf16x2 r = __builtin_convertvector(s, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}

template <int DT> __device__ __forceinline__ u32x4 add_vec(u32x4 x, u32x4 y);

template <> __device__ __forceinline__ u32x4 add_vec<0>(u32x4 x, u32x4 y)
{
    f32x4 a = __builtin_bit_cast(f32x4, x), b = __builtin_bit_cast(f32x4, y);
    f32x4 s;
    s.x = a.x + b.x; s.y = a.y + b.y; s.z = a.z + b.z; s.w = a.w + b.w;
    return __builtin_bit_cast(u32x4, s);
}
// fp16: the IEEE half add itself (what the HIP header's operator+ on _Float16 is);
// it equals fp32-upcast + add + round-to-nearest-even for every finite pair.
template <> __device__ __forceinline__ u32x4 add_vec<1>(u32x4 x, u32x4 y)
{
    f16x8 a = __builtin_bit_cast(f16x8, x), b = __builtin_bit_cast(f16x8, y);
    f16x8 s = a + b;
    return __builtin_bit_cast(u32x4, s);
}
template <> __device__ __forceinline__ u32x4 add_vec<2>(u32x4 x, u32x4 y)
{
    u32x4 r;
    r.x = add_bf16x2(x.x, y.x); r.y = add_bf16x2(x.y, y.y);
    r.z = add_bf16x2(x.z, y.z); r.w = add_bf16x2(x.w, y.w);
    return r;
}

template <int DT> struct Elem;
template <> struct Elem<0> { typedef float T; static __device__ __forceinline__ T add(T a, T b) { return a + b; } };
template <> struct Elem<1> { typedef _Float16 T; static __device__ __forceinline__ T add(T a, T b) { return a + b; } };
template <> struct Elem<2> {
    typedef uint16_t T;
    static __device__ __forceinline__ T add(T a, T b)
    {
        float s = __uint_as_float((uint32_t)a << 16) + __uint_as_float((uint32_t)b << 16);
        __bf16 r = (__bf16)s;
        return __builtin_bit_cast(uint16_t, r);
    }
};

// ---------------------------------------------------------------- signalling helpers

__device__ __forceinline__ void store_sys(unsigned long long* p, unsigned long long v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Every thread of the block calls this after its last store.  `bid` of `nblk` is the
// block's index among the blocks being counted (the whole grid, or one part of a merged
// launch).  When the last of them gets here, all their stores are visible system wide
// and `word` is set to `seq`.
//
// Blocks are counted in two levels so that no single address takes one atomic
// per block (same-address atomics retire one at a time): groups of kGroup blocks
// count on their own 64-byte line, and the last block of a group counts on the
// top line.  `ctr` points to the slot's counter lines (line 0 = top, line 1+g =
// group g, 16 words apart); every counter is put back to 0 by its last arriver.
//
// mode 0: the destination is uncached memory: stores bypass the L2, so each wave
//         only has to see its own stores acknowledged before the block is counted.
//         (The workgroup-scope release inside __syncthreads does not wait for the
//         store counter on gfx950, hence the explicit wait.)
// mode 1: the destination may be cached: the block leader also writes the L2 back
//         system wide after the barrier (one write-back per block).
// mode 2: every wave writes back system wide before the barrier (most conservative).
static constexpr unsigned kGroup = 32;
static constexpr unsigned kCtrLine = 16;       // words per counter line (64 bytes)

// Returns true in thread 0 of the block that found itself the last one (false everywhere else).
//
// `keep` (mode 0 only; block-uniform): the wave's last `keep` memory operations are stores that need not be counted
// (a fused body's output stores, issued after all of its bounce stores).  A wave's memory operations complete in the
// order they were issued, so waiting until only `keep` are outstanding has seen every counted store acknowledged.
__device__ __forceinline__ bool grid_complete(unsigned long long* word, unsigned long long seq,
                                              unsigned int* ctr, unsigned int bid, unsigned int nblk, int mode, int keep = 0)
{
    bool was_last = false;
    if (mode == 2) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
    if (mode == 0 && keep == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    else if (mode == 0 && keep == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        if (mode == 1) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");
        bool last = true;
        if (nblk > 1) {
            // groups of 32 blocks; of 64 when the grid is larger than 32 groups' lines can count
            const unsigned G = nblk > kGroup * (kCounterWords / kCtrLine - 1) ? 2 * kGroup : kGroup;
            const unsigned g = bid / G, ngroups = (nblk + G - 1) / G;
            const unsigned pop = min(G, nblk - g * G);
            unsigned int* gc = ctr + kCtrLine * (1 + g);
            last = false;
            if (__hip_atomic_fetch_add(gc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == pop - 1) {
                __hip_atomic_store(gc, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (ngroups == 1) last = true;
                else if (__hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ngroups - 1) {
                    __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    last = true;
                }
            }
        }
        // Modes 1 and 2 have written the L2 back above.  In mode 0 the counted stores went to uncached memory and
        // every wave waited for their acknowledgements before its block was counted, so they are in memory already:
        // a release here would only make this wave write back an L2 that holds none of them.
        if (last) {
            if (mode == 0) __hip_atomic_store(word, seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            else store_sys(word, seq);
        }
        was_last = last;
    }
    return was_last;
}

// Gate of a kernel on a host-visible word reaching seq.  Only block 0's leader
// polls the host word (each poll crosses PCIe); it republishes the value in a
// device word (`relay`) that the other blocks' leaders poll at L2 latency.  Block
// 0 never waits on another block, so the gate cannot deadlock however many blocks
// are resident.  Every wait is bounded by a tick count of the constant-rate wall
// clock (100 MHz on gfx950; the host passes ticks computed from the device's
// reported rate), so every wave leaves the kernel even if nobody raises the word.
// `also` (optional) is a device word the polling block waits for as well before it republishes: the pack relay of
// a launch whose pack blocks must all be done before its sum blocks may store (output aliasing the local tensor).
// Whoever raises it never waits itself, so this adds no way to deadlock.
__device__ __forceinline__ void gate_wait_as(unsigned bid, const unsigned long long* flag, unsigned long long seq,
                                             unsigned long long limit, unsigned long long* relay,
                                             unsigned long long* fp, bool acquire, const unsigned long long* also = nullptr,
                                             bool relay_may_be_up = false)
{
    if (threadIdx.x == 0) {
        const unsigned long long t0 = wall_clock64();
        if (bid == 0 || !relay) {
            if (fp && bid == 0) store_sys(fp + FP_WAIT_IN, seq);
            // relaxed polls: an acquire load in the loop would invalidate the caches on every iteration, for this
            // kernel and for whatever is writing the payload; one acquire fence follows the barrier below.
            // (relay_may_be_up: a block of the same launch that looked at the flag earlier may have published it already;
            // one look at device memory then saves the first read of host memory.)
            const bool up = relay_may_be_up && relay && !also && __hip_atomic_load(relay, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= seq;
            while (!up && __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) < seq) {
                __builtin_amdgcn_s_sleep(1);
                if (wall_clock64() - t0 > limit) {
                    if (fp) store_sys(fp + FP_WAIT_TIMEOUT, seq);
                    break;
                }
            }
            if (also) {
                while (__hip_atomic_load(also, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < seq) {
                    __builtin_amdgcn_s_sleep(1);
                    if (wall_clock64() - t0 > limit) break;
                }
            }
            if (relay) __hip_atomic_store(relay, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            if (fp && bid == 0) store_sys(fp + FP_WAIT_OUT, seq);
        } else {
            while (__hip_atomic_load(relay, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < seq) {
                __builtin_amdgcn_s_sleep(2);
                if (wall_clock64() - t0 > limit + limit / 8 + 1000000ull) break;
            }
        }
    }
    __syncthreads();
    // The payload was written before the flag: from here on no stale line of it may be read.  A system-scope acquire
    // invalidates the caches from every wave that executes it, which costs a gated 4 MiB sum 6.5 us (2.5 -> 9 us), so
    // it is skipped when the payload lies in uncached memory, which no cache holds lines of.
    if (acquire) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
}

// The same for a whole grid: block 0 of the grid polls.  (gate_wait_as is for kernels in which only a part of the
// grid waits; `bid` is then the block's index within that part.)
__device__ __forceinline__ void gate_wait(const unsigned long long* flag, unsigned long long seq,
                                          unsigned long long limit, unsigned long long* relay,
                                          unsigned long long* fp, bool acquire = true)
{
    gate_wait_as(blockIdx.x, flag, seq, limit, relay, fp, acquire);
}

// Arguments of the step kernels (pack, sum, pack+sum, merged launch, one-kernel small call, row kernels).
struct StepArgs {
    // pack
    u32x4* bounce; unsigned long long* cflag; unsigned int* pack_arrive; unsigned long long* tagp;
    // sum
    u32x4* out; const u32x4* b;
    const unsigned long long* wait_flag; unsigned long long* relay; unsigned long long spin_limit;
    unsigned long long* done; unsigned int* done_arrive;
    // common
    const u32x4* a; size_t nbytes; unsigned long long seq; unsigned long long* fp; int sigmode;
    unsigned long long* pre_word; unsigned long long pre_seq;
    unsigned pack_blocks;       // merged launch: blocks [0, pack_blocks) pack, the rest sum
    unsigned long long* pack_relay;   // device word: the pack part stores seq here when its last block is done; the sum part of
                                      // the same launch waits for it (beside its flag) when the output aliases the local tensor
    int b_uncached;             // the received payload lies in uncached memory: the gate needs no cache invalidation
    unsigned tiles;             // sum part of a pipeline launch: tiles of blockDim x US vectors, taken in turn by its blocks
    int out_through;            // codec kernels: results are written through the L2 (streaming profile)
};

}  // namespace tbv
