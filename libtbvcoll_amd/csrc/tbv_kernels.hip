// gfx950 kernels of the all-reduce data path: the pack copy with its completion
// signal, the two-operand sum, the fused pack+sum, and the small diagnostic
// kernels.  Everything is elementwise and HBM-bound: 128-bit accesses, several
// independent loads in flight per lane, no LDS, no MFMA.
//
// What each kernel replaces in the reference:
//   k_step<.., PACK, ..>  k_copy_sig  step4/libtbvcoll.cpp:126-140
//   k_step<.., SUM, ..>   k_acc<T>    step4/libtbvcoll.cpp:162-166
//   k_waitflag            k_waitflag  step4/libtbvcoll.cpp:155-160
//   k_tagchk / k_mark     k_tagchk / k_mark  step4/libtbvcoll.cpp:143-150,161
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include "tbv_kernels.h"
#include "tbv_device.h"

namespace tbv {

// ---------------------------------------------------------------- the step kernel
//
// One body for pack-only, sum-only and pack+sum.  Work unit = one 16-byte vector
// per lane; a block covers blockDim*U consecutive vectors per iteration with the
// U loads of a lane blockDim vectors apart, so each wavefront instruction touches
// 1 KiB of consecutive memory and a lane has U (x2 for the sum) loads in flight.


// The bytes past the last whole vector (at most 15), by the first lanes of one block.
template <int DT, bool PACK, bool SUM>
__device__ __forceinline__ void step_tail(const StepArgs& g)
{
    const unsigned tid = threadIdx.x;
    const unsigned tail = (unsigned)(g.nbytes & 15);
    if (!tail) return;
    const size_t off = (g.nbytes >> 4) << 4;
    if (PACK && tid < tail) ((unsigned char*)g.bounce)[off + tid] = ((const unsigned char*)g.a)[off + tid];
    if (SUM) {
        typedef typename Elem<DT>::T T;
        const unsigned ne = tail / sizeof(T);
        if (tid < ne) {
            const T* pa = (const T*)((const char*)g.a + off);
            const T* pb = (const T*)((const char*)g.b + off);
            T* po = (T*)((char*)g.out + off);
            po[tid] = Elem<DT>::add(pa[tid], pb[tid]);
        }
    }
}

// Block `bid` of `nblk` does its share of the payload; block 0 also does the bytes past the last whole vector.
template <int DT, int U, bool PACK, bool SUM, bool STREAM>
__device__ __forceinline__ void step_body(const StepArgs& g, unsigned bid, unsigned nblk)
{
    const unsigned tid = threadIdx.x, nthr = blockDim.x;
    const size_t nvec = g.nbytes >> 4;
    const size_t tile = (size_t)nthr * U;
    for (size_t base = (size_t)bid * tile; base < nvec; base += (size_t)nblk * tile) {
        u32x4 x[U], y[U];
        if (base + tile <= nvec) {                       // whole tile: no per-vector bounds checks
#pragma unroll
            for (int u = 0; u < U; u++) {
                const size_t i = base + (size_t)u * nthr + tid;
                x[u] = ld_a<STREAM, PACK && SUM>(g.a + i);
                if (SUM) y[u] = ld_b<STREAM>(g.b + i);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const size_t i = base + (size_t)u * nthr + tid;
                if (PACK) st_bounce<STREAM>(g.bounce + i, x[u]);
                if (SUM) st_out<STREAM>(g.out + i, add_vec<DT>(x[u], y[u]));
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const size_t i = base + (size_t)u * nthr + tid;
                if (i < nvec) {
                    x[u] = ld_a<STREAM, PACK && SUM>(g.a + i);
                    if (SUM) y[u] = ld_b<STREAM>(g.b + i);
                    if (PACK) st_bounce<STREAM>(g.bounce + i, x[u]);
                    if (SUM) st_out<STREAM>(g.out + i, add_vec<DT>(x[u], y[u]));
                }
            }
        }
    }
    if (bid == 0) step_tail<DT, PACK, SUM>(g);
}

template <int DT, int U, bool PACK, bool SUM, bool STREAM>
__global__ __launch_bounds__(kMaxSmallThreads, (U <= 2 ? 8 : 1)) void k_step(StepArgs g)
{
    const unsigned tid = threadIdx.x;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);     // deferred signal of the kernel before
    if (PACK && g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    if (SUM && g.wait_flag) gate_wait(g.wait_flag, g.seq, g.spin_limit, g.relay, g.fp, !g.b_uncached);
    step_body<DT, U, PACK, SUM, STREAM>(g, blockIdx.x, gridDim.x);
    if (PACK) {
        if (g.tagp && blockIdx.x == 0 && tid == 0) *g.tagp = g.seq;
        if (g.cflag) grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, gridDim.x, g.sigmode);
    }
    if (SUM && g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

// ---------------------------------------------------------------- pack and sum in one body
//
// One lane loads a[i] once, stores it to the bounce slot and stores a[i] + b[i]: 4 bytes per payload byte, and
// the one form of the step that is safe when the output IS the local tensor (the reference's outp == NULL).
// Only legal when the received payload is already in place (no gate), and only for an uncached bounce.
// The bounce stores of a tile are issued before its output stores, and memory operations of a wave complete
// in the order they were issued, so the pack's completion only has to wait until the U output stores are
// the wave's last outstanding operations: every bounce store is acknowledged by then, and the block is counted
// while its output stores are still on their way (16 MiB cache-cold: 13.9 us with every block counted after
// all of its stores, four vectors per lane, 1024 blocks -> 12.8 us this way with two vectors per lane, one pass).
template <int DT, int U, bool STREAM>
__global__ __launch_bounds__(kMaxSmallThreads, 8) void k_fused(StepArgs g)
{
    const unsigned tid = threadIdx.x, nthr = blockDim.x, bid = blockIdx.x;
    if (g.pre_word && bid == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && bid == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    const size_t nvec = g.nbytes >> 4;
    const size_t tile = (size_t)nthr * U;
    bool ordered = true;        // the wave's last U memory operations are output stores (or it has issued none at all)
    const bool in_place = (const void*)g.out == (const void*)g.a;
    for (size_t base = (size_t)bid * tile; base < nvec; base += (size_t)gridDim.x * tile) {
        u32x4 x[U], y[U];
        if (base + tile <= nvec) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const size_t i = base + (size_t)u * nthr + tid;
                x[u] = ld_a<STREAM, true>(g.a + i);
                y[u] = ld_b<STREAM>(g.b + i);
            }
#pragma unroll
            for (int u = 0; u < U; u++) st_bounce<STREAM>(g.bounce + base + (size_t)u * nthr + tid, x[u]);
            asm volatile("" ::: "memory");      // the output stores stay behind the bounce stores
#pragma unroll
            for (int u = 0; u < U; u++) st_out_at<STREAM>(g.out + base + (size_t)u * nthr + tid, add_vec<DT>(x[u], y[u]), in_place);
            ordered = true;
        } else {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const size_t i = base + (size_t)u * nthr + tid;
                if (i < nvec) {
                    x[u] = ld_a<STREAM, true>(g.a + i);
                    y[u] = ld_b<STREAM>(g.b + i);
                    st_bounce<STREAM>(g.bounce + i, x[u]);
                    st_out_at<STREAM>(g.out + i, add_vec<DT>(x[u], y[u]), in_place);
                }
            }
            ordered = false;
        }
    }
    if (bid == 0 && (g.nbytes & 15)) { step_tail<DT, true, true>(g); ordered = false; }
    if (g.tagp && bid == 0 && tid == 0) { *g.tagp = g.seq; ordered = false; }
    if (g.cflag) grid_complete(g.cflag, g.seq, g.pack_arrive, bid, gridDim.x, 0, ordered ? U : 0);
    if (g.done) grid_complete(g.done, g.seq, g.done_arrive, bid, gridDim.x, 1);
}

// ---------------------------------------------------------------- the merged launch
//
// Pack and sum of one call in ONE launch, as two sets of blocks: blocks [0, P) copy the
// local tensor into the bounce slot and count themselves complete (the pack's completion
// word is raised as soon as those P blocks are done, not at the end of the kernel), the
// remaining blocks sum.  Every kernel in a stream costs about 2.4 us of launch-to-launch
// time on this GPU whatever it does, so the 16 MiB step drops from 14.1 us (two launches)
// to 12.7 us on cache-cold buffers and from 10.9 to 9.6 us on resident ones.  The sum
// blocks read the local tensor themselves: the step still moves 5 bytes per payload byte,
// but pack block b and sum block P+b work on the same vectors and, with P a multiple of
// 8, land on the same XCD (blocks go to the eight XCDs round-robin), so the second read
// is served by that XCD's L2 (counters: 4.007 bytes per payload byte cross the fabric).
// Only legal when the received payload is already in place: there is no gate in this kernel.
template <int DT, int UP, int US, bool STREAM>
__global__ __launch_bounds__(kMaxSmallThreads, ((UP <= 2 && US <= 2) ? 8 : 1)) void k_merged(StepArgs g)
{
    const unsigned tid = threadIdx.x, P = g.pack_blocks;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    if (blockIdx.x < P) {
        step_body<DT, UP, true, false, STREAM>(g, blockIdx.x, P);
        if (g.tagp && blockIdx.x == 0 && tid == 0) *g.tagp = g.seq;
        if (g.cflag) grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, P, g.sigmode);
    } else {
        const unsigned bid = blockIdx.x - P, S = gridDim.x - P;
        step_body<DT, US, false, true, STREAM>(g, bid, S);
        if (g.done) grid_complete(g.done, g.seq, g.done_arrive, bid, S, 1);
    }
}

// The same launch for the common case, stripped: a payload that one pass covers (up to the counters' 8128 blocks
// per part), default block size, no diagnostics, no deferred signal of an earlier kernel, no done word.  Every block
// runs straight code on a whole tile; only a block among the last eight of its part looks at the byte count at all
// (tile_kind below).  The general kernel carries 208 bytes of arguments, four conditional stores and a
// bounds-checked loop; without them the 16 MiB cold launch is 0.3 us shorter (replicas on one box: 11.87 us lean, 12.05 with the general kernel's arguments and
// conditional stores, 12.21 with its loop and bounds as well; the general kernel itself 12.15).
// Their arguments are separate kernel parameters, the ones a wave needs first in front: this file is compiled with
// kernel-argument preloading, which hands the first 14 dwords of scalar and pointer parameters to every wave in
// registers at launch instead of having it load them (a structure passed by value is not preloaded).  A wave of
// these kernels lives about 5 us, and the load of its arguments stood in front of its first data load: the same
// lean launch measures 11.85 us with its arguments loaded and 11.59 us with them preloaded.
struct LeanArgs {
    const u32x4* a; const u32x4* b; u32x4* bounce; u32x4* out;
    unsigned long long* cflag; unsigned int* pack_arrive; unsigned long long seq; unsigned pack_blocks;
    size_t nbytes;
};
// A payload that is not a whole number of tiles ends in a ragged one: its vectors are bounds-checked and the bytes past
// the last whole vector follow, all by the one block that owns that tile (the last of its part of the grid).  Every
// other block runs the straight code; `nbytes` is looked at by the last block only.
// The parts of these grids are a multiple of eight blocks long, so that the pack block and the sum block of a tile
// always land on the same XCD (12 MiB + 2 bytes, 1537 tiles: 10.6 us with 1537 blocks per part, the second read of
// the local tensor then coming from memory, against 9.7 for 12 MiB).  A block among the last eight of its part finds
// out what it has: a whole tile (0), the ragged one (1), or nothing at all (2).
template <int U>
__device__ __forceinline__ int tile_kind(unsigned t, unsigned P, size_t nbytes)
{
    constexpr size_t kTileBytes = (size_t)kThreads * U * 16;
    if (t + 8 <= P) return 0;
    const size_t tiles = (nbytes + kTileBytes - 1) / kTileBytes;
    return t >= tiles ? 2 : (t == tiles - 1 && (nbytes & (kTileBytes - 1))) ? 1 : 0;
}
template <int DT, int U, bool STREAM, bool PACK, bool SUM>
__device__ __forceinline__ void ragged_tile(const u32x4* a, const u32x4* b, u32x4* bounce, u32x4* out, size_t first_vec, size_t nbytes, bool in_place)
{
    const unsigned tid = threadIdx.x;
    const size_t nvec = nbytes >> 4;
#pragma unroll
    for (int u = 0; u < U; u++) {
        const size_t i = first_vec + (size_t)u * kThreads + tid;
        if (i < nvec) {
            const u32x4 x = ld_a<STREAM, PACK && SUM>(a + i);
            if (PACK) st_bounce<STREAM>(bounce + i, x);
            if (SUM) st_out_at<STREAM>(out + i, add_vec<DT>(x, ld_b<STREAM>(b + i)), in_place);
        }
    }
    const unsigned tail = (unsigned)(nbytes & 15);
    if (tail) {
        const size_t off = nvec << 4;
        typedef typename Elem<DT>::T T;
        if (PACK && tid < tail) ((unsigned char*)bounce)[off + tid] = ((const unsigned char*)a)[off + tid];
        if (SUM) __syncthreads();        // in place: the bytes above are read before any of them is overwritten
        if (SUM && tid < tail / sizeof(T))
            ((T*)((char*)out + off))[tid] = Elem<DT>::add(((const T*)((const char*)a + off))[tid], ((const T*)((const char*)b + off))[tid]);
    }
}
template <int DT, int U, bool STREAM>
__global__ __launch_bounds__(kThreads) void k_merged_lean(unsigned P, const u32x4* a, const u32x4* b, u32x4* bounce, u32x4* out,
                                                           unsigned long long* cflag, unsigned int* pack_arrive, unsigned long long seq,
                                                           size_t nbytes)
{
    const unsigned tid = threadIdx.x;
    if (blockIdx.x < P) {
        const int kind = tile_kind<U>(blockIdx.x, P, nbytes);
        if (kind == 1) {
            ragged_tile<DT, U, STREAM, true, false>(a, b, bounce, out, (size_t)blockIdx.x * (kThreads * U), nbytes, false);
        } else if (kind == 0) {
            const size_t base = (size_t)blockIdx.x * (kThreads * U) + tid;
            u32x4 x[U];
#pragma unroll
            for (int u = 0; u < U; u++) x[u] = ld_a<STREAM, false>(a + base + u * kThreads);
#pragma unroll
            for (int u = 0; u < U; u++) st_bounce<STREAM>(bounce + base + u * kThreads, x[u]);
        }
        grid_complete(cflag, seq, pack_arrive, blockIdx.x, P, 0);
        return;
    }
    const int kind = tile_kind<U>(blockIdx.x - P, P, nbytes);
    if (kind == 1) {
        ragged_tile<DT, U, STREAM, false, true>(a, b, bounce, out, (size_t)(blockIdx.x - P) * (kThreads * U), nbytes, false);
    } else if (kind == 0) {
        const size_t base = (size_t)(blockIdx.x - P) * (kThreads * U) + tid;
        u32x4 x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; u++) { x[u] = ld_a<STREAM, false>(a + base + u * kThreads); y[u] = ld_b<STREAM>(b + base + u * kThreads); }
#pragma unroll
        for (int u = 0; u < U; u++) st_out<STREAM>(out + base + u * kThreads, add_vec<DT>(x[u], y[u]));
    }
}

// The fused body and the staged launch for the same common case (one pass of tiles of two vectors per lane, no
// diagnostics, no done word, no earlier kernel's signal).
template <int DT, bool STREAM>
__global__ __launch_bounds__(kThreads) void k_fused_lean(unsigned nblk_ragged, const u32x4* a, const u32x4* b, u32x4* bounce, u32x4* out,
                                                          unsigned long long* cflag, unsigned int* pack_arrive, unsigned long long seq,
                                                          size_t nbytes)
{
    // The number of blocks, and in its top bit whether the last tile is ragged, come as the first argument, preloaded
    // with the pointers: nothing a block has to load (the grid's dimensions, the byte count) stands between its start
    // and its first data load unless it is that last block.
    constexpr int U = 2;
    const unsigned nblk = nblk_ragged & 0x7fffffffu;
    if (nblk_ragged == ((blockIdx.x + 1) | 0x80000000u)) {
        ragged_tile<DT, U, STREAM, true, true>(a, b, bounce, out, (size_t)blockIdx.x * (kThreads * U), nbytes, (const void*)out == (const void*)a);
        grid_complete(cflag, seq, pack_arrive, blockIdx.x, nblk, 0);
        return;
    }
    const size_t base = (size_t)blockIdx.x * (kThreads * U) + threadIdx.x;
    u32x4 x[U], y[U];
#pragma unroll
    for (int u = 0; u < U; u++) { x[u] = ld_a<STREAM, true>(a + base + u * kThreads); y[u] = ld_b<STREAM>(b + base + u * kThreads); }
#pragma unroll
    for (int u = 0; u < U; u++) st_bounce<STREAM>(bounce + base + u * kThreads, x[u]);
    asm volatile("" ::: "memory");      // the output stores stay behind the bounce stores
    const bool in_place = (const void*)out == (const void*)a;
#pragma unroll
    for (int u = 0; u < U; u++) st_out_at<STREAM>(out + base + u * kThreads, add_vec<DT>(x[u], y[u]), in_place);
    grid_complete(cflag, seq, pack_arrive, blockIdx.x, nblk, 0, U);
}

struct LeanGateArgs {
    LeanArgs w;
    const unsigned long long* wait_flag; unsigned long long* relay; unsigned long long spin_limit;
    unsigned tiles;             // tiles of the sum part, taken in turn by its blocks
};
// (the received payload lies in uncached memory: the gate needs no cache invalidation; the host checks that)
template <int DT, bool STREAM>
__global__ __launch_bounds__(kThreads) void k_pipe_lean(unsigned P, const u32x4* a, const u32x4* b, u32x4* out, unsigned long long* relay,
                                                         unsigned long long seq, u32x4* bounce, const unsigned long long* wait_flag,
                                                         unsigned long long* cflag, unsigned int* pack_arrive, unsigned long long spin_limit, unsigned tiles,
                                                         size_t nbytes)
{
    constexpr int U = 2;
    constexpr size_t kTileBytes = (size_t)kThreads * U * 16;
    const unsigned tid = threadIdx.x;
    if (blockIdx.x < P) {
        if (blockIdx.x == 0 && tid == 0 && __hip_atomic_load(wait_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) >= seq)
            __hip_atomic_store(relay, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);       // one look, as in k_pipe
        const int kind = tile_kind<U>(blockIdx.x, P, nbytes);
        if (kind == 1) {
            ragged_tile<DT, U, STREAM, true, false>(a, b, bounce, out, (size_t)blockIdx.x * (kThreads * U), nbytes, false);
        } else if (kind == 0) {
            const size_t base = (size_t)blockIdx.x * (kThreads * U) + tid;
            u32x4 x[U];
#pragma unroll
            for (int u = 0; u < U; u++) x[u] = ld_a<STREAM, false>(a + base + u * kThreads);
#pragma unroll
            for (int u = 0; u < U; u++) st_bounce<STREAM>(bounce + base + u * kThreads, x[u]);
        }
        grid_complete(cflag, seq, pack_arrive, blockIdx.x, P, 0);
    } else {
        const unsigned bid = blockIdx.x - P, S = gridDim.x - P;
        gate_wait_as(bid, wait_flag, seq, spin_limit, relay, nullptr, false, nullptr, true);
        for (unsigned t = bid; t < tiles; t += S) {
            if (t == tiles - 1 && (nbytes & (kTileBytes - 1))) {
                ragged_tile<DT, U, STREAM, false, true>(a, b, bounce, out, (size_t)t * (kThreads * U), nbytes, false);
                break;
            }
            const size_t base = (size_t)t * (kThreads * U) + tid;
            u32x4 x[U], y[U];
#pragma unroll
            for (int u = 0; u < U; u++) { x[u] = ld_a<STREAM, false>(a + base + u * kThreads); y[u] = ld_b<STREAM>(b + base + u * kThreads); }
#pragma unroll
            for (int u = 0; u < U; u++) st_out<STREAM>(out + base + u * kThreads, add_vec<DT>(x[u], y[u]));
        }
    }
}

// ---------------------------------------------------------------- the pipeline step
//
// Pack blocks and GATED sum blocks in one launch, each set with its own arguments.  Blocks [0, P) pack and raise
// the pack's completion word; the rest wait for a flag (block P polls the host word and relays it) and sum.  The
// pack blocks have the lower indices, so they are placed first and never wait: a rank always sends before it waits,
// so two ranks running this against each other cannot deadlock.  Two uses:
//   chunked pipeline   pack of chunk i+depth + sum of chunk i: per chunk the caller's thread pays one launch instead of
//                      a pack launch, a stream wait and a sum launch (3.5 us of host time instead of 11)
//   one staged call    pack and sum of the SAME call when the peer's payload is not there yet (what two real ranks
//                      see): one launch instead of pack, stream gate, sum.  When the output aliases the local tensor
//                      the sum blocks also wait for the last pack block (sm.pack_relay), since a sum block may
//                      otherwise store out[i] while a pack block has yet to read a[i].
template <int DT, int UP, int US, bool STREAM>
__global__ __launch_bounds__(kMaxSmallThreads, ((UP <= 2 && US <= 2) ? 8 : 1)) void k_pipe(StepArgs pk, StepArgs sm)
{
    const unsigned tid = threadIdx.x, P = pk.pack_blocks;
    if (pk.pre_word && blockIdx.x == 0 && tid == 0) store_sys(pk.pre_word, pk.pre_seq);
    if (blockIdx.x < P) {
        // One look at the flag by the first block's first lane before its own work, without polling: when the peer was
        // early, the relay word is up before the first sum block is placed (they follow the pack blocks by 2-3 us) and
        // the gate costs the sum blocks one poll of device memory instead of a read of host memory.  This is a single
        // load, bounded by memory latency, not a wait for the peer.  (Not with an output that aliases the local
        // tensor: those sum blocks must see the pack relay first, which only the polling block republishes.)
        if (blockIdx.x == 0 && tid == 0 && sm.wait_flag && sm.relay && !sm.pack_relay &&
            __hip_atomic_load(sm.wait_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) >= sm.seq)
            __hip_atomic_store(sm.relay, sm.seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        step_body<DT, UP, true, false, STREAM>(pk, blockIdx.x, P);
        if (pk.cflag) {
            const bool last = grid_complete(pk.cflag, pk.seq, pk.pack_arrive, blockIdx.x, P, pk.sigmode);
            if (last && pk.pack_relay) __hip_atomic_store(pk.pack_relay, pk.seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        // The sum part works on `tiles` tiles of blockDim x US vectors; its blocks (capped in number, because a waiting
        // block holds its wave slots) take tiles bid, bid + S, ...  (Tried and dropped, neither changed the 14.0 us of a
        // 16 MiB launch whose flag is up beforehand: blocks behind the waiting ones that look at the relay once and take
        // the waiting blocks' second tiles if it is up; loading the first tile of the local tensor ahead of the gate.)
        const unsigned bid = blockIdx.x - P, S = gridDim.x - P, T = sm.tiles;
        if (sm.wait_flag) gate_wait_as(bid, sm.wait_flag, sm.seq, sm.spin_limit, sm.relay, sm.fp, !sm.b_uncached, sm.pack_relay, true);
        for (unsigned t = bid; t < T; t += S) step_body<DT, US, false, true, STREAM>(sm, t, T);
        if (sm.done) grid_complete(sm.done, sm.seq, sm.done_arrive, bid, S, 1);
    }
}

// ---------------------------------------------------------------- the one-kernel small call
//
// A whole small call in one launch: pack this block's vectors into the bounce slot,
// count the blocks and raise the pack's completion word, poll the flag, then sum with
// the local vectors still in registers.  The signal precedes the wait inside the same
// kernel, so two ranks running this against each other cannot wait for one another's
// data before having sent their own.  One vector per lane; the host keeps the grid to
// a handful of blocks so that all of them are resident together (a block that has
// not started cannot be counted, and the counted total gates everyone's flag).
template <int DT>
__global__ __launch_bounds__(kMaxSmallThreads) void k_small_call(StepArgs g)
{
    const unsigned tid = threadIdx.x;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    const size_t nvec = g.nbytes >> 4;
    const size_t i = (size_t)blockIdx.x * blockDim.x + tid;
    const bool mine = i < nvec;
    const unsigned tail = (unsigned)(g.nbytes & 15);
    const size_t off = nvec << 4;
    u32x4 x = {0, 0, 0, 0};
    if (mine) { x = ld_a<false, true>(g.a + i); st_bounce<false>(g.bounce + i, x); }
    if (tail && blockIdx.x == 0 && tid < tail) ((unsigned char*)g.bounce)[off + tid] = ((const unsigned char*)g.a)[off + tid];
    grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, gridDim.x, g.sigmode);
    if (g.wait_flag) gate_wait(g.wait_flag, g.seq, g.spin_limit, g.relay, g.fp, !g.b_uncached);
    if (mine) st_out<false>(g.out + i, add_vec<DT>(x, ld_b<false>(g.b + i)));
    if (tail && blockIdx.x == 0) {
        typedef typename Elem<DT>::T T;
        const unsigned ne = tail / sizeof(T);
        if (tid < ne) {
            const T* pa = (const T*)((const char*)g.a + off);
            const T* pb = (const T*)((const char*)g.b + off);
            T* po = (T*)((char*)g.out + off);
            po[tid] = Elem<DT>::add(pa[tid], pb[tid]);
        }
    }
    if (g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

// Fallback bodies for caller pointers that are not 16-byte aligned: element (sum)
// or 4/1-byte (pack) grid-stride loops.  Same results, lower bandwidth.
template <typename W>
__global__ __launch_bounds__(kThreads) void k_pack_narrow(PackArgs a)
{
    if (a.pre.word && blockIdx.x == 0 && threadIdx.x == 0) store_sys(a.pre.word, a.pre.seq);
    if (a.fp && blockIdx.x == 0 && threadIdx.x == 0) store_sys(a.fp + FP_PACK, a.seq);
    const size_t n = a.nbytes / sizeof(W);
    const W* s = (const W*)a.src; W* d = (W*)a.dst;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) d[i] = s[i];
    const unsigned tail = (unsigned)(a.nbytes - n * sizeof(W));
    if (blockIdx.x == 0 && threadIdx.x < tail)
        ((unsigned char*)a.dst)[n * sizeof(W) + threadIdx.x] = ((const unsigned char*)a.src)[n * sizeof(W) + threadIdx.x];
    if (a.tagp && blockIdx.x == 0 && threadIdx.x == 0) *a.tagp = a.seq;
    if (a.cflag) grid_complete(a.cflag, a.seq, a.arrive, blockIdx.x, gridDim.x, a.sigmode);
}

template <int DT>
__global__ __launch_bounds__(kThreads) void k_sum_narrow(SumArgs a)
{
    typedef typename Elem<DT>::T T;
    if (a.pre.word && blockIdx.x == 0 && threadIdx.x == 0) store_sys(a.pre.word, a.pre.seq);
    if (a.wait_flag) gate_wait(a.wait_flag, a.seq, a.spin_limit_ticks, a.relay, a.fp, !a.b_uncached);
    const size_t n = a.nbytes / sizeof(T);
    const T* x = (const T*)a.a; const T* y = (const T*)a.b; T* o = (T*)a.out;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        o[i] = Elem<DT>::add(x[i], y[i]);
    if (a.done) grid_complete(a.done, a.seq, a.done_arrive, blockIdx.x, gridDim.x, 1);
}

// ---------------------------------------------------------------- diagnostics

__global__ void k_waitflag(const unsigned long long* flag, unsigned long long seq, unsigned long long limit,
                           unsigned long long* fp)
{
    gate_wait(flag, seq, limit, nullptr, fp);
}

// Re-reads the sequence tag the pack kernel appended to the payload, once with a
// plain load and once with a system-scope load, and counts disagreements.
// dbg: [checks, plain mismatches, system mismatches, first bad seq, first plain value, first system value]
__global__ void k_tagchk(const unsigned long long* tag, unsigned long long seq, unsigned long long* dbg)
{
    unsigned long long v1 = *(const volatile unsigned long long*)tag;
    unsigned long long v2 = __hip_atomic_load(tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_fetch_add(dbg + 0, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (v1 != seq) __hip_atomic_fetch_add(dbg + 1, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (v2 != seq) __hip_atomic_fetch_add(dbg + 2, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if ((v1 != seq || v2 != seq) && dbg[3] == 0) { dbg[3] = seq; dbg[4] = v1; dbg[5] = v2; }
}

__global__ void k_mark(unsigned long long* fp, int i, unsigned long long seq) { store_sys(fp + i, seq); }

__global__ void k_fill_u32(unsigned int* p, unsigned int v, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}

// ---------------------------------------------------------------- launch geometry
//
// Measured on MI355X with the 16 MiB step (two launches, microseconds per step, cache-cold
// / cache-resident buffers): resident hints, one vector per lane, 1024 blocks 15.98 / 10.86;
// streaming hints, four vectors per lane, 1024 blocks 14.18 / 11.18; more blocks (2048,
// 4096) or 512/1024-lane blocks change nothing; fewer (256, 512) lose 10-40 %.

static int g_unroll = 0;        // vectors per lane per iteration for the large path; 0 = the profile's choice
// the completion counters have one line per group of blocks (32, or 64 for the largest grids): no grid may be larger
static constexpr int kMostBlocks = (int)(2 * kGroup * (kCounterWords / kCtrLine - 1));
static int g_grid_cap = 1024;
static bool g_grid_cap_given = false;   // a cap from the environment applies to every launch shape
static int g_block = kThreads;
static bool g_stream = false;   // streaming profile (see the cache hints above)
static int g_gated_cap = kGatedMaxGrid;     // most blocks of a grid (or part of one) that waits for a flag inside
// The cap is held in waves as well: whatever block size is in use, the waiting part of a grid never takes more than half
// of the GPU's 8192 wave slots (a cap counted in blocks alone would let 1024 blocks of 512 lanes fill every slot, and the
// kernel whose completion raises the flag could then never be placed).
static constexpr int kGatedMaxWaves = 4096;
static inline int gated_cap_for(int block)
{
    const int by_waves = kGatedMaxWaves / ((block + 63) / 64);
    const int cap = g_gated_cap < by_waves ? g_gated_cap : by_waves;
    return cap < 1 ? 1 : cap;
}
static int g_gated_unroll = 2;

struct Geom { int grid, block, unroll; };

static Geom geom_for(size_t nbytes, bool writeback = false, bool merged = false)
{
    size_t nvec = nbytes >> 4;
    Geom g;
    if (nvec <= (size_t)kMaxSmallThreads) {
        // one block, one vector per lane: no cross-block arrival counting on the latency path
        int thr = (int)((nvec + 63) / 64 * 64);
        if (thr < 64) thr = 64;
        g.grid = 1; g.block = thr; g.unroll = 1;
        return g;
    }
    g.block = g_block;
    int cap = g_grid_cap;
    if (g_unroll) g.unroll = (nvec >= (size_t)kThreads * 16) ? g_unroll : 1;
    else if (merged) {
        // the halves of a merged launch run side by side and do best when every block makes a single pass of two
        // vectors per lane (16 MiB, cold / resident: 12.75 / 9.55 us against 13.05 / 10.2 with 1024 blocks of one)
        // (32 - 256 MiB: one pass of up to 8128 blocks per half 7.1-7.2 TB/s on 5N, 2048 looping blocks 6.8-7.05)
        g.unroll = nvec >= (size_t)2 * g_block * 1024 ? 2 : 1;
        if (!g_grid_cap_given) cap = kMostBlocks;
    } else {
        // the streaming profile keeps four loads per lane in flight, as long as that still leaves a block for every
        // grid position, and makes one pass where the counters can count the blocks (64 MiB two-launch step 50.6 ->
        // 49.2 us, 256 MiB 194.9 -> 189.5 us); the resident profile keeps to four blocks per CU
        g.unroll = (g_stream && nvec >= (size_t)4 * g_block * g_grid_cap) ? 4 : 1;
        if (g_stream && !g_grid_cap_given) cap = kMostBlocks;
    }
    // an L2 write-back per block is dear and they run one after another: use one fat block per CU
    if (writeback) { cap = 256; g.unroll = 8; }
    size_t tile = (size_t)g.block * g.unroll;
    size_t tiles = (nvec + tile - 1) / tile;
    g.grid = (int)(tiles < (size_t)cap ? tiles : (size_t)cap);
    if (g.grid < 1) g.grid = 1;
    return g;
}

int pack_grid(size_t nbytes) { return geom_for(nbytes).grid; }
int sum_grid(size_t nbytes, int) { return geom_for(nbytes).grid; }

void set_gated_tuning(int cap, int unroll)
{
    // a waiting block holds its wave slots: never more than half of the GPU's 8192 (1024 blocks of 4 waves)
    g_gated_cap = cap >= 1 ? (cap > 1024 ? 1024 : cap) : kGatedMaxGrid;
    g_gated_unroll = (unroll == 1 || unroll == 2 || unroll == 4) ? unroll : 2;
}

void set_tuning(int unroll, int grid_cap, int block, int streaming)
{
    g_block = (block == 512 || block == 1024) ? block : kThreads;
    g_unroll = (unroll == 1 || unroll == 2 || unroll == 4 || unroll == 8) ? unroll : 0;
    g_grid_cap = grid_cap >= 1 ? (grid_cap < kMostBlocks ? grid_cap : kMostBlocks) : 1024;
    g_grid_cap_given = grid_cap >= 1;
    g_stream = streaming != 0;
}

bool streaming_profile() { return g_stream; }

static inline bool al16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// One launch of a kernel that takes a single argument struct; with `t` the
// dispatch's own start/end timestamps land in t->start / t->stop.
template <typename A>
static hipError_t launch1(void (*kernel)(A), int grid, int block, hipStream_t st, const Timing* t, const A& arg)
{
    if (t && t->start && t->stop) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, t->start, t->stop, 0, arg);
    else hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, arg);
    return hipGetLastError();
}

// The same for a kernel that takes its arguments one by one.
template <typename... P, typename... A>
static hipError_t launch_each(void (*kernel)(P...), int grid, int block, hipStream_t st, const Timing* t, A... args)
{
    if (t && t->start && t->stop) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, t->start, t->stop, 0, static_cast<P>(args)...);
    else hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, static_cast<P>(args)...);
    return hipGetLastError();
}

template <int DT, bool PACK, bool SUM, bool STREAM>
static hipError_t launch_step_u(const StepArgs& s, const Geom& g, hipStream_t st, const Timing* t)
{
    switch (g.unroll) {
        case 1: return launch1(k_step<DT, 1, PACK, SUM, STREAM>, g.grid, g.block, st, t, s);
        case 2: return launch1(k_step<DT, 2, PACK, SUM, STREAM>, g.grid, g.block, st, t, s);
        case 8: return launch1(k_step<DT, 8, PACK, SUM, STREAM>, g.grid, g.block, st, t, s);
        default: return launch1(k_step<DT, 4, PACK, SUM, STREAM>, g.grid, g.block, st, t, s);
    }
}

template <bool PACK, bool SUM>
static hipError_t launch_step(int dtype, const StepArgs& s, const Geom& g, hipStream_t st, const Timing* t)
{
    if (g_stream) {
        if (!SUM) return launch_step_u<0, PACK, SUM, true>(s, g, st, t);      // the copy does not depend on the element type
        switch (dtype) {
            case 0: return launch_step_u<0, PACK, SUM, true>(s, g, st, t);
            case 1: return launch_step_u<1, PACK, SUM, true>(s, g, st, t);
            case 2: return launch_step_u<2, PACK, SUM, true>(s, g, st, t);
        }
        return hipErrorInvalidValue;
    }
    if (!SUM) return launch_step_u<0, PACK, SUM, false>(s, g, st, t);
    switch (dtype) {
        case 0: return launch_step_u<0, PACK, SUM, false>(s, g, st, t);
        case 1: return launch_step_u<1, PACK, SUM, false>(s, g, st, t);
        case 2: return launch_step_u<2, PACK, SUM, false>(s, g, st, t);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_pack(const PackArgs& a, hipStream_t st, const Timing* t)
{
    if (!a.dst || !a.src || (a.cflag && !a.arrive) || !al16(a.dst)) return hipErrorInvalidValue;
    if (al16(a.src)) {
        StepArgs s{};
        s.bounce = (u32x4*)a.dst; s.cflag = a.cflag; s.pack_arrive = a.arrive; s.tagp = a.tagp;
        s.a = (const u32x4*)a.src; s.nbytes = a.nbytes; s.seq = a.seq; s.fp = a.fp; s.sigmode = a.sigmode;
        s.pre_word = a.pre.word; s.pre_seq = a.pre.seq;
        return launch_step<true, false>(0, s, geom_for(a.nbytes, a.sigmode != 0), st, t);
    }
    size_t units = a.nbytes / 4 + 1;
    int grid = (int)((units + kThreads - 1) / kThreads); if (grid > 1024) grid = 1024;
    if ((((uintptr_t)a.src) & 3) == 0) return launch1(k_pack_narrow<uint32_t>, grid, kThreads, st, t, a);
    return launch1(k_pack_narrow<unsigned char>, grid, kThreads, st, t, a);
}

hipError_t launch_sum(const SumArgs& a, hipStream_t st, const Timing* t)
{
    if (!a.out || !a.a || !a.b || a.dtype < 0 || a.dtype > 2) return hipErrorInvalidValue;
    if (a.done && !a.done_arrive) return hipErrorInvalidValue;
    if (al16(a.out) && al16(a.a) && al16(a.b)) {
        StepArgs s{};
        s.out = (u32x4*)a.out; s.b = (const u32x4*)a.b; s.wait_flag = a.wait_flag; s.relay = a.relay; s.spin_limit = a.spin_limit_ticks; s.b_uncached = a.b_uncached;
        s.done = a.done; s.done_arrive = a.done_arrive;
        s.a = (const u32x4*)a.a; s.nbytes = a.nbytes; s.seq = a.seq; s.fp = a.fp;
        s.pre_word = a.pre.word; s.pre_seq = a.pre.seq;
        Geom g = geom_for(a.nbytes);
        if (a.wait_flag && g.grid > gated_cap_for(g.block)) g.grid = gated_cap_for(g.block);
        return launch_step<false, true>(a.dtype, s, g, st, t);
    }
    size_t esz = a.dtype == 0 ? 4 : 2, n = a.nbytes / esz;
    int grid = (int)((n + kThreads - 1) / kThreads); if (grid > kMaxGrid) grid = kMaxGrid; if (grid < 1) grid = 1;
    if (a.wait_flag && grid > gated_cap_for(kThreads)) grid = gated_cap_for(kThreads);
    switch (a.dtype) {
        case 0: return launch1(k_sum_narrow<0>, grid, kThreads, st, t, a);
        case 1: return launch1(k_sum_narrow<1>, grid, kThreads, st, t, a);
        default: return launch1(k_sum_narrow<2>, grid, kThreads, st, t, a);
    }
}

static bool overlaps(const void* x, size_t nx, const void* y, size_t ny)
{
    const uintptr_t a = (uintptr_t)x, b = (uintptr_t)y;
    return a < b + ny && b < a + nx;
}

// `two_readers`: pack and sum are done by different blocks, each reading the local tensor itself; then the output must
// not overlap the local tensor (a sum block could store out[i] before the pack block has read a[i]).  With one reader
// (the fused body: one lane loads a[i] once and does both stores) an output equal to the local tensor is fine.
static bool fill_pack_sum(StepArgs& s, const PackArgs& p, const SumArgs& q, bool two_readers = false)
{
    if (two_readers && overlaps(q.out, q.nbytes, p.src, p.nbytes)) return false;
    if (!(al16(p.src) && al16(p.dst) && al16(q.out) && al16(q.b)) || p.src != q.a || p.nbytes != q.nbytes || !p.dst || !q.out || !q.b)
        return false;
    if (q.dtype < 0 || q.dtype > 2 || (q.done && !q.done_arrive) || (p.cflag && !p.arrive)) return false;
    if (q.wait_flag) return false;     // waiting for the peer before sending to it would deadlock two real ranks
    s.bounce = (u32x4*)p.dst; s.cflag = p.cflag; s.pack_arrive = p.arrive; s.tagp = p.tagp;
    s.out = (u32x4*)q.out; s.b = (const u32x4*)q.b; s.wait_flag = nullptr; s.relay = nullptr; s.spin_limit = 0;
    s.done = q.done; s.done_arrive = q.done_arrive;
    s.a = (const u32x4*)p.src; s.nbytes = p.nbytes; s.seq = p.seq; s.fp = p.fp; s.sigmode = p.sigmode;
    s.pre_word = p.pre.word; s.pre_seq = p.pre.seq;
    return true;
}

template <int DT, bool STREAM>
static hipError_t launch_fused_u(const StepArgs& s, const Geom& g, hipStream_t st, const Timing* t)
{
    if (g.unroll == 2) return launch1(k_fused<DT, 2, STREAM>, g.grid, g.block, st, t, s);
    return launch1(k_fused<DT, 1, STREAM>, g.grid, g.block, st, t, s);
}

hipError_t launch_pack_sum(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t)
{
    StepArgs s{};
    if (!fill_pack_sum(s, p, q)) return hipErrorInvalidValue;
    // a cached bounce needs its L2 write-back per block: the general step kernel with its fat blocks
    if (p.sigmode != 0 || (p.nbytes >> 4) <= (size_t)kMaxSmallThreads || (g_unroll && g_unroll != 1 && g_unroll != 2))
        return launch_step<true, true>(q.dtype, s, geom_for(p.nbytes, p.sigmode != 0), st, t);
    // uncached bounce: the shape of one half of the merged launch (one pass of two vectors per lane where the counters
    // can count the blocks), completion counted on the bounce stores alone
    Geom g = geom_for(p.nbytes, false, true);
    if (g.unroll != 2) g.unroll = 1;
    // one pass, nothing but the step itself: the stripped kernel
    const size_t lean_blocks = (s.nbytes + (size_t)kThreads * 2 * 16 - 1) / ((size_t)kThreads * 2 * 16);
    if (g.unroll == 2 && g.block == kThreads && lean_blocks <= (size_t)(g_grid_cap_given ? g_grid_cap : kMostBlocks) &&
        s.cflag && !s.pre_word && !s.fp && !s.tagp && !s.done) {
        g.grid = (int)lean_blocks;
        const LeanArgs w{s.a, s.b, s.bounce, s.out, s.cflag, s.pack_arrive, s.seq, (unsigned)g.grid, s.nbytes};
        if (g_stream) {
            switch (q.dtype) {
                case 0: return launch_each(k_fused_lean<0, true>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
                case 1: return launch_each(k_fused_lean<1, true>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
                default: return launch_each(k_fused_lean<2, true>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
            }
        }
        switch (q.dtype) {
            case 0: return launch_each(k_fused_lean<0, false>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
            case 1: return launch_each(k_fused_lean<1, false>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
            default: return launch_each(k_fused_lean<2, false>, g.grid, kThreads, st, t, w.pack_blocks | ((w.nbytes & 8191) ? 0x80000000u : 0u), w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
        }
    }
    if (g_stream) {
        switch (q.dtype) {
            case 0: return launch_fused_u<0, true>(s, g, st, t);
            case 1: return launch_fused_u<1, true>(s, g, st, t);
            default: return launch_fused_u<2, true>(s, g, st, t);
        }
    }
    switch (q.dtype) {
        case 0: return launch_fused_u<0, false>(s, g, st, t);
        case 1: return launch_fused_u<1, false>(s, g, st, t);
        default: return launch_fused_u<2, false>(s, g, st, t);
    }
}

template <int DT, bool STREAM>
static hipError_t launch_merged_u(const StepArgs& s, int grid, int block, int unroll, hipStream_t st, const Timing* t)
{
    switch (unroll) {
        case 2: return launch1(k_merged<DT, 2, 2, STREAM>, grid, block, st, t, s);
        case 4: return launch1(k_merged<DT, 4, 4, STREAM>, grid, block, st, t, s);
        default: return launch1(k_merged<DT, 1, 1, STREAM>, grid, block, st, t, s);
    }
}

template <int DT, bool STREAM>
static hipError_t launch_merged_lean(const LeanArgs& w, int grid, int unroll, hipStream_t st, const Timing* t)
{
    if (unroll == 2) return launch_each(k_merged_lean<DT, 2, STREAM>, grid, kThreads, st, t, w.pack_blocks, w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
    return launch_each(k_merged_lean<DT, 1, STREAM>, grid, kThreads, st, t, w.pack_blocks, w.a, w.b, w.bounce, w.out, w.cflag, w.pack_arrive, w.seq, w.nbytes);
}

static hipError_t launch_merged_one(int dtype, StepArgs& s, hipStream_t st, const Timing* t)
{
    Geom g = geom_for(s.nbytes, false, true);
    // each part a multiple of eight blocks long: pack block b and sum block P + b then share an XCD and its L2
    if (!g_grid_cap_given && g.grid > 8) g.grid = (g.grid + 7) & ~7;
    s.pack_blocks = (unsigned)g.grid;
    int grid = 2 * g.grid;
    const int u = g.unroll == 8 ? 4 : g.unroll;
    // one pass, nothing but the step itself: the stripped kernel (a last tile that is not whole goes to one block's slow path)
    const size_t lean_blocks = (s.nbytes + (size_t)kThreads * u * 16 - 1) / ((size_t)kThreads * u * 16);
    if ((u == 1 || u == 2) && g.block == kThreads && lean_blocks <= (size_t)(g_grid_cap_given ? g_grid_cap : kMostBlocks) &&
        s.cflag && s.sigmode == 0 && !s.pre_word && !s.fp && !s.tagp && !s.done) {
        const unsigned part = (unsigned)((lean_blocks + 7) & ~(size_t)7);       // a multiple of eight (so is the cap)
        grid = 2 * (int)part;
        const LeanArgs w{s.a, s.b, s.bounce, s.out, s.cflag, s.pack_arrive, s.seq, part, s.nbytes};
        if (g_stream) {
            switch (dtype) {
                case 0: return launch_merged_lean<0, true>(w, grid, u, st, t);
                case 1: return launch_merged_lean<1, true>(w, grid, u, st, t);
                default: return launch_merged_lean<2, true>(w, grid, u, st, t);
            }
        }
        switch (dtype) {
            case 0: return launch_merged_lean<0, false>(w, grid, u, st, t);
            case 1: return launch_merged_lean<1, false>(w, grid, u, st, t);
            default: return launch_merged_lean<2, false>(w, grid, u, st, t);
        }
    }
    if (g_stream) {
        switch (dtype) {
            case 0: return launch_merged_u<0, true>(s, grid, g.block, u, st, t);
            case 1: return launch_merged_u<1, true>(s, grid, g.block, u, st, t);
            default: return launch_merged_u<2, true>(s, grid, g.block, u, st, t);
        }
    }
    switch (dtype) {
        case 0: return launch_merged_u<0, false>(s, grid, g.block, u, st, t);
        case 1: return launch_merged_u<1, false>(s, grid, g.block, u, st, t);
        default: return launch_merged_u<2, false>(s, grid, g.block, u, st, t);
    }
}

// The two halves of a merged launch share the local tensor through the L2 only while they stay close in time, and the
// pack half (2 bytes per payload byte) runs ahead of the sum half (3): at 1 GiB one launch moves 5.1-5.45 TB/s against
// 7.2 at 256 MiB.  A payload beyond the segment size therefore goes out as several merged launches one after the other
// on the stream, each over its own segment; only the last one raises the completion words (stream order has finished
// the earlier segments, stores included, before it starts).
static size_t g_merge_segment = (size_t)256 << 20;
void set_merge_segment(size_t bytes) { g_merge_segment = bytes >= ((size_t)1 << 20) ? (bytes & ~(size_t)4095) : (size_t)256 << 20; }

hipError_t launch_pack_sum_merged(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t)
{
    StepArgs s{};
    if (!fill_pack_sum(s, p, q, true) || p.sigmode != 0) return hipErrorInvalidValue;
    const size_t seg = g_merge_segment, n = p.nbytes;
    if (n <= seg) return launch_merged_one(q.dtype, s, st, t);
    for (size_t off = 0; off < n; off += seg) {
        const bool first = off == 0, last = off + seg >= n;
        StepArgs x = s;
        x.a = (const u32x4*)((const char*)s.a + off); x.b = (const u32x4*)((const char*)s.b + off);
        x.bounce = (u32x4*)((char*)s.bounce + off); x.out = (u32x4*)((char*)s.out + off);
        x.nbytes = last ? n - off : seg;
        if (!first) { x.pre_word = nullptr; x.fp = nullptr; }
        if (!last) { x.cflag = nullptr; x.tagp = nullptr; x.done = nullptr; }
        const hipError_t e = launch_merged_one(q.dtype, x, st, last ? t : nullptr);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <typename A, typename B>
static hipError_t launch2(void (*kernel)(A, B), int grid, int block, hipStream_t st, const Timing* t, const A& a, const B& b)
{
    if (t && t->start && t->stop) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, t->start, t->stop, 0, a, b);
    else hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, a, b);
    return hipGetLastError();
}

template <int DT, bool STREAM>
static hipError_t launch_pipe_u(int up, int us, int grid, int block, hipStream_t st, const Timing* t, const StepArgs& pk, const StepArgs& sm)
{
    if (up == 2) {
        switch (us) {
            case 1: return launch2(k_pipe<DT, 2, 1, STREAM>, grid, block, st, t, pk, sm);
            case 2: return launch2(k_pipe<DT, 2, 2, STREAM>, grid, block, st, t, pk, sm);
            default: return launch2(k_pipe<DT, 2, 4, STREAM>, grid, block, st, t, pk, sm);
        }
    }
    switch (us) {
        case 1: return launch2(k_pipe<DT, 1, 1, STREAM>, grid, block, st, t, pk, sm);
        case 2: return launch2(k_pipe<DT, 1, 2, STREAM>, grid, block, st, t, pk, sm);
        default: return launch2(k_pipe<DT, 1, 4, STREAM>, grid, block, st, t, pk, sm);
    }
}

hipError_t launch_pipe(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t, unsigned long long* pack_relay)
{
    if (!p.dst || !p.src || !p.cflag || !p.arrive || p.sigmode != 0 || p.tagp || !al16(p.dst) || !al16(p.src)) return hipErrorInvalidValue;
    if (!q.out || !q.a || !q.b || !al16(q.out) || !al16(q.a) || !al16(q.b) || q.dtype < 0 || q.dtype > 2 || (q.done && !q.done_arrive) ||
        (q.wait_flag && !q.relay))
        return hipErrorInvalidValue;
    // The two parts read and write at the same time.  Different chunks of one tensor never overlap; pack and sum of the
    // same bytes do when the call is in place, and are then ordered through the pack relay (which needs the gate's poll).
    const bool same = overlaps(q.out, q.nbytes, p.src, p.nbytes);
    if (same && !(pack_relay && q.wait_flag)) return hipErrorInvalidValue;
    StepArgs pk{}, sm{};
    pk.bounce = (u32x4*)p.dst; pk.cflag = p.cflag; pk.pack_arrive = p.arrive; pk.a = (const u32x4*)p.src; pk.nbytes = p.nbytes;
    pk.seq = p.seq; pk.sigmode = p.sigmode; pk.pre_word = p.pre.word; pk.pre_seq = p.pre.seq;
    sm.out = (u32x4*)q.out; sm.a = (const u32x4*)q.a; sm.b = (const u32x4*)q.b; sm.nbytes = q.nbytes; sm.seq = q.seq; sm.fp = q.fp;
    sm.wait_flag = q.wait_flag; sm.relay = q.relay; sm.spin_limit = q.spin_limit_ticks; sm.done = q.done; sm.done_arrive = q.done_arrive;
    sm.b_uncached = q.b_uncached;
    if (same) { pk.pack_relay = pack_relay; sm.pack_relay = pack_relay; }
    // one block size for both parts; tiny chunks take the generic size too (their single-block shapes do not mix)
    const int block = g_block;
    // pack part: one vector per lane, or two from 8 MiB so that the part stays within 2048 blocks in one pass up to 16 MiB
    const size_t pvec = p.nbytes >> 4, svec = q.nbytes >> 4;
    const int up = pvec >= (size_t)2 * block * 1024 ? 2 : 1;
    const int us = q.wait_flag ? g_gated_unroll : 4;
    int P = (int)((pvec + (size_t)block * up - 1) / ((size_t)block * up));
    if (P < 1) P = 1;
    const int pcap = g_grid_cap_given ? g_grid_cap : 2048;
    if (P > pcap) P = pcap;
    // sum part: T tiles, taken in turn by at most `wcap` blocks (see k_pipe)
    size_t T = (svec + (size_t)block * us - 1) / ((size_t)block * us);
    if (T < 1) T = 1;
    if (T > 0x7fffffffu) return hipErrorInvalidValue;
    const size_t wcap = (size_t)(q.wait_flag ? gated_cap_for(block) : g_grid_cap);
    int S = (int)(T < wcap ? T : wcap);
    sm.tiles = (unsigned)T;
    pk.pack_blocks = (unsigned)P;
    // one staged call that one pass covers, out of place, nothing but the step itself: the stripped kernel
    if (p.src == q.a && p.nbytes == q.nbytes && !same && q.wait_flag && q.b_uncached && up == 2 && us == 2 && block == kThreads &&
        (p.nbytes + 8191) / 8192 <= (size_t)pcap && !p.pre.word && !q.pre.word && !q.fp && !q.done && !p.fp) {
        T = (p.nbytes + 8191) / 8192;                        // tiles of 8 KiB, the last one possibly ragged
        P = (int)((T + 7) & ~(size_t)7);                      // the pack part a multiple of eight blocks long (pairs on one XCD)
        S = (int)(T < wcap ? T : wcap);
        if (S > 8) S &= ~7;
        const LeanGateArgs w{LeanArgs{pk.a, sm.b, pk.bounce, sm.out, pk.cflag, pk.pack_arrive, pk.seq, (unsigned)P, p.nbytes},
                              q.wait_flag, q.relay, q.spin_limit_ticks, (unsigned)T};
        if (g_stream) {
            switch (q.dtype) {
                case 0: return launch_each(k_pipe_lean<0, true>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
                case 1: return launch_each(k_pipe_lean<1, true>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
                default: return launch_each(k_pipe_lean<2, true>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
            }
        }
        switch (q.dtype) {
            case 0: return launch_each(k_pipe_lean<0, false>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
            case 1: return launch_each(k_pipe_lean<1, false>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
            default: return launch_each(k_pipe_lean<2, false>, P + S, kThreads, st, t, w.w.pack_blocks, w.w.a, w.w.b, w.w.out, w.relay, w.w.seq, w.w.bounce, w.wait_flag, w.w.cflag, w.w.pack_arrive, w.spin_limit, w.tiles, w.w.nbytes);
        }
    }
    if (g_stream) {
        switch (q.dtype) {
            case 0: return launch_pipe_u<0, true>(up, us, P + S, block, st, t, pk, sm);
            case 1: return launch_pipe_u<1, true>(up, us, P + S, block, st, t, pk, sm);
            default: return launch_pipe_u<2, true>(up, us, P + S, block, st, t, pk, sm);
        }
    }
    switch (q.dtype) {
        case 0: return launch_pipe_u<0, false>(up, us, P + S, block, st, t, pk, sm);
        case 1: return launch_pipe_u<1, false>(up, us, P + S, block, st, t, pk, sm);
        default: return launch_pipe_u<2, false>(up, us, P + S, block, st, t, pk, sm);
    }
}

int small_call_blocks(size_t nbytes)
{
    const size_t nvec = nbytes >> 4;
    return (int)((nvec + kMaxSmallThreads - 1) / kMaxSmallThreads) + (nvec == 0 ? 1 : 0);
}

hipError_t launch_small_call(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t)
{
    if (!(al16(p.src) && al16(p.dst) && al16(q.out) && al16(q.b)) || p.src != q.a || p.nbytes != q.nbytes || !p.cflag ||
        !p.arrive || q.dtype < 0 || q.dtype > 2)
        return hipErrorInvalidValue;
    if (q.done && !q.done_arrive) return hipErrorInvalidValue;
    const int grid = small_call_blocks(p.nbytes);
    if (grid > kSmallCallMaxBlocks) return hipErrorInvalidValue;
    const size_t nvec = p.nbytes >> 4;
    int block = grid > 1 ? kMaxSmallThreads : (int)((nvec + 63) / 64 * 64);
    if (block < 64) block = 64;
    StepArgs s{};
    s.bounce = (u32x4*)p.dst; s.cflag = p.cflag; s.pack_arrive = p.arrive; s.tagp = nullptr;
    s.out = (u32x4*)q.out; s.b = (const u32x4*)q.b; s.wait_flag = q.wait_flag; s.relay = q.relay; s.spin_limit = q.spin_limit_ticks;
    s.b_uncached = q.b_uncached;
    s.done = q.done; s.done_arrive = q.done_arrive;
    s.a = (const u32x4*)p.src; s.nbytes = p.nbytes; s.seq = p.seq; s.fp = p.fp; s.sigmode = p.sigmode;
    s.pre_word = p.pre.word; s.pre_seq = p.pre.seq;
    switch (q.dtype) {
        case 0: return launch1(k_small_call<0>, grid, block, st, t, s);
        case 1: return launch1(k_small_call<1>, grid, block, st, t, s);
        default: return launch1(k_small_call<2>, grid, block, st, t, s);
    }
}

hipError_t launch_waitflag(const unsigned long long* flag, unsigned long long seq, unsigned long long limit,
                           unsigned long long* fp, hipStream_t st)
{
    hipLaunchKernelGGL(k_waitflag, dim3(1), dim3(64), 0, st, flag, seq, limit, fp);
    return hipGetLastError();
}
hipError_t launch_tagchk(const unsigned long long* tag, unsigned long long seq, unsigned long long* dbg, hipStream_t st)
{
    hipLaunchKernelGGL(k_tagchk, dim3(1), dim3(1), 0, st, tag, seq, dbg);
    return hipGetLastError();
}
hipError_t launch_mark(unsigned long long* fp, int i, unsigned long long seq, hipStream_t st)
{
    hipLaunchKernelGGL(k_mark, dim3(1), dim3(1), 0, st, fp, i, seq);
    return hipGetLastError();
}
hipError_t launch_fill_u32(unsigned int* p, unsigned int v, size_t n, hipStream_t st)
{
    int grid = (int)((n + kThreads - 1) / kThreads); if (grid < 1) grid = 1; if (grid > 1024) grid = 1024;
    hipLaunchKernelGGL(k_fill_u32, dim3(grid), dim3(kThreads), 0, st, p, v, n);
    return hipGetLastError();
}

}  // namespace tbv
