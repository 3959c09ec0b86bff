// Host engine of libtbvcoll.so for MI355X: ring, progress threads, enqueue halves.
//
// What it does per call (async mode, the default): take the next sequence
// number and ring slot, launch the pack kernel on the caller's stream (copy into
// the send bounce slot + completion word), hand one work item to each rail's
// progress thread, gate the caller's stream on the slot's 64-bit flag, launch
// the sum kernel.  A rail's progress thread waits for the pack's completion word,
// runs the transfer (wire_xfer, the one seam to the transport), and the last rail
// to see its arrival raises the flag the GPU waits on.  Every host wait is bounded
// by the watchdog, and the flag is raised even on error so the GPU never waits
// forever.
//
// Engine replaced: step4/libtbvcoll.cpp:64-117 (state), :226-277 (progress_rail),
// :279-342 and :405-413 (allocation half of tbv_ar_init), :417-508 (enqueue).
#include "tbv_engine.h"

#include <sched.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>

#include "tbv_dma.h"
#include "tbv_sock.h"

namespace tbv {

Engine G;

namespace {

// Uncached slabs are never returned to the driver once a kernel has read them;
// they are kept here and handed out again on the next initialisation.
struct SlabCache { char* ptr = nullptr; size_t size = 0; };
SlabCache g_uc_send, g_uc_recv;

void timed_wait(pthread_cond_t* cv)          // caller holds G.mx; naps at most 2 ms
{
    struct timespec t2;
    clock_gettime(CLOCK_REALTIME, &t2);
    t2.tv_nsec += 2000000;
    if (t2.tv_nsec >= 1000000000) { t2.tv_sec++; t2.tv_nsec -= 1000000000; }
    pthread_cond_timedwait(cv, &G.mx, &t2);
}

// Wake sleepers on `cv`.  Skipped when nobody is (about to be) asleep: a waiter sets its
// `napping` flag before it re-checks its condition under G.mx, and the waker publishes the
// condition before it reads the flag (both sequentially consistent), so one of the two always
// sees the other; a nap is 2 ms at most in any case.
// The broadcast comes after the mutex has been released again: taking it once is what orders this wake against a
// waiter between its re-check and its wait, and the woken threads then do not run into a mutex the waker still holds.
void wake_if(std::atomic<int>& napping, pthread_cond_t* cv)
{
    std::atomic_thread_fence(std::memory_order_seq_cst);
    if (!napping.load(std::memory_order_seq_cst)) return;
    pthread_mutex_lock(&G.mx);
    pthread_mutex_unlock(&G.mx);
    pthread_cond_broadcast(cv);
}

inline bool queue_empty(const Rail& x)
{
    return x.q_head.load(std::memory_order_seq_cst) == x.q_tail.load(std::memory_order_relaxed);
}

// Called by whichever thread completes the last rail of a call: raise the flag
// the GPU waits on.  With the latency probe on, also time release -> sum done.
void release_gpu(const Item& it)
{
    G.rails_done[it.slot].store(0u, std::memory_order_relaxed);
    const int probe = G.probe.load(std::memory_order_relaxed);
    const double t0 = probe ? nowt() : 0.0;
    st_rel(gflag(it.slot), it.seq);
    // only now may the caller reuse the slot: an early peer's call raises this same flag to its own, higher
    // sequence number on entry, and that store must not be overtaken by the one above
    G.released[it.slot].store(it.seq, std::memory_order_release);
    if (probe && !G.err.load()) {
        const unsigned long long* dw = doneword(it.slot);
        double t1 = t0;
        while (ld_acq(dw) < it.seq) { t1 = nowt(); if (t1 - t0 > 0.25) break; }
        t1 = nowt();
        std::lock_guard<std::mutex> lk(G.logmx);
        if (G.latencies.size() < LOG_MAX) G.latencies.push_back((t1 - t0) * 1e6);
    }
}

// ---- progress thread, one per rail (replaces progress_rail, step4/libtbvcoll.cpp:226-277) ----

// The pack's completion word of one item (every rail watches the same one), bounded by the watchdog counted
// from `since`.  Returns 1 when it is up, 0 when not yet, -1 when the watchdog has run out (error flag set).
int pack_complete(const Rail& x, const Item& it, double since, int NS)
{
    if (ld_acq(cflag(it.slot)) >= it.seq) return 1;
    if (nowt() - since <= G.wdog) return 0;
    unsigned long long* fp = footprints();
    LOGF("watchdog: rail%d pack completion word not seen for %.0fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq);
    LOGF("  GPU footprints wait-in=%llu wait-out=%llu pack=%llu sum-done=%llu wait-timeout=%llu host-seq=%llu cflag=%llu gflag[prev]=%llu",
         fp[0], fp[1], fp[2], fp[3], fp[4], (unsigned long long)G.seq, *cflag(it.slot), *gflag((int)((it.seq - 1) % NS)));
    G.err.store(1);
    return -1;
}

// An item is over for this rail: its own flag (per-rail sums start on their own arrival; raised on error too),
// the GPU's flag when this was the call's last rail (error or not; the counter is put back to 0 by that rail
// itself), and the queue slot back to the caller.
void finish_item(Rail& x, const Item& it, uint64_t tail)
{
    st_rel(rflag(x.idx, it.slot), it.seq);
    if (G.rails_done[it.slot].fetch_add(1u, std::memory_order_acq_rel) + 1u >= (unsigned)it.R) release_gpu(it);
    x.q_tail.store(tail + 1, std::memory_order_seq_cst);
    wake_if(G.caller_napping, &G.cv_room);
}

// Two ways through the queue.  The default keeps several transfers in flight, as a NIC with several work
// requests posted does: every queued item whose pack is complete gets its deposit and arrival signal posted at
// once (posting does not wait), and items are finished in order as their arrival words come up; sixteen
// 4 MiB chunks then cost one posting each (5-6 us) instead of posting plus arrival (12 us) one after the other.
// One item at a time, post then wait (the reference's do_xfer_rail, step4/libtbvcoll.cpp:172-211), remains for
// the copy-engine wire, whose copies block, for event signalling, and whenever a test hook is set.
void* progress_rail(void* arg)
{
    Rail& x = *(Rail*)arg;
    (void)hipSetDevice(G.device);
    if (G.cpu >= 0) {
        cpu_set_t cs; CPU_ZERO(&cs); CPU_SET((G.cpu + x.idx) % CPU_SETSIZE, &cs);
        if (pthread_setaffinity_np(pthread_self(), sizeof cs, &cs)) LOGF("rail%d: could not pin to cpu %d", x.idx, G.cpu + x.idx);
    }
    const int NS = G.nslot;
    uint64_t posted = 0;                        // items [q_tail, posted) have their transfer in flight
    double t_watch = 0;                         // since when the item at `posted` has been waiting for its pack
    double t_post0[MAXSLOT], t_post1[MAXSLOT];  // per queue position: posting started / returned
    bool owns[MAXSLOT];
    while (G.run.load(std::memory_order_acquire)) {
        if (queue_empty(x)) {
            // Spin, then sleep.  The reference spins 30 us (step4/libtbvcoll.cpp:54,236-243); a caller that makes a call
            // every few hundred microseconds then finds the thread asleep every time and pays a wake (a system call,
            // and now and then 20-50 us when the woken thread is placed on the caller's core) on its own thread at the
            // start of each burst.  So while the recent gaps between items have been short, the thread spins through
            // gaps of up to twice their smoothed length; sparse callers get the reference's 30 us.
            const double ts = nowt();
            double spin = G.spin_us;
            if (x.gap_us > 0 && 2 * x.gap_us <= G.spin_max_us && 2 * x.gap_us > spin) spin = 2 * x.gap_us;
            while (nowt() - ts < spin * 1e-6 && queue_empty(x) && G.run.load(std::memory_order_relaxed)) { }
            if (queue_empty(x)) {
                pthread_mutex_lock(&G.mx);
                x.napping.store(1, std::memory_order_seq_cst);
                while (G.run.load(std::memory_order_relaxed) && queue_empty(x)) timed_wait(&G.cv_item);
                x.napping.store(0, std::memory_order_relaxed);
                pthread_mutex_unlock(&G.mx);
            }
            if (!G.run.load(std::memory_order_relaxed)) break;
            if (queue_empty(x)) continue;
            // (a gap counts as TBV_SPINMAX at most: one long pause of a busy caller does not send the threads to sleep
            // for its next several bursts, and a sparse caller's gaps settle at the cap, beyond the spinning range)
            const double gap = std::min((nowt() - ts) * 1e6, G.spin_max_us);
            x.gap_us = x.gap_us > 0 ? 0.75 * x.gap_us + 0.25 * gap : gap;
        }
        const uint64_t tail = x.q_tail.load(std::memory_order_relaxed);
        const uint64_t head = x.q_head.load(std::memory_order_acquire);
        if (posted < tail) { posted = tail; t_watch = 0; }

        const Item& oldest = x.q[tail % NS];
        const bool one_at_a_time = G.hooks || !G.gpusig || oldest.host_wire || G.peer_tcp || G.err.load(std::memory_order_relaxed);
        if (one_at_a_time && posted == tail) {
            const Item it = oldest;
            if (G.gpusig) {
                const double tw = nowt();
                int pc;
                while ((pc = pack_complete(x, it, tw, NS)) == 0) { }
                const double w = nowt() - tw;
                if (w > 1.0 && x.idx == 0) LOGF("pack completion word took %.1fs seq=%llu", w, (unsigned long long)it.seq);
            } else if (hipEventSynchronize(G.ev[it.slot]) != hipSuccess) {
                G.err.store(1);
            }
            if (!G.err.load() && wire_xfer(x, it) != 0) G.err.store(1);
            finish_item(x, it, tail);
            posted = tail + 1; t_watch = 0;
            continue;
        }

        // post the next one that is ready, in order; one per turn, so that an arrival is never left unseen behind
        // several postings (a posting is a kernel launch, 3 us and more)
        if (posted < head && !G.err.load(std::memory_order_relaxed)) {
            const Item& it = x.q[posted % NS];
            if (!it.host_wire && !G.hooks && !G.peer_tcp) {          // else it goes one at a time, once it is the oldest
                if (t_watch == 0) t_watch = nowt();
                if (pack_complete(x, it, t_watch, NS) == 1) {
                    const int k = (int)(posted % NS);
                    t_post0[k] = nowt();
                    if (wire_post(x, it, &owns[k]) != 0) G.err.store(1);
                    else { t_post1[k] = nowt(); posted++; t_watch = 0; }
                }
            }
        }
        // finish the oldest one when its fragment has arrived
        if (posted > tail) {
            const Item it = oldest;
            const int k = (int)(tail % NS);
            bool over = !owns[k] || wire_arrived(x, it);
            if (!over && nowt() - t_post0[k] > G.wdog) {
                LOGF("watchdog: rail%d transfer exceeded %.1fs seq=%llu", x.idx, nowt() - t_post0[k], (unsigned long long)it.seq);
                G.err.store(1);
            }
            if (over || G.err.load(std::memory_order_relaxed)) {
                if (over && owns[k]) wire_done(x, it, t_post0[k], t_post1[k]);
                finish_item(x, it, tail);
            }
        } else if (G.err.load(std::memory_order_relaxed) && posted == tail && tail < head) {
            continue;                                                // the error path above takes it from here
        }
    }
    return nullptr;
}

int count_rails(const char* devs)
{
    if (!devs) return 0;
    int n = 1;
    for (const char* p = devs; *p; p++) if (*p == ',') n++;
    return n;
}

bool alloc_slab(char** out, size_t span, bool uncached, SlabCache& cache)
{
    if (!uncached) return hipMalloc((void**)out, span) == hipSuccess;
    if (cache.ptr && cache.size >= span) { *out = cache.ptr; return true; }
    char* p = nullptr;
    if (hipExtMallocWithFlags((void**)&p, span, hipDeviceMallocUncached) != hipSuccess) return false;
    cache.ptr = p; cache.size = span;       // an older, smaller slab stays allocated on purpose
    *out = p;
    return true;
}

void free_slab(char* p, const SlabCache& cache)
{
    if (p && p != cache.ptr) (void)hipFree(p);
}

// Event pair for one kernel launch when kernel timing is on (pool grows on demand).
// The events are handed to the launch itself, so they carry that dispatch's own
// start and end timestamps.
struct KTimer {
    Timing t;
    bool on;
    explicit KTimer(int which) : on(G.ktime != 0)
    {
        if (!on) return;
        auto& pool = G.kev[which];
        if (G.kev_used[which] == pool.size()) {
            hipEvent_t a, b;
            if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) { on = false; return; }
            pool.emplace_back(a, b);
        }
        t.start = pool[G.kev_used[which]].first;
        t.stop = pool[G.kev_used[which]].second;
        G.kev_used[which]++;
    }
    const Timing* get() const { return on ? &t : nullptr; }
};

// Back-pressure as in the reference (step4/libtbvcoll.cpp:441-443): no rail this call uses may be a full ring behind.
int wait_for_room(int R)
{
    auto full = [&]() {
        for (int r = 0; r < R; r++)
            if (G.rr[r].q_head.load(std::memory_order_relaxed) - G.rr[r].q_tail.load(std::memory_order_seq_cst) >= (uint64_t)G.nslot) return true;
        return false;
    };
    if (!full()) return 0;
    const double ts = nowt();
    while (nowt() - ts < SPIN_US * 1e-6 && full() && !G.err.load()) { }
    if (full() && !G.err.load()) {
        pthread_mutex_lock(&G.mx);
        G.caller_napping.store(1, std::memory_order_seq_cst);
        while (!G.err.load() && full()) timed_wait(&G.cv_room);
        G.caller_napping.store(0, std::memory_order_relaxed);
        pthread_mutex_unlock(&G.mx);
    }
    if (G.err.load()) FAIL("transfer error while waiting for room in the ring");
    return 0;
}

// The slot's previous user (call seq - NSLOT) must have had its GPU flag raised before the slot
// takes a new call.  Queue depth alone does not say so: a rail's queue only holds the calls that
// use that rail, so a one-rail call can find room while rail 1 still owes the slot's previous,
// two-rail call its fragment; the two calls would then share the slot's rail counter, and a flag
// raised for the newer one (as soon as the call is made, when its peer payload arrived early)
// would pass the older one's gate as well.
int wait_for_slot(uint64_t seq, int slot)
{
    if (seq <= (uint64_t)G.nslot) return 0;
    const uint64_t prev = seq - (uint64_t)G.nslot;
    if (G.released[slot].load(std::memory_order_acquire) >= prev) return 0;
    const double ts = nowt();
    while (G.released[slot].load(std::memory_order_acquire) < prev) {
        if (G.err.load()) FAIL("transfer error while waiting for slot %d", slot);
        if (nowt() - ts > G.wdog + 1.0) FAIL("watchdog: slot %d still belongs to call %llu", slot, (unsigned long long)prev);
        if (nowt() - ts > SPIN_US * 1e-6) sched_yield();
    }
    return 0;
}

// The completion signal a kernel about to be launched on `st` has to deliver for its predecessor.
PreSignal take_pending(hipStream_t st)
{
    PreSignal p;
    if (G.pending.word) {
        if (G.pending_stream == st) p = G.pending;
        else (void)launch_mark(G.pending.word, 0, G.pending.seq, G.pending_stream);   // other stream: deliver it there
        G.pending = PreSignal{};
        G.pending_stream = nullptr;
    }
    return p;
}

}  // namespace

// A deferred signal must not outlive the call that made it.
int flush_pending()
{
    if (!G.pending.word) return 0;
    hipError_t e = launch_mark(G.pending.word, 0, G.pending.seq, G.pending_stream);
    G.pending = PreSignal{};
    G.pending_stream = nullptr;
    return e == hipSuccess ? 0 : -1;
}

// ---- configuration ---------------------------------------------------------------------

int configure(const char* devs, size_t cap)
{
    auto geti = [](const char* k, int d) { const char* e = getenv(k); return e ? atoi(e) : d; };
    auto getz = [](const char* k, size_t d) { const char* e = getenv(k); return e ? (size_t)strtoull(e, 0, 10) : d; };
    // tbv_ar_cap() reports the cap as an int (step4/libtbvcoll.cpp:537): larger caps cannot be told to the caller
    if (cap > (size_t)0x7ffff000) FAIL("cap %zu B is above what tbv_ar_cap can report (2 GiB - 4 KiB)", cap);
    G.cap = (cap + 4095) & ~(size_t)4095;
    G.async = geti("TBV_ASYNC", 1);
    G.gpusig = geti("TBV_GPUSIG", 1);
    G.kwait = geti("TBV_KWAIT", 0);
    { int v = geti("TBV_NSLOT", 8); if (v < 2) v = 2; if (v > MAXSLOT) v = MAXSLOT; G.nslot = v; }
    G.chunkb = getz("TBV_CHUNK", 0);
    G.rail1max = getz("TBV_RAIL1MAX", 96u * 1024u);
    G.cpu = geti("TBV_CPU", -1);
    { const char* e = getenv("TBV_WDOG"); G.wdog = (e && atof(e) > 0) ? atof(e) : 10.0; }
    { const char* e = getenv("TBV_SPIN"); G.spin_us = (e && atof(e) >= 0) ? atof(e) : SPIN_US; }
    { const char* e = getenv("TBV_SPINMAX"); G.spin_max_us = (e && atof(e) >= 0) ? atof(e) : 1000.0; }
    G.tag = (geti("TBV_TAG", 0) && G.async && G.gpusig) ? 1 : 0;
    // bit 0: send ring uncached (the reference's default, step4/libtbvcoll.cpp:314); bit 1: receive ring uncached, the
    // kind of memory a peer's writes land in (costs the sum nothing: 12.9 us per 16 MiB step either way)
    G.uncached = geti("TBV_UNCACHED", 3);
    G.railsum = geti("TBV_RAILSUM", 0);
    G.fuse = geti("TBV_FUSE", 0);
    // uncached bounce: waves only drain their stores; cached bounce: block leader writes the L2 back
    G.packsig = geti("TBV_PACKSIG", (G.uncached & 1) ? 0 : 1);
    // decode-size messages (up to 1 MiB: batch 128 x hidden 4096 x 2 B is 1 MiB) poll their flag inside the kernel
    G.fusewait_max = getz("TBV_FUSEWAIT", (size_t)1 << 20);
    G.defer = geti("TBV_DEFERSIG", 1);
    G.onekernel = geti("TBV_ONEKERNEL", 1);
    { const char* e = getenv("TBV_WIRE");
      G.wire_mode = (e && !strcmp(e, "stream")) ? 1 : (e && !strcmp(e, "host")) ? 2 : 0; }
    G.stride = G.cap + (G.tag ? 4096 : 0);
    { size_t per_item = G.chunkb ? ((G.cap + G.chunkb - 1) / G.chunkb + 1) : 1;
      G.wr_hwm = (int)std::min<size_t>(96, (size_t)(G.nslot - 1) * per_item); if (G.wr_hwm < 1) G.wr_hwm = 1; }
    G.R = count_rails(devs);
    if (G.R < 1 || G.R > MAXRAIL) FAIL("rail count %d out of range 1..%d", G.R, MAXRAIL);
    G.merge = geti("TBV_MERGE", 1);
    G.merge_max = getz("TBV_MERGEMAX", (size_t)256 << 20);
    if (G.merge_max < ((size_t)1 << 20)) G.merge_max = (size_t)1 << 20;      // segments of a merged launch: whole MiB at least
    set_merge_segment(G.merge_max);
    // a call whose peer payload has not arrived yet, above the one-kernel size: pack blocks + gated sum blocks in one launch
    G.staged_merge = geti("TBV_STAGEDMERGE", 1);
    G.force_gate = geti("TBV_FORCEGATE", 0);
    { const char* e = getenv("TBV_PEER"); G.peer_tcp = (e && !strcmp(e, "tcp")) ? 1 : 0; }
    set_gated_tuning(geti("TBV_GATEDGRID", 0), geti("TBV_GATEDUNROLL", 0));
    set_row_grid_cap(geti("TBV_ROWGRID", 0));
    set_codec_grid_cap(geti("TBV_CODECGRID", 0));
    G.codec = geti("TBV_CODEC", 0);
    G.codec_min = getz("TBV_CODEC_MIN", (size_t)512 << 10);
    // Cache-hint profile: when both rings plus one local and one output tensor fit in three quarters of the
    // 256 MB Infinity Cache they stay resident from call to call; beyond that every operand streams from HBM.
    { const size_t working_set = 2 * (size_t)G.nslot * G.stride + 2 * G.cap;
      G.streaming = geti("TBV_STREAMING", working_set > ((size_t)192 << 20) ? 1 : 0); }
    set_tuning(geti("TBV_UNROLL", 0), geti("TBV_GRIDCAP", 0), geti("TBV_BLOCK", 0), G.streaming);
    G.configured = 1;
    return 0;
}

// ---- enqueue halves --------------------------------------------------------------------

// First half of a call: sequence number, slot, pack kernel, work items.
// `sum_out`/`dtype` are only used when the sum can share the pack's launch.
int enqueue_pack(const void* ptr, void* sum_out, size_t nbytes, int dtype, hipStream_t st, Call* c, const NormArgs* nm, PackArgs* hold)
{
    const size_t tagoff = tag_offset(nbytes);
    c->nbytes = nbytes;
    c->xbytes = G.tag ? tagoff + 8 : nbytes;
    c->R = rails_for(nbytes);
    c->seq = ++G.seq;
    c->slot = (int)(c->seq % (uint64_t)G.nslot);
    c->fused = false;
    c->deferred = false;
    c->host_wire = G.async && use_host_wire(st);
    // The int8 codec applies from a size threshold upwards (below it the wire is a small part of a call), to
    // whole 16-byte vectors, and not together with the modes that cut or extend the payload on the wire.
    c->codec = G.codec && G.async && G.gpusig && nbytes >= G.codec_min && !(nbytes & 15) && !G.tag && G.kwait != 1 &&
               !(G.railsum && c->R > 1) && !nm && !(((uintptr_t)ptr | (uintptr_t)sum_out) & 15) && !c->out_unaligned &&
               codec_image_bytes(nbytes, dtype) <= G.stride;
    if (c->codec) c->xbytes = codec_image_bytes(nbytes, dtype);

    const char* peer = nullptr;
    if (peer_assign(c, nbytes, dtype, &peer) != 0) return -1;

    PackArgs pa{};
    pa.dst = slot_send(c->slot); pa.src = ptr; pa.nbytes = nbytes;
    pa.cflag = cflag(c->slot); pa.seq = c->seq; pa.arrive = pack_counters(c->slot);
    pa.tagp = G.tag ? (unsigned long long*)(slot_send(c->slot) + tagoff) : nullptr;
    pa.fp = G.kwait ? footprints() : nullptr;
    pa.sigmode = G.packsig;

    if (G.async) {
        if (wait_for_room(c->R) != 0) return -1;
        if (wait_for_slot(c->seq, c->slot) != 0) return -1;
        if (c->resident) st_rel(gflag(c->slot), c->seq);      // the peer was early: its flag is already up
        if (G.gpusig) {
            const bool aligned = !(((uintptr_t)ptr | (uintptr_t)sum_out) & 15);
            const bool plain = sum_out && !G.tag && G.kwait != 1 && !(G.railsum && c->R > 1) && aligned && !c->codec;
            // in place (the output IS the local tensor), or an output that overlaps it in some other way
            const bool inplace = sum_out == ptr;
            const bool overlap = sum_out && (uintptr_t)sum_out < (uintptr_t)ptr + nbytes && (uintptr_t)ptr < (uintptr_t)sum_out + nbytes;
            // measurement aid (TBV_FORCEGATE=1): an early peer's large calls take the gated one-launch form too, so that
            // form can be timed with its flag already up when the kernel starts
            const bool gate_resident = G.force_gate && c->resident && nbytes > G.fusewait_max;
            const bool in_place_already = c->resident;      // the slot's flag is raised by this rank's own progress thread, never before the call
            const bool fuse_wanted = G.fuse && in_place_already && plain && !nm && !gate_resident;
            // One launch for a small call: pack, completion word, flag poll and sum in a single kernel whose
            // few blocks are all resident (a decode-size reduction pays one flag wait and one kernel).
            const bool one_kernel = G.onekernel && !fuse_wanted && plain && G.can_wait_value && nbytes <= G.fusewait_max &&
                                    (nm ? nm->rows <= (unsigned)kRowNormMaxSmallRows : small_call_blocks(nbytes) <= kSmallCallMaxBlocks);
            // Payload already in place and too large for the one-kernel call: pack blocks and sum blocks in one
            // launch (a launch costs about 2.4 us of stream time whatever it does).
            // (payloads beyond TBV_MERGEMAX as several such launches, one per segment: the two halves share the local
            // tensor through the L2 only while they stay close in time)
            const bool mergeable = G.merge && !fuse_wanted && !one_kernel && in_place_already && !gate_resident && plain && G.packsig == 0 && !nm;
            // Pack blocks and sum blocks read the local tensor independently, so a sum block may store out[i] before
            // the pack block has read a[i]: an output that overlaps the local tensor cannot take the merged launch.
            // In place it takes the fused body instead (one lane loads a[i] once and does both stores); any other
            // overlap gets two launches.
            const bool can_merge = mergeable && !overlap;
            const bool can_fuse = fuse_wanted || (mergeable && inplace);
            // The peer's payload is not there yet and the call is too large for the one-kernel form: still one launch,
            // pack blocks first, then sum blocks that wait for the flag inside the kernel (instead of pack launch, stream
            // gate, sum launch).  In place, the sum blocks also wait for the last pack block.
            const bool staged_one = G.staged_merge && G.merge && (!in_place_already || gate_resident) && !one_kernel && plain && G.can_wait_value && G.packsig == 0 &&
                                    !nm && !hold && nbytes <= G.merge_max && (!overlap || inplace);
            // With the int8 codec and the peer's image already in place: quantise, decode both images and sum in one
            // kernel that reads the local tensor once and never reads its own image back.
            const bool coded_one = c->codec && G.merge && in_place_already && !gate_resident && sum_out && G.packsig == 0 && !hold &&
                                   (!overlap || inplace);
            // Deferred signal: counting the pack's blocks costs about 1.5 us at the end of the kernel.
            // When the next kernel on the stream is one of ours and will not wait behind a stream gate
            // (payload already there, or the flag is polled inside the sum kernel), the pack leaves its
            // completion word alone and that next kernel raises it first thing.
            const bool will_poll_in_kernel = nbytes <= G.fusewait_max;
            c->deferred = G.defer && !can_fuse && !can_merge && !one_kernel && !staged_one && !coded_one && !G.tag && G.kwait != 1 && G.can_wait_value &&
                          !(G.railsum && c->R > 1) && (c->resident || will_poll_in_kernel);
            pa.pre = take_pending(st);
            // test hook: this call's pack never raises its completion word
            const bool mute_pack = G.hooks && G.withhold_seq.load() == c->seq && G.withhold_rail.load() < 0;
            if (mute_pack) {
                pa.cflag = nullptr;
                c->deferred = false;
                if (launch_pack(pa, st) != hipSuccess) FAIL("pack kernel launch failed");
            } else if (one_kernel || can_fuse || can_merge || staged_one || coded_one) {
                SumArgs sa{};
                sa.out = sum_out; sa.a = ptr; sa.b = slot_recv(c->slot); sa.b_uncached = (G.uncached & 2) != 0; sa.nbytes = nbytes; sa.dtype = dtype; sa.seq = c->seq;
                sa.fp = pa.fp;
                if ((one_kernel && !c->resident) || staged_one) {
                    sa.wait_flag = gflag(c->slot); sa.relay = relay_word(c->slot);
                    sa.spin_limit_ticks = (unsigned long long)((G.wdog * 2.0 + 1.0) * G.tick_hz);
                }
                if (G.probe.load(std::memory_order_relaxed)) { sa.done = doneword(c->slot); sa.done_arrive = done_counters(c->slot); }
                KTimer kt(1);
                const double tq = nowt();
                const hipError_t e = coded_one ? launch_coded_step(pa, sa, st, kt.get())
                                   : one_kernel ? (nm ? launch_row_norm(2, &pa, sa, *nm, st, kt.get()) : launch_small_call(pa, sa, st, kt.get()))
                                   : staged_one ? launch_pipe(pa, sa, st, kt.get(), relay_word(c->slot) + 1)
                                   : can_fuse ? launch_pack_sum(pa, sa, st, kt.get()) : launch_pack_sum_merged(pa, sa, st, kt.get());
                if (e != hipSuccess)
                    FAIL("%s launch failed: %s (%zu B)", coded_one ? "coded step" : one_kernel ? "one-kernel call" : staged_one ? "pack + gated sum kernel" : "pack+sum kernel",
                         hipGetErrorName(e), nbytes);
                G.t_post += nowt() - tq;                       // the launch that carries the sum
                c->fused = true;
            } else if (hold && !c->codec && G.packsig == 0 && !G.tag && G.kwait != 1 && !(((uintptr_t)ptr) & 15)) {
                // the chunked pipeline launches this pack together with an earlier chunk's sum: hand the arguments back
                c->deferred = false;
                c->held = true;
                *hold = pa;
            } else {
                if (c->deferred) pa.cflag = nullptr;
                KTimer kt(0);
                if ((c->codec ? launch_quant(pa, dtype, st, kt.get()) : launch_pack(pa, st, kt.get())) != hipSuccess) FAIL("pack kernel launch failed");
                if (c->deferred) { G.pending.word = cflag(c->slot); G.pending.seq = c->seq; G.pending_stream = st; }
            }
        } else {
            if (hipMemcpyAsync(slot_send(c->slot), ptr, nbytes, hipMemcpyDeviceToDevice, st) != hipSuccess) FAIL("copy into send slot failed");
            if (hipEventRecord(G.ev[c->slot], st) != hipSuccess) FAIL("event record failed");
        }
        // rails_done[slot] is never cleared here: the last rail of the previous user of the slot does it
        for (int r = 0; r < c->R; r++) {
            Rail& x = G.rr[r];
            uint64_t h = x.q_head.load(std::memory_order_relaxed);
            x.q[h % G.nslot] = Item{c->seq, c->slot, nbytes, c->R, c->xbytes, peer, c->resident, c->host_wire};
            x.q_head.store(h + 1, std::memory_order_seq_cst);
        }
        // the rails sleep on one condition variable: one broadcast wakes all of them (a wake is a system call, and the
        // first call after an idle spell pays it on the caller's thread)
        for (int r = 0; r < c->R; r++)
            if (G.rr[r].napping.load(std::memory_order_seq_cst)) { wake_if(G.rr[r].napping, &G.cv_item); break; }
    } else {
        // synchronous mode: the caller thread does everything (step4/libtbvcoll.cpp:482-493)
        if (hipMemcpyAsync(slot_send(c->slot), ptr, nbytes, hipMemcpyDeviceToDevice, st) != hipSuccess) FAIL("copy into send slot failed");
        const double tp = nowt();
        for (;;) {
            hipError_t e = hipStreamQuery(st);
            if (e == hipSuccess) break;
            if (e != hipErrorNotReady) FAIL("stream query failed");
            if (nowt() - tp > G.wdog) FAIL("watchdog: stream did not drain");
        }
        G.t_pre += nowt() - tp;
        Item it{c->seq, c->slot, nbytes, c->R, c->xbytes, peer, c->resident, false};
        for (int r = 0; r < c->R; r++) if (wire_xfer(G.rr[r], it) != 0) { G.err.store(1); FAIL("transfer failed"); }
        const double tdr = nowt();          // nothing to reap: the emulated sends complete with their arrival
        G.t_drain += nowt() - tdr;
    }
    return 0;
}

// Second half: gate the stream on the flag(s), then the sum.
// `with_pack`: a later chunk's pack that enqueue_pack handed back, to be launched with this sum (or before it,
// where the two cannot share a launch).
int enqueue_wait_sum(const void* ptr, void* outp, int dtype, hipStream_t st, const Call& c, const NormArgs* nm, const PackArgs* with_pack)
{
    if (c.fused) return 0;
    const bool railsum_path = G.async && G.railsum && c.R > 1 && !G.tag;
    const bool pipe = with_pack && !railsum_path && !c.codec && !nm && !G.tag && G.kwait != 1 && G.async && G.can_wait_value &&
                      !(((uintptr_t)ptr | (uintptr_t)outp) & 15);
    if (with_pack && !pipe) {
        PackArgs pa = *with_pack;
        if (!pa.pre.word) pa.pre = take_pending(st);
        KTimer kt(0);
        if (launch_pack(pa, st, kt.get()) != hipSuccess) FAIL("pack kernel launch failed");
    }
    const char* rb = slot_recv(c.slot);
    const unsigned long long spin_ticks = (unsigned long long)((G.wdog * 2.0 + 1.0) * G.tick_hz);
    const bool probe = G.probe.load(std::memory_order_relaxed) != 0;
    const size_t esz = dtype == 0 ? 4 : 2;

    auto sum_piece = [&](size_t off, size_t len, const unsigned long long* gate, bool last) -> int {
        SumArgs sa{};
        sa.out = (char*)outp + off; sa.a = (const char*)ptr + off; sa.b = rb + off; sa.b_uncached = (G.uncached & 2) != 0;
        sa.nbytes = len; sa.dtype = dtype; sa.seq = c.seq;
        sa.wait_flag = gate; sa.relay = gate ? relay_word(c.slot) : nullptr; sa.spin_limit_ticks = spin_ticks;
        sa.fp = G.kwait ? footprints() : nullptr;
        if (probe && last) { sa.done = doneword(c.slot); sa.done_arrive = done_counters(c.slot); }
        sa.pre = take_pending(st);
        KTimer kt(1);
        // with a norm to follow and the whole payload in this piece, the sum kernel is the row kernel that also normalises
        const bool with_norm = nm && off == 0 && len == c.nbytes;
        if (c.codec) sa.a = slot_send(c.slot);               // this rank's own payload as the peer sees it: its image
        if (pipe) {
            PackArgs pa = *with_pack;
            if (!pa.pre.word) pa.pre = sa.pre;               // at most one signal is pending at a time: the held pack may hold it already
            sa.pre = PreSignal{};
            if (gate) { sa.wait_flag = gate; sa.relay = relay_word(c.slot); }
            const hipError_t pe = launch_pipe(pa, sa, st, kt.get());
            if (pe != hipSuccess)
                FAIL("pipeline kernel launch failed: %s (pack %p -> %p %zu B seq %llu; sum %p + %p -> %p %zu B seq %llu%s)", hipGetErrorName(pe),
                     pa.src, pa.dst, pa.nbytes, pa.seq, sa.a, sa.b, sa.out, sa.nbytes, sa.seq, gate ? ", gated" : "");
            return 0;
        }
        if ((c.codec ? launch_sum_quant(sa, st, kt.get())
             : with_norm ? launch_row_norm(1, nullptr, sa, *nm, st, kt.get()) : launch_sum(sa, st, kt.get())) != hipSuccess)
            FAIL("sum kernel launch failed");
        return 0;
    };
    auto gate_stream = [&](unsigned long long* flag) -> int {
        if (flush_pending() != 0) FAIL("deferred signal launch failed");     // never park a pending signal behind a gate
        if (G.kwait == 1 || !G.can_wait_value) {
            if (launch_waitflag(flag, c.seq, spin_ticks, G.kwait ? footprints() : nullptr, st) != hipSuccess) FAIL("wait kernel launch failed");
        } else if (hipStreamWaitValue64(st, flag, c.seq, hipStreamWaitValueGte, 0xffffffffffffffffull) != hipSuccess)
            FAIL("hipStreamWaitValue64 failed");
        return 0;
    };

    double tq;
    if (G.async && G.railsum && c.R > 1 && !G.tag) {
        // each rail's half is summed as soon as that rail's own flag is up
        tq = nowt();
        int pieces = 0, total = 0;
        size_t off, len;
        for (int r = 0; r < c.R; r++) if (rail_fragment(c.xbytes, c.R, r, &off, &len)) total++;
        for (int r = 0; r < c.R; r++) {
            if (!rail_fragment(c.xbytes, c.R, r, &off, &len)) continue;
            if (gate_stream(rflag(r, c.slot)) != 0) return -1;
            pieces++;
            size_t l = (len / esz) * esz;
            if (off + len >= c.nbytes) l = ((c.nbytes - off) / esz) * esz;
            if (sum_piece(off, l, nullptr, pieces == total) != 0) return -1;
        }
        if (nm) {                            // per-rail sums cannot normalise whole rows: normalise the finished output
            SumArgs sa{};
            sa.a = outp; sa.nbytes = c.nbytes; sa.dtype = dtype; sa.seq = c.seq;
            if (launch_row_norm(0, nullptr, sa, *nm, st) != hipSuccess) FAIL("norm kernel launch failed");
        }
    } else {
        // The flag may already be up when the call is made (the peer was early): the payload is then in
        // place before the sum is even launched and the stream needs no gate at all.
        const bool arrived = G.async && !G.tag && G.kwait != 1 && ld_acq(gflag(c.slot)) >= c.seq;
        const bool fusewait = G.async && !arrived && (pipe || c.held || c.deferred || c.nbytes <= G.fusewait_max) && !G.tag && G.kwait != 1;
        if (G.async && !arrived && !fusewait && gate_stream(gflag(c.slot)) != 0) return -1;
        if (G.async && G.tag) {
            if (launch_tagchk((const unsigned long long*)(rb + tag_offset(c.nbytes)), c.seq, dbgwords(), st) != hipSuccess)
                FAIL("tag check launch failed");
        }
        tq = nowt();
        if (sum_piece(0, c.nbytes, fusewait ? gflag(c.slot) : nullptr, true) != 0) return -1;
    }
    if (G.kwait && launch_mark(footprints(), FP_SUM_DONE, c.seq, st) != hipSuccess) FAIL("footprint launch failed");
    G.t_post += nowt() - tq;
    return 0;
}

// Bookkeeping of the caller's streams.  On a switch the new stream is made to wait for what the library
// queued on the old one: call N+NSLOT reuses call N's receive slot, and stream order is all that keeps
// its deposit behind call N's sum.
void note_stream(void* stream, size_t nbytes)
{
    if (stream == G.last_stream) return;
    if (G.seq > 0) {
        G.n_stream_sw++;
        if (!G.switch_ev && hipEventCreateWithFlags(&G.switch_ev, hipEventDisableTiming) != hipSuccess) G.switch_ev = nullptr;
        if (G.switch_ev && hipEventRecord(G.switch_ev, (hipStream_t)G.last_stream) == hipSuccess)
            (void)hipStreamWaitEvent((hipStream_t)stream, G.switch_ev, 0);
        (void)hipGetLastError();             // the old stream may be gone: then there is nothing left to wait for
    }
    G.last_stream = stream;
    bool seen = false;
    for (int i = 0; i < G.nseen; i++) if (G.seen_streams[i] == stream) { seen = true; break; }
    if (!seen && G.nseen < 16) {
        G.seen_streams[G.nseen++] = stream;
        LOGF("new stream #%d %p seq=%llu nbytes=%zu", G.nseen, stream, (unsigned long long)(G.seq + 1), nbytes);
    } else if (G.n_stream_sw <= 20) {
        LOGF("stream switch %p seq=%llu", stream, (unsigned long long)(G.seq + 1));
    }
}

bool rails_idle()
{
    for (int r = 0; r < G.R; r++)
        if (G.rr[r].q_head.load(std::memory_order_acquire) != G.rr[r].q_tail.load(std::memory_order_acquire)) return false;
    return true;
}

int drain_rails()
{
    const double t0 = nowt();
    while (G.async && G.run.load() && !rails_idle()) {
        if (nowt() - t0 > G.wdog + 1.0) return -1;
        sched_yield();
    }
    return 0;
}

// ---- initialisation and teardown (allocation half of tbv_ar_init, step4/libtbvcoll.cpp:279-342,405-413) ----

int init_impl(int rank, const char* devs, const char* peer_ip, int port, size_t cap)
{
    if (configure(devs, cap) != 0) return -1;
    if (G.peer_tcp && rank != 0 && rank != 1) FAIL("two-process mode has ranks 0 and 1, not %d", rank);
    G.rank = rank;
    if (hipGetDevice(&G.device) != hipSuccess) FAIL("no HIP device");
    { int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeCanUseStreamWaitValue, G.device) != hipSuccess) v = 0;
      G.can_wait_value = v;
      int khz = 0;
      if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, G.device) == hipSuccess && khz > 0) G.tick_hz = khz * 1e3;
      (void)hipGetLastError(); }

    if (!noalloc_bind_device()) FAIL("built-in counter array not addressable on device %d", G.device);
    const size_t span = G.stride * (size_t)G.nslot;
    if (!alloc_slab(&G.sendbase, span, (G.uncached & 1) != 0, g_uc_send)) FAIL("send bounce allocation failed (%zu B)", span);
    if (!alloc_slab(&G.recvbase, span, (G.uncached & 2) != 0, g_uc_recv)) FAIL("receive bounce allocation failed (%zu B)", span);
    const size_t wbytes = (size_t)W_BLOCKS * MAXSLOT * FLAG_STRIDE;
    if (hipHostMalloc((void**)&G.hostwords, wbytes, hipHostMallocCoherent) != hipSuccess) FAIL("host flag block allocation failed");
    memset(G.hostwords, 0, wbytes);
    // [2 x MAXSLOT counter blocks][one block's worth of relay words][MAXRAIL x MAXSLOT counter blocks]
    const size_t cbytes = sizeof(unsigned int) * ((size_t)2 * MAXSLOT + 1 + (size_t)MAXRAIL * MAXSLOT) * kCounterWords;
    if (hipMalloc((void**)&G.counters, cbytes) != hipSuccess) FAIL("counter allocation failed");
    if (hipMemset(G.counters, 0, cbytes) != hipSuccess) FAIL("counter clear failed");
    for (int i = 0; i < G.nslot; i++) {
        if (hipEventCreateWithFlags(&G.ev[i], hipEventReleaseToSystem | hipEventDisableTiming) != hipSuccess) {
            (void)hipGetLastError();
            if (hipEventCreateWithFlags(&G.ev[i], hipEventDisableTiming) != hipSuccess) FAIL("event creation failed");
        }
    }
    for (int r = 0; r < G.R; r++) {
        Rail& x = G.rr[r];
        x.idx = r; x.q_head.store(0); x.q_tail.store(0); x.script_pos = 0; x.napping.store(0); x.gap_us = 0;
        x.rl_post = x.rl_arr = 0; x.rl_n = 0;
        if (hipStreamCreateWithFlags(&x.wire, hipStreamNonBlocking) != hipSuccess) FAIL("side stream creation failed");
    }
    if (G.codec && hipStreamCreateWithFlags(&G.util, hipStreamNonBlocking) != hipSuccess) FAIL("utility stream creation failed");
    for (int i = 0; i < MAXSLOT; i++) { G.rails_done[i].store(0); G.released[i].store(0); G.resident_ok[i] = false; }
    G.caller_napping.store(0);
    for (int r = 0; r < MAXRAIL; r++) G.hold[r].store(0);
    const bool dma = dma_init(G.recvbase, MAXRAIL);
    // does a stream-ordered 64-bit write reach the host block? otherwise signal with a one-thread kernel
    G.can_write_value = 1;
    if (hipStreamWriteValue64(G.rr[0].wire, scratchword(), 0x5eedull, 0) != hipSuccess ||
        hipStreamSynchronize(G.rr[0].wire) != hipSuccess || *scratchword() != 0x5eedull) {
        (void)hipGetLastError();
        G.can_write_value = 0;
    }
    G.seq = 0; G.err.store(0);
    // two processes on this GPU: meet the peer before any thread of this rank starts (as the reference brings its
    // queue pairs up before it spawns its progress threads, step4/libtbvcoll.cpp:371-407)
    if (G.peer_tcp && sock_start(rank, peer_ip, port) != 0) return -1;
    if (G.async) {
        G.run.store(1);
        for (int r = 0; r < G.R; r++) {
            if (pthread_create(&G.rr[r].th, nullptr, progress_rail, &G.rr[r])) FAIL("pthread_create failed");
            G.rr[r].started = true;
        }
    }
    G.inited = 1;
    LOGF("rank%d ready: %d rail(s), cap=%zu KiB, %d slots, mode %s", rank, G.R, G.cap / 1024, G.nslot,
         G.async ? (G.gpusig ? (G.kwait ? "ASYNC+GPUSIG+KWAIT" : "ASYNC+GPUSIG") : "ASYNC+EVENT") : "SYNC");
    LOGF("  %s on device %d; stream wait value %s, stream write value %s; uncached=%d tag=%d railsum=%d fuse=%d fusewait<=%zu",
         G.peer_tcp ? "peer = a second process" : "emulated peer", G.device, G.can_wait_value ? "yes" : "no (wait kernel)", G.can_write_value ? "yes" : "no (mark kernel)",
         G.uncached, G.tag, G.railsum, G.fuse, G.fusewait_max);
    LOGF("  wire %s; copy-engine access for the host wire: %s", G.wire_mode == 1 ? "stream" : G.wire_mode == 2 ? "host" : "auto", dma ? "yes" : "no");
    LOGF("  small calls (<= %zu B) in one kernel: %s", G.fusewait_max, G.onekernel ? "yes" : "no");
    LOGF("  deferred pack signal %s", G.defer ? "on (early peer, or flag polled inside the sum kernel)" : "off");
    if (G.codec) LOGF("  int8 payload codec for payloads of at least %zu B (group 128, asymmetric, 0.53 of a 2-byte payload on the wire)", G.codec_min);
    LOGF("  cache hints: %s profile; early peer above the one-kernel size: %s", G.streaming ? "streaming" : "resident",
         G.fuse ? "pack+sum fused (4N)" : G.merge ? "pack and sum blocks in one launch" : "two launches");
    return 0;
}

void stop_progress()
{
    if (G.async && G.run.load()) {
        G.run.store(0);
        pthread_mutex_lock(&G.mx);
        pthread_cond_broadcast(&G.cv_item);
        pthread_mutex_unlock(&G.mx);
        for (int r = 0; r < G.R; r++)
            if (G.rr[r].started) { pthread_join(G.rr[r].th, nullptr); G.rr[r].started = false; }
    }
}

// Releases whatever exists, whether or not initialisation completed.
void teardown()
{
    // let the GPU finish what is queued (flags are raised even after an error), then stop the threads
    (void)hipDeviceSynchronize();
    stop_progress();
    sock_stop();
    for (int r = 0; r < MAXRAIL; r++) if (G.rr[r].wire) { (void)hipStreamDestroy(G.rr[r].wire); G.rr[r].wire = nullptr; }
    peer_teardown();
    if (G.util) { (void)hipStreamDestroy(G.util); G.util = nullptr; }
    for (int i = 0; i < MAXSLOT; i++) if (G.ev[i]) { (void)hipEventDestroy(G.ev[i]); G.ev[i] = nullptr; }
    if (G.switch_ev) { (void)hipEventDestroy(G.switch_ev); G.switch_ev = nullptr; }
    free_slab(G.sendbase, g_uc_send); G.sendbase = nullptr;
    free_slab(G.recvbase, g_uc_recv); G.recvbase = nullptr;
    if (G.hostwords) { (void)hipHostFree(G.hostwords); G.hostwords = nullptr; }
    if (G.counters) { (void)hipFree(G.counters); G.counters = nullptr; }
    for (int w = 0; w < 2; w++) {
        for (auto& p : G.kev[w]) { (void)hipEventDestroy(p.first); (void)hipEventDestroy(p.second); }
        G.kev[w].clear(); G.kev_used[w] = 0;
    }
    G.ktime = 0;
    G.pending = PreSignal{}; G.pending_stream = nullptr;
    G.probe.store(0);
    G.t_pre = G.t_post = G.t_enq = G.t_drain = 0;
    { std::lock_guard<std::mutex> lk(G.smx);
      G.t_acc = 0; G.n_acc = 0;
      for (int b = 0; b < 32; b++) { G.hb_t[b] = 0; G.hb_n[b] = 0; G.hb_r[b] = 0; } }
    G.last_stream = nullptr; G.n_stream_sw = 0; G.nseen = 0;
    G.seq = 0; G.err.store(0);
    G.inited = 0; G.configured = 0;
}

}  // namespace tbv
