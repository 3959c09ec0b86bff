// Host engine and C ABI of libtbvcoll.so for MI355X.
//
// What it does per call (async mode, the default): take the next sequence
// number and ring slot, launch the pack kernel on the caller's stream (copy into
// the send bounce slot + completion word), hand one work item to each rail's
// progress thread, gate the caller's stream on the slot's 64-bit flag, launch
// the sum kernel.  A rail's progress thread waits for the pack's completion word,
// plays the peer (side-stream copy of the peer fragment into the receive slot,
// then a 64-bit arrival word on that stream), and the last rail to see its
// arrival raises the flag the GPU waits on.  Every host wait is bounded by the
// watchdog, and the flag is raised even on error so the GPU never waits forever.
//
// Interface replaced: step4/libtbvcoll.cpp:279-566 (the extern "C" block) and the
// engine behind it, :64-117, :168-277.  The wire (ibverbs queue pairs, dmabuf
// registration, TCP rendezvous, :172-224, :343-403) is replaced by the emulated
// peer; see include/tbvcoll.h part 2.
#include <hip/hip_runtime.h>

#include <errno.h>
#include <pthread.h>
#include <sched.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <algorithm>
#include <atomic>
#include <deque>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/tbvcoll.h"
#include "tbv_dma.h"
#include "tbv_kernels.h"

namespace {

constexpr int MAXRAIL = 4;
constexpr int MAXSLOT = 32;
constexpr double SPIN_US = 30.0;          // short spin before sleeping on a condition variable
constexpr size_t FLAG_STRIDE = 64;        // one cache line per host-visible word
constexpr size_t LOG_MAX = 1u << 20;

double nowt()
{
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + (double)t.tv_nsec * 1e-9;
}

#define LOGF(...) do { fprintf(stderr, "[tbvcoll] " __VA_ARGS__); fputc('\n', stderr); } while (0)
#define FAIL(...) do { LOGF(__VA_ARGS__); return -1; } while (0)

struct Item {
    uint64_t seq;
    int slot;
    size_t nbytes;
    int R;
    size_t xbytes;            // bytes on the wire: payload, plus the tag when tagging
    const char* peer;         // staged peer payload, or null: mirror this rank's send slot
    bool resident;            // peer payload is already in the receive slot
    bool host_wire;           // deposit with copy-engine transfers only (no GPU queue involved)
};

struct Rail {
    int idx = 0;
    Item q[MAXSLOT];
    std::atomic<uint64_t> q_head{0}, q_tail{0};
    pthread_t th{};
    bool started = false;
    hipStream_t wire = nullptr;               // side stream that plays the peer's writes
    size_t script_pos = 0;                    // next position to look at in the arrival script
    // per-rail transfer statistics (guarded by Engine::smx)
    double rl_post = 0, rl_arr = 0;
    uint64_t rl_n = 0;
};

struct Staged { const char* ptr; size_t nbytes; bool owned; };

struct Engine {
    // configuration
    int configured = 0, inited = 0, rank = 0, R = 0, async = 1, nslot = 8, gpusig = 1, kwait = 0;
    int uncached = 1, tag = 0, cpu = -1, wr_hwm = 8, device = 0, railsum = 0, fuse = 0, packsig = 0;
    int merge = 1;                            // resident peer: pack and sum blocks in one launch (TBV_MERGE)
    int streaming = 0;                        // cache-hint profile of the large kernels (TBV_STREAMING, default by ring size)
    size_t cap = 0, stride = 0, rail1max = 96u * 1024u, chunkb = 0, fusewait_max = 0;
    double wdog = 10.0;
    double tick_hz = 1e8;                     // rate of the constant clock the kernels bound their waits with
    int can_wait_value = 1, can_write_value = 1;
    // memory
    char* sendbase = nullptr;
    char* recvbase = nullptr;
    char* hostwords = nullptr;                // one coherent host block holding every flag word
    unsigned int* counters = nullptr;         // device: per slot one counter block for the pack, one for the sum
    hipEvent_t ev[MAXSLOT] = {};
    // protocol state
    Rail rr[MAXRAIL];
    uint64_t seq = 0;
    std::atomic<unsigned> rails_done[MAXSLOT];
    std::atomic<int> run{0};
    std::atomic<int> err{0};
    pthread_mutex_t mx = PTHREAD_MUTEX_INITIALIZER;
    pthread_cond_t cv_item = PTHREAD_COND_INITIALIZER;    // caller -> progress: new item
    pthread_cond_t cv_room = PTHREAD_COND_INITIALIZER;    // progress -> caller: room in the ring
    void* last_stream = nullptr;
    uint64_t n_stream_sw = 0;
    void* seen_streams[16] = {};
    int nseen = 0;
    // emulated peer
    std::deque<Staged> staged;
    Staged repeat{nullptr, 0, false};
    // device copies of payloads that were staged from host memory: (buffer, last call that reads it; 0 = not yet assigned)
    std::vector<std::pair<char*, uint64_t>> owned;
    size_t resident_bytes = 0;
    std::vector<int> script;
    std::atomic<size_t> turn{0};
    std::atomic<uint64_t> withhold_seq{0};
    std::atomic<int> withhold_rail{0};
    std::mutex logmx;
    std::vector<std::pair<uint64_t, int>> arrivals;
    std::atomic<int> probe{0};
    std::vector<double> latencies;
    // a pack's completion word that its kernel did not raise: the next kernel on the same stream raises it
    tbv::PreSignal pending;
    hipStream_t pending_stream = nullptr;
    int defer = 1;                            // allow deferring (TBV_DEFERSIG)
    int onekernel = 1;                        // small calls as one launch: pack, signal, flag poll, sum (TBV_ONEKERNEL)
    int wire_mode = 0;                        // TBV_WIRE: 0 auto (probe each new caller stream), 1 stream, 2 host
    std::vector<std::pair<void*, bool>> stream_wire;   // caller stream -> use the host wire
    // optional per-kernel timing with events on the caller's stream: [0]=pack, [1]=sum
    int ktime = 0;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> kev[2];
    size_t kev_used[2] = {0, 0};
    // statistics (guarded by smx)
    std::mutex smx;
    double t_acc = 0, t_pre = 0, t_post = 0, t_enq = 0, t_drain = 0;
    uint64_t n_acc = 0;
    double hb_t[32] = {};
    uint64_t hb_n[32] = {}, hb_r[32] = {};
};

Engine G;

// Uncached slabs are never returned to the driver once a kernel has read them;
// they are kept here and handed out again on the next initialisation.
struct SlabCache { char* ptr = nullptr; size_t size = 0; };
SlabCache g_uc_send, g_uc_recv;

// ---- host-visible words: layout inside Engine::hostwords --------------------------------
enum WordBlock { W_GFLAG = 0, W_CFLAG = 1, W_DONE = 2, W_AFLAG0 = 3 /* .. +MAXRAIL */, W_RFLAG0 = 3 + MAXRAIL,
                 W_MISC = 3 + 2 * MAXRAIL, W_BLOCKS = 4 + 2 * MAXRAIL };
inline unsigned long long* word(int block, int slot)
{
    return (unsigned long long*)(G.hostwords + ((size_t)block * MAXSLOT + (size_t)slot) * FLAG_STRIDE);
}
inline unsigned long long* gflag(int s) { return word(W_GFLAG, s); }
inline unsigned long long* cflag(int s) { return word(W_CFLAG, s); }
inline unsigned long long* doneword(int s) { return word(W_DONE, s); }
inline unsigned long long* aflag(int rail, int s) { return word(W_AFLAG0 + rail, s); }
inline unsigned long long* rflag(int rail, int s) { return word(W_RFLAG0 + rail, s); }
inline unsigned long long* footprints() { return word(W_MISC, 0); }     // 8 words
inline unsigned long long* dbgwords() { return word(W_MISC, 2); }       // 8 words
inline unsigned long long* scratchword() { return word(W_MISC, 4); }

inline uint64_t ld_acq(const unsigned long long* p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
inline void st_rel(unsigned long long* p, uint64_t v) { __atomic_store_n(p, (unsigned long long)v, __ATOMIC_RELEASE); }

inline unsigned int* pack_counters(int s) { return G.counters + (size_t)s * tbv::kCounterWords; }
inline unsigned long long* relay_word(int s) { return (unsigned long long*)(G.counters + (size_t)2 * MAXSLOT * tbv::kCounterWords) + (size_t)s * 8; }
inline unsigned int* done_counters(int s) { return G.counters + (size_t)(MAXSLOT + s) * tbv::kCounterWords; }
inline char* slot_send(int s) { return G.sendbase + (size_t)s * G.stride; }
inline char* slot_recv(int s) { return G.recvbase + (size_t)s * G.stride; }
inline size_t tag_offset(size_t nbytes) { return (nbytes + 7) & ~(size_t)7; }

// Rail r of R owns [off, off+len) of an xbytes transfer.  Same split as the
// reference (step4/libtbvcoll.cpp:173-177) except that the chunk is the rounded-up
// CEILING of xbytes/R: the reference rounds the floor, which leaves the last
// xbytes % R bytes without an owner when the quotient is a multiple of 4096.
inline bool rail_fragment(size_t xbytes, int R, int idx, size_t* off, size_t* len)
{
    size_t chunk = (((xbytes + (size_t)R - 1) / (size_t)R) + 4095) & ~(size_t)4095;
    size_t roff = (size_t)idx * chunk;
    if (roff >= xbytes) return false;
    *off = roff;
    *len = std::min(chunk, xbytes - roff);
    return true;
}
inline int rails_for(size_t nbytes) { return nbytes <= G.rail1max ? 1 : G.R; }

void record_arrival(uint64_t seq, int rail)
{
    std::lock_guard<std::mutex> lk(G.logmx);
    if (G.arrivals.size() < LOG_MAX) G.arrivals.emplace_back(seq, rail);
}

void wake(pthread_cond_t* cv)
{
    pthread_mutex_lock(&G.mx);
    pthread_cond_broadcast(cv);
    pthread_mutex_unlock(&G.mx);
}

void timed_wait(pthread_cond_t* cv)          // caller holds G.mx; naps at most 2 ms
{
    struct timespec t2;
    clock_gettime(CLOCK_REALTIME, &t2);
    t2.tv_nsec += 2000000;
    if (t2.tv_nsec >= 1000000000) { t2.tv_sec++; t2.tv_nsec -= 1000000000; }
    pthread_cond_timedwait(cv, &G.mx, &t2);
}

// Raise a 64-bit word from a side stream after everything queued on it so far:
// the stand-in for the completion an RDMA write-with-immediate delivers.
hipError_t stream_bump(hipStream_t st, unsigned long long* w, uint64_t v)
{
    if (G.can_write_value) return hipStreamWriteValue64(st, w, v, 0);
    return tbv::launch_mark(w, 0, v, st);
}

// Host wire deposit of one rail fragment (see wire_xfer): device-to-device copy-engine
// transfers issued and awaited by this thread.  Two rules keep it from ever waiting on the
// stream it is meant to release.  No HIP call is made here: one can block on a runtime lock
// held by the caller thread while that thread waits for the gated stream.  And nothing is
// read from host memory: the runtime's host-to-device engine works in order, so a transfer
// would queue behind a copy the caller has issued on the gated stream (payloads staged from
// host memory are moved to the device when they are staged; the peer's tag, which equals this
// rank's, is taken from this rank's send slot where the pack kernel wrote it).
int host_deposit(Rail& x, const Item& it, size_t off, size_t len, double t0)
{
    if (!tbv::dma_ready()) { LOGF("rail%d: no copy-engine access for the host wire", x.idx); return -1; }
    size_t n = len;
    if (it.peer && off + n > it.nbytes) n = it.nbytes > off ? it.nbytes - off : 0;        // staged payload has no tag
    const char* src = it.peer ? it.peer + off : slot_send(it.slot) + off;
    auto left = [&]() { double r = G.wdog - (nowt() - t0); return r > 0.001 ? r : 0.001; };
    // TBV_CHUNK: the fragment travels as several writes, the completion only after the last
    // (step4/libtbvcoll.cpp:181-194)
    const size_t ck = G.chunkb ? G.chunkb : (n ? n : 1);
    int rc = 0;
    for (size_t o = 0; o < n && rc == 0; o += ck)
        rc = tbv::dma_copy(x.idx, slot_recv(it.slot) + off + o, tbv::DMA_DEVICE, src + o, tbv::DMA_DEVICE, std::min(ck, n - o), left());
    if (rc == 0 && it.peer && G.tag) {       // the peer's own tag travels at the end of its payload
        const size_t to = tag_offset(it.nbytes);
        if (to >= off && to < off + len)
            rc = tbv::dma_copy(x.idx, slot_recv(it.slot) + to, tbv::DMA_DEVICE, slot_send(it.slot) + to, tbv::DMA_DEVICE, 8, left());
    }
    if (rc == -2) LOGF("watchdog: rail%d host wire copy exceeded %.1fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq);
    else if (rc != 0) LOGF("rail%d host wire copy failed seq=%llu", x.idx, (unsigned long long)it.seq);
    return rc == 0 ? 0 : -1;
}

// ---- the emulated transfer of one rail (replaces do_xfer_rail, step4/libtbvcoll.cpp:172-211) ----
// Posts this rail's fragment of the peer payload into the receive slot and waits
// for its arrival word.  Returns 0, or -1 on error / watchdog.
int wire_xfer(Rail& x, const Item& it)
{
    size_t off = 0, len = 0;
    if (!rail_fragment(it.xbytes, it.R, x.idx, &off, &len)) return 0;       // this rail owns nothing
    const double t0 = nowt();
    unsigned long long* aw = aflag(x.idx, it.slot);

    // arrival script: hold this rail's deposit until its turn
    size_t my_turn = (size_t)-1;
    if (!G.script.empty()) {
        size_t p = x.script_pos;
        while (p < G.script.size() && G.script[p] != x.idx) p++;
        if (p < G.script.size()) {
            my_turn = p;
            x.script_pos = p + 1;
            while (G.turn.load(std::memory_order_acquire) != my_turn) {
                if (nowt() - t0 > G.wdog) { LOGF("watchdog: rail%d waited %.1fs for its turn %zu in the arrival script seq=%llu",
                                                 x.idx, G.wdog, my_turn, (unsigned long long)it.seq); return -1; }
                if (!G.run.load(std::memory_order_relaxed) && G.async) return -1;
                sched_yield();
            }
        }
    }

    const bool withheld = (G.withhold_seq.load() == it.seq && G.withhold_rail.load() == x.idx);
    if (!it.resident && it.host_wire) {
        // Host wire: the fragment goes straight into the receive slot with a copy-engine transfer that
        // this thread waits for, and this thread raises the arrival word itself.  Nothing is placed on
        // one of our compute queues, so this works even when the caller's gated stream and the side
        // stream are multiplexed onto the same hardware queue.
        if (host_deposit(x, it, off, len, t0) != 0) return -1;
        if (!withheld) st_rel(aw, it.seq);
    } else if (!it.resident) {
        const char* src = it.peer ? it.peer + off : slot_send(it.slot) + off;
        size_t n = len;
        if (it.peer && off + n > it.nbytes) n = it.nbytes > off ? it.nbytes - off : 0;   // staged payload has no tag
        // TBV_CHUNK: the fragment travels as several writes, the completion signal only after the last
        // (step4/libtbvcoll.cpp:181-194)
        const size_t ck = G.chunkb ? G.chunkb : (n ? n : 1);
        for (size_t o = 0; o < n; o += ck)
            if (hipMemcpyAsync(slot_recv(it.slot) + off + o, src + o, std::min(ck, n - o), hipMemcpyDefault, x.wire) != hipSuccess) {
                LOGF("rail%d peer deposit failed seq=%llu", x.idx, (unsigned long long)it.seq); return -1; }
        if (it.peer && G.tag) {              // the peer's own tag travels at the end of its payload
            size_t to = tag_offset(it.nbytes);
            if (to >= off && to < off + len &&
                stream_bump(x.wire, (unsigned long long*)(slot_recv(it.slot) + to), it.seq) != hipSuccess) return -1;
        }
        if (!withheld && stream_bump(x.wire, aw, it.seq) != hipSuccess) {
            LOGF("rail%d arrival signal failed seq=%llu", x.idx, (unsigned long long)it.seq); return -1; }
    } else if (!withheld) {
        st_rel(aw, it.seq);                  // payload already in place: arrival is immediate
    }
    const double tp = nowt();

    // wait for the arrival word, as the reference polls its completion queue
    while (ld_acq(aw) < it.seq) {
        if (nowt() - t0 > G.wdog) {
            LOGF("watchdog: rail%d transfer exceeded %.1fs seq=%llu", x.idx, nowt() - t0, (unsigned long long)it.seq);
            if (my_turn != (size_t)-1) G.turn.store(my_turn + 1, std::memory_order_release);
            return -1;
        }
    }
    const double d = nowt() - t0;
    record_arrival(it.seq, x.idx);
    if (my_turn != (size_t)-1) G.turn.store(my_turn + 1, std::memory_order_release);
    {
        std::lock_guard<std::mutex> lk(G.smx);
        x.rl_post += tp - t0; x.rl_arr += d; x.rl_n++;
        if (x.idx == 0) {
            G.t_acc += d; G.n_acc++;
            int b = 0; { size_t v = it.nbytes; while (v >>= 1) b++; } if (b > 31) b = 31;
            G.hb_t[b] += d; G.hb_n[b]++; G.hb_r[b] += (uint64_t)it.R;
        }
    }
    return 0;
}

// Called by whichever thread completes the last rail of a call: raise the flag
// the GPU waits on.  With the latency probe on, also time release -> sum done.
void release_gpu(const Item& it)
{
    G.rails_done[it.slot].store(0u, std::memory_order_relaxed);
    const int probe = G.probe.load(std::memory_order_relaxed);
    const double t0 = probe ? nowt() : 0.0;
    st_rel(gflag(it.slot), it.seq);
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
void* progress_rail(void* arg)
{
    Rail& x = *(Rail*)arg;
    (void)hipSetDevice(G.device);
    if (G.cpu >= 0) {
        cpu_set_t cs; CPU_ZERO(&cs); CPU_SET((G.cpu + x.idx) % CPU_SETSIZE, &cs);
        if (pthread_setaffinity_np(pthread_self(), sizeof cs, &cs)) LOGF("rail%d: could not pin to cpu %d", x.idx, G.cpu + x.idx);
    }
    const int NS = G.nslot;
    while (G.run.load(std::memory_order_acquire)) {
        if (x.q_head.load(std::memory_order_acquire) == x.q_tail.load(std::memory_order_relaxed)) {
            const double ts = nowt();
            while (nowt() - ts < SPIN_US * 1e-6 && x.q_head.load(std::memory_order_acquire) == x.q_tail.load(std::memory_order_relaxed)
                   && G.run.load(std::memory_order_relaxed)) { }
            if (x.q_head.load(std::memory_order_acquire) == x.q_tail.load(std::memory_order_relaxed)) {
                pthread_mutex_lock(&G.mx);
                while (G.run.load(std::memory_order_relaxed) &&
                       x.q_head.load(std::memory_order_acquire) == x.q_tail.load(std::memory_order_relaxed))
                    timed_wait(&G.cv_item);
                pthread_mutex_unlock(&G.mx);
            }
            if (!G.run.load(std::memory_order_relaxed)) break;
            if (x.q_head.load(std::memory_order_acquire) == x.q_tail.load(std::memory_order_relaxed)) continue;
        }
        const uint64_t tail = x.q_tail.load(std::memory_order_relaxed);
        const Item it = x.q[tail % NS];

        // the pack's completion word: every rail watches the same one
        if (G.gpusig) {
            const double tw = nowt();
            while (ld_acq(cflag(it.slot)) < it.seq) {
                if (nowt() - tw > G.wdog) {
                    unsigned long long* fp = footprints();
                    LOGF("watchdog: rail%d pack completion word not seen for %.0fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq);
                    LOGF("  GPU footprints wait-in=%llu wait-out=%llu pack=%llu sum-done=%llu wait-timeout=%llu host-seq=%llu cflag=%llu gflag[prev]=%llu",
                         fp[0], fp[1], fp[2], fp[3], fp[4], (unsigned long long)G.seq, *cflag(it.slot),
                         *gflag((int)((it.seq - 1) % NS)));
                    G.err.store(1);
                    break;
                }
            }
            const double w = nowt() - tw;
            if (w > 1.0 && x.idx == 0) LOGF("pack completion word took %.1fs seq=%llu", w, (unsigned long long)it.seq);
        } else if (hipEventSynchronize(G.ev[it.slot]) != hipSuccess) {
            G.err.store(1);
        }
        if (!G.err.load() && wire_xfer(x, it) != 0) G.err.store(1);
        // this rail's own flag (per-rail sums start on their own arrival); raised on error too
        st_rel(rflag(x.idx, it.slot), it.seq);
        // the last rail to finish releases the GPU, error or not, and puts the counter back to 0 itself
        if (G.rails_done[it.slot].fetch_add(1u, std::memory_order_acq_rel) + 1u >= (unsigned)it.R) release_gpu(it);
        x.q_tail.store(tail + 1, std::memory_order_release);
        wake(&G.cv_room);
    }
    return nullptr;
}

// ---- configuration ---------------------------------------------------------------------

int count_rails(const char* devs)
{
    if (!devs) return 0;
    int n = 1;
    for (const char* p = devs; *p; p++) if (*p == ',') n++;
    return n;
}

int configure(const char* devs, size_t cap)
{
    auto geti = [](const char* k, int d) { const char* e = getenv(k); return e ? atoi(e) : d; };
    auto getz = [](const char* k, size_t d) { const char* e = getenv(k); return e ? (size_t)strtoull(e, 0, 10) : d; };
    G.cap = (cap + 4095) & ~(size_t)4095;
    G.async = geti("TBV_ASYNC", 1);
    G.gpusig = geti("TBV_GPUSIG", 1);
    G.kwait = geti("TBV_KWAIT", 0);
    { int v = geti("TBV_NSLOT", 8); if (v < 2) v = 2; if (v > MAXSLOT) v = MAXSLOT; G.nslot = v; }
    G.chunkb = getz("TBV_CHUNK", 0);
    G.rail1max = getz("TBV_RAIL1MAX", 96u * 1024u);
    G.cpu = geti("TBV_CPU", -1);
    { const char* e = getenv("TBV_WDOG"); G.wdog = (e && atof(e) > 0) ? atof(e) : 10.0; }
    G.tag = (geti("TBV_TAG", 0) && G.async && G.gpusig) ? 1 : 0;
    G.uncached = geti("TBV_UNCACHED", 1);
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
    // Cache-hint profile: when both rings plus one local and one output tensor fit in three quarters of the
    // 256 MB Infinity Cache they stay resident from call to call; beyond that every operand streams from HBM.
    { const size_t working_set = 2 * (size_t)G.nslot * G.stride + 2 * G.cap;
      G.streaming = geti("TBV_STREAMING", working_set > ((size_t)192 << 20) ? 1 : 0); }
    tbv::set_tuning(geti("TBV_UNROLL", 0), geti("TBV_GRIDCAP", 0), geti("TBV_BLOCK", 0), G.streaming);
    G.configured = 1;
    return 0;
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

// ---- enqueue halves --------------------------------------------------------------------

bool use_host_wire(hipStream_t st);

// Event pair for one kernel launch when kernel timing is on (pool grows on demand).
// The events are handed to the launch itself, so they carry that dispatch's own
// start and end timestamps.
struct KTimer {
    tbv::Timing t;
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
    const tbv::Timing* get() const { return on ? &t : nullptr; }
};

struct Call {
    uint64_t seq; int slot; int R; size_t nbytes, xbytes; bool resident; bool fused; bool deferred; bool host_wire;
};

int wait_for_room(int R)
{
    auto full = [&]() {
        for (int r = 0; r < R; r++)
            if (G.rr[r].q_head.load(std::memory_order_relaxed) - G.rr[r].q_tail.load(std::memory_order_acquire) >= (uint64_t)G.nslot) return true;
        return false;
    };
    if (!full()) return 0;
    const double ts = nowt();
    while (nowt() - ts < SPIN_US * 1e-6 && full() && !G.err.load()) { }
    pthread_mutex_lock(&G.mx);
    while (!G.err.load() && full()) timed_wait(&G.cv_room);
    pthread_mutex_unlock(&G.mx);
    if (G.err.load()) FAIL("transfer error while waiting for room in the ring");
    return 0;
}

// The completion signal a kernel about to be launched on `st` has to deliver for its predecessor.
tbv::PreSignal take_pending(hipStream_t st)
{
    tbv::PreSignal p;
    if (G.pending.word) {
        if (G.pending_stream == st) p = G.pending;
        else (void)tbv::launch_mark(G.pending.word, 0, G.pending.seq, G.pending_stream);   // other stream: deliver it there
        G.pending = tbv::PreSignal{};
        G.pending_stream = nullptr;
    }
    return p;
}

// A deferred signal must not outlive the call that made it.
int flush_pending()
{
    if (!G.pending.word) return 0;
    hipError_t e = tbv::launch_mark(G.pending.word, 0, G.pending.seq, G.pending_stream);
    G.pending = tbv::PreSignal{};
    G.pending_stream = nullptr;
    return e == hipSuccess ? 0 : -1;
}

// First half of a call: sequence number, slot, pack kernel, work items.
// `sum_out`/`dtype` are only used when the pack can be fused with the sum.
int enqueue_pack(const void* ptr, void* sum_out, size_t nbytes, int dtype, hipStream_t st, Call* c)
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

    // whose payload plays the peer for this call
    const char* peer = nullptr;
    c->resident = false;
    if (!G.staged.empty()) {
        Staged s = G.staged.front(); G.staged.pop_front();
        if (s.nbytes < nbytes) FAIL("staged peer payload (%zu B) is shorter than the call (%zu B)", s.nbytes, nbytes);
        peer = s.ptr;
        if (s.owned) for (auto& o : G.owned) if (o.first == s.ptr) o.second = c->seq;
    } else if (G.resident_bytes >= nbytes && G.resident_bytes) {
        c->resident = true;
    } else if (G.repeat.ptr) {
        if (G.repeat.nbytes < nbytes) FAIL("repeat peer payload (%zu B) is shorter than the call (%zu B)", G.repeat.nbytes, nbytes);
        peer = G.repeat.ptr;
    }

    tbv::PackArgs pa{};
    pa.dst = slot_send(c->slot); pa.src = ptr; pa.nbytes = nbytes;
    pa.cflag = cflag(c->slot); pa.seq = c->seq; pa.arrive = pack_counters(c->slot);
    pa.tagp = G.tag ? (unsigned long long*)(slot_send(c->slot) + tagoff) : nullptr;
    pa.fp = G.kwait ? footprints() : nullptr;
    pa.sigmode = G.packsig;

    if (G.async) {
        // An early flag must not release an older call of this slot that some rail has not finished:
        // with the payload resident, wait until every rail (not only this call's) is less than a ring behind.
        if (wait_for_room(c->resident ? G.R : c->R) != 0) return -1;
        if (c->resident) st_rel(gflag(c->slot), c->seq);      // the peer was early: its flag is already up
        if (G.gpusig) {
            const bool can_fuse = G.fuse && c->resident && sum_out && !G.tag &&
                                  !(((uintptr_t)ptr | (uintptr_t)sum_out) & 15);
            // One launch for a small call: pack, completion word, flag poll and sum in a single kernel whose
            // few blocks are all resident (a decode-size reduction pays one flag wait and one kernel).
            const bool one_kernel = G.onekernel && !can_fuse && sum_out && !G.tag && G.kwait != 1 && G.can_wait_value &&
                                    !(G.railsum && c->R > 1) && nbytes <= G.fusewait_max &&
                                    tbv::small_call_blocks(nbytes) <= tbv::kSmallCallMaxBlocks &&
                                    !(((uintptr_t)ptr | (uintptr_t)sum_out) & 15);
            // Payload already in place and too large for the one-kernel call: pack blocks and sum blocks in one
            // launch (a launch costs about 2.4 us of stream time whatever it does).
            const bool can_merge = G.merge && !can_fuse && !one_kernel && c->resident && sum_out && !G.tag && G.kwait != 1 &&
                                   G.packsig == 0 && !(G.railsum && c->R > 1) && !(((uintptr_t)ptr | (uintptr_t)sum_out) & 15);
            // Deferred signal: counting the pack's blocks costs about 1.5 us at the end of the kernel.
            // When the next kernel on the stream is one of ours and will not wait behind a stream gate
            // (payload already there, or the flag is polled inside the sum kernel), the pack leaves its
            // completion word alone and that next kernel raises it first thing.
            const bool will_poll_in_kernel = nbytes <= G.fusewait_max;
            c->deferred = G.defer && !can_fuse && !can_merge && !one_kernel && !G.tag && G.kwait != 1 && G.can_wait_value &&
                          !(G.railsum && c->R > 1) && (c->resident || will_poll_in_kernel);
            pa.pre = take_pending(st);
            // fault injection from the host: this call's pack never raises its completion word
            const bool mute_pack = G.withhold_seq.load() == c->seq && G.withhold_rail.load() < 0;
            if (mute_pack) {
                pa.cflag = nullptr;
                c->deferred = false;
                if (tbv::launch_pack(pa, st) != hipSuccess) FAIL("pack kernel launch failed");
            } else if (one_kernel) {
                tbv::SumArgs sa{};
                sa.out = sum_out; sa.a = ptr; sa.b = slot_recv(c->slot); sa.nbytes = nbytes; sa.dtype = dtype; sa.seq = c->seq;
                if (!c->resident) {
                    sa.wait_flag = gflag(c->slot); sa.relay = relay_word(c->slot);
                    sa.spin_limit_ticks = (unsigned long long)((G.wdog * 2.0 + 1.0) * G.tick_hz);
                }
                if (G.probe.load()) { sa.done = doneword(c->slot); sa.done_arrive = done_counters(c->slot); }
                KTimer kt(1);
                const double tq = nowt();
                if (tbv::launch_small_call(pa, sa, st, kt.get()) != hipSuccess) FAIL("one-kernel call launch failed");
                { std::lock_guard<std::mutex> lk(G.smx); G.t_post += nowt() - tq; }      // the launch that carries the sum
                c->fused = true;
            } else if (can_fuse || can_merge) {
                tbv::SumArgs sa{};
                sa.out = sum_out; sa.a = ptr; sa.b = slot_recv(c->slot); sa.nbytes = nbytes; sa.dtype = dtype; sa.seq = c->seq;
                if (G.probe.load()) { sa.done = doneword(c->slot); sa.done_arrive = done_counters(c->slot); }
                KTimer kt(1);
                const double tq = nowt();
                if ((can_fuse ? tbv::launch_pack_sum(pa, sa, st, kt.get()) : tbv::launch_pack_sum_merged(pa, sa, st, kt.get())) != hipSuccess)
                    FAIL("pack+sum kernel launch failed");
                { std::lock_guard<std::mutex> lk(G.smx); G.t_post += nowt() - tq; }
                c->fused = true;
            } else {
                if (c->deferred) pa.cflag = nullptr;
                KTimer kt(0);
                if (tbv::launch_pack(pa, st, kt.get()) != hipSuccess) FAIL("pack kernel launch failed");
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
            x.q_head.store(h + 1, std::memory_order_release);
        }
        wake(&G.cv_item);
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
        { std::lock_guard<std::mutex> lk(G.smx); G.t_pre += nowt() - tp; }
        Item it{c->seq, c->slot, nbytes, c->R, c->xbytes, peer, c->resident, false};
        for (int r = 0; r < c->R; r++) if (wire_xfer(G.rr[r], it) != 0) { G.err.store(1); FAIL("transfer failed"); }
        const double tdr = nowt();          // nothing to reap: the emulated sends complete with their arrival
        { std::lock_guard<std::mutex> lk(G.smx); G.t_drain += nowt() - tdr; }
    }
    return 0;
}

// Second half: gate the stream on the flag(s), then the sum.
int enqueue_wait_sum(const void* ptr, void* outp, int dtype, hipStream_t st, const Call& c)
{
    if (c.fused) return 0;
    const char* rb = slot_recv(c.slot);
    const unsigned long long spin_ticks = (unsigned long long)((G.wdog * 2.0 + 1.0) * G.tick_hz);
    const bool probe = G.probe.load() != 0;
    const size_t esz = dtype == 0 ? 4 : 2;

    auto sum_piece = [&](size_t off, size_t len, const unsigned long long* gate, bool last) -> int {
        tbv::SumArgs sa{};
        sa.out = (char*)outp + off; sa.a = (const char*)ptr + off; sa.b = rb + off;
        sa.nbytes = len; sa.dtype = dtype; sa.seq = c.seq;
        sa.wait_flag = gate; sa.relay = gate ? relay_word(c.slot) : nullptr; sa.spin_limit_ticks = spin_ticks;
        sa.fp = G.kwait ? footprints() : nullptr;
        if (probe && last) { sa.done = doneword(c.slot); sa.done_arrive = done_counters(c.slot); }
        sa.pre = take_pending(st);
        KTimer kt(1);
        if (tbv::launch_sum(sa, st, kt.get()) != hipSuccess) FAIL("sum kernel launch failed");
        return 0;
    };
    auto gate_stream = [&](unsigned long long* flag) -> int {
        if (flush_pending() != 0) FAIL("deferred signal launch failed");     // never park a pending signal behind a gate
        if (G.kwait == 1 || !G.can_wait_value) {
            if (tbv::launch_waitflag(flag, c.seq, spin_ticks, G.kwait ? footprints() : nullptr, st) != hipSuccess) FAIL("wait kernel launch failed");
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
    } else {
        // The flag may already be up when the call is made (the peer was early): the payload is then in
        // place before the sum is even launched and the stream needs no gate at all.
        const bool arrived = G.async && !G.tag && G.kwait != 1 && ld_acq(gflag(c.slot)) >= c.seq;
        const bool fusewait = G.async && !arrived && (c.deferred || c.nbytes <= G.fusewait_max) && !G.tag && G.kwait != 1;
        if (G.async && !arrived && !fusewait && gate_stream(gflag(c.slot)) != 0) return -1;
        if (G.async && G.tag) {
            if (tbv::launch_tagchk((const unsigned long long*)(rb + tag_offset(c.nbytes)), c.seq, dbgwords(), st) != hipSuccess)
                FAIL("tag check launch failed");
        }
        tq = nowt();
        if (sum_piece(0, c.nbytes, fusewait ? gflag(c.slot) : nullptr, true) != 0) return -1;
    }
    if (G.kwait && tbv::launch_mark(footprints(), tbv::FP_SUM_DONE, c.seq, st) != hipSuccess) FAIL("footprint launch failed");
    { std::lock_guard<std::mutex> lk(G.smx); G.t_post += nowt() - tq; }
    return 0;
}

// Do this caller stream and a rail's side stream end up on the same hardware queue?  The runtime
// multiplexes streams onto a few hardware queues; two streams on one queue run in submission order,
// so a side-stream copy submitted after the caller's gate would sit behind the gate it is meant to
// release.  Probe: a wait kernel bounded to 300 us goes on the caller's stream, the word it waits
// for is raised from the side stream; on separate queues the wait ends at once, on a shared queue it
// runs to its bound.  Every kernel involved exits by itself.
bool shares_queue_with_wire(hipStream_t st)
{
    if (hipStreamSynchronize(st) != hipSuccess) { (void)hipGetLastError(); return true; }   // measure queues, not backlog
    for (int r = 0; r < G.R; r++) {
        unsigned long long* w = scratchword();
        st_rel(w, 0);
        if (tbv::launch_waitflag(w, 1, (unsigned long long)(300e-6 * G.tick_hz), nullptr, st) != hipSuccess) return true;
        const double t0 = nowt();
        if (stream_bump(G.rr[r].wire, w, 1) != hipSuccess) { (void)hipStreamSynchronize(st); return true; }
        while (hipStreamQuery(st) == hipErrorNotReady && nowt() - t0 < 0.05) { }
        const double dt = nowt() - t0;
        (void)hipStreamSynchronize(G.rr[r].wire);
        (void)hipStreamSynchronize(st);
        (void)hipGetLastError();
        if (dt > 200e-6) {
            LOGF("stream %p shares a hardware queue with rail%d's side stream (probe %.0f us): using the host wire for it",
                 (void*)st, r, dt * 1e6);
            return true;
        }
        LOGF("stream %p and rail%d's side stream run on separate hardware queues (probe %.0f us)", (void*)st, r, dt * 1e6);
    }
    return false;
}

bool use_host_wire(hipStream_t st)
{
    if (G.wire_mode == 2) return true;
    if (G.wire_mode == 1) return false;
    for (auto& p : G.stream_wire) if (p.first == (void*)st) return p.second;
    const bool host = shares_queue_with_wire(st) && tbv::dma_ready();
    G.stream_wire.emplace_back((void*)st, host);
    return host;
}

void note_stream(void* stream, size_t nbytes)
{
    if (stream == G.last_stream) return;
    if (G.last_stream) G.n_stream_sw++;
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

}  // namespace

// ========================================================================== C ABI, part 1

static void teardown();

static int init_impl(int rank, const char* devs, size_t cap)
{
    if (configure(devs, cap) != 0) return -1;
    G.rank = rank;
    if (hipGetDevice(&G.device) != hipSuccess) FAIL("no HIP device");
    { int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeCanUseStreamWaitValue, G.device) != hipSuccess) v = 0;
      G.can_wait_value = v;
      int khz = 0;
      if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, G.device) == hipSuccess && khz > 0) G.tick_hz = khz * 1e3;
      (void)hipGetLastError(); }

    if (!tbv::noalloc_bind_device()) FAIL("built-in counter array not addressable on device %d", G.device);
    const size_t span = G.stride * (size_t)G.nslot;
    if (!alloc_slab(&G.sendbase, span, (G.uncached & 1) != 0, g_uc_send)) FAIL("send bounce allocation failed (%zu B)", span);
    if (!alloc_slab(&G.recvbase, span, (G.uncached & 2) != 0, g_uc_recv)) FAIL("receive bounce allocation failed (%zu B)", span);
    const size_t wbytes = (size_t)W_BLOCKS * MAXSLOT * FLAG_STRIDE;
    if (hipHostMalloc((void**)&G.hostwords, wbytes, hipHostMallocCoherent) != hipSuccess) FAIL("host flag block allocation failed");
    memset(G.hostwords, 0, wbytes);
    const size_t cbytes = sizeof(unsigned int) * 2 * MAXSLOT * tbv::kCounterWords + (size_t)MAXSLOT * 64;
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
        x.idx = r; x.q_head.store(0); x.q_tail.store(0); x.script_pos = 0;
        x.rl_post = x.rl_arr = 0; x.rl_n = 0;
        if (hipStreamCreateWithFlags(&x.wire, hipStreamNonBlocking) != hipSuccess) FAIL("side stream creation failed");
    }
    for (int i = 0; i < MAXSLOT; i++) G.rails_done[i].store(0);
    const bool dma = tbv::dma_init(G.recvbase, MAXRAIL);
    // does a stream-ordered 64-bit write reach the host block? otherwise signal with a one-thread kernel
    G.can_write_value = 1;
    if (hipStreamWriteValue64(G.rr[0].wire, scratchword(), 0x5eedull, 0) != hipSuccess ||
        hipStreamSynchronize(G.rr[0].wire) != hipSuccess || *scratchword() != 0x5eedull) {
        (void)hipGetLastError();
        G.can_write_value = 0;
    }
    G.seq = 0; G.err.store(0);
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
    LOGF("  emulated peer on device %d; stream wait value %s, stream write value %s; uncached=%d tag=%d railsum=%d fuse=%d fusewait<=%zu",
         G.device, G.can_wait_value ? "yes" : "no (wait kernel)", G.can_write_value ? "yes" : "no (mark kernel)",
         G.uncached, G.tag, G.railsum, G.fuse, G.fusewait_max);
    LOGF("  wire %s; copy-engine access for the host wire: %s", G.wire_mode == 1 ? "stream" : G.wire_mode == 2 ? "host" : "auto", dma ? "yes" : "no");
    LOGF("  small calls (<= %zu B) in one kernel: %s", G.fusewait_max, G.onekernel ? "yes" : "no");
    LOGF("  deferred pack signal %s", G.defer ? "on (early peer, or flag polled inside the sum kernel)" : "off");
    LOGF("  cache hints: %s profile; early peer above the one-kernel size: %s", G.streaming ? "streaming" : "resident",
         G.fuse ? "pack+sum fused (4N)" : G.merge ? "pack and sum blocks in one launch" : "two launches");
    return 0;
}

extern "C" int tbv_ar_init(int rank, const char* devs, const char* peer_ip, int port, size_t cap)
{
    (void)peer_ip; (void)port;
    if (G.inited) return 0;
    const int rc = init_impl(rank, devs, cap);
    if (rc != 0) teardown();               // a failed initialisation leaves nothing allocated and no thread running
    return rc;
}

extern "C" int tbv_ar_allreduce(void* ptr, void* outp, size_t nbytes, int dtype, void* stream)
{
    if (!G.inited) FAIL("not initialised");
    if (G.err.load()) FAIL("an earlier transfer failed; the library cannot recover");
    if (nbytes > G.cap) return -2;                    // caller falls back to its own collective
    if (dtype < 0 || dtype > 2) FAIL("unknown dtype %d", dtype);
    if (G.async && !G.run.load()) FAIL("progress threads were stopped by tbv_ar_fini");
    if (!outp) outp = ptr;
    hipStream_t st = (hipStream_t)stream;
    note_stream(stream, nbytes);
    const double te = nowt();
    Call c;
    if (enqueue_pack(ptr, outp, nbytes, dtype, st, &c) != 0) return -1;
    if (enqueue_wait_sum(ptr, outp, dtype, st, c) != 0) return -1;
    if (flush_pending() != 0) FAIL("deferred signal launch failed");
    { std::lock_guard<std::mutex> lk(G.smx); G.t_enq += nowt() - te; }
    return 0;
}

extern "C" void tbv_ar_stats(double* avg_us, unsigned long long* count)
{
    std::lock_guard<std::mutex> lk(G.smx);
    if (avg_us) *avg_us = G.n_acc ? G.t_acc / (double)G.n_acc * 1e6 : 0.0;
    if (count) *count = G.n_acc;
    G.t_acc = 0; G.n_acc = 0;
}

extern "C" void tbv_ar_stats5(double* pre_us, double* xfer_us, double* post_us, double* enq_us, double* drain_us,
                              unsigned long long* count)
{
    std::lock_guard<std::mutex> lk(G.smx);
    const double n = G.n_acc ? (double)G.n_acc : 1.0;
    if (pre_us) *pre_us = G.t_pre / n * 1e6;
    if (xfer_us) *xfer_us = G.t_acc / n * 1e6;
    if (post_us) *post_us = G.t_post / n * 1e6;
    if (enq_us) *enq_us = G.t_enq / n * 1e6;
    if (drain_us) *drain_us = G.t_drain / n * 1e6;
    if (count) *count = G.n_acc;
    G.t_pre = G.t_acc = G.t_post = G.t_enq = G.t_drain = 0; G.n_acc = 0;
}

extern "C" void tbv_ar_stats4(double* pre_us, double* xfer_us, double* post_us, double* enq_us, unsigned long long* count)
{
    std::lock_guard<std::mutex> lk(G.smx);
    const double n = G.n_acc ? (double)G.n_acc : 1.0;
    if (pre_us) *pre_us = G.t_pre / n * 1e6;
    if (xfer_us) *xfer_us = G.t_acc / n * 1e6;
    if (post_us) *post_us = G.t_post / n * 1e6;
    if (enq_us) *enq_us = G.t_enq / n * 1e6;
    if (count) *count = G.n_acc;
    G.t_pre = G.t_acc = G.t_post = G.t_enq = 0; G.n_acc = 0;      // drain keeps accumulating, as in the reference
}

extern "C" int tbv_ar_cap(void) { return (int)G.cap; }
extern "C" int tbv_ar_async(void) { return G.async; }
extern "C" int tbv_ar_err(void) { return G.err.load(); }

extern "C" void tbv_ar_rails(void)
{
    std::lock_guard<std::mutex> lk(G.smx);
    LOGF("per rail (post done / peer arrival, us):");
    for (int r = 0; r < G.R; r++) {
        Rail& x = G.rr[r];
        if (!x.rl_n) continue;
        LOGF("  rail%d: post %7.1f   arrival %7.1f   (%llu calls)", r, x.rl_post / (double)x.rl_n * 1e6,
             x.rl_arr / (double)x.rl_n * 1e6, (unsigned long long)x.rl_n);
        x.rl_post = 0; x.rl_arr = 0; x.rl_n = 0;
    }
}

extern "C" void tbv_ar_hist(void)
{
    LOGF("stream switches: %llu", (unsigned long long)G.n_stream_sw);
    if (G.tag && G.inited) {
        (void)hipDeviceSynchronize();
        unsigned long long* d = dbgwords();
        LOGF("tag checks %llu  plain-load mismatches %llu  system-load mismatches %llu  first bad seq=%llu plain=%llu system=%llu",
             d[0], d[1], d[2], d[3], d[4], d[5]);
    }
    std::lock_guard<std::mutex> lk(G.smx);
    LOGF("transfers by size (bucket = at least 1<<b bytes):");
    for (int b = 0; b < 32; b++) {
        if (!G.hb_n[b]) continue;
        LOGF("  %8zu B~ : %7llu calls  mean %7.1f us  mean rails %.2f", (size_t)1 << b, (unsigned long long)G.hb_n[b],
             G.hb_t[b] / (double)G.hb_n[b] * 1e6, (double)G.hb_r[b] / (double)G.hb_n[b]);
        G.hb_t[b] = 0; G.hb_n[b] = 0; G.hb_r[b] = 0;
    }
}

extern "C" void tbv_ar_fini(void)
{
    if (G.async && G.run.load()) {
        G.run.store(0);
        wake(&G.cv_item);
        for (int r = 0; r < G.R; r++)
            if (G.rr[r].started) { pthread_join(G.rr[r].th, nullptr); G.rr[r].started = false; }
    }
}

// ========================================================================== C ABI, part 2

namespace {
bool pointer_is_host(const void* p)
{
    hipPointerAttribute_t at;
    if (hipPointerGetAttributes(&at, p) != hipSuccess) { (void)hipGetLastError(); return true; }   // unknown to HIP: plain host memory
    return at.type == hipMemoryTypeHost;
}

// Every rail has finished every call up to this sequence number.
uint64_t calls_done()
{
    // each rail's tail counts the items it has completed; a call is done when all its rails are.  The
    // cheap conservative answer: nothing is in flight when every queue is empty.
    for (int r = 0; r < G.R; r++)
        if (G.rr[r].q_head.load(std::memory_order_acquire) != G.rr[r].q_tail.load(std::memory_order_acquire)) return 0;
    return G.seq;
}

// Device copies of host-staged payloads are released on the caller's thread once no call can read them.
void reap_owned()
{
    if (G.owned.empty()) return;
    const uint64_t done = calls_done();
    if (!done) return;
    size_t k = 0;
    for (auto& o : G.owned) {
        if (o.second && o.second <= done) (void)hipFree(o.first);
        else G.owned[k++] = o;
    }
    G.owned.resize(k);
}

// A payload in host memory is moved to the device when it is staged (see host_deposit for why the
// wire never reads host memory).  Returns the device pointer, or null on failure.
const char* to_device(const void* src, size_t nbytes)
{
    char* d = nullptr;
    if (hipMalloc((void**)&d, nbytes ? nbytes : 1) != hipSuccess) return nullptr;
    if (nbytes && hipMemcpy(d, src, nbytes, hipMemcpyHostToDevice) != hipSuccess) { (void)hipFree(d); return nullptr; }
    G.owned.emplace_back(d, 0);
    return d;
}
}  // namespace

extern "C" int tbv_emu_configure(const char* devs, size_t cap)
{
    if (G.inited) return 0;
    return configure(devs, cap);
}

extern "C" int tbv_emu_plan(size_t nbytes, size_t* off, size_t* len)
{
    if (!G.configured) return -1;
    const int R = rails_for(nbytes);
    const size_t xbytes = G.tag ? tag_offset(nbytes) + 8 : nbytes;
    for (int r = 0; r < R; r++) {
        size_t o = 0, l = 0;
        if (!rail_fragment(xbytes, R, r, &o, &l)) { o = xbytes; l = 0; }
        if (off) off[r] = o;
        if (len) len[r] = l;
    }
    return R;
}

extern "C" int tbv_emu_nslot(void) { return G.nslot; }
extern "C" size_t tbv_emu_stride(void) { return G.stride; }
extern "C" void* tbv_emu_send_slot(int slot) { return (G.inited && slot >= 0 && slot < G.nslot) ? slot_send(slot) : nullptr; }
extern "C" void* tbv_emu_recv_slot(int slot) { return (G.inited && slot >= 0 && slot < G.nslot) ? slot_recv(slot) : nullptr; }
extern "C" unsigned long long tbv_emu_seq(void) { return G.seq; }

extern "C" int tbv_emu_stage_peer(const void* src, size_t nbytes)
{
    if (!G.inited || !src) return -1;
    if (G.staged.size() >= LOG_MAX) return -1;
    reap_owned();
    const bool host = pointer_is_host(src);
    const char* p = host ? to_device(src, nbytes) : (const char*)src;
    if (!p) return -1;
    G.staged.push_back(Staged{p, nbytes, host});
    return 0;
}

extern "C" int tbv_emu_stage_peer_repeat(const void* src, size_t nbytes)
{
    if (!G.inited) return -1;
    if (src && pointer_is_host(src)) { src = to_device(src, nbytes); if (!src) return -1; G.owned.back().second = ~0ull; }   // kept until shutdown
    G.repeat = Staged{(const char*)src, src ? nbytes : 0, false};
    return 0;
}

// The peer's payload is already sitting in every receive slot ("the peer ran
// ahead"): each following call of at most nbytes finds its flag up on entry.
// src == NULL ends the mode.
extern "C" int tbv_emu_peer_resident(const void* src, size_t nbytes)
{
    if (!G.inited) return -1;
    if (!src) { G.resident_bytes = 0; return 0; }
    if (nbytes > G.cap) return -2;
    if (drain_rails() != 0) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;        // no earlier sum may still be reading a slot
    for (int s = 0; s < G.nslot; s++)
        if (hipMemcpy(slot_recv(s), src, nbytes, hipMemcpyDefault) != hipSuccess) return -1;
    G.resident_bytes = nbytes;
    return 0;
}

extern "C" int tbv_emu_arrival_script(const int* rails, size_t n)
{
    if (!G.inited) return -1;
    if (drain_rails() != 0) return -1;
    for (size_t i = 0; i < n; i++) if (rails[i] < 0 || rails[i] >= G.R) return -1;
    G.script.assign(rails, rails + n);
    G.turn.store(0);
    for (int r = 0; r < G.R; r++) G.rr[r].script_pos = 0;
    return 0;
}

extern "C" int tbv_emu_withhold(unsigned long long seq, int rail)
{
    G.withhold_rail.store(rail);
    G.withhold_seq.store(seq);
    return 0;
}

extern "C" size_t tbv_emu_arrival_log(unsigned long long* seqs, int* rails, size_t max)
{
    std::lock_guard<std::mutex> lk(G.logmx);
    size_t n = std::min(max, G.arrivals.size());
    for (size_t i = 0; i < n; i++) { if (seqs) seqs[i] = G.arrivals[i].first; if (rails) rails[i] = G.arrivals[i].second; }
    G.arrivals.erase(G.arrivals.begin(), G.arrivals.begin() + (long)n);
    return n;
}

extern "C" int tbv_emu_latency_probe(int on)
{
    if (drain_rails() != 0) return -1;
    G.probe.store(on ? 1 : 0);
    return 0;
}

extern "C" size_t tbv_emu_latencies(double* us, size_t max)
{
    std::lock_guard<std::mutex> lk(G.logmx);
    size_t n = std::min(max, G.latencies.size());
    for (size_t i = 0; i < n; i++) us[i] = G.latencies[i];
    G.latencies.erase(G.latencies.begin(), G.latencies.begin() + (long)n);
    return n;
}

// Per-kernel timing with events recorded on the caller's stream right before and
// after each pack (which 0) and sum / pack+sum (which 1) launch.
extern "C" int tbv_emu_kernel_timing(int on)
{
    if (!G.inited) return -1;
    G.ktime = on ? 1 : 0;
    return 0;
}

// Mean, minimum and count of the recorded launches of one kernel; synchronises the
// device, then forgets the samples.  Returns the count.
extern "C" size_t tbv_emu_kernel_times(int which, double* mean_us, double* min_us)
{
    if (!G.inited || which < 0 || which > 1) return 0;
    (void)hipDeviceSynchronize();
    double sum = 0, mn = 1e30;
    size_t n = 0;
    for (size_t i = 0; i < G.kev_used[which]; i++) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, G.kev[which][i].first, G.kev[which][i].second) != hipSuccess) continue;
        sum += ms * 1e3; mn = std::min(mn, (double)ms * 1e3); n++;
    }
    G.kev_used[which] = 0;
    if (mean_us) *mean_us = n ? sum / (double)n : 0.0;
    if (min_us) *min_us = n ? mn : 0.0;
    return n;
}

extern "C" void tbv_emu_footprints(unsigned long long out[5])
{
    for (int i = 0; i < 5; i++) out[i] = G.inited ? footprints()[i] : 0;
}

extern "C" void tbv_emu_tag_counts(unsigned long long* checks, unsigned long long* bad_plain, unsigned long long* bad_system)
{
    unsigned long long z[3] = {0, 0, 0};
    unsigned long long* d = (G.inited && G.tag) ? dbgwords() : z;
    if (checks) *checks = d[0];
    if (bad_plain) *bad_plain = d[1];
    if (bad_system) *bad_system = d[2];
}

extern "C" void tbv_emu_shutdown(void)
{
    if (!G.inited) { G.configured = 0; return; }
    teardown();
}

// Releases whatever exists, whether or not initialisation completed.
static void teardown()
{
    // let the GPU finish what is queued (flags are raised even after an error), then stop the threads
    (void)hipDeviceSynchronize();
    tbv_ar_fini();
    for (int r = 0; r < MAXRAIL; r++) if (G.rr[r].wire) { (void)hipStreamDestroy(G.rr[r].wire); G.rr[r].wire = nullptr; }
    for (auto& o : G.owned) (void)hipFree(o.first);
    G.owned.clear();
    G.stream_wire.clear();
    for (int i = 0; i < MAXSLOT; i++) if (G.ev[i]) { (void)hipEventDestroy(G.ev[i]); G.ev[i] = nullptr; }
    free_slab(G.sendbase, g_uc_send); G.sendbase = nullptr;
    free_slab(G.recvbase, g_uc_recv); G.recvbase = nullptr;
    if (G.hostwords) { (void)hipHostFree(G.hostwords); G.hostwords = nullptr; }
    if (G.counters) { (void)hipFree(G.counters); G.counters = nullptr; }
    for (int w = 0; w < 2; w++) {
        for (auto& p : G.kev[w]) { (void)hipEventDestroy(p.first); (void)hipEventDestroy(p.second); }
        G.kev[w].clear(); G.kev_used[w] = 0;
    }
    G.ktime = 0;
    G.pending = tbv::PreSignal{}; G.pending_stream = nullptr;
    G.staged.clear(); G.repeat = Staged{nullptr, 0, false}; G.resident_bytes = 0;
    G.script.clear(); G.turn.store(0); G.withhold_seq.store(0);
    { std::lock_guard<std::mutex> lk(G.logmx); G.arrivals.clear(); G.latencies.clear(); }
    G.probe.store(0);
    { std::lock_guard<std::mutex> lk(G.smx);
      G.t_acc = G.t_pre = G.t_post = G.t_enq = G.t_drain = 0; G.n_acc = 0;
      for (int b = 0; b < 32; b++) { G.hb_t[b] = 0; G.hb_n[b] = 0; G.hb_r[b] = 0; } }
    G.last_stream = nullptr; G.n_stream_sw = 0; G.nseen = 0;
    G.seq = 0; G.err.store(0);
    G.inited = 0; G.configured = 0;
}

extern "C" int tbv_ar_allreduce_chunked(void* ptr, void* outp, size_t nbytes, int dtype, void* stream)
{
    if (!G.inited) FAIL("not initialised");
    if (G.err.load()) FAIL("an earlier transfer failed; the library cannot recover");
    if (dtype < 0 || dtype > 2) FAIL("unknown dtype %d", dtype);
    if (!G.async) FAIL("the chunked pipeline needs async mode");
    if (!G.run.load()) FAIL("progress threads were stopped by tbv_ar_fini");
    if (!outp) outp = ptr;
    if (nbytes == 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    note_stream(stream, nbytes);
    const size_t esz = dtype == 0 ? 4 : 2;
    const size_t chunk = (G.cap / esz) * esz;
    const size_t n = (nbytes + chunk - 1) / chunk;
    const size_t depth = std::min<size_t>((size_t)G.nslot - 1, n);
    std::vector<Call> calls(n);
    auto piece = [&](size_t i, size_t* off, size_t* len) { *off = i * chunk; *len = std::min(chunk, nbytes - *off); };
    const double te = nowt();
    size_t off, len;
    for (size_t i = 0; i < depth; i++) {
        piece(i, &off, &len);
        if (enqueue_pack((const char*)ptr + off, nullptr, len, dtype, st, &calls[i]) != 0) return -1;
    }
    for (size_t i = 0; i < n; i++) {
        piece(i, &off, &len);
        if (enqueue_wait_sum((const char*)ptr + off, (char*)outp + off, dtype, st, calls[i]) != 0) return -1;
        if (i + depth < n) {
            piece(i + depth, &off, &len);
            if (enqueue_pack((const char*)ptr + off, nullptr, len, dtype, st, &calls[i + depth]) != 0) return -1;
        }
    }
    if (flush_pending() != 0) FAIL("deferred signal launch failed");
    { std::lock_guard<std::mutex> lk(G.smx); G.t_enq += nowt() - te; }
    return 0;
}

extern "C" int tbv_emu_run_pack(const void* src, size_t nbytes, int slot, void* stream)
{
    if (!G.inited || slot < 0 || slot >= G.nslot || nbytes > G.cap) return -1;
    tbv::PackArgs pa{};
    pa.dst = slot_send(slot); pa.src = src; pa.nbytes = nbytes;
    pa.cflag = word(W_MISC, 8 + slot % 16);          // a completion word nobody waits on
    pa.seq = 1; pa.arrive = pack_counters(slot); pa.sigmode = G.packsig;
    return tbv::launch_pack(pa, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}

extern "C" int tbv_emu_run_sum(void* out, const void* a, const void* b, size_t nbytes, int dtype, void* stream)
{
    if (dtype < 0 || dtype > 2) return -1;
    tbv::SumArgs sa{};
    sa.out = out; sa.a = a; sa.b = b; sa.nbytes = nbytes; sa.dtype = dtype;
    return tbv::launch_sum(sa, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}
