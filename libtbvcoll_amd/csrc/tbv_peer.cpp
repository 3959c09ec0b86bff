// The emulated peer: the only code that knows there is no second machine.
//
// The reference's peer is reached through RDMA write-with-immediate over ibverbs queue
// pairs set up by a TCP rendezvous (step4/libtbvcoll.cpp:172-224 transfer and reaping,
// :343-403 bring-up).  Here the peer is played on the same GPU: for every call, each
// rail's progress thread copies that rail's fragment of the peer payload into the receive
// slot (a copy kernel on the rail's side stream whose last block raises the arrival word;
// side-stream copies plus a stream write into a cached ring; or a copy-engine transfer)
// and the 64-bit arrival word is the signal the immediate's completion gave.  wire_xfer()
// and its non-blocking halves wire_post() / wire_arrived() / wire_done() are the seam a
// real transport would replace; everything else in this file feeds them (payload staging,
// the early-peer mode, arrival scripts, held rails and withheld signals for tests).
#include "tbv_engine.h"

#include <sched.h>

#include <algorithm>

#include "../../include/tbvcoll_emu.h"
#include "tbv_dma.h"
#include "tbv_sock.h"

namespace tbv {

namespace {

void record_arrival(uint64_t seq, int rail)
{
    std::lock_guard<std::mutex> lk(G.logmx);
    if (G.arrivals.size() < LOG_MAX) G.arrivals.emplace_back(seq, rail);
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
    if (!dma_ready()) { LOGF("rail%d: no copy-engine access for the host wire", x.idx); return -1; }
    size_t n = len;
    if (it.peer && off + n > it.nbytes) n = it.nbytes > off ? it.nbytes - off : 0;        // staged payload has no tag
    const char* src = it.peer ? it.peer + off : slot_send(it.slot) + off;
    auto left = [&]() { double r = G.wdog - (nowt() - t0); return r > 0.001 ? r : 0.001; };
    // TBV_CHUNK: the fragment travels as several writes, the completion only after the last
    // (step4/libtbvcoll.cpp:181-194)
    const size_t ck = G.chunkb ? G.chunkb : (n ? n : 1);
    int rc = 0;
    for (size_t o = 0; o < n && rc == 0; o += ck)
        rc = dma_copy(x.idx, slot_recv(it.slot) + off + o, DMA_DEVICE, src + o, G.peer_tcp ? DMA_HOST : DMA_DEVICE, std::min(ck, n - o), left());
    if (rc == 0 && it.peer && G.tag) {       // the peer's own tag travels at the end of its payload
        const size_t to = tag_offset(it.nbytes);
        if (to >= off && to < off + len)
            rc = dma_copy(x.idx, slot_recv(it.slot) + to, DMA_DEVICE, slot_send(it.slot) + to, DMA_DEVICE, 8, left());
    }
    if (rc == -2) LOGF("watchdog: rail%d host wire copy exceeded %.1fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq);
    else if (rc != 0) LOGF("rail%d host wire copy failed seq=%llu", x.idx, (unsigned long long)it.seq);
    return rc == 0 ? 0 : -1;
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
        if (launch_waitflag(w, 1, (unsigned long long)(300e-6 * G.tick_hz), nullptr, st) != hipSuccess) return true;
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

bool pointer_is_host(const void* p)
{
    hipPointerAttribute_t at;
    if (hipPointerGetAttributes(&at, p) != hipSuccess) { (void)hipGetLastError(); return true; }   // unknown to HIP: plain host memory
    return at.type == hipMemoryTypeHost;
}

// Device buffers the emulated peer owns (copies of host-staged payloads, int8 images) are released on the
// caller's thread once the call that reads them has been released: only the wire reads them, and a call is
// released after its last rail has seen its fragment arrive.
void reap_owned()
{
    if (G.owned.empty()) return;
    size_t k = 0;
    for (auto& o : G.owned) {
        const bool over = o.second && o.second != ~0ull &&
                          G.released[(int)(o.second % (uint64_t)G.nslot)].load(std::memory_order_acquire) >= o.second;
        if (over) (void)hipFree(o.first);
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

// The int8 image of a peer payload, made the way the peer's own pack kernel would make it (on the caller's
// thread, on the utility stream, waited for).  The buffer is released once call `seq` is over.
const char* peer_image(const char* payload, size_t nbytes, int dtype, uint64_t seq)
{
    char* img = nullptr;
    if (hipMalloc((void**)&img, codec_image_bytes(nbytes, dtype)) != hipSuccess) return nullptr;
    PackArgs pa{};
    pa.dst = img; pa.src = payload; pa.nbytes = nbytes; pa.seq = seq;
    if (launch_quant(pa, dtype, G.util) != hipSuccess || hipStreamSynchronize(G.util) != hipSuccess) { (void)hipFree(img); return nullptr; }
    G.owned.emplace_back(img, seq);
    return img;
}

// Put the resident payload into every receive slot in the wanted form: raw (-1) or as its int8 image for `form`.
int resident_refill(int form)
{
    if (drain_rails() != 0) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;         // no earlier sum may still be reading a slot
    for (int s = 0; s < G.nslot; s++) {
        if (form < 0) {
            if (hipMemcpy(slot_recv(s), G.resident_src, G.resident_bytes, hipMemcpyDeviceToDevice) != hipSuccess) return -1;
        } else {
            PackArgs pa{};
            pa.dst = slot_recv(s); pa.src = G.resident_src; pa.nbytes = G.resident_bytes;
            if (!G.util || launch_quant(pa, form, G.util) != hipSuccess) return -1;
        }
        G.resident_ok[s] = true;
    }
    if (form >= 0 && hipStreamSynchronize(G.util) != hipSuccess) return -1;
    G.resident_form = form;
    return 0;
}

// Stream wire deposit of one rail fragment: side-stream copies of the fragment into the receive slot, then
// the 64-bit arrival word on the same stream.  Nothing here waits.
int stream_deposit(Rail& x, const Item& it, size_t off, size_t len, bool withheld)
{
    unsigned long long* aw = aflag(x.idx, it.slot);
    const char* src = it.peer ? it.peer + off : slot_send(it.slot) + off;
    size_t n = len;
    if (it.peer && off + n > it.nbytes) n = it.nbytes > off ? it.nbytes - off : 0;   // staged payload has no tag
    // One launch when the receive ring is uncached: the library's own copy kernel writes the fragment and its last
    // block raises the arrival word, as the pack raises its completion word (stores to uncached memory are visible
    // once acknowledged; into a cached ring the signal has to wait for the end of the copy kernel instead, below).
    // Every HIP call of the three threads involved goes through the runtime's locks, so calls per transfer count.
    if ((G.uncached & 2) && !G.chunkb && !(it.peer && G.tag)) {
        PackArgs pa{};
        pa.dst = slot_recv(it.slot) + off; pa.src = src; pa.nbytes = n; pa.seq = it.seq;
        pa.cflag = withheld ? nullptr : aw; pa.arrive = wire_counters(x.idx, it.slot);
        if (launch_pack(pa, x.wire) != hipSuccess) { LOGF("rail%d peer deposit failed seq=%llu", x.idx, (unsigned long long)it.seq); return -1; }
        return 0;
    }
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
    return 0;
}

void account_arrival(Rail& x, const Item& it, double t0, double tp, double ta)
{
    record_arrival(it.seq, x.idx);
    std::lock_guard<std::mutex> lk(G.smx);
    x.rl_post += tp - t0; x.rl_arr += ta - t0; x.rl_n++;
    if (x.idx == 0) {
        G.t_acc += ta - t0; G.n_acc++;
        int b = 0; { size_t v = it.nbytes; while (v >>= 1) b++; } if (b > 31) b = 31;
        G.hb_t[b] += ta - t0; G.hb_n[b]++; G.hb_r[b] += (uint64_t)it.R;
    }
}

void refresh_hooks()
{
    int h = (!G.script.empty() || G.withhold_seq.load() != 0) ? 1 : 0;
    for (int r = 0; r < MAXRAIL; r++) if (G.hold[r].load()) h = 1;
    G.hooks = h;
}

}  // namespace

// Raise a 64-bit word from a side stream after everything queued on it so far:
// the stand-in for the completion an RDMA write-with-immediate delivers.
hipError_t stream_bump(hipStream_t st, unsigned long long* w, uint64_t v)
{
    if (G.can_write_value) return hipStreamWriteValue64(st, w, v, 0);
    return launch_mark(w, 0, v, st);
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

    // test hooks, off the default path: an arrival script holds this rail's deposit until its turn,
    // and one chosen signal can be withheld for good
    size_t my_turn = (size_t)-1;
    bool withheld = false;
    if (G.hooks) {
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
        withheld = (G.withhold_seq.load() == it.seq && G.withhold_rail.load() == x.idx);
        while (G.hold[x.idx].load(std::memory_order_acquire)) {          // the host holds this rail back for now
            if (nowt() - t0 > G.wdog) { LOGF("watchdog: rail%d held for %.1fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq); return -1; }
            if (!G.run.load(std::memory_order_relaxed) && G.async) return -1;
            sched_yield();
        }
    }

    // Two processes: this rail's fragment goes to the peer over its connection and the peer's comes back into pinned
    // host memory; from there it is deposited like an emulated peer's payload (same copy, same arrival word).
    Item tcp_item = it;
    if (G.peer_tcp) {
        const char* staged = nullptr;
        if (sock_exchange(x, it, off, len, t0, &staged) != 0) return -1;
        tcp_item.peer = staged - off;               // the deposit adds the fragment's offset
        tcp_item.resident = false;
    }
    const Item& dep = G.peer_tcp ? tcp_item : it;
    if (!dep.resident && dep.host_wire) {
        // Host wire: the fragment goes straight into the receive slot with a copy-engine transfer that
        // this thread waits for, and this thread raises the arrival word itself.  Nothing is placed on
        // one of our compute queues, so this works even when the caller's gated stream and the side
        // stream are multiplexed onto the same hardware queue.
        if (host_deposit(x, dep, off, len, t0) != 0) return -1;
        if (!withheld) st_rel(aw, it.seq);
    } else if (!dep.resident) {
        if (stream_deposit(x, dep, off, len, withheld) != 0) return -1;
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
    if (G.peer_tcp) sock_consumed(x, it);
    account_arrival(x, it, t0, tp, nowt());      // logged before the next rail in the script may go
    if (my_turn != (size_t)-1) G.turn.store(my_turn + 1, std::memory_order_release);
    return 0;
}

// The two non-blocking halves of the stream wire, for a progress thread that keeps several transfers in
// flight (a NIC with several work requests posted): post the deposit and its arrival signal; later ask
// whether the signal has come.  *owns = false when this rail has no fragment of the call.
int wire_post(Rail& x, const Item& it, bool* owns)
{
    size_t off = 0, len = 0;
    *owns = rail_fragment(it.xbytes, it.R, x.idx, &off, &len);
    if (!*owns) return 0;
    if (it.resident) { st_rel(aflag(x.idx, it.slot), it.seq); return 0; }
    return stream_deposit(x, it, off, len, false);
}

bool wire_arrived(const Rail& x, const Item& it) { return ld_acq(aflag(x.idx, it.slot)) >= it.seq; }

void wire_done(Rail& x, const Item& it, double t0, double tp) { account_arrival(x, it, t0, tp, nowt()); }

bool use_host_wire(hipStream_t st)
{
    if (G.wire_mode == 2) return true;
    if (G.wire_mode == 1) return false;
    if ((void*)st == G.wire_stream) return G.wire_stream_host;        // the usual case: the stream of the call before
    bool host = false, known = false;
    for (auto& p : G.stream_wire) if (p.first == (void*)st) { host = p.second; known = true; break; }
    if (!known) {
        host = shares_queue_with_wire(st) && dma_ready();
        G.stream_wire.emplace_back((void*)st, host);
    }
    G.wire_stream = (void*)st; G.wire_stream_host = host;
    return host;
}

// Whose payload plays the peer for this call: a staged one (FIFO), the resident one (already in the
// receive slot, or put back through the wire when another payload went through that slot since),
// the repeat payload, or none (mirror: the peer echoes this rank's bounce slot).
int peer_assign(Call* c, size_t nbytes, int dtype, const char** peer)
{
    *peer = nullptr;
    c->resident = false;
    if (G.peer_tcp) return 0;                    // the payload comes from the peer process, over the wire
    bool from_resident = false;
    if (!G.staged.empty()) {
        Staged s = G.staged.front(); G.staged.pop_front();
        if (s.nbytes < nbytes) FAIL("staged peer payload (%zu B) is shorter than the call (%zu B)", s.nbytes, nbytes);
        *peer = s.ptr;
        if (s.owned) for (auto& o : G.owned) if (o.first == s.ptr) o.second = c->seq;
    } else if (G.resident_bytes && G.resident_bytes >= nbytes) {
        // the receive slots hold either the raw payload or its int8 image for one dtype and exactly its size
        const int form = c->codec ? dtype : -1;
        if (c->codec && G.resident_bytes != nbytes) FAIL("with the int8 codec an early peer's payload must have the call's size (%zu B, call %zu B)", G.resident_bytes, nbytes);
        if (form != G.resident_form && resident_refill(form) != 0) return -1;
        if (G.resident_ok[c->slot]) c->resident = true;
        else { *peer = G.resident_src; from_resident = true; }
    } else if (G.repeat.ptr) {
        if (G.repeat.nbytes < nbytes) FAIL("repeat peer payload (%zu B) is shorter than the call (%zu B)", G.repeat.nbytes, nbytes);
        *peer = G.repeat.ptr;
    }
    // With the codec the peer's pack kernel would have quantised its payload: do that for it now.
    if (c->codec && *peer) {
        reap_owned();
        const char* img = peer_image(*peer, nbytes, dtype, c->seq);
        if (!img) FAIL("could not quantise the peer's payload");
        *peer = img;
    }
    // Any call that deposits into its slot replaces the resident image there; the image counts as restored
    // only when the resident payload itself went through the wire in full.
    if (G.resident_bytes && !c->resident)
        G.resident_ok[c->slot] = (from_resident && nbytes >= G.resident_bytes);
    return 0;
}

void peer_teardown()
{
    for (auto& o : G.owned) (void)hipFree(o.first);
    G.owned.clear();
    if (G.resident_src) { (void)hipFree(G.resident_src); G.resident_src = nullptr; }
    G.resident_bytes = 0;
    G.stream_wire.clear(); G.wire_stream = nullptr; G.wire_stream_host = false;
    G.staged.clear(); G.repeat = Staged{nullptr, 0, false};
    G.script.clear(); G.turn.store(0); G.withhold_seq.store(0); G.hooks = 0;
    for (int r = 0; r < MAXRAIL; r++) G.hold[r].store(0);
    std::lock_guard<std::mutex> lk(G.logmx);
    G.arrivals.clear(); G.latencies.clear();
}

}  // namespace tbv

using namespace tbv;

// ========================================================================== C ABI, part 2: the emulated peer

extern "C" int tbv_emu_stage_peer(const void* src, size_t nbytes)
{
    if (!G.inited || !src) return -1;
    if (G.peer_tcp) FAIL("two-process mode: the peer's payload comes from the peer process, it cannot be staged");
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
    if (G.peer_tcp && src) FAIL("two-process mode: the peer's payload comes from the peer process, it cannot be staged");
    if (src && pointer_is_host(src)) { src = to_device(src, nbytes); if (!src) return -1; G.owned.back().second = ~0ull; }   // kept until shutdown
    G.repeat = Staged{(const char*)src, src ? nbytes : 0, false};
    return 0;
}

// The peer's payload is already sitting in every receive slot ("the peer ran ahead"): each following
// call of at most nbytes with no queued payload finds its flag up on entry.  A copy of the payload is
// kept so that a slot another payload went through can get the resident image back (through the wire,
// as part of the next call that wants it).  src == NULL ends the mode.
extern "C" int tbv_emu_peer_resident(const void* src, size_t nbytes)
{
    if (!G.inited) return -1;
    if (G.peer_tcp && src) FAIL("two-process mode: the peer's payload comes from the peer process, it cannot be made resident");
    if (src && nbytes > G.cap) return -2;
    if (drain_rails() != 0) return -1;
    if (hipDeviceSynchronize() != hipSuccess) return -1;        // no earlier sum may still be reading a slot or the old copy
    if (G.resident_src) { (void)hipFree(G.resident_src); G.resident_src = nullptr; }
    G.resident_bytes = 0;
    if (!src || !nbytes) return 0;
    if (hipMalloc((void**)&G.resident_src, nbytes) != hipSuccess) { G.resident_src = nullptr; return -1; }
    if (hipMemcpy(G.resident_src, src, nbytes, hipMemcpyDefault) != hipSuccess) return -1;
    for (int s = 0; s < G.nslot; s++) {
        if (hipMemcpy(slot_recv(s), G.resident_src, nbytes, hipMemcpyDeviceToDevice) != hipSuccess) return -1;
        G.resident_ok[s] = true;
    }
    G.resident_bytes = nbytes;
    G.resident_form = -1;
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
    refresh_hooks();
    return 0;
}

extern "C" int tbv_emu_withhold(unsigned long long seq, int rail)
{
    if (G.inited && drain_rails() != 0) return -1;              // the hook switch is read by the progress threads
    G.withhold_rail.store(rail);
    G.withhold_seq.store(seq);
    refresh_hooks();
    return 0;
}

// Test hook: while `hold` is non-zero, rail `rail` deposits nothing (each held transfer is bounded by the
// watchdog).  Setting a hold needs idle rails; lifting one may be done at any time, from any thread.
extern "C" int tbv_emu_hold_rail(int rail, int hold)
{
    if (!G.inited || rail < 0 || rail >= G.R) return -1;
    if (hold) {
        if (drain_rails() != 0) return -1;
        G.hold[rail].store(1);
        refresh_hooks();
    } else {
        G.hold[rail].store(0, std::memory_order_release);               // hooks stay on until the next idle change
    }
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
