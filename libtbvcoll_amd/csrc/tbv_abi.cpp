// The extern "C" surface of libtbvcoll.so (declared in include/tbvcoll.h and include/tbvcoll_emu.h).
//
// Part 1 is what the reference's ctypes binding loads (step4/tbvcoll.py:19-30), replacing
// step4/libtbvcoll.cpp:279-566; part 2 holds this build's additions that are not about the
// emulated peer itself (those live beside wire_xfer in tbv_peer.cpp).
#include <unistd.h>

#include <algorithm>

#include "../../include/tbvcoll_emu.h"
#include "tbv_engine.h"
#include "tbv_sock.h"

using namespace tbv;

// ========================================================================== part 1: the drop-in boundary

namespace {
// The sequence number, the ring slots and the rails' queues have one producer (as in the reference, which
// increments its sequence number without a lock, step4/libtbvcoll.cpp:435): calls may come from any thread, but
// from one at a time.  Two at once would share a slot; say so instead.
struct OneCaller {
    bool ok;
    OneCaller() : ok(G.in_call.exchange(1, std::memory_order_acquire) == 0) {}
    ~OneCaller() { if (ok) G.in_call.store(0, std::memory_order_release); }
};
}  // namespace
#define ONE_CALLER() OneCaller one_caller; if (!one_caller.ok) FAIL("two threads inside the library at once: calls must come from one thread at a time")

extern "C" int tbv_ar_init(int rank, const char* devs, const char* peer_ip, int port, size_t cap)
{
    if (G.inited) return 0;
    const int rc = init_impl(rank, devs, peer_ip, port, cap);
    if (rc != 0) teardown();               // a failed initialisation leaves nothing allocated and no thread running
    return rc;
}

extern "C" int tbv_ar_allreduce(void* ptr, void* outp, size_t nbytes, int dtype, void* stream)
{
    if (!G.inited) FAIL("not initialised");
    if (G.err.load(std::memory_order_relaxed)) FAIL("an earlier transfer failed; the library cannot recover");
    if (nbytes > G.cap) return -2;                    // caller falls back to its own collective
    if (dtype < 0 || dtype > 2) FAIL("unknown dtype %d", dtype);
    if (G.async && !G.run.load(std::memory_order_relaxed)) FAIL("progress threads were stopped by tbv_ar_fini");
    ONE_CALLER();
    if (!outp) outp = ptr;
    hipStream_t st = (hipStream_t)stream;
    note_stream(stream, nbytes);
    const double te = nowt();
    Call c{};
    if (enqueue_pack(ptr, outp, nbytes, dtype, st, &c) != 0) return -1;
    if (enqueue_wait_sum(ptr, outp, dtype, st, c) != 0) return -1;
    if (flush_pending() != 0) FAIL("deferred signal launch failed");
    G.t_enq += nowt() - te;
    return 0;
}

// The three statistics readers share one body: per-call averages over the transfers rail 0 has completed
// since the last read (step4/libtbvcoll.cpp:510-536; a count of zero divides by one, :518,529).
namespace {
void read_stats(double* pre_us, double* xfer_us, double* post_us, double* enq_us, double* drain_us,
                unsigned long long* count, bool reset_drain)
{
    double acc; uint64_t n_acc;
    { std::lock_guard<std::mutex> lk(G.smx); acc = G.t_acc; n_acc = G.n_acc; G.t_acc = 0; G.n_acc = 0; }
    const double n = n_acc ? (double)n_acc : 1.0;
    if (pre_us) *pre_us = G.t_pre / n * 1e6;
    if (xfer_us) *xfer_us = acc / n * 1e6;
    if (post_us) *post_us = G.t_post / n * 1e6;
    if (enq_us) *enq_us = G.t_enq / n * 1e6;
    if (drain_us) *drain_us = G.t_drain / n * 1e6;
    if (count) *count = n_acc;
    G.t_pre = G.t_post = G.t_enq = 0;
    if (reset_drain) G.t_drain = 0;
}
}  // namespace

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
    read_stats(pre_us, xfer_us, post_us, enq_us, drain_us, count, true);
}

extern "C" void tbv_ar_stats4(double* pre_us, double* xfer_us, double* post_us, double* enq_us, unsigned long long* count)
{
    read_stats(pre_us, xfer_us, post_us, enq_us, nullptr, count, false);     // drain keeps accumulating, as in the reference
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

extern "C" void tbv_ar_fini(void) { stop_progress(); }

// ========================================================================== part 2: additions

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

// The rendezvous of the two-process mode alone (sockets only, no GPU): needs tbv_emu_configure first.
extern "C" int tbv_emu_rendezvous(int rank, const char* peer_ip, int port, double timeout_s)
{
    if (!G.configured || G.inited) return -1;
    int fds[MAXRAIL];
    const int rc = sock_rendezvous(rank, peer_ip, port, fds, timeout_s);
    for (int r = 0; r < MAXRAIL; r++) if (fds[r] >= 0) close(fds[r]);
    return rc;
}

extern "C" int tbv_emu_nslot(void) { return G.nslot; }
extern "C" size_t tbv_emu_stride(void) { return G.stride; }
extern "C" void* tbv_emu_send_slot(int slot) { return (G.inited && slot >= 0 && slot < G.nslot) ? slot_send(slot) : nullptr; }
extern "C" void* tbv_emu_recv_slot(int slot) { return (G.inited && slot >= 0 && slot < G.nslot) ? slot_recv(slot) : nullptr; }
extern "C" unsigned long long tbv_emu_seq(void) { return G.seq; }

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

// Per-kernel timing: every pack launch (which 0) and every launch that carries a sum (which 1) gets the
// dispatch's own start and end timestamps.
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

// Start and end of every recorded launch of one kind, in microseconds after the start of the first one (the
// dispatches' own timestamps); synchronises the device and keeps the samples.  Returns how many were written.
extern "C" size_t tbv_emu_kernel_timeline(int which, double* start_us, double* stop_us, size_t max)
{
    if (!G.inited || which < 0 || which > 1 || !start_us || !stop_us) return 0;
    (void)hipDeviceSynchronize();
    size_t n = 0;
    for (size_t i = 0; i < G.kev_used[which] && n < max; i++) {
        float a = 0, b = 0;
        if (hipEventElapsedTime(&a, G.kev[which][0].first, G.kev[which][i].first) != hipSuccess ||
            hipEventElapsedTime(&b, G.kev[which][0].first, G.kev[which][i].second) != hipSuccess) continue;
        start_us[n] = a * 1e3; stop_us[n] = b * 1e3; n++;
    }
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

extern "C" int tbv_ar_allreduce_chunked(void* ptr, void* outp, size_t nbytes, int dtype, void* stream)
{
    if (!G.inited) FAIL("not initialised");
    if (G.err.load()) FAIL("an earlier transfer failed; the library cannot recover");
    if (dtype < 0 || dtype > 2) FAIL("unknown dtype %d", dtype);
    if (!G.async) FAIL("the chunked pipeline needs async mode");
    if (!G.run.load()) FAIL("progress threads were stopped by tbv_ar_fini");
    if (!outp) outp = ptr;
    if (nbytes == 0) return 0;
    ONE_CALLER();
    hipStream_t st = (hipStream_t)stream;
    note_stream(stream, nbytes);
    const size_t esz = dtype == 0 ? 4 : 2;
    const size_t chunk = (G.cap / esz) * esz;
    const size_t n = (nbytes + chunk - 1) / chunk;
    const size_t depth = std::min<size_t>((size_t)G.nslot - 1, n);
    std::vector<Call> calls(n);
    for (auto& k : calls) k.out_unaligned = (((uintptr_t)outp) & 15) != 0;    // chunk offsets keep the base's alignment or the codec is off anyway
    auto piece = [&](size_t i, size_t* off, size_t* len) { *off = i * chunk; *len = std::min(chunk, nbytes - *off); };
    const double te = nowt();
    size_t off, len;
    for (size_t i = 0; i < depth; i++) {
        piece(i, &off, &len);
        if (enqueue_pack((const char*)ptr + off, nullptr, len, dtype, st, &calls[i]) != 0) return -1;
    }
    for (size_t i = 0; i < n; i++) {
        // the pack of chunk i+depth shares a launch with the sum of chunk i wherever the mode allows
        PackArgs held{};
        bool have_held = false;
        if (i + depth < n) {
            piece(i + depth, &off, &len);
            if (enqueue_pack((const char*)ptr + off, nullptr, len, dtype, st, &calls[i + depth], nullptr, &held) != 0) return -1;
            have_held = calls[i + depth].held;
        }
        piece(i, &off, &len);
        if (enqueue_wait_sum((const char*)ptr + off, (char*)outp + off, dtype, st, calls[i], nullptr, have_held ? &held : nullptr) != 0) return -1;
    }
    if (flush_pending() != 0) FAIL("deferred signal launch failed");
    G.t_enq += nowt() - te;
    return 0;
}

// The all-reduce followed by the RMSNorm of its result, in one pass over the hidden state (planned, not built,
// in the reference: reports/12_references.md:136).
extern "C" int tbv_ar_allreduce_rmsnorm(void* ptr, void* outp, void* normed, const void* weight, float eps,
                                        size_t rows, size_t hidden, int dtype, void* stream)
{
    if (!G.inited) FAIL("not initialised");
    if (G.err.load(std::memory_order_relaxed)) FAIL("an earlier transfer failed; the library cannot recover");
    if (dtype < 0 || dtype > 2) FAIL("unknown dtype %d", dtype);
    const size_t esz = dtype == 0 ? 4 : 2;
    if (rows == 0 || hidden == 0) return 0;
    if (hidden > ((size_t)1 << 40) / rows) return -2;
    const size_t nbytes = rows * hidden * esz;
    if (nbytes > G.cap) return -2;                    // caller falls back to its own collective and norm
    if (!row_norm_shape_ok(rows, hidden, dtype)) FAIL("rmsnorm rows must be a multiple of 16 bytes and at most %d bytes", kRowNormMaxVecs * 16);
    if (!normed || !weight || !ptr) FAIL("null buffer");
    if (!outp) outp = ptr;
    if (((uintptr_t)ptr | (uintptr_t)outp | (uintptr_t)normed | (uintptr_t)weight) & 15) FAIL("rmsnorm buffers must be 16-byte aligned");
    if (G.async && !G.run.load(std::memory_order_relaxed)) FAIL("progress threads were stopped by tbv_ar_fini");
    ONE_CALLER();
    hipStream_t st = (hipStream_t)stream;
    note_stream(stream, nbytes);
    NormArgs nm{weight, normed, eps, (unsigned)(hidden * esz / 16), (unsigned)rows, G.streaming};
    const double te = nowt();
    Call c{};
    if (enqueue_pack(ptr, outp, nbytes, dtype, st, &c, &nm) != 0) return -1;
    if (enqueue_wait_sum(ptr, outp, dtype, st, c, &nm) != 0) return -1;
    if (flush_pending() != 0) FAIL("deferred signal launch failed");
    G.t_enq += nowt() - te;
    return 0;
}

// Standalone row kernel for benches and tests: mode 0 normalises `a`; mode 1 writes out = a + b and normalises it;
// + 4: the operands are cache-cold (what the engine derives from its ring size: the streaming profile's hints).
extern "C" int tbv_emu_run_sum_norm(int mode, void* out, const void* a, const void* b, void* normed, const void* weight, float eps,
                                    size_t rows, size_t hidden, int dtype, void* stream)
{
    const int cold = (mode & 4) ? 1 : 0;
    if (mode >= 0) mode &= 3;
    if (dtype < 0 || dtype > 2 || mode < 0 || mode > 1 || !row_norm_shape_ok(rows, hidden, dtype)) return -1;
    const size_t esz = dtype == 0 ? 4 : 2;
    SumArgs sa{};
    sa.out = out; sa.a = a; sa.b = b; sa.nbytes = rows * hidden * esz; sa.dtype = dtype;
    NormArgs nm{weight, normed, eps, (unsigned)(hidden * esz / 16), (unsigned)rows, cold};
    return launch_row_norm(mode, nullptr, sa, nm, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}

// int8 payload codec, standalone for benches and tests (the reference plans the codec, reports/12_references.md:134).
extern "C" size_t tbv_emu_codec_image_bytes(size_t nbytes, int dtype)
{
    return (dtype < 0 || dtype > 2) ? 0 : codec_image_bytes(nbytes, dtype);
}

extern "C" int tbv_emu_run_quant(void* image, const void* src, size_t nbytes, int dtype, void* stream)
{
    PackArgs pa{};
    pa.dst = image; pa.src = src; pa.nbytes = nbytes; pa.seq = 1;
    return launch_quant(pa, dtype, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}

extern "C" int tbv_emu_run_sum_quant(void* out, const void* own_image, const void* recv_image, size_t nbytes, int dtype, void* stream)
{
    SumArgs sa{};
    sa.out = out; sa.a = own_image; sa.b = recv_image; sa.nbytes = nbytes; sa.dtype = dtype;
    return launch_sum_quant(sa, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}

extern "C" int tbv_emu_run_pack(const void* src, size_t nbytes, int slot, void* stream)
{
    if (!G.inited || slot < 0 || slot >= G.nslot || nbytes > G.cap) return -1;
    PackArgs pa{};
    pa.dst = slot_send(slot); pa.src = src; pa.nbytes = nbytes;
    pa.cflag = word(W_MISC, 8 + slot % 16);          // a completion word nobody waits on
    pa.seq = 1; pa.arrive = pack_counters(slot); pa.sigmode = G.packsig;
    return launch_pack(pa, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}

extern "C" int tbv_emu_run_sum(void* out, const void* a, const void* b, size_t nbytes, int dtype, void* stream)
{
    if (dtype < 0 || dtype > 2) return -1;
    SumArgs sa{};
    sa.out = out; sa.a = a; sa.b = b; sa.nbytes = nbytes; sa.dtype = dtype;
    return launch_sum(sa, (hipStream_t)stream) == hipSuccess ? 0 : -1;
}
