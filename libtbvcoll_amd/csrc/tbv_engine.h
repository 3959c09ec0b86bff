// Internal state and seams of the host engine, shared by
//   tbv_engine.cpp  ring, progress threads, enqueue halves, init/teardown
//                   (replaces step4/libtbvcoll.cpp:64-117, :226-342, :417-508)
//   tbv_peer.cpp    the emulated peer: everything that crossed a wire in the reference
//                   (step4/libtbvcoll.cpp:172-224, :343-403) behind one function, wire_xfer()
//   tbv_abi.cpp     the extern "C" surface (step4/libtbvcoll.cpp:279-566 as seen by step4/tbvcoll.py)
#pragma once
#include <hip/hip_runtime.h>

#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <time.h>

#include <atomic>
#include <deque>
#include <mutex>
#include <utility>
#include <vector>

#include "tbv_kernels.h"

namespace tbv {

constexpr int MAXRAIL = 4;
constexpr int MAXSLOT = 32;
constexpr double SPIN_US = 30.0;          // short spin before sleeping on a condition variable
constexpr size_t FLAG_STRIDE = 64;        // one cache line per host-visible word
constexpr size_t LOG_MAX = 1u << 20;

inline double nowt()
{
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + (double)t.tv_nsec * 1e-9;
}

#define LOGF(...) do { fprintf(stderr, "[tbvcoll] " __VA_ARGS__); fputc('\n', stderr); } while (0)
#define FAIL(...) do { LOGF(__VA_ARGS__); return -1; } while (0)

// One call's work for one rail's progress thread.
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
    std::atomic<int> napping{0};              // the progress thread is (about to be) asleep on cv_item
    double gap_us = 0;                        // recent idle gaps between items, smoothed (progress thread only)
    pthread_t th{};
    bool started = false;
    hipStream_t wire = nullptr;               // side stream that plays the peer's writes
    size_t script_pos = 0;                    // next position to look at in the arrival script
    // per-rail transfer statistics (guarded by Engine::smx)
    double rl_post = 0, rl_arr = 0;
    uint64_t rl_n = 0;
};

struct Staged { const char* ptr; size_t nbytes; bool owned; };

// What enqueue_pack decides about a call and enqueue_wait_sum needs to know.
struct Call {
    uint64_t seq; int slot; int R; size_t nbytes, xbytes; bool resident; bool fused; bool deferred; bool host_wire;
    bool codec;               // the payload travels as its int8 image (decided by enqueue_pack)
    bool out_unaligned;       // set by the caller before enqueue_pack when the output is not 16-byte aligned
    bool held;                // enqueue_pack handed the pack's arguments back instead of launching it
};

struct Engine {
    // configuration
    int configured = 0, inited = 0, rank = 0, R = 0, async = 1, nslot = 8, gpusig = 1, kwait = 0;
    int uncached = 1, tag = 0, cpu = -1, wr_hwm = 8, device = 0, railsum = 0, fuse = 0, packsig = 0;
    int merge = 1;                            // resident peer: pack and sum blocks in one launch (TBV_MERGE)
    size_t merge_max = (size_t)256 << 20;     // TBV_MERGEMAX: largest payload of one merged or staged launch (larger early-peer calls: one merged launch per segment)
    int peer_tcp = 0;                         // TBV_PEER=tcp: the peer is a second process on this GPU, reached over TCP (tbv_sock.cpp)
    int force_gate = 0;                       // measurement aid: early-peer large calls take the gated one-launch form (TBV_FORCEGATE)
    int staged_merge = 1;                     // peer not there yet: pack blocks + gated sum blocks in one launch (TBV_STAGEDMERGE)
    int streaming = 0;                        // cache-hint profile of the large kernels (TBV_STREAMING, default by ring size)
    int codec = 0;                            // int8 payload codec for payloads of at least codec_min bytes (TBV_CODEC, off by default)
    size_t codec_min = (size_t)512 << 10;     // TBV_CODEC_MIN
    size_t cap = 0, stride = 0, rail1max = 96u * 1024u, chunkb = 0, fusewait_max = 0;
    double wdog = 10.0;
    double spin_us = SPIN_US;                 // how long a progress thread spins on an empty queue before it sleeps (TBV_SPIN)
    double spin_max_us = 1000.0;              // while calls keep coming at gaps of up to half of this, the threads spin through the gaps (TBV_SPINMAX; 0 = never)
    double tick_hz = 1e8;                     // rate of the constant clock the kernels bound their waits with
    int can_wait_value = 1, can_write_value = 1;
    // memory
    char* sendbase = nullptr;
    char* recvbase = nullptr;
    char* hostwords = nullptr;                // one coherent host block holding every flag word
    unsigned int* counters = nullptr;         // device: per slot a counter block for the pack and one for the sum, the relay words,
                                              // and a counter block per (rail, slot) for the emulated peer's deposit kernel
    hipEvent_t ev[MAXSLOT] = {};
    // protocol state
    Rail rr[MAXRAIL];
    uint64_t seq = 0;
    std::atomic<unsigned> rails_done[MAXSLOT];
    std::atomic<uint64_t> released[MAXSLOT];  // last call of each slot whose GPU flag has been raised
    std::atomic<int> run{0};
    std::atomic<int> err{0};
    pthread_mutex_t mx = PTHREAD_MUTEX_INITIALIZER;
    pthread_cond_t cv_item = PTHREAD_COND_INITIALIZER;    // caller -> progress: new item
    pthread_cond_t cv_room = PTHREAD_COND_INITIALIZER;    // progress -> caller: room in the ring
    std::atomic<int> caller_napping{0};                   // the caller is (about to be) asleep on cv_room
    std::atomic<int> in_call{0};                          // a thread is inside one of the all-reduce entry points
    void* last_stream = nullptr;
    hipEvent_t switch_ev = nullptr;           // orders a new caller stream behind the previous one
    uint64_t n_stream_sw = 0;
    void* seen_streams[16] = {};
    int nseen = 0;
    // emulated peer (tbv_peer.cpp)
    std::deque<Staged> staged;
    Staged repeat{nullptr, 0, false};
    // device copies of payloads that were staged from host memory: (buffer, last call that reads it; 0 = not yet assigned)
    std::vector<std::pair<char*, uint64_t>> owned;
    size_t resident_bytes = 0;
    char* resident_src = nullptr;             // device copy of the resident payload, to restore a slot another payload went through
    bool resident_ok[MAXSLOT] = {};           // the receive slot still holds the resident payload
    int resident_form = -1;                   // what the receive slots hold of it: -1 the raw bytes, else the int8 image for this dtype
    hipStream_t util = nullptr;               // caller-thread stream for the emulated peer's own preparation work
    int hooks = 0;                            // an arrival script or a withheld signal is set (test hooks, off the default path)
    std::vector<int> script;
    std::atomic<size_t> turn{0};
    std::atomic<int> hold[MAXRAIL];           // test hook: a rail's deposits wait while its entry is set
    std::atomic<uint64_t> withhold_seq{0};
    std::atomic<int> withhold_rail{0};
    std::mutex logmx;
    std::vector<std::pair<uint64_t, int>> arrivals;
    std::atomic<int> probe{0};
    std::vector<double> latencies;
    int wire_mode = 0;                        // TBV_WIRE: 0 auto (probe each new caller stream), 1 stream, 2 host
    void* wire_stream = nullptr;              // the caller stream of the verdict below (the usual case: one stream)
    bool wire_stream_host = false;
    std::vector<std::pair<void*, bool>> stream_wire;   // every probed caller stream -> use the host wire
    // a pack's completion word that its kernel did not raise: the next kernel on the same stream raises it
    PreSignal pending;
    hipStream_t pending_stream = nullptr;
    int defer = 1;                            // allow deferring (TBV_DEFERSIG)
    int onekernel = 1;                        // small calls as one launch: pack, signal, flag poll, sum (TBV_ONEKERNEL)
    // optional per-kernel timing with events on the caller's stream: [0]=pack, [1]=sum
    int ktime = 0;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> kev[2];
    size_t kev_used[2] = {0, 0};
    // statistics.  The caller thread alone writes and reads the first row (one caller thread at a time is the
    // library's rule), so it needs no lock; the progress threads write the rest under smx.
    double t_pre = 0, t_post = 0, t_enq = 0, t_drain = 0;
    std::mutex smx;
    double t_acc = 0;
    uint64_t n_acc = 0;
    double hb_t[32] = {};
    uint64_t hb_n[32] = {}, hb_r[32] = {};
};

extern Engine G;

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

inline unsigned int* pack_counters(int s) { return G.counters + (size_t)s * kCounterWords; }
inline unsigned int* done_counters(int s) { return G.counters + (size_t)(MAXSLOT + s) * kCounterWords; }
inline unsigned int* wire_counters(int rail, int s) { return G.counters + ((size_t)2 * MAXSLOT + 1 + (size_t)rail * MAXSLOT + s) * kCounterWords; }
inline unsigned long long* relay_word(int s) { return (unsigned long long*)(G.counters + (size_t)2 * MAXSLOT * kCounterWords) + (size_t)s * 8; }
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
    *len = chunk < xbytes - roff ? chunk : xbytes - roff;
    return true;
}
inline int rails_for(size_t nbytes) { return nbytes <= G.rail1max ? 1 : G.R; }

// ---- tbv_engine.cpp -------------------------------------------------------------------
int configure(const char* devs, size_t cap);
int init_impl(int rank, const char* devs, const char* peer_ip, int port, size_t cap);
void teardown();
void stop_progress();
int enqueue_pack(const void* ptr, void* sum_out, size_t nbytes, int dtype, hipStream_t st, Call* c, const NormArgs* nm = nullptr,
                 PackArgs* hold = nullptr);
int enqueue_wait_sum(const void* ptr, void* outp, int dtype, hipStream_t st, const Call& c, const NormArgs* nm = nullptr,
                     const PackArgs* with_pack = nullptr);
int flush_pending();
void note_stream(void* stream, size_t nbytes);
bool rails_idle();
int drain_rails();

// ---- tbv_peer.cpp: the only code that knows the peer is emulated ----------------------
// The transfer of one rail's fragment of one call and the wait for the peer's fragment
// (replaces do_xfer_rail, step4/libtbvcoll.cpp:172-211).  Returns 0, or -1 on error / watchdog.
int wire_xfer(Rail& x, const Item& it);
// Its two non-blocking halves (stream wire only, no test hooks), for a progress thread that keeps several
// transfers in flight, and the bookkeeping of a completed one (t0 = post started, tp = post returned).
int wire_post(Rail& x, const Item& it, bool* owns);
bool wire_arrived(const Rail& x, const Item& it);
void wire_done(Rail& x, const Item& it, double t0, double tp);
// Whose payload plays the peer for call `c` of `nbytes`: sets *peer (null = mirror) and c->resident.
int peer_assign(Call* c, size_t nbytes, int dtype, const char** peer);
// Must this caller stream's calls be deposited by copy engines rather than a side stream?
bool use_host_wire(hipStream_t st);
hipError_t stream_bump(hipStream_t st, unsigned long long* w, uint64_t v);
void peer_teardown();

}  // namespace tbv
