// Two processes on one GPU: the wire between the ranks is a TCP connection per rail.
//
// The reference brings its ranks together over TCP (rank 0 listens, rank 1 connects with
// retries, step4/libtbvcoll.cpp:371-379), swaps one 32-byte record per rail that tells the
// peer where to write (queue pair, key, address; :64, :380-385), ends with a one-byte
// barrier (:403) and from then on moves payloads with RDMA writes.  Here the same
// rendezvous swaps a 40-byte record per rail that holds what the two ranks must agree on
// (cap, slots, rails, the modes that change what travels), and the payloads travel over the
// rails' connections themselves: the rail's progress thread copies its fragment of the send
// slot to pinned host memory and writes it to the socket; a receiver thread per rail reads
// the peer's fragments into pinned staging buffers, one per ring slot; the progress thread
// then deposits the staged fragment into the receive slot the way the emulated peer does
// (copy + 64-bit arrival word).  Nothing here is fast and nothing needs to be: this is the
// wire, which the data path only meets through wire_xfer().  It exists so that two-rank
// drivers written against the reference (RANK=0/1 processes that never hand the library a
// peer payload) run unchanged on one GPU.
#include "tbv_sock.h"

#include <arpa/inet.h>
#include <errno.h>
#include <netdb.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <poll.h>
#include <sched.h>
#include <stdlib.h>
#include <string.h>
#include <sys/socket.h>
#include <unistd.h>

#include "tbv_dma.h"

namespace tbv {

namespace {

constexpr uint32_t kMagic = 0x54425643u;           // "TBVC"

// One per rail, both ways, before anything else travels (in the place of the reference's `exch`, step4/libtbvcoll.cpp:64).
struct __attribute__((packed)) Hello {
    uint32_t magic, rail;
    uint64_t cap;
    uint32_t nslot, rails, flags, rail1max_kib;
    uint32_t chunk_kib, rank;
};
static_assert(sizeof(Hello) == 40, "Hello layout");

// Ahead of every fragment.
struct __attribute__((packed)) FragHeader {
    uint32_t magic, rail;
    uint64_t seq, off, len, xbytes;
};

struct SockRail {
    int fd = -1;
    pthread_t rx_th{};
    bool rx_started = false;
    char* tx = nullptr;                            // pinned: this rail's outgoing fragment
    char* rx[MAXSLOT] = {};                        // pinned: the peer's fragment of the call in that ring slot
    std::atomic<uint64_t> rx_ready[MAXSLOT];       // sequence number whose fragment sits in rx[slot]
    std::atomic<uint64_t> rx_taken[MAXSLOT];       // sequence number whose fragment has been deposited: the buffer is free again
    uint64_t rx_off[MAXSLOT] = {}, rx_len[MAXSLOT] = {};
};

struct Sock {
    SockRail r[MAXRAIL];
    std::atomic<int> run{0};
    std::atomic<int> err{0};
    int listen_fd = -1;
    size_t buf_bytes = 0;
} S;

bool full_write(int fd, const void* p, size_t n, double deadline)
{
    const char* c = (const char*)p;
    while (n) {
        ssize_t k = send(fd, c, n, MSG_NOSIGNAL);
        if (k > 0) { c += k; n -= (size_t)k; continue; }
        if (k < 0 && (errno == EINTR)) continue;
        if (k < 0 && (errno == EAGAIN || errno == EWOULDBLOCK)) { if (nowt() > deadline) return false; continue; }
        return false;
    }
    return true;
}

// Reads exactly n bytes; returns 1, 0 when `keep_going` turned false or the deadline passed before the first byte, -1 on error / EOF.
int full_read(int fd, void* p, size_t n, double deadline, const std::atomic<int>* keep_going)
{
    char* c = (char*)p;
    size_t got = 0;
    while (got < n) {
        struct pollfd pf{fd, POLLIN, 0};
        const int pr = poll(&pf, 1, 100);
        if (pr < 0 && errno == EINTR) continue;
        if (pr < 0) return -1;
        if (pr == 0) {
            if (keep_going && !keep_going->load(std::memory_order_relaxed)) return 0;
            if (nowt() > deadline) return got ? -1 : 0;
            continue;
        }
        ssize_t k = recv(fd, c + got, n - got, 0);
        if (k > 0) { got += (size_t)k; continue; }
        if (k < 0 && (errno == EINTR || errno == EAGAIN)) continue;
        return -1;                                  // error, or the peer closed the connection
    }
    return 1;
}

void tune(int fd)
{
    int one = 1;
    (void)setsockopt(fd, IPPROTO_TCP, TCP_NODELAY, &one, sizeof one);
    int big = 8 << 20;
    (void)setsockopt(fd, SOL_SOCKET, SO_SNDBUF, &big, sizeof big);
    (void)setsockopt(fd, SOL_SOCKET, SO_RCVBUF, &big, sizeof big);
    struct timeval tv{0, 200000};                   // a blocked send wakes up to look at its deadline
    (void)setsockopt(fd, SOL_SOCKET, SO_SNDTIMEO, &tv, sizeof tv);
}

Hello my_hello(int rank, int rail)
{
    Hello h{};
    h.magic = kMagic; h.rail = (uint32_t)rail; h.cap = G.cap; h.nslot = (uint32_t)G.nslot; h.rails = (uint32_t)G.R;
    h.flags = (G.tag ? 1u : 0u) | (G.codec ? 2u : 0u) | ((uint32_t)(G.codec_min >> 10) << 8);
    h.rail1max_kib = (uint32_t)(G.rail1max >> 10);
    h.chunk_kib = (uint32_t)(G.chunkb >> 10);
    h.rank = (uint32_t)rank;
    return h;
}

bool hello_matches(const Hello& a, const Hello& b, int rail)
{
    if (b.magic != kMagic) { LOGF("rendezvous: rail%d: the peer does not speak this protocol", rail); return false; }
    if (b.rank == a.rank) { LOGF("rendezvous: both processes say they are rank %u", a.rank); return false; }
    if (a.cap != b.cap || a.nslot != b.nslot || a.rails != b.rails || a.flags != b.flags || a.rail1max_kib != b.rail1max_kib ||
        a.chunk_kib != b.chunk_kib) {
        LOGF("rendezvous: rail%d: the ranks disagree (cap %llu/%llu, slots %u/%u, rails %u/%u, tag+codec %#x/%#x, rail1max %u/%u KiB, chunk %u/%u KiB)",
             rail, (unsigned long long)a.cap, (unsigned long long)b.cap, a.nslot, b.nslot, a.rails, b.rails, a.flags, b.flags,
             a.rail1max_kib, b.rail1max_kib, a.chunk_kib, b.chunk_kib);
        return false;
    }
    return true;
}

void close_all(int* fds, int n)
{
    for (int i = 0; i < n; i++) if (fds[i] >= 0) { close(fds[i]); fds[i] = -1; }
    if (S.listen_fd >= 0) { close(S.listen_fd); S.listen_fd = -1; }
}

// The peer's fragments of this rail, one after the other, into the staging buffer of their ring slot.
void* rx_main(void* arg)
{
    SockRail& x = *(SockRail*)arg;
    const int rail = (int)(&x - S.r);
    const double forever = 1e300;
    while (S.run.load(std::memory_order_acquire)) {
        FragHeader h{};
        const int hr = full_read(x.fd, &h, sizeof h, forever, &S.run);
        if (hr == 0) continue;                      // stopping (the loop condition says so)
        if (hr < 0) { if (S.run.load()) { LOGF("rail%d: connection to the peer lost", rail); S.err.store(1); } break; }
        const int slot = (int)(h.seq % (uint64_t)G.nslot);
        if (h.magic != kMagic || (int)h.rail != rail || h.len > S.buf_bytes || h.seq == 0) {
            LOGF("rail%d: bad fragment header from the peer (seq %llu, %llu bytes)", rail, (unsigned long long)h.seq, (unsigned long long)h.len);
            S.err.store(1); break;
        }
        // the buffer is free once whatever this thread last put there has been deposited (not every call uses every rail,
        // so the slot's previous call need not be the buffer's previous user)
        const double t0 = nowt();
        while (S.run.load(std::memory_order_relaxed) &&
               x.rx_taken[slot].load(std::memory_order_acquire) < x.rx_ready[slot].load(std::memory_order_relaxed)) {
            if (nowt() - t0 > 1e-4) sched_yield();
        }
        if (!S.run.load()) break;
        if (full_read(x.fd, x.rx[slot], (size_t)h.len, forever, &S.run) != 1) {
            if (S.run.load()) { LOGF("rail%d: connection to the peer lost inside a fragment", rail); S.err.store(1); }
            break;
        }
        x.rx_off[slot] = h.off; x.rx_len[slot] = h.len;
        x.rx_ready[slot].store(h.seq, std::memory_order_release);
    }
    return nullptr;
}

}  // namespace

// ---- rendezvous: sockets only, no GPU --------------------------------------------------------

int sock_rendezvous(int rank, const char* peer_ip, int port, int fds[MAXRAIL], double timeout_s)
{
    const int R = G.R;
    for (int i = 0; i < MAXRAIL; i++) fds[i] = -1;
    const double deadline = nowt() + timeout_s;
    if (rank == 0) {
        // rank 0 listens (step4/libtbvcoll.cpp:371-375) and takes one connection per rail
        S.listen_fd = socket(AF_INET, SOCK_STREAM, 0);
        if (S.listen_fd < 0) FAIL("rendezvous: socket() failed: %s", strerror(errno));
        int one = 1;
        (void)setsockopt(S.listen_fd, SOL_SOCKET, SO_REUSEADDR, &one, sizeof one);
        struct sockaddr_in a{};
        a.sin_family = AF_INET; a.sin_port = htons((uint16_t)port);
        a.sin_addr.s_addr = htonl(INADDR_ANY);
        if (bind(S.listen_fd, (struct sockaddr*)&a, sizeof a) != 0 || listen(S.listen_fd, MAXRAIL) != 0) {
            LOGF("rendezvous: cannot listen on port %d: %s", port, strerror(errno));
            close_all(fds, MAXRAIL); return -1;
        }
        for (int k = 0; k < R; k++) {
            int fd = -1;
            while (fd < 0) {
                struct pollfd pf{S.listen_fd, POLLIN, 0};
                const int pr = poll(&pf, 1, 100);
                if (pr > 0) fd = accept(S.listen_fd, nullptr, nullptr);
                if (fd < 0 && nowt() > deadline) { LOGF("rendezvous: no peer connected within %.0f s", timeout_s); close_all(fds, MAXRAIL); return -1; }
            }
            tune(fd);
            Hello theirs{};
            if (full_read(fd, &theirs, sizeof theirs, deadline, nullptr) != 1 || theirs.rail >= (uint32_t)R || fds[theirs.rail] >= 0) {
                LOGF("rendezvous: bad greeting from the peer"); close(fd); close_all(fds, MAXRAIL); return -1;
            }
            const Hello mine = my_hello(rank, (int)theirs.rail);
            const bool sent = full_write(fd, &mine, sizeof mine, deadline);
            if (!sent || !hello_matches(mine, theirs, (int)theirs.rail)) { close(fd); close_all(fds, MAXRAIL); return -1; }
            fds[theirs.rail] = fd;
        }
        close(S.listen_fd); S.listen_fd = -1;
    } else {
        // rank 1 connects, retrying every 250 ms while rank 0 is not there yet (step4/libtbvcoll.cpp:376-379)
        if (!peer_ip || !*peer_ip) FAIL("rendezvous: rank %d needs the address of rank 0", rank);
        struct addrinfo hints{}, *res = nullptr;
        hints.ai_family = AF_INET; hints.ai_socktype = SOCK_STREAM;
        char ports[16]; snprintf(ports, sizeof ports, "%d", port);
        if (getaddrinfo(peer_ip, ports, &hints, &res) != 0 || !res) FAIL("rendezvous: cannot resolve %s", peer_ip);
        for (int k = 0; k < R; k++) {
            int fd = -1;
            for (;;) {
                fd = socket(AF_INET, SOCK_STREAM, 0);
                if (fd >= 0 && connect(fd, res->ai_addr, res->ai_addrlen) == 0) break;
                if (fd >= 0) close(fd);
                fd = -1;
                if (nowt() > deadline) { LOGF("rendezvous: rank 0 at %s:%d did not answer within %.0f s", peer_ip, port, timeout_s); freeaddrinfo(res); close_all(fds, MAXRAIL); return -1; }
                usleep(timeout_s < 2.0 ? 20000 : 250000);
            }
            tune(fd);
            const Hello mine = my_hello(rank, k);
            Hello theirs{};
            if (!full_write(fd, &mine, sizeof mine, deadline) || full_read(fd, &theirs, sizeof theirs, deadline, nullptr) != 1 ||
                !hello_matches(mine, theirs, k)) {
                if (theirs.magic == 0) LOGF("rendezvous: rank 0 closed rail%d's connection", k);
                close(fd); freeaddrinfo(res); close_all(fds, MAXRAIL); return -1;
            }
            fds[k] = fd;
        }
        freeaddrinfo(res);
    }
    // one byte each way on rail 0: both ranks are through (the reference's barrier, step4/libtbvcoll.cpp:403)
    char s = 'S', got = 0;
    if (!full_write(fds[0], &s, 1, deadline) || full_read(fds[0], &got, 1, deadline, nullptr) != 1 || got != 'S') {
        LOGF("rendezvous: barrier with the peer failed"); close_all(fds, MAXRAIL); return -1;
    }
    return 0;
}

// ---- the wire ------------------------------------------------------------------------------------

int sock_start(int rank, const char* peer_ip, int port)
{
    const char* e = getenv("TBV_RDV_TIMEOUT");
    const double timeout_s = (e && atof(e) > 0) ? atof(e) : 60.0;
    int fds[MAXRAIL];
    if (sock_rendezvous(rank, peer_ip, port, fds, timeout_s) != 0) return -1;
    S.buf_bytes = G.stride;
    S.err.store(0);
    for (int r = 0; r < G.R; r++) S.r[r].fd = fds[r];     // owned by sock_stop() from here on, whatever fails below
    for (int r = 0; r < G.R; r++) {
        SockRail& x = S.r[r];
        if (hipHostMalloc((void**)&x.tx, S.buf_bytes, hipHostMallocDefault) != hipSuccess) FAIL("two-process wire: pinned staging allocation failed");
        for (int s = 0; s < G.nslot; s++) {
            if (hipHostMalloc((void**)&x.rx[s], S.buf_bytes, hipHostMallocDefault) != hipSuccess) FAIL("two-process wire: pinned staging allocation failed");
            x.rx_ready[s].store(0); x.rx_taken[s].store(0);
        }
    }
    S.run.store(1);
    for (int r = 0; r < G.R; r++) {
        if (pthread_create(&S.r[r].rx_th, nullptr, rx_main, &S.r[r])) FAIL("two-process wire: pthread_create failed");
        S.r[r].rx_started = true;
    }
    LOGF("  two processes: rank%d %s, %d connection(s) to the peer on port %d, %zu KiB of pinned staging per rail", rank,
         rank == 0 ? "listened" : "connected", G.R, port, (S.buf_bytes * (size_t)(G.nslot + 1)) >> 10);
    return 0;
}

void sock_stop()
{
    S.run.store(0);
    for (int r = 0; r < MAXRAIL; r++) {
        SockRail& x = S.r[r];
        if (x.fd >= 0) (void)shutdown(x.fd, SHUT_RDWR);
        if (x.rx_started) { pthread_join(x.rx_th, nullptr); x.rx_started = false; }
        if (x.fd >= 0) { close(x.fd); x.fd = -1; }
        if (x.tx) { (void)hipHostFree(x.tx); x.tx = nullptr; }
        for (int s = 0; s < MAXSLOT; s++) if (x.rx[s]) { (void)hipHostFree(x.rx[s]); x.rx[s] = nullptr; }
    }
    if (S.listen_fd >= 0) { close(S.listen_fd); S.listen_fd = -1; }
}

// This rail's fragment [off, off+len) of call `it` goes to the peer; then the peer's fragment of the same call is
// awaited.  On success *staged points at it (pinned host memory, readable by the GPU).  Bounded by the watchdog.
int sock_exchange(Rail& x, const Item& it, size_t off, size_t len, double t0, const char** staged)
{
    SockRail& s = S.r[x.idx];
    if (s.fd < 0 || S.err.load()) { LOGF("rail%d: no connection to the peer", x.idx); return -1; }
    if (len > S.buf_bytes) { LOGF("rail%d: fragment of %zu bytes exceeds the staging buffers", x.idx, len); return -1; }
    const double deadline = t0 + G.wdog;
    // out of the send slot into pinned host memory: a copy-engine transfer when this caller's stream shares a hardware
    // queue with the rail's side stream, else a copy on that side stream
    if (it.host_wire) {
        const int rc = dma_copy(x.idx, s.tx, DMA_HOST, slot_send(it.slot) + off, DMA_DEVICE, len, G.wdog);
        if (rc != 0) { LOGF("rail%d: copy of the fragment to host memory failed seq=%llu", x.idx, (unsigned long long)it.seq); return -1; }
    } else if (hipMemcpyAsync(s.tx, slot_send(it.slot) + off, len, hipMemcpyDeviceToHost, x.wire) != hipSuccess ||
               hipStreamSynchronize(x.wire) != hipSuccess) {
        LOGF("rail%d: copy of the fragment to host memory failed seq=%llu", x.idx, (unsigned long long)it.seq); return -1;
    }
    FragHeader h{kMagic, (uint32_t)x.idx, it.seq, off, len, it.xbytes};
    if (!full_write(s.fd, &h, sizeof h, deadline) || !full_write(s.fd, s.tx, len, deadline)) {
        LOGF("%srail%d: sending to the peer failed seq=%llu", nowt() > deadline ? "watchdog: " : "", x.idx, (unsigned long long)it.seq); return -1;
    }
    while (s.rx_ready[it.slot].load(std::memory_order_acquire) < it.seq) {
        if (S.err.load()) return -1;
        if (nowt() > deadline) { LOGF("watchdog: rail%d: nothing from the peer for %.1fs seq=%llu", x.idx, G.wdog, (unsigned long long)it.seq); return -1; }
        if (!G.run.load(std::memory_order_relaxed) && G.async) return -1;
    }
    if (s.rx_ready[it.slot].load() != it.seq || s.rx_off[it.slot] != off || s.rx_len[it.slot] != len) {
        LOGF("rail%d: the peer's fragment does not match this rank's (seq %llu/%llu, offset %llu/%zu, %llu/%zu bytes): the ranks made different calls",
             x.idx, (unsigned long long)s.rx_ready[it.slot].load(), (unsigned long long)it.seq, (unsigned long long)s.rx_off[it.slot], off,
             (unsigned long long)s.rx_len[it.slot], len);
        return -1;
    }
    *staged = s.rx[it.slot];
    return 0;
}

void sock_consumed(Rail& x, const Item& it) { S.r[x.idx].rx_taken[it.slot].store(it.seq, std::memory_order_release); }

}  // namespace tbv
