// Two-process wire (tbv_sock.cpp): TCP rendezvous of the two ranks and a connection per rail that
// carries the fragments (replaces the bring-up and transfer of step4/libtbvcoll.cpp:343-403, :172-211
// for two processes that share one GPU).
#pragma once
#include "tbv_engine.h"

namespace tbv {

// Rank 0 listens on `port` and takes one connection per rail, rank 1 connects to peer_ip:port (retrying while
// rank 0 is not there yet); per rail the ranks swap and compare what they must agree on, then a one-byte barrier.
// Sockets only: needs tbv's configuration (configure()) but no GPU.  fds[r] = rail r's connection.  0 or -1.
int sock_rendezvous(int rank, const char* peer_ip, int port, int fds[MAXRAIL], double timeout_s);
// Rendezvous, pinned staging buffers, one receiver thread per rail.  0 or -1 (teardown() cleans up).
int sock_start(int rank, const char* peer_ip, int port);
void sock_stop();
// Send this rail's fragment of call `it`, wait for the peer's; *staged = where it sits (pinned host memory).
int sock_exchange(Rail& x, const Item& it, size_t off, size_t len, double t0, const char** staged);
// The staged fragment has been deposited: its buffer may take the slot's next call.
void sock_consumed(Rail& x, const Item& it);

}  // namespace tbv
