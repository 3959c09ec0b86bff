/*
 * tbvcoll_emu.h -- the emulated peer of libtbvcoll.so's single-GPU build, its test hooks and its
 * measurement aids.  None of these symbols exist in the reference and none belong to the drop-in
 * boundary (tbvcoll.h): a transport that reaches a real second GPU replaces what they drive.
 *
 * The reference's peer is a second machine reached through RDMA write-with-immediate
 * (step4/libtbvcoll.cpp:181-203).  Here the peer is played on the same GPU: for every call, each
 * rail's progress thread copies that rail's fragment of the peer payload into the receive slot on a
 * side stream and then raises a 64-bit arrival word, which is the signal the immediate's completion
 * gave.  Like tbv_ar_allreduce these functions are to be called from the one caller thread.
 */
#ifndef TBVCOLL_EMU_H
#define TBVCOLL_EMU_H

#include "tbvcoll.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ the peer's payload and its arrival */
/* Queue the peer's payload for the next call that has none yet (FIFO, one entry per
 * call).  `src` holds at least the call's nbytes.  A device pointer is read when
 * the call's transfer runs and must stay valid until that call's result is
 * complete; host memory is copied to the device right here (the emulated wire
 * never reads host memory) and may be reused at once.  Calls
 * with no queued payload fall back to the repeat payload, then to mirror mode
 * (the peer sends back this rank's own bounce slot, so out = 2 * in). */
int tbv_emu_stage_peer(const void* src, size_t nbytes);

/* Payload used by every call with an empty queue; NULL restores mirror mode. */
int tbv_emu_stage_peer_repeat(const void* src, size_t nbytes);

/* The peer ran ahead: copy `src` (nbytes <= cap) into every receive slot now and
 * treat it as the already-arrived payload of each following call of at most
 * nbytes that has no queued payload: such a call finds its flag up on entry, so
 * its stream pays the pack, an already-satisfied wait and the sum.  Blocks until
 * the copies are done.  src == NULL ends the mode. */
int tbv_emu_peer_resident(const void* src, size_t nbytes);

/* Arrival order: `rails[k]` is the rail whose fragment arrives k-th from now on.
 * Each rail consumes its own occurrences in order and holds its signal until its
 * turn (bounded by the watchdog).  n == 0 clears the script (free-running). */
int tbv_emu_arrival_script(const int* rails, size_t n);

/* Fault injection from the host: the peer never signals rail `rail` of call `seq`
 * (seq counts calls from 1); with rail == -1 it is the pack kernel of call `seq`
 * that never raises its completion word.  The watchdog must then trip.
 * seq == 0 clears. */
int tbv_emu_withhold(unsigned long long seq, int rail);

/* Test hook: while `hold` is non-zero, rail `rail` deposits nothing; each held transfer is
 * bounded by the watchdog.  Setting a hold needs idle rails; lifting it may be done at
 * any time and from any thread (the one emulated-peer call that may be made while
 * another thread is inside tbv_ar_allreduce). */
int tbv_emu_hold_rail(int rail, int hold);

/* Sequence number of the last call issued (0 before the first). */
unsigned long long tbv_emu_seq(void);

/* Rail plan of a payload under the current settings: returns the rail count R and
 * fills off[r], len[r] for r < R (len 0 when a rail owns nothing).  Pure host
 * arithmetic; works without a GPU once TBV_* are read by tbv_emu_configure. */
int tbv_emu_plan(size_t nbytes, size_t* off, size_t* len);

/* Read the TBV_* environment and the rail count without touching the GPU, so the
 * host logic (tbv_emu_plan, slot/cap arithmetic) can be exercised on a CPU box. */
int tbv_emu_configure(const char* devs, size_t cap);

/* Slot geometry and addresses (device pointers) for tests and benches. */
int tbv_emu_nslot(void);
size_t tbv_emu_stride(void);
void* tbv_emu_send_slot(int slot);
void* tbv_emu_recv_slot(int slot);

/* Observed arrivals since the last read: fills up to `max` (seq, rail) pairs in
 * the order the arrival words were seen; returns the count. */
size_t tbv_emu_arrival_log(unsigned long long* seqs, int* rails, size_t max);

/* Release-to-done latency probe.  When on, the sum kernel stores the call's seq
 * to a host-visible word when its last block retires, and the progress thread
 * that releases the GPU records (time it saw that word) - (time just before it
 * raised the flag).  tbv_emu_latencies copies out up to `max` samples in
 * microseconds and clears them. */
int tbv_emu_latency_probe(int on);
size_t tbv_emu_latencies(double* us, size_t max);

/* Per-kernel timing: when on, every pack launch (which = 0) and every sum or
 * pack+sum launch (which = 1) is bracketed by two events on the caller's stream.
 * tbv_emu_kernel_times synchronises the device, returns the number of recorded
 * launches and their mean and minimum duration in microseconds, then forgets them. */
int tbv_emu_kernel_timing(int on);
size_t tbv_emu_kernel_times(int which, double* mean_us, double* min_us);
/* The recorded launches one by one: start and end of each, in microseconds after the start of the first
 * (up to `max`; the samples are kept).  Shows where a short burst of calls loses time between launches. */
size_t tbv_emu_kernel_timeline(int which, double* start_us, double* stop_us, size_t max);

/* GPU footprints (kept with TBV_KWAIT=1, as the reference's, step4/libtbvcoll.cpp:98):
 * sequence numbers of the last [wait entered, wait passed, pack started, sum done,
 * wait that ran into its bound]. */
void tbv_emu_footprints(unsigned long long out[5]);

/* Stale-data detector counters (TBV_TAG=1): checks, plain-load mismatches,
 * system-scope-load mismatches. */
void tbv_emu_tag_counts(unsigned long long* checks, unsigned long long* bad_plain,
                        unsigned long long* bad_system);

/* Full teardown so a process can re-initialise with other settings: joins threads,
 * destroys streams, releases buffers (the uncached bounce slab is kept for reuse,
 * never freed), clears the sticky error. */
void tbv_emu_shutdown(void);

/* ------------------------------------------------------------------ two processes on one GPU
 *
 * With TBV_PEER=tcp in the environment of both processes, tbv_ar_init(rank, devs, peer_ip, port, cap) meets a real
 * peer process instead of emulating one: rank 0 listens on `port`, rank 1 connects to peer_ip:port (retrying for up
 * to TBV_RDV_TIMEOUT seconds, default 60, while rank 0 is not there yet), per rail the ranks swap and compare what they
 * must agree on (cap, TBV_NSLOT, rail count, TBV_TAG, TBV_CODEC, TBV_RAIL1MAX, TBV_CHUNK; a mismatch fails both
 * inits), then one byte each way as a barrier: the shape of the reference's bring-up (step4/libtbvcoll.cpp:371-385,
 * :403).  Each rail's connection then carries that rail's fragments, through pinned host memory on both sides; the
 * receive side deposits them into the receive slot and raises the arrival word like the emulated peer.  A two-rank
 * driver written against the reference (RANK=0/1 processes that call init and all_reduce and nothing else) runs
 * unchanged.  The tbv_emu_stage_* / tbv_emu_peer_resident calls are refused in this mode.
 *
 * tbv_emu_rendezvous runs that rendezvous alone and closes the connections again (sockets only, no GPU; needs
 * tbv_emu_configure first).  Returns 0, or -1 after a "[tbvcoll] rendezvous: ..." line. */
int tbv_emu_rendezvous(int rank, const char* peer_ip, int port, double timeout_s);

/* ------------------------------------------------------------------ kernels run alone, for benches and tests */

/* The int8 codec's kernels: the image size of a payload, payload -> image, and two images -> sum. */
size_t tbv_emu_codec_image_bytes(size_t nbytes, int dtype);
int tbv_emu_run_quant(void* image, const void* src, size_t nbytes, int dtype, void* stream);
int tbv_emu_run_sum_quant(void* out, const void* own_image, const void* recv_image, size_t nbytes, int dtype, void* stream);

/* Standalone row kernel for benches and tests: mode 0: normed = rmsnorm(a) * weight;
 * mode 1: out = a + b, normed = rmsnorm(out) * weight.  mode + 4: the operands are cache-cold (buffers beyond
 * the caches, read once): the hints the engine takes in its streaming profile.  Same bits either way. */
int tbv_emu_run_sum_norm(int mode, void* out, const void* a, const void* b, void* normed, const void* weight, float eps,
                         size_t rows, size_t hidden, int dtype, void* stream);

/* Standalone kernel entry points for benches and tests: run only the pack copy
 * (into send slot `slot`, with completion signal) or only the sum, on `stream`. */
int tbv_emu_run_pack(const void* src, size_t nbytes, int slot, void* stream);
int tbv_emu_run_sum(void* out, const void* a, const void* b, size_t nbytes, int dtype, void* stream);

/* What plain streaming kernels reach on this GPU, as measured denominators beside the
 * published HBM peak (no counterpart in the reference).  tbv_emu_hbm_probe streams
 * `bytes` per launch (kind 0 read, 1 write, 2 copy with non-temporal loads, 3 plain
 * copy) `reps` times through successive windows of a pool of `pool_bytes` that it
 * allocates and frees itself, and returns the mean and minimum launch duration in
 * microseconds.  tbv_emu_launch_floor returns the launch-to-launch time of an empty
 * kernel in one stream.  Both return 0, or -1 on bad arguments or a HIP error. */
int tbv_emu_hbm_probe(int kind, size_t bytes, size_t pool_bytes, int reps, double* mean_us, double* min_us);
int tbv_emu_launch_floor(int reps, double* us_per_launch);

/* The floor under every form of the step: device time per launch, in microseconds, of a kernel that
 * only moves the step's four streams (reads `bytes` of local tensor and of received payload, writes
 * the uncached bounce and the bf16 sum; no block counting, no completion word, no gate), `reps`
 * launches back to back over 12 rotating local/output tensors and 16 rotating received/bounce
 * buffers that it allocates itself (the uncached ones are kept until the process ends).
 * bytes: whole tiles of 8 KiB, up to 64 MiB.  Returns 0, or -1. */
int tbv_emu_step_floor(size_t bytes, int reps, double* us_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* TBVCOLL_EMU_H */
