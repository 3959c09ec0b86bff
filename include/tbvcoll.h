/*
 * tbvcoll.h -- C ABI of libtbvcoll.so, the MI355X (gfx950) build of the 2-rank
 * tensor-parallel all-reduce data path.
 *
 * Part 1 is the drop-in boundary: the eleven symbols a caller of the reference
 * library binds through ctypes (step4/tbvcoll.py:19-30), with the same argument
 * meaning, return codes and threading rules.  Part 2 is additive: the emulated
 * peer that stands in for everything that crossed a wire in the reference
 * (step4/libtbvcoll.cpp:172-224,343-403), and a pipelined many-chunk entry point.
 *
 * Plain C types only.  Device pointers are raw HIP device addresses; `stream` is a
 * raw hipStream_t.  The library never owns caller memory and touches caller
 * buffers only from kernels launched on the caller's stream.
 */
#ifndef TBVCOLL_H
#define TBVCOLL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ Part 1: drop-in boundary */

/* dtype codes of tbv_ar_allreduce (step4/libtbvcoll.cpp:416). */
#define TBV_DT_F32 0
#define TBV_DT_F16 1
#define TBV_DT_BF16 2

/*
 * Replaces tbv_ar_init (step4/libtbvcoll.cpp:279-414).
 * rank: 0 or 1 (label only here).  devs: comma list naming the rails; only the
 * count matters (1..4).  peer_ip/port: kept for signature parity, unused by the
 * emulated peer.  cap: largest payload in bytes, rounded up to 4096.
 * Reads TBV_ASYNC, TBV_GPUSIG, TBV_KWAIT, TBV_NSLOT, TBV_CHUNK, TBV_RAIL1MAX,
 * TBV_CPU, TBV_WDOG, TBV_TAG, TBV_UNCACHED (the reference's switches) and this
 * build's own tuning switches once.  Idempotent: a second call
 * returns 0 and changes nothing.  Returns 0, or -1 after a "[tbvcoll] ..." line
 * on stderr.
 */
int tbv_ar_init(int rank, const char* devs, const char* peer_ip, int port, size_t cap);

/*
 * Replaces tbv_ar_allreduce (step4/libtbvcoll.cpp:417-508).
 * out = ptr + peer, element-wise in `dtype`, for nbytes bytes; outp == NULL means
 * in place.  Asynchronous: the result is valid in `stream` order.  Returns 0;
 * -2 when nbytes exceeds the cap (caller falls back to its own collective);
 * -1 when not initialised, after any earlier transfer error (sticky), or on a
 * launch failure.  One caller thread at a time: a call that arrives while another
 * thread is inside the library is refused with -1.
 */
int tbv_ar_allreduce(void* ptr, void* outp, size_t nbytes, int dtype, void* stream);

/* Replace tbv_ar_stats / tbv_ar_stats4 / tbv_ar_stats5 (step4/libtbvcoll.cpp:510-536):
 * per-call averages in microseconds since the last read; any pointer may be NULL;
 * reading resets. */
void tbv_ar_stats(double* avg_us, unsigned long long* count);
void tbv_ar_stats4(double* pre_us, double* xfer_us, double* post_us, double* enq_us,
                   unsigned long long* count);
void tbv_ar_stats5(double* pre_us, double* xfer_us, double* post_us, double* enq_us,
                   double* drain_us, unsigned long long* count);

/* Replace tbv_ar_cap / tbv_ar_async / tbv_ar_err (step4/libtbvcoll.cpp:537-539). */
int tbv_ar_cap(void);
int tbv_ar_async(void);
int tbv_ar_err(void);

/* Replace tbv_ar_rails / tbv_ar_hist (step4/libtbvcoll.cpp:542-561): dump per-rail
 * and per-size transfer averages to stderr, then reset them. */
void tbv_ar_rails(void);
void tbv_ar_hist(void);

/* Replaces tbv_ar_fini (step4/libtbvcoll.cpp:562-566): stops and joins the
 * progress threads.  Frees nothing; the library stays initialised. */
void tbv_ar_fini(void);

/* ------------------------------------------------------------------ Part 2: emulated peer (additive)
 *
 * The reference's peer is a second machine reached through RDMA
 * write-with-immediate (step4/libtbvcoll.cpp:181-203).  Here the peer is played
 * on the same GPU: for every call, each rail's progress thread copies that
 * rail's fragment of the peer payload into the receive slot on a side stream and
 * then raises a 64-bit arrival word on that stream, which is the signal the
 * immediate's completion gave.  None of these symbols exist in the reference.
 * Like tbv_ar_allreduce they are to be called from the one caller thread.
 */

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

/* Pipelined all-reduce of a payload larger than the cap: split into cap-sized
 * chunks, each an ordinary call (own sequence number, slot and rail split), with
 * up to NSLOT-1 chunks packed ahead so that the sum of chunk i overlaps the
 * arrival of chunks i+1...  Queued peer payloads are consumed one per chunk.
 * Same return codes as tbv_ar_allreduce, except that no size is over the cap. */
int tbv_ar_allreduce_chunked(void* ptr, void* outp, size_t nbytes, int dtype, void* stream);

/* The all-reduce followed by the RMSNorm of its result in one pass over the hidden state.
 * The reference plans this fusion but does not have it (reports/12_references.md:136:
 * the all-reduce tail k_acc fused with the next RMSNorm); the arithmetic is that of the
 * fused add + RMSNorm of its caller (vLLM): with T the storage type,
 *   out    = ptr + peer                      (as tbv_ar_allreduce, bit for bit; outp NULL = in place)
 *   normed = T(float(out) * s) * weight      (product in T), s = 1 / sqrt(mean(float(out)^2 over a row) + eps)
 * for `rows` rows of `hidden` elements; `weight` holds `hidden` elements of T.  The sum of
 * squares is taken in fp32 in a fixed order, so results are reproducible.  A row must be a
 * multiple of 16 bytes and at most 64 KiB, and all buffers 16-byte aligned (-1 otherwise).
 * Return codes as tbv_ar_allreduce (-2: rows * hidden exceeds the cap). */
int tbv_ar_allreduce_rmsnorm(void* ptr, void* outp, void* normed, const void* weight, float eps,
                             size_t rows, size_t hidden, int dtype, void* stream);

/* int8 payload codec (TBV_CODEC=1, off by default; payloads of at least TBV_CODEC_MIN bytes,
 * default 512 KiB, made of whole 16-byte vectors).  The reference plans it as its next feature
 * and has no code for it (reports/12_references.md:134: bf16 -> int8 blockwise, group 128,
 * asymmetric; behind a size threshold since it changes the numerics, :140-142).  With the codec
 * on, tbv_ar_allreduce's pack kernel writes the int8 image of the local tensor into the bounce
 * slot (groups of 128 elements: scale = (max - min) / 255 and min as fp32, one code byte per
 * element; 2176 bytes per 2048 elements = 0.53 of a 2-byte payload on the wire) and its sum kernel
 * writes out = T(decode(own image) + decode(received image)): every rank decodes its own payload
 * too, so the two ranks of a pair compute the same bits.  |decode(x) - x| <= scale / 2 per
 * element.  An emulated peer's payload is quantised for it; with tbv_emu_peer_resident it must
 * have exactly the call's size.
 * The three functions below run the codec kernels alone, for benches and tests: the image size of
 * a payload, payload -> image, and two images -> sum. */
size_t tbv_emu_codec_image_bytes(size_t nbytes, int dtype);
int tbv_emu_run_quant(void* image, const void* src, size_t nbytes, int dtype, void* stream);
int tbv_emu_run_sum_quant(void* out, const void* own_image, const void* recv_image, size_t nbytes, int dtype, void* stream);

/* Standalone row kernel for benches and tests: mode 0: normed = rmsnorm(a) * weight;
 * mode 1: out = a + b, normed = rmsnorm(out) * weight. */
int tbv_emu_run_sum_norm(int mode, void* out, const void* a, const void* b, void* normed, const void* weight, float eps,
                         size_t rows, size_t hidden, int dtype, void* stream);

/* Standalone kernel entry points for benches and tests: run only the pack copy
 * (into send slot `slot`, with completion signal) or only the sum, on `stream`. */
int tbv_emu_run_pack(const void* src, size_t nbytes, int slot, void* stream);
int tbv_emu_run_sum(void* out, const void* a, const void* b, size_t nbytes, int dtype, void* stream);

/* One step of the data path with no allocation anywhere.  It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It needs no tbv_ar_init.
 *   bounce <- local (nbytes), then *pack_word = seq once every byte of it is visible;
 *   out <- local + received in `dtype`, then *done_word = seq.
 * All five buffers are the caller's, 16-byte aligned device memory; out may alias local.
 * bounce_uncached != 0 says that `bounce` is uncached (fine-grained) memory.  pack_word
 * and done_word are host-visible or device words, either may be NULL.  The kernels count
 * their blocks in a 16 KiB device array built into the library (one copy per GPU, held
 * until the process ends), so no hipMalloc, hipFree or other allocating call is made.
 * Calls that overlap in time on one GPU share that array and race: issue them on one
 * stream, or otherwise one after the other.  Returns 0; -2 when nbytes exceeds
 * TBV_NOALLOC_MAX_BYTES; -1 for bad arguments or a launch failure ("[tbvcoll] ..." on
 * stderr says which). */
#define TBV_NOALLOC_MAX_BYTES ((size_t)1 << 30)
int tbv_step_noalloc(void* out, const void* local, const void* received, void* bounce, int bounce_uncached,
                     size_t nbytes, int dtype, unsigned long long* pack_word, unsigned long long* done_word,
                     unsigned long long seq, void* stream);

/* What plain streaming kernels reach on this GPU, as measured denominators beside the
 * published HBM peak (no counterpart in the reference).  tbv_emu_hbm_probe streams
 * `bytes` per launch (kind 0 read, 1 write, 2 copy with non-temporal loads, 3 plain
 * copy) `reps` times through successive windows of a pool of `pool_bytes` that it
 * allocates and frees itself, and returns the mean and minimum launch duration in
 * microseconds.  tbv_emu_launch_floor returns the launch-to-launch time of an empty
 * kernel in one stream.  Both return 0, or -1 on bad arguments or a HIP error. */
int tbv_emu_hbm_probe(int kind, size_t bytes, size_t pool_bytes, int reps, double* mean_us, double* min_us);
int tbv_emu_launch_floor(int reps, double* us_per_launch);

#ifdef __cplusplus
}
#endif
#endif /* TBVCOLL_H */
