/*
 * tbvcoll.h -- C ABI of libtbvcoll.so, the MI355X (gfx950) build of the 2-rank
 * tensor-parallel all-reduce data path.
 *
 * Part 1 is the drop-in boundary: the eleven symbols a caller of the reference
 * library binds through ctypes (step4/tbvcoll.py:19-30), with the same argument
 * meaning, return codes and threading rules.  Part 2 holds entry points the
 * reference does not have (a pipelined many-chunk call, the all-reduce fused with
 * the RMSNorm that follows it, a step that allocates nothing).  The emulated peer
 * that stands in for everything that crossed a wire in the reference, with its
 * test hooks and measurement aids, is declared apart, in tbvcoll_emu.h.
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

/* ------------------------------------------------------------------ Part 2: entry points the reference does not have */

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
 * Accuracy: the step of a group is (max - min) / 255, so ONE outlier stretches the step of all 128
 * elements around it; on activations with rare large outliers the error relative to the typical
 * element is large: about 16 % relative error on the non-outlier elements of a tensor drawn from
 * N(0, 0.02^2) with 0.1 % of its elements at +-8, against 0.6 % when there are no outliers (bench.py's
 * codec leg prints these figures).  tbvcoll_emu.h declares functions that run the codec kernels alone. */

/* One step of the data path with no allocation anywhere.  It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It needs no tbv_ar_init, but the
 * FIRST call on a device looks up the address of the library's built-in counter array, which
 * may make the runtime load code and set the array up: that call (or tbv_ar_init, which does
 * the same look-up) must happen on the device before any stream capture begins; a first call
 * made while `stream` is capturing is refused with -1.
 *   bounce <- local (nbytes), then *pack_word = seq once every byte of it is visible;
 *   out <- local + received in `dtype`, then *done_word = seq.
 * All five buffers are the caller's, 16-byte aligned device memory; out may be local itself
 * (in place: the step then runs as one fused kernel body; an output that overlaps local in
 * any other way gets pack and sum as two launches).
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

#ifdef __cplusplus
}
#endif
#endif /* TBVCOLL_H */
