// Internal interface between the host engine and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace tbv {

// Footprint words the kernels leave in host-visible memory (same four the
// reference keeps, step4/libtbvcoll.cpp:98): wait entered, wait passed, pack
// started, sum done.
enum Footprint { FP_WAIT_IN = 0, FP_WAIT_OUT = 1, FP_PACK = 2, FP_SUM_DONE = 3, FP_WAIT_TIMEOUT = 4 };

// A completion word some earlier kernel on the same stream left unsignalled: the
// next kernel stores `seq` to it as its first action (the earlier kernel is
// complete by then, so its stores are globally visible).
struct PreSignal { unsigned long long* word = nullptr; unsigned long long seq = 0; };

struct PackArgs {
    void* dst;                  // send slot (16-byte aligned)
    const void* src;            // caller tensor
    size_t nbytes;
    unsigned long long* cflag;  // host-visible completion word of the slot; null: do not signal (deferred to the next kernel)
    unsigned long long seq;
    unsigned int* arrive;       // the slot's counter lines (kCounterWords words), all return to 0
    unsigned long long* tagp;   // where to store seq after the payload, or null
    unsigned long long* fp;     // footprints or null
    int sigmode;                // how block stores are made visible before the block is counted (see grid_complete)
    PreSignal pre;
};

struct SumArgs {
    void* out;
    const void* a;              // caller tensor (may alias out)
    const void* b;              // received payload
    size_t nbytes;
    int dtype;                  // 0 f32, 1 f16, 2 bf16
    // optional in-kernel gate: block-leaders poll *wait_flag until >= seq
    const unsigned long long* wait_flag;
    unsigned long long* relay;  // device word: block 0 polls wait_flag and republishes it here for the other blocks
    bool b_uncached = false;    // `b` lies in uncached memory: passing the gate needs no cache invalidation
    unsigned long long seq;
    unsigned long long spin_limit_ticks;   // bound of the in-kernel wait, in ticks of the device's constant wall clock
    // optional completion word (latency probe / footprint): last block stores seq
    unsigned long long* done;
    unsigned int* done_arrive;  // counter lines (kCounterWords words), all return to 0
    unsigned long long* fp;
    PreSignal pre;
};

// Optional exact timing of one launch: the two events receive the start and end
// timestamps of that dispatch itself (hipExtLaunchKernel), not of the gaps around it.
struct Timing { hipEvent_t start = nullptr, stop = nullptr; };

// Words of device memory one grid-completion counter block needs (top line + group lines).
static constexpr size_t kCounterWords = 16 * 128;

// Launch geometry is exposed so the host can log and test it.
int pack_grid(size_t nbytes);
int sum_grid(size_t nbytes, int dtype);
// Tuning: vectors per lane per iteration (1,2,4,8; 0 = chosen by the profile), the grid cap and threads per
// block (0 = defaults), and the cache-hint profile (0 = operands stay cache resident, 1 = streaming from HBM).
// Every call sets all four.
void set_tuning(int unroll, int grid_cap, int block, int streaming);
bool streaming_profile();       // the cache-hint profile set_tuning was last given

hipError_t launch_pack(const PackArgs& a, hipStream_t st, const Timing* t = nullptr);
hipError_t launch_sum(const SumArgs& a, hipStream_t st, const Timing* t = nullptr);
// One kernel that does pack (with completion signal) and sum: legal only when the
// received payload is already in place.
hipError_t launch_pack_sum(const PackArgs& p, const SumArgs& s, hipStream_t st, const Timing* t = nullptr);
// Pack and sum in one launch as two sets of blocks (the pack blocks raise the completion word when they
// are done, the sum blocks read the local tensor themselves); same legality rule as launch_pack_sum, and
// the bounce must be uncached (sigmode 0).
hipError_t launch_pack_sum_merged(const PackArgs& p, const SumArgs& s, hipStream_t st, const Timing* t = nullptr);
// One launch of the chunked pipeline: pack `p` (a later chunk; uncached bounce, completion word raised by its own
// blocks) and sum `s` (an earlier chunk, optionally gated inside on s.wait_flag with s.relay) as two sets of blocks.
// p and s may belong to the same call (one launch for a call whose peer payload has not arrived yet); when s.out then
// overlaps p.src, `pack_relay` (a device word) must be given: the sum blocks wait for the pack blocks through it.
hipError_t launch_pipe(const PackArgs& p, const SumArgs& s, hipStream_t st, const Timing* t = nullptr,
                       unsigned long long* pack_relay = nullptr);
// Most blocks, and vectors per lane, of a grid (or the part of one) that waits for a flag inside the kernel.
void set_merge_segment(size_t bytes);     // largest payload of ONE merged launch; larger ones go out as several
void set_gated_tuning(int cap, int unroll);
// A whole small call (pack, signal, flag poll, sum) in one launch; at most kSmallCallMaxBlocks
// blocks of 1024 lanes, one 16-byte vector per lane.
static constexpr int kSmallCallMaxBlocks = 64;       // 1 MiB; 64 x 16 waves = an eighth of the GPU's wave slots
int small_call_blocks(size_t nbytes);
hipError_t launch_small_call(const PackArgs& p, const SumArgs& s, hipStream_t st, const Timing* t = nullptr);
hipError_t launch_waitflag(const unsigned long long* flag, unsigned long long seq,
                           unsigned long long spin_limit_ticks, unsigned long long* fp, hipStream_t st);
hipError_t launch_tagchk(const unsigned long long* tag, unsigned long long seq, unsigned long long* dbg,
                         hipStream_t st);
hipError_t launch_mark(unsigned long long* fp, int i, unsigned long long seq, hipStream_t st);
hipError_t launch_fill_u32(unsigned int* p, unsigned int v, size_t n, hipStream_t st);

// Row-wise RMSNorm fused with the sum (tbv_norm.hip).  A row is `row_vecs` 16-byte vectors; `weight` holds one row.
struct NormArgs {
    const void* weight;
    void* normed;
    float eps;
    unsigned row_vecs;
    unsigned rows;
    int cold = 0;               // host side only: the operands come from HBM, not from a cache (streaming profile)
};
static constexpr int kRowNormMaxVecs = 4096;          // 64 KiB per row: 1024 lanes x 4 vectors
static constexpr int kRowNormMaxSmallRows = 128;      // one-launch form: every block must be resident while it waits
bool row_norm_shape_ok(size_t rows, size_t hidden, int dtype);
void set_row_grid_cap(int cap);                       // most blocks of a row-kernel launch (0 = default)
// mode 0: normed = rmsnorm(s.a) * weight.   mode 1: out = a + b (s.wait_flag optional), normed = rmsnorm(out) * weight.
// mode 2: the whole small call in one launch (pack `p`, completion word, flag poll, sum, norm).
hipError_t launch_row_norm(int mode, const PackArgs* p, const SumArgs& s, const NormArgs& n, hipStream_t st, const Timing* t = nullptr);

// int8 payload codec (tbv_codec.hip): groups of 128 elements, 16 groups to a superblock of 2176 bytes.
static constexpr unsigned kCodecGroup = 128;
static constexpr unsigned kCodecSuper = 2048;          // elements per superblock
static constexpr unsigned kCodecSuperBytes = 2176;     // 16 x 8 header bytes + 2048 code bytes
size_t codec_image_bytes(size_t nbytes, int dtype);
void set_codec_grid_cap(int cap);                      // most blocks of a codec launch (0 = default)
hipError_t launch_quant(const PackArgs& a, int dtype, hipStream_t st, const Timing* t = nullptr);
hipError_t launch_sum_quant(const SumArgs& s, hipStream_t st, const Timing* t = nullptr);
// Quantise + dequantising sum of one call in a single launch (peer image already in place; p.src == q.a is the local tensor).
hipError_t launch_coded_step(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t = nullptr);

// Looks up this device's copy of the built-in counter array of tbv_step_noalloc (once per device).
bool noalloc_bind_device();

}  // namespace tbv
