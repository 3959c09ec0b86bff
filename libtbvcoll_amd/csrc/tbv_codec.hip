// int8 payload codec of the all-reduce: the pack kernel quantises the local tensor into the
// bounce slot (what goes over the wire shrinks to 0.53 of a 2-byte payload), the sum kernel
// dequantises both ranks' images.
//
// The reference plans this as its next feature and has no code for it ("all-reduce payload
// quantisation, bf16 -> int8 blockwise, group 128, asymmetric", reports/12_references.md:134;
// it changes the numerics, so it must sit behind a size threshold, :140-142).  Format and
// arithmetic, all in IEEE fp32 so that a CPU restatement reproduces every byte:
//
//   group      128 consecutive elements; mn = min, mx = max of float(x) over the group
//   scale      (mx - mn) / 255, or 1 when mx == mn;  inv = 255 / (mx - mn), or 0 when mx == mn
//   code       q = rint((float(x) - mn) * inv) clamped to [0, 255], one byte (mn -> 0, mx -> 255)
//   decode     r = fma(float(q), scale, mn)
//   superblock 16 groups: 16 x (scale, mn) as two fp32 each = 128 bytes, then 16 x 128 code bytes
//              = 2176 bytes for 2048 elements; the image of n elements is ceil(n / 2048)
//              superblocks (absent elements: code 0, absent groups: scale 0, mn 0)
//   sum        out = T(decode(own image) + decode(received image)): each rank decodes its OWN
//              payload too, so both ranks of a pair compute the same bits
//
// One lane per pair of 16-byte input vectors (16 elements of a 2-byte type, 8 of fp32); the 8 (16) lanes
// of a group reduce min and max with xor shuffles; a block of 256 lanes takes two (one) superblocks per iteration.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "tbv_device.h"
#include "tbv_kernels.h"

namespace tbv {

namespace {

template <int DT> struct Vec;
template <> struct Vec<0> {
    static constexpr int EPV = 4;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float* f)
    {
        u32x4 r = {__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
        return r;
    }
};
template <> struct Vec<1> {
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        f16x8 h = __builtin_bit_cast(f16x8, v);
#pragma unroll
        for (int i = 0; i < 8; i++) f[i] = (float)h[i];
    }
    static __device__ __forceinline__ u32x4 pack(const float* f)
    {
        f16x8 h;
#pragma unroll
        for (int i = 0; i < 8; i++) h[i] = (_Float16)f[i];
        return __builtin_bit_cast(u32x4, h);
    }
};
template <> struct Vec<2> {
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) { f[2 * i] = __uint_as_float(u[i] << 16); f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u); }
    }
    static __device__ __forceinline__ u32x4 pack(const float* f)
    {
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x2 s = {f[2 * i], f[2 * i + 1]};
            bf16x2 r = __builtin_convertvector(s, bf16x2);
            o[i] = __builtin_bit_cast(uint32_t, r);
        }
        u32x4 r = {o[0], o[1], o[2], o[3]};
        return r;
    }
};

static constexpr unsigned kSbHeader = 128;      // 16 x (scale, mn)
static constexpr unsigned kCodecBlock = 256;    // lanes per block

// A lane owns two consecutive 16-byte input vectors (16 elements of a 2-byte type, 8 of fp32): the min/max of a
// group then needs three (four) shuffle steps per 16 (8) elements, and the codes of a 2-byte type leave as one
// 16-byte store.  A superblock takes 128 (fp32: 256) lanes, so a block of 256 lanes works on two (one) at a time.
template <int DT, int U>
__global__ __launch_bounds__(kCodecBlock) void k_quant(StepArgs g)
{
    constexpr int EPV = Vec<DT>::EPV, EPL = 2 * EPV;        // elements per vector, per lane
    constexpr unsigned LPS = kCodecSuper / EPL;             // lanes per superblock: 128 or 256
    constexpr unsigned LPG = kCodecGroup / EPL;             // lanes per group: 8 or 16
    constexpr unsigned SPB = kCodecBlock / LPS;             // superblocks per block and pass: 2 or 1
    const unsigned tid = threadIdx.x, lt = tid % LPS;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    const size_t nvec = g.nbytes >> 4;
    const size_t nsb = (nvec * EPV + kCodecSuper - 1) / kCodecSuper;
    const size_t stride = (size_t)gridDim.x * SPB;
    unsigned char* image = (unsigned char*)g.bounce;
    // U passes' loads go out together (measured: no gain, see the grid cap's comment)
    for (size_t sb0 = (size_t)blockIdx.x * SPB + tid / LPS; sb0 < nsb; sb0 += stride * U) {
        u32x4 v0[U], v1[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t sb = sb0 + (size_t)u * stride, i = sb * (kCodecSuper / EPV) + (size_t)lt * 2;
            const u32x4 zero = {0, 0, 0, 0};
            v0[u] = (sb < nsb && i < nvec) ? g.a[i] : zero;
            v1[u] = (sb < nsb && i + 1 < nvec) ? g.a[i + 1] : zero;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t sb = sb0 + (size_t)u * stride;
            if (sb >= nsb) break;                              // uniform over the wave: a wave lies within one superblock
            const size_t i = sb * (kCodecSuper / EPV) + (size_t)lt * 2;
            const bool have0 = i < nvec, have1 = i + 1 < nvec;
            float f[EPL];
            float mn = __builtin_inff(), mx = -__builtin_inff();
            Vec<DT>::unpack(v0[u], f);
            Vec<DT>::unpack(v1[u], f + EPV);
            if (have0) {
#pragma unroll
                for (int e = 0; e < EPV; e++) { mn = __builtin_fminf(mn, f[e]); mx = __builtin_fmaxf(mx, f[e]); }
            }
            if (have1) {
#pragma unroll
                for (int e = EPV; e < EPL; e++) { mn = __builtin_fminf(mn, f[e]); mx = __builtin_fmaxf(mx, f[e]); }
            }
#pragma unroll
            for (unsigned off = LPG / 2; off >= 1; off >>= 1) {
                mn = __builtin_fminf(mn, __shfl_xor(mn, off, 64));
                mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, 64));
            }
            const bool group_has = mn <= mx;                       // false when every lane of the group is past the end
            mn += 0.0f;                                            // a minimum of -0 is stored as +0, whichever zero the reduction met first
            const float range = mx - mn;
            const float scale = !group_has ? 0.0f : (range > 0.0f ? range / 255.0f : 1.0f);
            const float inv = (group_has && range > 0.0f) ? 255.0f / range : 0.0f;
            if (!group_has) mn = 0.0f;
            unsigned char* sbp = image + sb * kCodecSuperBytes;
            if ((lt % LPG) == 0) {
                f32x2 hdr = {scale, mn};
                *(f32x2*)(sbp + (lt / LPG) * 8) = hdr;
            }
            uint32_t c[EPL / 4];
#pragma unroll
            for (int k = 0; k < EPL / 4; k++) c[k] = 0;
#pragma unroll
            for (int e = 0; e < EPL; e++) {
                const bool have = e < EPV ? have0 : have1;
                float t = __builtin_rintf((f[e] - mn) * inv);
                t = __builtin_fminf(__builtin_fmaxf(t, 0.0f), 255.0f);
                const uint32_t q = have ? (uint32_t)t : 0u;
                c[e / 4] |= q << (8 * (e % 4));
            }
            unsigned char* cp = sbp + kSbHeader + (size_t)lt * EPL;
            if (EPL == 16) { u32x4 cv = {c[0], c[1], c[2 % (EPL / 4)], c[3 % (EPL / 4)]}; st_bounce<true>((u32x4*)cp, cv); }
            else { uint2 cv = {c[0], c[1]}; *(uint2*)cp = cv; }
        }
    }
    if (g.cflag) grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, gridDim.x, g.sigmode);
}

// What one lane needs of one superblock image to decode its vector: the group's header and its code bytes.
struct LaneCodes { f32x2 hdr; uint32_t lo, hi; };

template <int EPV>
__device__ __forceinline__ LaneCodes load_codes(const unsigned char* sbp, unsigned tid, unsigned lpg)
{
    LaneCodes c;
    c.hdr = *(const f32x2*)(sbp + (tid / lpg) * 8);
    c.hi = 0;
    if (EPV == 8) { const uint2 v = *(const uint2*)(sbp + kSbHeader + (size_t)tid * 8); c.lo = v.x; c.hi = v.y; }
    else c.lo = *(const uint32_t*)(sbp + kSbHeader + (size_t)tid * 4);
    return c;
}

template <int EPV>
__device__ __forceinline__ void decode_codes(const LaneCodes& c, float* r)
{
#pragma unroll
    for (int e = 0; e < EPV; e++) {
        const uint32_t q = ((e < 4 ? c.lo >> (8 * e) : c.hi >> (8 * (e - 4))) & 0xffu);
        r[e] = __builtin_fmaf((float)q, c.hdr.x, c.hdr.y);
    }
}

// out = T(decode(own image) + decode(received image)); g.a = own image, g.b = received image.  One output vector per
// lane, so every load and store of a wave is one contiguous run (a lane that owns two consecutive vectors would
// store with a 32-byte stride, which costs this kernel a quarter of its rate).  A block takes U superblocks per
// iteration and issues all their loads before the first store (measured: no gain, see the grid cap's comment).
template <int DT, int U>
__global__ __launch_bounds__(512) void k_sum_quant(StepArgs g)
{
    constexpr int EPV = Vec<DT>::EPV;
    constexpr unsigned LPG = kCodecGroup / EPV;
    const unsigned tid = threadIdx.x;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.wait_flag) gate_wait(g.wait_flag, g.seq, g.spin_limit, g.relay, g.fp, !g.b_uncached);
    const size_t nvec = g.nbytes >> 4;
    const size_t nsb = (nvec * EPV + kCodecSuper - 1) / kCodecSuper;
    const unsigned char* ia = (const unsigned char*)g.a;
    const unsigned char* ib = (const unsigned char*)g.b;
    for (size_t sb0 = (size_t)blockIdx.x * U; sb0 < nsb; sb0 += (size_t)gridDim.x * U) {
        LaneCodes ca[U], cb[U];
        bool have[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t sb = sb0 + u, i = sb * blockDim.x + tid;
            have[u] = sb < nsb && i < nvec;
            if (have[u]) {
                ca[u] = load_codes<EPV>(ia + sb * kCodecSuperBytes, tid, LPG);
                cb[u] = load_codes<EPV>(ib + sb * kCodecSuperBytes, tid, LPG);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (!have[u]) continue;
            float x[EPV], y[EPV];
            decode_codes<EPV>(ca[u], x);
            decode_codes<EPV>(cb[u], y);
#pragma unroll
            for (int e = 0; e < EPV; e++) x[e] = x[e] + y[e];
            st_result(g.out + (sb0 + u) * blockDim.x + tid, Vec<DT>::pack(x), g.out_through);
        }
    }
    if (g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

// The whole coded step in one kernel, for a call whose peer image is already in the receive slot: a lane loads its
// vector of the local tensor once, the lanes of a group agree on min and max, the lane stores its codes (and the
// group's leader the header) into the bounce slot, decodes them again from its registers (the same fma on the same
// numbers as a decode of the stored image), decodes the peer's codes of the same elements, adds and stores the
// output.  Bytes per payload byte of a 2-byte type: read 1, write 0.53, read 0.53, write 1 = 3.06 against 4.6 for
// the quantise kernel followed by the dequantising sum (which reads this rank's image back), and one launch instead
// of two.  One vector per lane (blockDim = vectors per superblock: 256, fp32 512), so every load and store of a wave
// is one contiguous run.  In place is fine: the lane that stores out[i] is the one that loaded a[i].
// min and max over the LPG (16 or 32) lanes of a group; every lane gets the result.  Within a row of 16 lanes by four
// rotations on the data-parallel path (no LDS traffic; rotating by 8, 4, 2, 1 and taking the minimum each time leaves
// every lane with the minimum of all 16, since min and max do not mind an element counted twice); the two rows of an
// fp32 group then swap through one xor shuffle.
template <unsigned LPG, bool DPP>
__device__ __forceinline__ void group_minmax(float& mn, float& mx)
{
    if (DPP) {
        // Written out, because the compiler turns each rotation into a move, a canonicalising max and the min (five
        // instructions a step with their wait states, against one here).  A lane-crossing read needs two wait states
        // after the write of the register it reads: the other chain's instruction and one s_nop provide them, and
        // the leading s_nop covers whatever wrote mn, mx or the exec mask just before.  Neither input can be a
        // signalling NaN (both come out of min/max instructions), so the missing canonicalisation changes nothing.
        asm("s_nop 4\n\t"
            "v_min_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
            "v_max_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0\n\t"
            "v_min_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
            "v_max_f32_dpp %1, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0\n\t"
            "v_min_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
            "v_max_f32_dpp %1, %1, %1 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 0\n\t"
            "v_min_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
            "v_max_f32_dpp %1, %1, %1 row_ror:1 row_mask:0xf bank_mask:0xf"
            : "+v"(mn), "+v"(mx));
        if (LPG == 32) {
            mn = __builtin_fminf(mn, __shfl_xor(mn, 16, 64));
            mx = __builtin_fmaxf(mx, __shfl_xor(mx, 16, 64));
        }
    } else {
#pragma unroll
        for (unsigned off = LPG / 2; off >= 1; off >>= 1) {
            mn = __builtin_fminf(mn, __shfl_xor(mn, off, 64));
            mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, 64));
        }
    }
}

// What a lane holds of one superblock between its loads and its work.
struct CodedIn { u32x4 v; LaneCodes cb; bool have; };

template <int DT>
__device__ __forceinline__ CodedIn coded_load(const StepArgs& g, size_t sb, size_t nsb, size_t nvec)
{
    constexpr int EPV = Vec<DT>::EPV;
    constexpr unsigned LPG = kCodecGroup / EPV;
    CodedIn in;
    const size_t i = sb * blockDim.x + threadIdx.x;
    in.have = sb < nsb && i < nvec;
    const u32x4 zero = {0, 0, 0, 0};
    in.v = in.have ? g.a[i] : zero;
    in.cb = LaneCodes{};
    if (in.have) in.cb = load_codes<EPV>((const unsigned char*)g.b + sb * kCodecSuperBytes, threadIdx.x, LPG);
    return in;
}

template <int DT, bool DPP>
__device__ __forceinline__ void coded_work(const StepArgs& g, size_t sb, const CodedIn& in)
{
    constexpr int EPV = Vec<DT>::EPV;
    constexpr unsigned LPG = kCodecGroup / EPV;             // lanes per group: 16, fp32 32
    const unsigned tid = threadIdx.x;
    float f[EPV];
    Vec<DT>::unpack(in.v, f);
    float mn = __builtin_inff(), mx = -__builtin_inff();
    if (in.have) {
#pragma unroll
        for (int e = 0; e < EPV; e++) { mn = __builtin_fminf(mn, f[e]); mx = __builtin_fmaxf(mx, f[e]); }
    }
    group_minmax<LPG, DPP>(mn, mx);
    const bool group_has = mn <= mx;                   // false when every lane of the group is past the end
    mn += 0.0f;                                        // a minimum of -0 is stored as +0
    const float range = mx - mn;
    const float scale = !group_has ? 0.0f : (range > 0.0f ? range / 255.0f : 1.0f);
    const float inv = (group_has && range > 0.0f) ? 255.0f / range : 0.0f;
    if (!group_has) mn = 0.0f;
    unsigned char* sbp = (unsigned char*)g.bounce + sb * kCodecSuperBytes;
    if ((tid % LPG) == 0) {
        f32x2 hdr = {scale, mn};
        *(f32x2*)(sbp + (tid / LPG) * 8) = hdr;
    }
    // rint first, so the conversion below meets whole numbers only (exact in any rounding mode); it saturates to
    // 0...255 and drops each code into its byte of the dword
    uint32_t c[2] = {0, 0};
#pragma unroll
    for (int e = 0; e < EPV; e++)
        c[e / 4] = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf((f[e] - mn) * inv), e % 4, c[e / 4]);
    if (!in.have) { c[0] = 0; c[1] = 0; }
    if (EPV == 8) { uint2 cv = {c[0], c[1]}; *(uint2*)(sbp + kSbHeader + (size_t)tid * 8) = cv; }
    else *(uint32_t*)(sbp + kSbHeader + (size_t)tid * 4) = c[0];
    if (in.have) {
        float x[EPV], y[EPV];
        LaneCodes own;
        own.hdr.x = scale; own.hdr.y = mn; own.lo = c[0]; own.hi = c[1];
        decode_codes<EPV>(own, x);                     // the decode of the image just made, from registers
        decode_codes<EPV>(in.cb, y);
#pragma unroll
        for (int e = 0; e < EPV; e++) x[e] = x[e] + y[e];
        st_result(g.out + sb * blockDim.x + tid, Vec<DT>::pack(x), g.out_through);
    }
}

// (Tried and dropped, 16 MiB bf16 cold, 12.55 us as it stood, 12.45 with the rotations written out: two superblocks'
// loads issued together 13.05; the next superblock's loads issued ahead of the work on the current one, with and without
// a branch around the loads, 13.7-14.1 (the compiler's waits at the head of such a loop still cover the stores issued
// before, whichever way the registers take turns); a branch-free copy of the work for superblocks in which every lane
// has a vector 13.9; one superblock per block in a stripped kernel with preloaded arguments 12.95 (10.95 against 11.7
// when the tensors are resident in the cache); the output stored without write-through 12.6; blocks that share a CU given
// different wave priorities or a staggered start 12.65-13.0.
// Taking the parts out one at a time says where the time goes: header stores 0.2 us, code stores 1.4, the peer's codes
// 1.2, decode + sum + output store 2.8, and 7.3 us remain for reading the local tensor and making the codes.)
template <int DT, bool DPP>
__global__ __launch_bounds__(512) void k_coded_step(StepArgs g)
{
    constexpr int EPV = Vec<DT>::EPV;
    const unsigned tid = threadIdx.x;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    const size_t nvec = g.nbytes >> 4;
    const size_t nsb = (nvec * EPV + kCodecSuper - 1) / kCodecSuper;
    for (size_t sb = blockIdx.x; sb < nsb; sb += gridDim.x) coded_work<DT, DPP>(g, sb, coded_load<DT>(g, sb, nsb, nvec));
    if (g.cflag) grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, gridDim.x, g.sigmode);
    if (g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

inline bool al16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

template <typename A>
hipError_t launch1(void (*kernel)(A), int grid, int block, hipStream_t st, const Timing* t, const A& arg)
{
    if (t && t->start && t->stop) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, t->start, t->stop, 0, arg);
    else hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, arg);
    return hipGetLastError();
}

// Measured with 16 MiB bf16, cache-cold (quantise / dequantising sum, us): 2048 blocks 7.3 / 8.1, 1024 blocks 7.1 / 7.9,
// 512 blocks 8.4 / 9.4; two or four passes' loads issued together (U = 2, 4): 7.5 / 8.4 and 7.9 / 9.0, so U stays 1.
int g_codec_grid_cap = 1024;
int g_coded_grid_cap = 1024;          // the one-launch coded step (measured: 768 blocks 12.9 us, 1024 and 1536 12.65, 2048 12.75, 4096 13.3)


// spb = superblocks one block takes per iteration
int codec_grid(size_t nbytes, int dtype, bool gated, size_t spb)
{
    const size_t epv = dtype == 0 ? 4 : 8, nsb = ((nbytes >> 4) * epv + kCodecSuper - 1) / kCodecSuper;
    const size_t want = (nsb + spb - 1) / spb;
    const size_t cap = gated ? 256 : (size_t)g_codec_grid_cap;
    return (int)(want < 1 ? 1 : want < cap ? want : cap);
}

}  // namespace

void set_codec_grid_cap(int cap)
{
    g_codec_grid_cap = cap >= 1 ? (cap > 8128 ? 8128 : cap) : 1024;
    g_coded_grid_cap = cap >= 1 ? (cap > 8128 ? 8128 : cap) : 1024;
}

size_t codec_image_bytes(size_t nbytes, int dtype)
{
    const size_t esz = dtype == 0 ? 4 : 2, n = nbytes / esz;
    return (n + kCodecSuper - 1) / kCodecSuper * kCodecSuperBytes;
}

// Quantise `a.src` (a.nbytes of `dtype`, whole 16-byte vectors) into the image at a.dst; completion signal as the pack's.
hipError_t launch_quant(const PackArgs& a, int dtype, hipStream_t st, const Timing* t)
{
    if (!a.dst || !a.src || (a.cflag && !a.arrive) || !al16(a.dst) || !al16(a.src) || (a.nbytes & 15) || dtype < 0 || dtype > 2 || a.tagp)
        return hipErrorInvalidValue;
    StepArgs s{};
    s.bounce = (u32x4*)a.dst; s.cflag = a.cflag; s.pack_arrive = a.arrive;
    s.a = (const u32x4*)a.src; s.nbytes = a.nbytes; s.seq = a.seq; s.fp = a.fp; s.sigmode = a.sigmode;
    s.pre_word = a.pre.word; s.pre_seq = a.pre.seq;
    const int grid = codec_grid(a.nbytes, dtype, false, dtype == 0 ? 1 : 2);
    switch (dtype) {
        case 0: return launch1(k_quant<0, 1>, grid, (int)kCodecBlock, st, t, s);
        case 1: return launch1(k_quant<1, 1>, grid, (int)kCodecBlock, st, t, s);
        default: return launch1(k_quant<2, 1>, grid, (int)kCodecBlock, st, t, s);
    }
}

// out = T(decode(q.a) + decode(q.b)) where q.a and q.b are images of q.nbytes of `dtype`.
hipError_t launch_sum_quant(const SumArgs& q, hipStream_t st, const Timing* t)
{
    if (!q.out || !q.a || !q.b || !al16(q.out) || !al16(q.a) || !al16(q.b) || (q.nbytes & 15) || q.dtype < 0 || q.dtype > 2 ||
        (q.done && !q.done_arrive))
        return hipErrorInvalidValue;
    StepArgs s{};
    s.out = (u32x4*)q.out; s.a = (const u32x4*)q.a; s.b = (const u32x4*)q.b; s.nbytes = q.nbytes; s.seq = q.seq; s.fp = q.fp;
    s.wait_flag = q.wait_flag; s.relay = q.relay; s.spin_limit = q.spin_limit_ticks; s.b_uncached = q.b_uncached;
    s.done = q.done; s.done_arrive = q.done_arrive;
    s.pre_word = q.pre.word; s.pre_seq = q.pre.seq;
    s.out_through = streaming_profile();
    const int grid = codec_grid(q.nbytes, q.dtype, q.wait_flag != nullptr, 1);
    switch (q.dtype) {
        case 0: return launch1(k_sum_quant<0, 1>, grid, 512, st, t, s);
        case 1: return launch1(k_sum_quant<1, 1>, grid, 256, st, t, s);
        default: return launch1(k_sum_quant<2, 1>, grid, 256, st, t, s);
    }
}

// The coded step in one launch (see k_coded_step): quantise p.src into the image at p.dst and write
// out = T(decode(that image) + decode(the received image q.b)).  No gate: for calls whose peer image is in place.
hipError_t launch_coded_step(const PackArgs& p, const SumArgs& q, hipStream_t st, const Timing* t)
{
    if (!p.dst || !p.src || !q.out || !q.b || p.src != q.a || p.nbytes != q.nbytes || (p.nbytes & 15) || p.tagp || q.wait_flag ||
        !al16(p.dst) || !al16(p.src) || !al16(q.out) || !al16(q.b) || q.dtype < 0 || q.dtype > 2 || (p.cflag && !p.arrive) ||
        (q.done && !q.done_arrive))
        return hipErrorInvalidValue;
    // an output that overlaps the local tensor without being it would be stored over vectors other lanes have yet to load
    const uintptr_t lo = (uintptr_t)p.src, oo = (uintptr_t)q.out;
    if (oo != lo && oo < lo + p.nbytes && lo < oo + p.nbytes) return hipErrorInvalidValue;
    StepArgs s{};
    s.bounce = (u32x4*)p.dst; s.cflag = p.cflag; s.pack_arrive = p.arrive; s.sigmode = p.sigmode;
    s.a = (const u32x4*)p.src; s.b = (const u32x4*)q.b; s.out = (u32x4*)q.out; s.nbytes = p.nbytes; s.seq = p.seq; s.fp = p.fp;
    s.done = q.done; s.done_arrive = q.done_arrive;
    s.pre_word = p.pre.word; s.pre_seq = p.pre.seq;
    s.out_through = streaming_profile();
    const size_t epv = q.dtype == 0 ? 4 : 8, nsb = ((p.nbytes >> 4) * epv + kCodecSuper - 1) / kCodecSuper;
    const size_t cap = (size_t)g_coded_grid_cap;
    const int grid = (int)(nsb < 1 ? 1 : nsb < cap ? nsb : cap);
    switch (q.dtype) {
        case 0: return launch1(k_coded_step<0, true>, grid, 512, st, t, s);
        case 1: return launch1(k_coded_step<1, true>, grid, 256, st, t, s);
        default: return launch1(k_coded_step<2, true>, grid, 256, st, t, s);
    }
}

}  // namespace tbv
