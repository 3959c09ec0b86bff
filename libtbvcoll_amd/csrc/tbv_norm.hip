// All-reduce tail fused with the RMSNorm that follows it: one pass over the hidden state
// writes both the reduced tensor (the residual stream) and its normalised form.
//
// The reference only plans this ("k_acc + next RMSNorm in one kernel: one launch and one
// hidden-state read/write less, 56 times per step", reports/12_references.md:136).  The
// arithmetic follows the fused add + RMSNorm of the reference's caller (vLLM's
// fused_add_rms_norm): z = local + received rounded to the storage type (exactly the sum
// kernel's result, step4/libtbvcoll.cpp:162-166), x = float(z), s = 1 / sqrt(mean(x^2) + eps),
// normed = T(x * s) * weight with the product taken in the storage type.
//
// One block per row at a time (L = 64..512 lanes; with more rows than blocks a block takes several rows in turn,
// keeps its part of the weight row in registers and loads the next row while it reduces the current one).  Lane t of L holds vectors t, t+L, ... of the row in registers, so the
// row is read once; the sum of squares is accumulated with fused multiply-adds in a fixed
// order (per lane: its vectors in order, elements in order; per wave: xor butterfly 32, 16,
// 8, 4, 2, 1; per block: the waves' totals in wave order), which makes the result
// reproducible and lets a CPU restatement match it bit for bit.  1/sqrt is the correctly
// rounded division of the correctly rounded square root.
//
// MODE 0: normalise `a` as it is (no sum; used after an all-reduce that ran unfused)
// MODE 1: z = a + b, write z to out, normalise z
// MODE 2: the whole small call in one launch: pack a into the bounce slot, count the blocks and
//         raise the pack's completion word, poll the flag, then as MODE 1 (grid small enough
//         for all blocks to be resident together, as for k_small_call)
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "tbv_device.h"
#include "tbv_kernels.h"

namespace tbv {

namespace {

template <int DT> struct Row;
// f32: 4 elements per vector
template <> struct Row<0> {
    static constexpr int EPV = 4;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    }
    static __device__ __forceinline__ u32x4 scale(u32x4 v, u32x4 w, float s)
    {
        float f[4], g[4]; unpack(v, f); unpack(w, g);
        u32x4 r;
        r.x = __float_as_uint((f[0] * s) * g[0]); r.y = __float_as_uint((f[1] * s) * g[1]);
        r.z = __float_as_uint((f[2] * s) * g[2]); r.w = __float_as_uint((f[3] * s) * g[3]);
        return r;
    }
};
// f16: 8 elements per vector; T(x*s) by round-to-nearest-even conversion, then the half multiply
template <> struct Row<1> {
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        f16x8 h = __builtin_bit_cast(f16x8, v);
#pragma unroll
        for (int i = 0; i < 8; i++) f[i] = (float)h[i];
    }
    static __device__ __forceinline__ u32x4 scale(u32x4 v, u32x4 w, float s)
    {
        f16x8 h = __builtin_bit_cast(f16x8, v), g = __builtin_bit_cast(f16x8, w), r;
#pragma unroll
        for (int i = 0; i < 8; i++) { _Float16 t = (_Float16)((float)h[i] * s); r[i] = t * g[i]; }
        return __builtin_bit_cast(u32x4, r);
    }
};
// bf16: 8 elements per vector; both roundings to nearest even from fp32
template <> struct Row<2> {
    static constexpr int EPV = 8;
    static __device__ __forceinline__ void unpack(u32x4 v, float* f)
    {
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) { f[2 * i] = __uint_as_float(u[i] << 16); f[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u); }
    }
    static __device__ __forceinline__ uint32_t bf16(float x)
    {
        __bf16 r = (__bf16)x;
        return (uint32_t)__builtin_bit_cast(uint16_t, r);
    }
    static __device__ __forceinline__ u32x4 scale(u32x4 v, u32x4 w, float s)
    {
        float f[8], g[8]; unpack(v, f); unpack(w, g);
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float t0 = __uint_as_float(bf16(f[2 * i] * s) << 16), t1 = __uint_as_float(bf16(f[2 * i + 1] * s) << 16);
            o[i] = bf16(t0 * g[2 * i]) | (bf16(t1 * g[2 * i + 1]) << 16);
        }
        u32x4 r = {o[0], o[1], o[2], o[3]};
        return r;
    }
};

// A row takes 512 lanes at most (4096 vectors at eight per lane), which leaves the compiler 256 registers per lane.
static constexpr int kRowMaxLanes = 512;

// Sum of squares of the block's row from the lanes' partial sums: wave butterfly, one LDS word per wave, the waves'
// totals added in wave order.  `slot` alternates between rows so that a fast wave's word for the next row cannot
// overwrite one a slow wave has yet to read (one barrier per row suffices).
__device__ __forceinline__ float row_total(float ssq, float (*wave_total)[kMaxSmallThreads / 64], int slot, unsigned tid, unsigned lanes)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
    if ((tid & 63) == 0) wave_total[slot][tid >> 6] = ssq;
    __syncthreads();
    float total = wave_total[slot][0];
    for (unsigned w = 1; w < (lanes >> 6); w++) total += wave_total[slot][w];
    return total;
}

// MODE 0 / MODE 1.  A block takes rows blockIdx.x, blockIdx.x + gridDim.x, ...  LOOP: the grid has fewer blocks than
// there are rows; the loads of the next row are then issued before the current row is reduced, so the reduction
// (shuffles, a barrier, a division and a square root) is covered by memory time.  (The second set of row registers
// costs occupancy, which is why the one-row form is a variant of its own.)  The weight row is read where it is used,
// after the reduction: it comes from the L2, and holding it in registers across rows, or asking for it at the start
// of the kernel (every block wants the same few lines then), measured slower: 2048 x 4096 bf16 cache-cold, 1024
// looping blocks, 12.58 us against 12.99 (weights first) and 13.27 (weights after the first row's loads); one block
// per row with the weights read after the reduction: 13.8 us.
// NT: the rows come from HBM and are read once (buffers beyond the caches): non-temporal loads of both operands.
// 2048 x 4096 bf16, 1024 looping blocks: cache-cold 13.9 -> 12.4 us; the same loads on rows that ARE resident in the
// Infinity Cache cost 2 us (8.9 -> 11.1), so the caller says which case it is (NormArgs::cold).
template <bool NT> __device__ __forceinline__ u32x4 ld_row(const u32x4* p) { return NT ? __builtin_nontemporal_load(p) : *p; }

template <int DT, int VPL, int MODE, bool LOOP, bool NT>
__global__ __launch_bounds__(kRowMaxLanes) void k_row_norm(StepArgs g, NormArgs nm)
{
    __shared__ float wave_total[2][kMaxSmallThreads / 64];
    const unsigned tid = threadIdx.x, lanes = blockDim.x, hv = nm.row_vecs;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    const u32x4 zero = {0, 0, 0, 0};
    u32x4 x[VPL], y[VPL];
    if (MODE == 1 && g.wait_flag) gate_wait(g.wait_flag, g.seq, g.spin_limit, g.relay, g.fp, !g.b_uncached);
    unsigned row = blockIdx.x;
    if (row < nm.rows) {
        const size_t r0 = (size_t)row * hv;
#pragma unroll
        for (int v = 0; v < VPL; v++) {
            const unsigned j = tid + (unsigned)v * lanes;
            x[v] = j < hv ? ld_row<NT>(g.a + r0 + j) : zero;
            if (MODE == 1) y[v] = j < hv ? ld_row<NT>(g.b + r0 + j) : zero;
        }
    }
    int slot = 0;
    for (; row < nm.rows; row += gridDim.x, slot ^= 1) {
        const size_t r0 = (size_t)row * hv;
        const unsigned nrow = row + gridDim.x;
        // (rows of more than two vectors per lane would spill with a second set of row registers: they load the
        // next row after the current one's stores instead)
        constexpr bool PRE = LOOP && VPL <= 2;
        u32x4 xn[PRE ? VPL : 1], yn[PRE ? VPL : 1];
        if (PRE && nrow < nm.rows) {                            // the next row's loads go out before this row's stores
            const size_t n0 = (size_t)nrow * hv;
#pragma unroll
            for (int v = 0; v < VPL; v++) {
                const unsigned j = tid + (unsigned)v * lanes;
                xn[PRE ? v : 0] = j < hv ? ld_row<NT>(g.a + n0 + j) : zero;
                if (MODE == 1) yn[PRE ? v : 0] = j < hv ? ld_row<NT>(g.b + n0 + j) : zero;
            }
        }
        if (MODE == 1) {
#pragma unroll
            for (int v = 0; v < VPL; v++) x[v] = add_vec<DT>(x[v], y[v]);   // lanes past the row: 0 + 0 = +0 in every type
        }
        float ssq = 0.0f;
#pragma unroll
        for (int v = 0; v < VPL; v++) {
            const unsigned j = tid + (unsigned)v * lanes;
            if (MODE == 1 && j < hv) __builtin_nontemporal_store(x[v], g.out + r0 + j);
            float f[Row<DT>::EPV];
            Row<DT>::unpack(x[v], f);                            // lanes past the row hold zeros: they add nothing
#pragma unroll
            for (int e = 0; e < Row<DT>::EPV; e++) ssq = __builtin_fmaf(f[e], f[e], ssq);
        }
        const float total = row_total(ssq, wave_total, slot, tid, lanes);
        const float s = 1.0f / __builtin_sqrtf(total / (float)((size_t)hv * Row<DT>::EPV) + nm.eps);
#pragma unroll
        for (int v = 0; v < VPL; v++) {
            const unsigned j = tid + (unsigned)v * lanes;
            if (j < hv) __builtin_nontemporal_store(Row<DT>::scale(x[v], ((const u32x4*)nm.weight)[j], s), (u32x4*)nm.normed + r0 + j);
        }
        if (!LOOP) break;
        if (nrow < nm.rows) {
            const size_t n0 = (size_t)nrow * hv;
#pragma unroll
            for (int v = 0; v < VPL; v++) {
                const unsigned j = tid + (unsigned)v * lanes;
                if (PRE) { x[v] = xn[PRE ? v : 0]; if (MODE == 1) y[v] = yn[PRE ? v : 0]; }
                else { x[v] = j < hv ? ld_row<NT>(g.a + n0 + j) : zero; if (MODE == 1) y[v] = j < hv ? ld_row<NT>(g.b + n0 + j) : zero; }
            }
        }
    }
    if (MODE == 1 && g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

// MODE 2: the whole small call in one launch, one block per row (all resident together): pack the row into the
// bounce slot, count the blocks and raise the pack's completion word, poll the flag, then sum and normalise.
template <int DT, int VPL>
__global__ __launch_bounds__(kMaxSmallThreads) void k_row_call(StepArgs g, NormArgs nm)
{
    __shared__ float wave_total[2][kMaxSmallThreads / 64];
    const unsigned tid = threadIdx.x, lanes = blockDim.x, hv = nm.row_vecs;
    const size_t row0 = (size_t)blockIdx.x * hv;
    if (g.pre_word && blockIdx.x == 0 && tid == 0) store_sys(g.pre_word, g.pre_seq);
    if (g.fp && blockIdx.x == 0 && tid == 0) store_sys(g.fp + FP_PACK, g.seq);
    const u32x4 zero = {0, 0, 0, 0};
    u32x4 x[VPL], w[VPL];
#pragma unroll
    for (int v = 0; v < VPL; v++) {
        const unsigned j = tid + (unsigned)v * lanes;
        x[v] = j < hv ? g.a[row0 + j] : zero;
        if (j < hv) g.bounce[row0 + j] = x[v];
    }
    grid_complete(g.cflag, g.seq, g.pack_arrive, blockIdx.x, gridDim.x, g.sigmode);
#pragma unroll
    for (int v = 0; v < VPL; v++) {                             // the weight row arrives while the flag is polled
        const unsigned j = tid + (unsigned)v * lanes;
        w[v] = j < hv ? ((const u32x4*)nm.weight)[j] : zero;
    }
    if (g.wait_flag) gate_wait(g.wait_flag, g.seq, g.spin_limit, g.relay, g.fp, !g.b_uncached);
    // all loads of the received row before the first store: `out` may alias anything, so a load placed after a
    // store waits for it
    u32x4 y[VPL];
#pragma unroll
    for (int v = 0; v < VPL; v++) {
        const unsigned j = tid + (unsigned)v * lanes;
        y[v] = j < hv ? g.b[row0 + j] : zero;
    }
#pragma unroll
    for (int v = 0; v < VPL; v++) x[v] = add_vec<DT>(x[v], y[v]);
    float ssq = 0.0f;
#pragma unroll
    for (int v = 0; v < VPL; v++) {
        const unsigned j = tid + (unsigned)v * lanes;
        if (j < hv) __builtin_nontemporal_store(x[v], g.out + row0 + j);
        float f[Row<DT>::EPV];
        Row<DT>::unpack(x[v], f);
#pragma unroll
        for (int e = 0; e < Row<DT>::EPV; e++) ssq = __builtin_fmaf(f[e], f[e], ssq);
    }
    const float total = row_total(ssq, wave_total, 0, tid, lanes);
    const float s = 1.0f / __builtin_sqrtf(total / (float)((size_t)hv * Row<DT>::EPV) + nm.eps);
#pragma unroll
    for (int v = 0; v < VPL; v++) {
        const unsigned j = tid + (unsigned)v * lanes;
        if (j < hv) __builtin_nontemporal_store(Row<DT>::scale(x[v], w[v], s), (u32x4*)nm.normed + row0 + j);
    }
    if (g.done) grid_complete(g.done, g.seq, g.done_arrive, blockIdx.x, gridDim.x, 1);
}

template <typename A, typename B>
hipError_t launch2(void (*kernel)(A, B), int grid, int block, hipStream_t st, const Timing* t, const A& a, const B& b)
{
    if (t && t->start && t->stop) hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, t->start, t->stop, 0, a, b);
    else hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, st, a, b);
    return hipGetLastError();
}

template <int DT, int MODE>
hipError_t launch_vpl(int vpl, int grid, int block, hipStream_t st, const Timing* t, const StepArgs& s, const NormArgs& n)
{
    if (MODE == 2) {
        switch (vpl) {
            case 1: return launch2(k_row_call<DT, 1>, grid, block, st, t, s, n);
            case 2: return launch2(k_row_call<DT, 2>, grid, block, st, t, s, n);
            case 4: return launch2(k_row_call<DT, 4>, grid, block, st, t, s, n);
            default: return launch2(k_row_call<DT, 8>, grid, block, st, t, s, n);
        }
    }
    constexpr int M = MODE == 2 ? 1 : MODE;
#define ROWK(V, L, N) launch2(k_row_norm<DT, V, M, L, N>, grid, block, st, t, s, n)
    if ((unsigned)grid < n.rows) {
        // the looping form is the one for payloads beyond the resident grid: the only one with a cache-cold variant
        if (n.cold) return vpl == 1 ? ROWK(1, true, true) : vpl == 2 ? ROWK(2, true, true) : vpl == 4 ? ROWK(4, true, true) : ROWK(8, true, true);
        return vpl == 1 ? ROWK(1, true, false) : vpl == 2 ? ROWK(2, true, false) : vpl == 4 ? ROWK(4, true, false) : ROWK(8, true, false);
    }
    return vpl == 1 ? ROWK(1, false, false) : vpl == 2 ? ROWK(2, false, false) : vpl == 4 ? ROWK(4, false, false) : ROWK(8, false, false);
#undef ROWK
}

template <int MODE>
hipError_t launch_dt(int dtype, int vpl, int grid, int block, hipStream_t st, const Timing* t, const StepArgs& s, const NormArgs& n)
{
    switch (dtype) {
        case 0: return launch_vpl<0, MODE>(vpl, grid, block, st, t, s, n);
        case 1: return launch_vpl<1, MODE>(vpl, grid, block, st, t, s, n);
        case 2: return launch_vpl<2, MODE>(vpl, grid, block, st, t, s, n);
    }
    return hipErrorInvalidValue;
}

inline bool al16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// Most blocks of a row-kernel launch: 0 = what is resident at once (see launch_row_norm), else a given number.
// Every block counted by grid_complete needs a place in the counter lines, which hold 8128 blocks.
int g_row_grid_cap = 0;
constexpr int kRowGatedWaves = 2048;    // a grid that waits for its flag inside holds at most a quarter of the GPU's 8192 wave slots

}  // namespace

void set_row_grid_cap(int cap) { g_row_grid_cap = cap >= 1 ? (cap > 8128 ? 8128 : cap) : 0; }

bool row_norm_shape_ok(size_t rows, size_t hidden, int dtype)
{
    const size_t esz = dtype == 0 ? 4 : 2, row_bytes = hidden * esz;
    return rows >= 1 && rows <= 0x7fffffffu && hidden >= 1 && (row_bytes & 15) == 0 && (row_bytes >> 4) <= (size_t)kRowNormMaxVecs;
}

hipError_t launch_row_norm(int mode, const PackArgs* p, const SumArgs& q, const NormArgs& nm, hipStream_t st, const Timing* t)
{
    if (mode < 0 || mode > 2 || q.dtype < 0 || q.dtype > 2 || !nm.weight || !nm.normed || !q.a) return hipErrorInvalidValue;
    const size_t esz = q.dtype == 0 ? 4 : 2;
    if (!nm.rows || !nm.row_vecs || nm.row_vecs > (unsigned)kRowNormMaxVecs || q.nbytes != (size_t)nm.rows * nm.row_vecs * 16) return hipErrorInvalidValue;
    if (!(al16(q.a) && al16(nm.weight) && al16(nm.normed))) return hipErrorInvalidValue;
    if (mode >= 1 && (!q.out || !q.b || !al16(q.out) || !al16(q.b) || (q.done && !q.done_arrive))) return hipErrorInvalidValue;
    if (mode == 2 && (!p || !p->dst || !al16(p->dst) || !p->cflag || !p->arrive || p->src != q.a || p->nbytes != q.nbytes ||
                      nm.rows > (unsigned)kRowNormMaxSmallRows)) return hipErrorInvalidValue;
    (void)esz;
    StepArgs s{};
    if (mode == 2) { s.bounce = (u32x4*)p->dst; s.cflag = p->cflag; s.pack_arrive = p->arrive; s.sigmode = p->sigmode; s.fp = p->fp;
                     s.pre_word = p->pre.word; s.pre_seq = p->pre.seq; }
    else { s.pre_word = q.pre.word; s.pre_seq = q.pre.seq; s.fp = q.fp; }
    s.out = (u32x4*)q.out; s.b = (const u32x4*)q.b; s.wait_flag = q.wait_flag; s.relay = q.relay; s.spin_limit = q.spin_limit_ticks;
    s.b_uncached = q.b_uncached;
    s.done = q.done; s.done_arrive = q.done_arrive;
    s.a = (const u32x4*)q.a; s.nbytes = q.nbytes; s.seq = q.seq;
    // Lanes per row: the fewest vectors per lane (1, 2, 4, 8) that bring a row down to 256 lanes, so that eight rows
    // fit a CU at once.  Measured with 2048 x 4096 bf16, cache-cold: 512 lanes x 1 vector 15.7 us, 256 x 2 14.0 us,
    // 128 x 4 13.6 us (but 128 decode rows 4.0 us instead of 3.6), 64 x 8 16.0 us.
    int vpl = 1;
    while (vpl < 8 && (nm.row_vecs + vpl - 1) / vpl > 256) vpl *= 2;
    int block = (int)(((nm.row_vecs + vpl - 1) / vpl + 63) / 64 * 64);
    if (block > kRowMaxLanes) return hipErrorInvalidValue;        // cannot happen for rows within kRowNormMaxVecs
    // One block per row up to the cap, beyond it the blocks loop over rows (and overlap one row's reduction with the
    // next row's loads), every block the same number of rows where that divides.  The cap is what is resident at once
    // at four waves per SIMD (the looping form's registers allow four to five): 4096 waves.  Measured with 2048 x 4096
    // bf16, cache-cold: 2048 blocks of one row 13.8 us, 1024 blocks of two rows 13.0, 768 13.4, 512 14.6.  A grid that
    // waits for its flag inside is kept to half of that; the one-launch call (mode 2) has one block per row by
    // construction (its row count is bounded).
    // (the norm-only form needs fewer registers: all 8192 wave slots hold a block of it)
    int cap = g_row_grid_cap > 0 ? g_row_grid_cap : (mode == 0 ? 8192 : 4096) / (block / 64);
    const int gated_cap = kRowGatedWaves / (block / 64);
    if (mode == 1 && q.wait_flag && cap > gated_cap) cap = gated_cap;
    if (cap < 1) cap = 1;
    const unsigned per_block = (nm.rows + (unsigned)cap - 1) / (unsigned)cap;
    const int grid = mode == 2 ? (int)nm.rows : (int)((nm.rows + per_block - 1) / per_block);
    switch (mode) {
        case 0: return launch_dt<0>(q.dtype, vpl, grid, block, st, t, s, nm);
        case 1: return launch_dt<1>(q.dtype, vpl, grid, block, st, t, s, nm);
        default: return launch_dt<2>(q.dtype, vpl, grid, block, st, t, s, nm);
    }
}

}  // namespace tbv
