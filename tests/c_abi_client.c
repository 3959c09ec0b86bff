/*
 * A plain C caller of the library: includes include/tbvcoll.h (through tbvcoll_emu.h) as C, links
 * libtbvcoll.so, and runs one all-reduce of each dtype code against a host
 * computed sum.  Built by tests/test_c_client.py (compile + link without a
 * GPU; run on the GPU box).  Inputs are small integers, so the sums are exact
 * in every dtype and the expected bits can be written down directly.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <stdint.h>

#include <hip/hip_runtime_api.h>

#include "tbvcoll_emu.h"      /* the emulated peer (includes tbvcoll.h, the boundary) */

#define CHECK(x) do { if ((x) != hipSuccess) { fprintf(stderr, "HIP call failed at line %d\n", __LINE__); return 2; } } while (0)

/* value v (|v| <= 256, integer) as fp32 / fp16 / bf16 bit patterns */
static uint32_t f32_bits(float v) { uint32_t u; memcpy(&u, &v, 4); return u; }
static uint16_t bf16_bits(float v) { return (uint16_t)(f32_bits(v) >> 16); }        /* exact: small integers fit 8 bits */
static uint16_t f16_bits(float v)
{
    uint32_t u = f32_bits(v), sign = (u >> 16) & 0x8000u;
    if ((u & 0x7fffffffu) == 0) return (uint16_t)sign;
    int e = (int)((u >> 23) & 0xff) - 127 + 15;
    return (uint16_t)(sign | ((uint32_t)e << 10) | ((u >> 13) & 0x3ffu));             /* exact for small integers */
}

static int run(int dtype, size_t n, void* stream)
{
    const size_t esz = dtype == TBV_DT_F32 ? 4 : 2, nbytes = n * esz;
    unsigned char *ha = malloc(nbytes), *hb = malloc(nbytes), *ho = malloc(nbytes), *hw = malloc(nbytes);
    for (size_t i = 0; i < n; i++) {
        float a = (float)((int)(i % 97) - 48), b = (float)((int)(i % 61) - 30), s = a + b;
        if (dtype == TBV_DT_F32) { uint32_t x = f32_bits(a), y = f32_bits(b), z = f32_bits(s);
            memcpy(ha + 4 * i, &x, 4); memcpy(hb + 4 * i, &y, 4); memcpy(hw + 4 * i, &z, 4); }
        else { uint16_t x = dtype == TBV_DT_F16 ? f16_bits(a) : bf16_bits(a), y = dtype == TBV_DT_F16 ? f16_bits(b) : bf16_bits(b),
                        z = dtype == TBV_DT_F16 ? f16_bits(s) : bf16_bits(s);
            if (s == 0.0f) z = 0;                                                       /* x + (-x) = +0 */
            memcpy(ha + 2 * i, &x, 2); memcpy(hb + 2 * i, &y, 2); memcpy(hw + 2 * i, &z, 2); }
    }
    void *da, *db, *dout;
    CHECK(hipMalloc(&da, nbytes)); CHECK(hipMalloc(&db, nbytes)); CHECK(hipMalloc(&dout, nbytes));
    CHECK(hipMemcpy(da, ha, nbytes, hipMemcpyHostToDevice)); CHECK(hipMemcpy(db, hb, nbytes, hipMemcpyHostToDevice));
    if (tbv_emu_stage_peer(db, nbytes) != 0) return 3;
    int rc = tbv_ar_allreduce(da, dout, nbytes, dtype, stream);
    if (rc != 0) { fprintf(stderr, "tbv_ar_allreduce rc=%d\n", rc); return 4; }
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(ho, dout, nbytes, hipMemcpyDeviceToHost));
    int bad = memcmp(ho, hw, nbytes) != 0;
    if (tbv_emu_stage_peer(db, nbytes) != 0) return 3;                                 /* in place */
    if (tbv_ar_allreduce(da, NULL, nbytes, dtype, stream) != 0) return 4;
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(ho, da, nbytes, hipMemcpyDeviceToHost));
    bad |= memcmp(ho, hw, nbytes) != 0;
    CHECK(hipFree(da)); CHECK(hipFree(db)); CHECK(hipFree(dout));
    free(ha); free(hb); free(ho); free(hw);
    printf("dtype %d n %zu: %s\n", dtype, n, bad ? "MISMATCH" : "exact");
    return bad;
}

int main(void)
{
    if (tbv_ar_cap() != 0) return 10;                                   /* nothing initialised yet */
    if (tbv_ar_allreduce(NULL, NULL, 16, 0, NULL) != -1) return 11;    /* not initialised */
    if (tbv_ar_init(0, "rail0,rail1", "", 18995, (size_t)1 << 20) != 0) return 12;
    if (tbv_ar_init(1, "x", "", 1, 4096) != 0 || tbv_ar_cap() != (1 << 20)) return 13;   /* idempotent */
    if (tbv_ar_async() != 1 || tbv_ar_err() != 0) return 14;
    hipStream_t st;
    CHECK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    int bad = 0;
    bad |= run(TBV_DT_F32, 4096, st);
    bad |= run(TBV_DT_F16, 100003, st);
    bad |= run(TBV_DT_BF16, 262144, NULL);
    if (tbv_ar_allreduce((void*)16, NULL, ((size_t)1 << 20) + 2, TBV_DT_BF16, st) != -2) return 15;   /* over the cap */
    double us; unsigned long long cnt;
    tbv_ar_stats(&us, &cnt);
    if (cnt != 6) { fprintf(stderr, "stats count %llu\n", cnt); return 16; }
    tbv_ar_rails(); tbv_ar_hist();
    tbv_ar_fini();
    if (tbv_ar_allreduce((void*)16, NULL, 64, 0, st) != -1) return 17;   /* progress threads are gone: refuse */
    tbv_emu_shutdown();
    printf(bad ? "FAILED\n" : "C client OK\n");
    return bad;
}
