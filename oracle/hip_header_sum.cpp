// hip_header_sum.cpp -- TEST INFRASTRUCTURE ONLY.
//
// Host-only build of the HIP headers' own operator+ for __half and
// __hip_bfloat16, i.e. the third-party arithmetic that the reference's sum
// kernel resolves to (step4/libtbvcoll.cpp:165 `out[i]=a[i]+b[i]`; ROCm
// amd_hip_bf16.h `operator+` -> `__hadd`, amd_hip_fp16.h `operator+`).  Both are
// declared __host__ __device__, so the host instantiation pins the oracle's
// bit-level restatement without a GPU.  Nothing here comes from the reference.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <cstdint>
#include <cstddef>
#include <cstring>

template <typename T> static void add_all(const uint16_t* a, const uint16_t* b, uint16_t* o, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        T x, y;
        memcpy(&x, a + i, 2);
        memcpy(&y, b + i, 2);
        T z = x + y;
        memcpy(o + i, &z, 2);
    }
}

extern "C" void hdr_sum_bf16(const uint16_t* a, const uint16_t* b, uint16_t* o, size_t n) { add_all<__hip_bfloat16>(a, b, o, n); }
extern "C" void hdr_sum_f16(const uint16_t* a, const uint16_t* b, uint16_t* o, size_t n) { add_all<__half>(a, b, o, n); }
