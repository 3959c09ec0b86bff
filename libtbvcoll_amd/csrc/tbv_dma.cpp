#include "tbv_dma.h"

#include <dlfcn.h>
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>
#include <time.h>

namespace tbv {
namespace {

struct Api {
    decltype(&hsa_iterate_agents) iterate_agents = nullptr;
    decltype(&hsa_agent_get_info) agent_get_info = nullptr;
    decltype(&hsa_signal_create) signal_create = nullptr;
    decltype(&hsa_signal_destroy) signal_destroy = nullptr;
    decltype(&hsa_signal_store_relaxed) signal_store_relaxed = nullptr;
    decltype(&hsa_signal_wait_scacquire) signal_wait_scacquire = nullptr;
    decltype(&hsa_amd_memory_async_copy) memory_async_copy = nullptr;
    decltype(&hsa_amd_pointer_info) pointer_info = nullptr;
};

constexpr int kMaxLanes = 8;
Api api;
hsa_agent_t gpu{}, cpu{};
hsa_signal_t sig[kMaxLanes] = {};
int nlanes = 0;
bool ready = false;

double nowt()
{
    struct timespec t;
    clock_gettime(CLOCK_MONOTONIC, &t);
    return (double)t.tv_sec + (double)t.tv_nsec * 1e-9;
}

template <typename F> bool bind(void* h, F& f, const char* name)
{
    f = (F)dlsym(h, name);
    return f != nullptr;
}

hsa_status_t pick_cpu(hsa_agent_t a, void* data)
{
    hsa_device_type_t t;
    if (api.agent_get_info(a, HSA_AGENT_INFO_DEVICE, &t) == HSA_STATUS_SUCCESS && t == HSA_DEVICE_TYPE_CPU) {
        *(hsa_agent_t*)data = a;
        return HSA_STATUS_INFO_BREAK;
    }
    return HSA_STATUS_SUCCESS;
}

}  // namespace

bool dma_ready() { return ready; }

bool dma_init(const void* device_ptr, int lanes)
{
    if (ready) return true;
    if (lanes < 1 || lanes > kMaxLanes) return false;
    // the runtime HIP is already using; never load a second copy
    void* h = dlopen("libhsa-runtime64.so.1", RTLD_NOW | RTLD_NOLOAD);
    if (!h) h = dlopen("libhsa-runtime64.so", RTLD_NOW | RTLD_NOLOAD);
    if (!h) return false;
    if (!(bind(h, api.iterate_agents, "hsa_iterate_agents") && bind(h, api.agent_get_info, "hsa_agent_get_info") &&
          bind(h, api.signal_create, "hsa_signal_create") && bind(h, api.signal_destroy, "hsa_signal_destroy") &&
          bind(h, api.signal_store_relaxed, "hsa_signal_store_relaxed") &&
          bind(h, api.signal_wait_scacquire, "hsa_signal_wait_scacquire") &&
          bind(h, api.memory_async_copy, "hsa_amd_memory_async_copy") && bind(h, api.pointer_info, "hsa_amd_pointer_info")))
        return false;
    hsa_amd_pointer_info_t info{};
    info.size = sizeof(info);
    if (api.pointer_info(device_ptr, &info, nullptr, nullptr, nullptr) != HSA_STATUS_SUCCESS) return false;
    if (info.type != HSA_EXT_POINTER_TYPE_HSA) return false;
    gpu = info.agentOwner;
    hsa_agent_t c{};
    hsa_status_t st = api.iterate_agents(pick_cpu, &c);
    if ((st != HSA_STATUS_INFO_BREAK && st != HSA_STATUS_SUCCESS) || c.handle == 0) return false;
    cpu = c;
    for (int i = 0; i < lanes; i++) {
        if (api.signal_create(0, 0, nullptr, &sig[i]) != HSA_STATUS_SUCCESS) {
            for (int j = 0; j < i; j++) api.signal_destroy(sig[j]);
            return false;
        }
    }
    nlanes = lanes;
    ready = true;
    return true;
}

void dma_fini()
{
    if (!ready) return;
    for (int i = 0; i < nlanes; i++) api.signal_destroy(sig[i]);
    nlanes = 0;
    ready = false;
}

// Pinned host memory belongs to the CPU agent of the NUMA node it was allocated on, which
// depends on the allocating thread; ask the runtime rather than assume the first CPU agent.
static hsa_agent_t host_agent_of(const void* p)
{
    hsa_amd_pointer_info_t info{};
    info.size = sizeof(info);
    if (api.pointer_info(p, &info, nullptr, nullptr, nullptr) == HSA_STATUS_SUCCESS &&
        info.type == HSA_EXT_POINTER_TYPE_HSA && info.agentOwner.handle != 0 && info.agentOwner.handle != gpu.handle)
        return info.agentOwner;
    return cpu;
}

int dma_copy(int lane, void* dst, DmaSide dst_side, const void* src, DmaSide src_side, size_t n, double timeout_s)
{
    if (!ready || lane < 0 || lane >= nlanes) return -1;
    if (n == 0) return 0;
    const hsa_agent_t da = dst_side == DMA_HOST ? host_agent_of(dst) : gpu;
    const hsa_agent_t sa = src_side == DMA_HOST ? host_agent_of(src) : gpu;
    api.signal_store_relaxed(sig[lane], 1);
    if (api.memory_async_copy(dst, da, src, sa, n, 0, nullptr, sig[lane]) != HSA_STATUS_SUCCESS) return -1;
    const double t0 = nowt();
    for (;;) {
        hsa_signal_value_t v = api.signal_wait_scacquire(sig[lane], HSA_SIGNAL_CONDITION_LT, 1, 1000000ull, HSA_WAIT_STATE_ACTIVE);
        if (v < 0) return -1;       // the engine reported an error
        if (v < 1) return 0;
        if (nowt() - t0 > timeout_s) return -2;
    }
}

}  // namespace tbv
