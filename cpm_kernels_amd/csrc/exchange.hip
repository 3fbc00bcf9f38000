// The packet pool of exchange.h and its host-side bookkeeping.
#include "exchange.h"
#include <atomic>
#include <mutex>

namespace cpmk {

static __device__ __align__(256) uint64_t g_xch_pool[(size_t)kXchRegions * kXchRegionWords];

int xch_begin(XchLaunch* out) {
    static std::mutex mu;
    static uint64_t* base[64] = {nullptr};      // the pool's address on each device
    static std::atomic<uint32_t> seq{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CPMK_EBADARG;
    uint64_t* p;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (base[dev] == nullptr) {
            void* sym = nullptr;
            e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_xch_pool));
            if (e != hipSuccess) return (int)e;
            base[dev] = (uint64_t*)sym;
        }
        p = base[dev];
    }
    uint32_t s = seq.fetch_add(1, std::memory_order_relaxed) + 1;
    if (s == 0) s = seq.fetch_add(1, std::memory_order_relaxed) + 1;   // tag 0 is what a fresh pool holds
    out->region = p + (size_t)(s % kXchRegions) * kXchRegionWords;
    out->tag = s;
    return 0;
}

}  // namespace cpmk
