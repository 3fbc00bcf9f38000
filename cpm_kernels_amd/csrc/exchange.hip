// The packet pool of exchange.h and its host-side bookkeeping.
#include "exchange.h"
#include <atomic>
#include <mutex>
#include <vector>

namespace cpmk {

// packets, then one counter per slot (a team uses the counter of its index within the launch's range)
static __device__ __align__(256) uint64_t g_xch_pool[(size_t)kXchPoolSlots * kXchVals + kXchPoolSlots];
static __device__ uint32_t g_xch_status;

namespace {

struct Held {             // a range of slots given to a launch that may still be running
    int32_t first, last;  // [first, last)
    hipEvent_t done;      // recorded after the launch; nullptr for a launch recorded during stream capture
};

struct DevicePool {
    uint64_t* base = nullptr;       // the pool's address on this device
    uint32_t* status = nullptr;
    int32_t head = 0;               // next free slot of the ring
    std::vector<Held> held;
    std::vector<hipEvent_t> spare;  // events ready for reuse
};

std::mutex g_mu;
DevicePool g_dev[64];
std::atomic<uint32_t> g_seq{0};

int device_pool(DevicePool** out) {      // g_mu held
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CPMK_EBADARG;
    DevicePool& d = g_dev[dev];
    if (d.base == nullptr) {
        void *pool = nullptr, *stat = nullptr;
        e = hipGetSymbolAddress(&pool, HIP_SYMBOL(g_xch_pool));
        if (e != hipSuccess) return (int)e;
        e = hipGetSymbolAddress(&stat, HIP_SYMBOL(g_xch_status));
        if (e != hipSuccess) return (int)e;
        d.status = (uint32_t*)stat;
        d.base = (uint64_t*)pool;
    }
    *out = &d;
    return 0;
}

bool capturing(hipStream_t st) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cs != hipStreamCaptureStatusNone;
}

}  // namespace

uint32_t xch_next_tag() {
    uint32_t s = g_seq.fetch_add(1, std::memory_order_relaxed) + 1;
    if (s == 0) s = g_seq.fetch_add(1, std::memory_order_relaxed) + 1;   // tag 0 is what a fresh pool holds
    return s;
}

int xch_status_word(uint32_t** out) {
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    if (int rc = device_pool(&d)) return rc;
    *out = d->status;
    return 0;
}

int xch_begin(XchLaunch* out, int64_t slots, hipStream_t st) {
    if (slots < 1 || slots > kXchSlots) return CPMK_ETOOBIG;
    const int32_t need = (int32_t)(ceil_div(slots, kXchGranule) * kXchGranule);
    const bool cap = capturing(st);
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    if (int rc = device_pool(&d)) return rc;
    if (d->head + need > kXchPoolSlots) d->head = 0;
    const int32_t first = d->head, last = first + need;
    d->head = last;
    // whoever last held any of these slots must have finished before this launch starts
    for (size_t i = 0; i < d->held.size();) {
        Held& h = d->held[i];
        if (h.first < last && first < h.last) {
            if (h.done != nullptr) {
                if (!cap) {
                    const hipError_t e = hipStreamWaitEvent(st, h.done, 0);
                    if (e != hipSuccess) return (int)e;
                }
                d->spare.push_back(h.done);
            }
            d->held[i] = d->held.back();
            d->held.pop_back();
        } else {
            ++i;
        }
    }
    const uint32_t s = xch_next_tag();
    out->region = d->base + (size_t)first * kXchVals;
    out->counters = d->base + (size_t)kXchPoolSlots * kXchVals + first;
    out->status = d->status;
    out->tag = s;
    out->first = first;
    // the slots are taken from now on, whether or not the launch succeeds
    d->held.push_back(Held{first, last, nullptr});
    return 0;
}

int xch_end(const XchLaunch& xl, hipStream_t st) {
    if (xl.first < 0) return 0;
    if (capturing(st)) return 0;         // a graph's replays are not tracked
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    if (int rc = device_pool(&d)) return rc;
    for (Held& h : d->held) {
        if (h.first != xl.first || h.done != nullptr) continue;
        hipEvent_t ev = nullptr;
        if (!d->spare.empty()) {
            ev = d->spare.back();
            d->spare.pop_back();
        } else {
            const hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
            if (e != hipSuccess) return (int)e;
        }
        const hipError_t e = hipEventRecord(ev, st);
        if (e != hipSuccess) {
            d->spare.push_back(ev);
            return (int)e;
        }
        h.done = ev;
        break;
    }
    return 0;
}

int xch_take_status(uint32_t* bits) {
    *bits = 0;
    uint32_t* status = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        DevicePool* d = nullptr;
        if (int rc = device_pool(&d)) return rc;
        status = d->status;
    }
    uint32_t v = 0;
    hipError_t e = hipMemcpy(&v, status, sizeof(v), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    if (v != 0) {
        e = hipMemset(status, 0, sizeof(v));
        if (e != hipSuccess) return (int)e;
    }
    *bits = v;
    return 0;
}

// One workgroup that waits `ticks` wall-clock ticks (100 MHz) for a packet nobody posts and then
// reports the time-out like the team kernels do: the way to exercise the failure path with a
// kernel that still ends normally.
__global__ void k_xch_selftest(XchLaunch xl, uint64_t ticks) {
    float v;
    if (threadIdx.x == 0 && !xch_wait(xl.region, xl.tag, wall_clock64() + ticks, v)) xch_flag(xl.status, kXchStatusTimeout);
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_async_status(void) {
    uint32_t bits = 0;
    if (int rc = xch_take_status(&bits)) return rc;
    return (bits & kXchStatusTimeout) ? CPMK_ETIMEOUT : 0;
}

int cpmk_selftest_exchange_timeout(int32_t microseconds, void* stream) {
    clear_stale_error();
    if (microseconds < 0 || microseconds > 100000) return CPMK_EBADARG;
    hipStream_t st = (hipStream_t)stream;
    XchLaunch xl;
    if (int rc = xch_begin(&xl, 1, st)) return rc;
    hipLaunchKernelGGL(k_xch_selftest, dim3(1), dim3(64), 0, st, xl, (uint64_t)microseconds * 100ull);
    const int e = launch_status();
    if (int rc = xch_end(xl, st)) return e ? e : rc;
    return e;
}

}  // extern "C"
