// The packet pool of exchange.h and its host-side bookkeeping.
#include "exchange.h"
#include <atomic>
#include <mutex>
#include <vector>

namespace cpmk {

// packets, then one counter per slot (a team uses the counter of its index within the launch's range)
static __device__ __align__(256) uint64_t g_xch_pool[(size_t)kXchPoolSlots * kXchVals + kXchPoolSlots];
static __device__ uint32_t g_xch_status;
static __device__ uint32_t g_xch_taken;       // where k_xch_take_status leaves what it took

// The host mirrors of the status words, one per device (nullptr until the device's pool is set up, or if
// pinned memory could not be had).  Read without the lock by async_failure().
static std::atomic<uint32_t*> g_host_status[64];

namespace {

struct Held {             // a range of ring slots given to a launch that may still be running
    int32_t first, last;  // [first, last)
    hipEvent_t done;      // recorded after the launch
};

// Slots of the capture reserve belong to one (recording, stream) pair for good.  Launches recorded on one stream
// during one capture become a chain of graph nodes that run one after the other, and every team launch leaves its
// slots clean, so they share one range (a graph of many tall layernorms takes the slots of one).
struct CaptureRange {
    unsigned long long id;
    hipStream_t stream;
    int32_t first, size;
};

struct DevicePool {
    uint64_t* base = nullptr;       // the pool's address on this device
    uint32_t* status = nullptr;
    uint32_t* taken = nullptr;
    int32_t head = 0;               // next free slot of the ring
    int32_t capture_head = kXchRingSlots;   // next slot of the capture reserve; they are never taken back
    std::vector<Held> held;
    std::vector<hipEvent_t> spare;  // events ready for reuse
    std::vector<CaptureRange> captured;
};

std::mutex g_mu;
DevicePool g_dev[64];
std::atomic<uint32_t> g_seq{0};

// Is `st` recording into a graph?  `id` then identifies the recording (unique per capture).
bool capturing(hipStream_t st, unsigned long long* id) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    *id = 0;
    if (hipStreamGetCaptureInfo(st, &cs, id) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cs != hipStreamCaptureStatusNone;
}

// `may_allocate`: the caller is not recording into a graph, so the one-time allocation of the status word's
// host mirror (64 bytes of pinned memory per device) may be made now; otherwise it is left for a later call.
int device_pool(DevicePool** out, int* device, bool may_allocate) {      // g_mu held
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return CPMK_EBADARG;
    DevicePool& d = g_dev[dev];
    if (d.base == nullptr) {
        void *pool = nullptr, *stat = nullptr, *taken = nullptr;
        e = hipGetSymbolAddress(&pool, HIP_SYMBOL(g_xch_pool));
        if (e != hipSuccess) return (int)e;
        e = hipGetSymbolAddress(&stat, HIP_SYMBOL(g_xch_status));
        if (e != hipSuccess) return (int)e;
        e = hipGetSymbolAddress(&taken, HIP_SYMBOL(g_xch_taken));
        if (e != hipSuccess) return (int)e;
        d.status = (uint32_t*)stat;
        d.taken = (uint32_t*)taken;
        d.base = (uint64_t*)pool;
    }
    if (may_allocate && g_host_status[dev].load(std::memory_order_acquire) == nullptr) {
        void* h = nullptr;
        if (hipHostMalloc(&h, 64, hipHostMallocDefault) == hipSuccess && h != nullptr) {
            *(volatile uint32_t*)h = 0;
            g_host_status[dev].store((uint32_t*)h, std::memory_order_release);
        } else {
            (void)hipGetLastError();      // no mirror: time-outs are then only seen by cpmk_async_status()
        }
    }
    *out = &d;
    if (device != nullptr) *device = dev;
    return 0;
}

__global__ void k_xch_take_status(uint32_t* status, uint32_t* taken) {
    *taken = __hip_atomic_exchange(status, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

int async_failure() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    const uint32_t* h = g_host_status[dev].load(std::memory_order_acquire);
    if (h == nullptr) return 0;
    return (__atomic_load_n(h, __ATOMIC_RELAXED) & kXchStatusTimeout) ? CPMK_ETIMEOUT : 0;
}

uint32_t xch_next_tag() {
    uint32_t s = g_seq.fetch_add(1, std::memory_order_relaxed) + 1;
    if (s == 0) s = g_seq.fetch_add(1, std::memory_order_relaxed) + 1;   // tag 0 is what a fresh pool holds
    return s;
}

int xch_status_words(uint32_t** device_word, uint32_t** host_word) {
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    int dev = 0;
    if (int rc = device_pool(&d, &dev, false)) return rc;      // (callers of this one may not allocate)
    *device_word = d->status;
    *host_word = g_host_status[dev].load(std::memory_order_acquire);
    return 0;
}

XchScope::~XchScope() {
    if (locked_) (void)end();      // a caller that left early: whatever it launched is still waited for by the next holder
}

int XchScope::begin(int64_t slots, hipStream_t st) {
    if (locked_) return CPMK_EBADARG;
    if (slots < 1 || slots > kXchSlots) return CPMK_ETOOBIG;
    const int32_t need = (int32_t)(ceil_div(slots, kXchGranule) * kXchGranule);
    unsigned long long cap_id = 0;
    const bool cap = capturing(st, &cap_id);
    g_mu.lock();
    locked_ = true;
    DevicePool* d = nullptr;
    int dev = 0;
    if (int rc = device_pool(&d, &dev, !cap)) return rc;
    int32_t first;
    if (cap) {
        // a graph may be replayed at any time: its slots are its own for good
        first = -1;
        for (const CaptureRange& c : d->captured)
            if (c.id == cap_id && c.stream == st && c.size >= need) first = c.first;
        if (first < 0) {
            if (d->capture_head + need > kXchPoolSlots) {
                g_mu.unlock();
                locked_ = false;
                return kXchFull;
            }
            first = d->capture_head;
            d->capture_head += need;
            d->captured.push_back(CaptureRange{cap_id, st, first, need});
        }
    } else {
        first = d->head + need > kXchRingSlots ? 0 : d->head;
        const int32_t last = first + need;
        // whoever last held any of these slots must have finished before this launch starts; nothing of the
        // bookkeeping changes until every wait is queued, so a failure here leaves the ring as it was
        for (const Held& h : d->held)
            if (h.first < last && first < h.last) {
                const hipError_t e = hipStreamWaitEvent(st, h.done, 0);
                if (e != hipSuccess) return (int)e;
            }
        // The new holder takes over what it overlaps.  Slots go out in rising order, so an earlier holder's range
        // never starts below `first` unless it ends there too: what is left of a range that is only partly
        // covered is its upper end, which stays on record with its event for whoever is given those slots next.
        for (size_t i = 0; i < d->held.size();) {
            Held& h = d->held[i];
            if (h.first < last && first < h.last) {
                if (h.last > last && h.first >= first) {
                    h.first = last;
                    ++i;
                    continue;
                }
                d->spare.push_back(h.done);
                d->held[i] = d->held.back();
                d->held.pop_back();
            } else {
                ++i;
            }
        }
        d->head = last;
    }
    xl.region = d->base + (size_t)first * kXchVals;
    xl.counters = d->base + (size_t)kXchPoolSlots * kXchVals + first;
    xl.status = d->status;
    xl.host_status = g_host_status[dev].load(std::memory_order_acquire);
    xl.tag = xch_next_tag();
    xl.first = first;
    last_ = first + need;
    st_ = st;
    captured_ = cap;
    return 0;
}

int XchScope::end() {
    if (!locked_) return 0;               // nothing was begun (a launch without packets)
    int rc = 0;
    if (!captured_ && xl.first >= 0) {
        // The slots are taken from now on, whether or not the launch succeeded: the next holder waits for
        // everything queued on this stream up to here.
        DevicePool* d = nullptr;
        rc = device_pool(&d, nullptr, false);
        if (rc == 0) {
            hipEvent_t ev = nullptr;
            if (!d->spare.empty()) {
                ev = d->spare.back();
                d->spare.pop_back();
            } else {
                const hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
                if (e != hipSuccess) rc = (int)e;
            }
            if (rc == 0) {
                const hipError_t e = hipEventRecord(ev, st_);
                if (e != hipSuccess) {
                    d->spare.push_back(ev);
                    rc = (int)e;
                } else {
                    d->held.push_back(Held{xl.first, last_, ev});
                }
            }
            // no event to wait for later: the slots must be idle before anyone else can be given them
            if (rc != 0) (void)hipStreamSynchronize(st_);
        }
    }
    g_mu.unlock();
    locked_ = false;
    return rc;
}

void xch_prepare() {
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    (void)device_pool(&d, nullptr, true);
}

int xch_capture_slots_left(int32_t* slots) {
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    if (int rc = device_pool(&d, nullptr, false)) return rc;
    *slots = kXchPoolSlots - d->capture_head;
    return 0;
}

int xch_take_status(uint32_t* bits) {
    *bits = 0;
    std::lock_guard<std::mutex> lock(g_mu);
    DevicePool* d = nullptr;
    int dev = 0;
    if (int rc = device_pool(&d, &dev, false)) return rc;
    // read and clear in one step on the device (a flag raised in between is kept for the next call) ...
    hipLaunchKernelGGL(k_xch_take_status, dim3(1), dim3(1), 0, nullptr, d->status, d->taken);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    uint32_t v = 0;
    e = hipMemcpy(&v, d->taken, sizeof(v), hipMemcpyDeviceToHost);       // (waits for the kernel: both use the null stream)
    if (e != hipSuccess) return (int)e;
    // ... and the mirror on the host
    uint32_t* h = g_host_status[dev].load(std::memory_order_acquire);
    if (h != nullptr) v |= __atomic_exchange_n(h, 0u, __ATOMIC_RELAXED);
    *bits = v;
    return 0;
}

// One workgroup that waits `ticks` wall-clock ticks (100 MHz) for a packet nobody posts and then
// reports the time-out like the team kernels do: the way to exercise the failure path with a
// kernel that still ends normally.
__global__ void k_xch_selftest(XchLaunch xl, uint64_t ticks) {
    float v;
    if (threadIdx.x == 0 && !xch_wait(xl.region, xl.tag, wall_clock64() + ticks, v)) xch_flag(xl, kXchStatusTimeout);
}

}  // namespace cpmk

using namespace cpmk;

extern "C" {

int cpmk_async_status(void) {
    uint32_t bits = 0;
    if (int rc = xch_take_status(&bits)) return rc;
    return (bits & kXchStatusTimeout) ? CPMK_ETIMEOUT : 0;
}

int cpmk_exchange_capture_slots_left(int32_t* slots) {
    if (slots == nullptr) return CPMK_EBADARG;
    return xch_capture_slots_left(slots);
}

int cpmk_selftest_exchange_timeout(int32_t microseconds, void* stream) {
    clear_stale_error();
    if (microseconds < 0 || microseconds > 100000) return CPMK_EBADARG;
    hipStream_t st = (hipStream_t)stream;
    XchScope xs;
    if (int rc = xs.begin(1, st)) return rc == kXchFull ? CPMK_ETOOBIG : rc;
    hipLaunchKernelGGL(k_xch_selftest, dim3(1), dim3(64), 0, st, xs.xl, (uint64_t)microseconds * 100ull);
    const int e = (int)hipGetLastError();
    const int rc = xs.end();
    return e ? e : rc;
}

}  // extern "C"
