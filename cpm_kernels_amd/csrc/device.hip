// Library and device queries of the C ABI (the part of cpm_kernels/library/cudart.py and
// cpm_kernels/device/__init__.py the path needs), plus error strings.
#include "exchange.h"
#include <string.h>

extern "C" {

int cpmk_version(void) { return 10000; }

const char* cpmk_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case CPMK_EBADARG: return "cpmk: invalid argument (negative size, bad batch combination or null pointer)";
        case CPMK_EALIGN: return "cpmk: size violates a divisibility precondition of the reference kernel";
        case CPMK_ETOOBIG: return "cpmk: problem exceeds a size limit of this library";
        case CPMK_ETIMEOUT: return "cpmk: a kernel gave up waiting for another workgroup of its launch; its output holds NaN (0 in int8 tensors)";
        default: return hipGetErrorString((hipError_t)code);
    }
}

int cpmk_device_count(int* count) { return (int)hipGetDeviceCount(count); }
int cpmk_get_device(int* device) { return (int)hipGetDevice(device); }
int cpmk_set_device(int device) {
    const hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) cpmk::xch_prepare();      // (the packet pool's one host allocation, outside any stream capture)
    return (int)e;
}

int cpmk_device_props(int device, char* name, int name_len, int* compute_units, int* lds_bytes, int* wavefront,
                      int* clock_khz, int* mem_clock_khz, int* mem_bus_bits, int* l2_bytes,
                      uint64_t* global_mem_bytes) {
    hipDeviceProp_t p;
    hipError_t e = hipGetDeviceProperties(&p, device);
    if (e != hipSuccess) return (int)e;
    if (name && name_len > 0) {
        strncpy(name, p.gcnArchName, (size_t)name_len - 1);
        name[name_len - 1] = 0;
        char* colon = strchr(name, ':');   // "gfx950:sramecc+:xnack-" -> "gfx950"
        if (colon) *colon = 0;
    }
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (lds_bytes) *lds_bytes = (int)p.sharedMemPerBlock;
    if (wavefront) *wavefront = p.warpSize;
    if (clock_khz) *clock_khz = p.clockRate;
    if (mem_clock_khz) *mem_clock_khz = p.memoryClockRate;
    if (mem_bus_bits) *mem_bus_bits = p.memoryBusWidth;
    if (l2_bytes) *l2_bytes = p.l2CacheSize;
    if (global_mem_bytes) *global_mem_bytes = (uint64_t)p.totalGlobalMem;
    return 0;
}

}  // extern "C"
