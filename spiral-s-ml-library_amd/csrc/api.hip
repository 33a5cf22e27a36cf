// Library-level entry points: error slot, device probing, kernel occupancy report.
#include "common.h"

#include <string.h>

#include <mutex>
#include <string>
#include <vector>

namespace sp {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

struct DeviceCache {
    bool probed = false;
    bool ok = false;
    int cus = 0;
    char arch[64] = {0};
};

static DeviceCache& device_cache(int dev) {
    static DeviceCache cache[64];
    return cache[dev < 0 || dev >= 64 ? 0 : dev];
}

static std::mutex g_mutex;

static int probe(DeviceCache** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipGetDevice failed: %s", hipGetErrorString(e));
    DeviceCache& c = device_cache(dev);
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!c.probed) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
        strncpy(c.arch, prop.gcnArchName, sizeof(c.arch) - 1);
        c.cus = prop.multiProcessorCount;
        c.ok = strncmp(c.arch, "gfx950", 6) == 0;
        c.probed = true;
    }
    *out = &c;
    return SP_OK;
}

int require_gfx950(const char* what) {
    DeviceCache* c = nullptr;
    int rc = probe(&c);
    if (rc != SP_OK) return rc;
    if (!c->ok)
        return fail(SP_ERR_DEVICE, "%s: this library is built for gfx950 (MI355X) only; current device is %s", what,
                    c->arch);
    return SP_OK;
}

int device_cu_count() {
    DeviceCache* c = nullptr;
    if (probe(&c) != SP_OK || c->cus <= 0) return 256;
    return c->cus;
}

// The opt-in to more than 64 KiB of dynamic LDS is per kernel and device.  Each host thread remembers the
// (kernel, device) pairs it has opted in (thread-local, so nothing is shared between threads; the HIP call
// itself is thread safe and idempotent, a second thread merely repeats it once).
int ensure_dynamic_lds(const void* kernel, int lds_bytes) {
    struct Seen { const void* kernel; int device; };
    static thread_local Seen seen[64];
    static thread_local int n_seen = 0;
    int dev = 0;
    (void)hipGetDevice(&dev);
    for (int i = 0; i < n_seen; ++i)
        if (seen[i].kernel == kernel && seen[i].device == dev) return SP_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipFuncSetAttribute(%d B LDS) failed: %s", lds_bytes, hipGetErrorString(e));
    if (n_seen < 64) seen[n_seen++] = Seen{kernel, dev};
    return SP_OK;
}

struct KernelEntry {
    std::string name;
    const void* fn;
    int threads;
};

static std::vector<KernelEntry>& registry() {
    static std::vector<KernelEntry> r;
    return r;
}

void register_kernel(const char* name, const void* fn, int threads) { registry().push_back({name, fn, threads}); }

// Every workgroup writes the number of the XCD it runs on, that XCD's shader clock counter (s_memtime: counts the
// cycles the compute units run at, so it slows down with the clock) and the constant 100 MHz counter (s_memrealtime).
// Every compute unit keeps a cycle counter of its own, and they are not in step (tens of millions of cycles apart even
// inside one XCD), so two samples can only be compared unit by unit: a workgroup writes its pair of counters into the
// slot of the unit it ran on -- XCD number and the unit's place in it (shader engine, shader array, unit, SIMD: bits
// 15:4 of the hardware id) -- and 8192 one-wave workgroups reach every SIMD of the chip.
constexpr int CLOCK_SAMPLE_GROUPS = 8192;
constexpr int CLOCK_SAMPLE_SLOTS = 8 * 4096;
__global__ void clock_sample_kernel(unsigned long long* out) {
    if (threadIdx.x == 0) {
        const unsigned long long cycles = __builtin_amdgcn_s_memtime();
        const unsigned long long ticks = __builtin_amdgcn_s_memrealtime();
        const unsigned xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 0x7u;   // HW_REG_XCC_ID, bits 3:0
        const unsigned hw = __builtin_amdgcn_s_getreg(4 | (4 << 6) | (11 << 11));          // HW_REG_HW_ID, bits 15:4
        typedef unsigned long long u64x2 __attribute__((ext_vector_type(2)));
        const u64x2 rec = {cycles, ticks};
        *reinterpret_cast<u64x2*>(out + 2 * (xcc * 4096 + (hw & 0xfffu))) = rec;              // one 16-byte store
    }
}

}  // namespace sp

using namespace sp;

extern "C" int sp_clock_sample(uint64_t* out, void* stream) {
    SP_REQUIRE_PTR(out);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    hipLaunchKernelGGL(clock_sample_kernel, dim3(CLOCK_SAMPLE_GROUPS), dim3(64), 0, (hipStream_t)stream, (unsigned long long*)out);
    return check_launch(__func__);
}

extern "C" const char* sp_last_error_string(void) { return error_buffer(); }

extern "C" int sp_device_info(sp_device_info_t* out) {
    if (out == nullptr) return fail(SP_ERR_NULL, "sp_device_info: out is NULL");
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipGetDevice failed: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipGetDeviceProperties failed: %s", hipGetErrorString(e));
    memset(out, 0, sizeof(*out));
    strncpy(out->name, prop.name, sizeof(out->name) - 1);
    strncpy(out->arch, prop.gcnArchName, sizeof(out->arch) - 1);
    out->compute_units = prop.multiProcessorCount;
    out->wavefront_size = prop.warpSize;
    out->lds_bytes_per_cu = (int32_t)prop.sharedMemPerBlock;
    out->max_clock_khz = prop.clockRate;
    out->hbm_bytes = (int64_t)prop.totalGlobalMem;
    out->l2_bytes = prop.l2CacheSize;
    return SP_OK;
}

extern "C" int sp_kernel_info(const char* kernel_family, sp_kernel_info_t* out) {
    if (kernel_family == nullptr || out == nullptr) return fail(SP_ERR_NULL, "sp_kernel_info: NULL argument");
    for (const KernelEntry& k : registry()) {
        if (k.name != kernel_family) continue;
        hipFuncAttributes attr;
        hipError_t e = hipFuncGetAttributes(&attr, k.fn);
        if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipFuncGetAttributes failed: %s", hipGetErrorString(e));
        out->vgprs = attr.numRegs;
        out->sgprs = 0;
        out->static_lds_bytes = (int32_t)attr.sharedSizeBytes;
        out->threads_per_block = k.threads;
        int blocks = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, k.fn, k.threads, 0);
        if (e != hipSuccess) return fail(SP_ERR_DEVICE, "occupancy query failed: %s", hipGetErrorString(e));
        out->max_blocks_per_cu = blocks;
        return SP_OK;
    }
    return fail(SP_ERR_ARG, "sp_kernel_info: unknown kernel family '%s'", kernel_family);
}
