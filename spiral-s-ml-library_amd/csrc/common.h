// Shared host/device helpers of libspiral_mi355.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include <type_traits>

#include "spiral_mi355.h"

namespace sp {

// ---- host: per-thread error slot ------------------------------------------------------------
char* error_buffer();  // 512 bytes, thread local (api.hip)

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define SP_REQUIRE_PTR(p)                                                        \
    do {                                                                         \
        if ((p) == nullptr) return sp::fail(SP_ERR_NULL, "%s: %s is NULL", __func__, #p); \
        if (!sp::aligned16(p)) return sp::fail(SP_ERR_ALIGN, "%s: %s is not 16-byte aligned", __func__, #p); \
    } while (0)

#define SP_OPTIONAL_PTR(p)                                                       \
    do {                                                                         \
        if ((p) != nullptr && !sp::aligned16(p))                                 \
            return sp::fail(SP_ERR_ALIGN, "%s: %s is not 16-byte aligned", __func__, #p); \
    } while (0)

inline int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return SP_OK;
}

// The kernels are built for gfx950 only; refuse to launch on anything else instead of faulting.
int require_gfx950(const char* what);
int device_cu_count();
// Name -> kernel registry behind sp_kernel_info().
void register_kernel(const char* name, const void* fn, int threads);

// ---- device: wave-level helpers (wave64) ----------------------------------------------------
#ifdef __HIPCC__
constexpr int WAVE = 64;

// Butterfly all-reduce inside aligned groups of T lanes (T a power of two <= 64).
template <int T, typename V, typename F>
__device__ __forceinline__ V group_allreduce(V v, F f) {
#pragma unroll
    for (int d = 1; d < T; d <<= 1) v = f(v, __shfl_xor(v, d, WAVE));
    return v;
}

// Hillis-Steele inclusive scan inside aligned groups of T lanes: for d = 1, 2, 4, ...:
// v_t = v_{t-d} + v_t for t >= d.  The association is part of the library's contract (the CPU
// checker restates it to compare cumulative distributions bit for bit).
template <int T, typename V>
__device__ __forceinline__ V group_inclusive_scan(V v, int lane_in_group) {
#pragma unroll
    for (int d = 1; d < T; d <<= 1) {
        V o = __shfl_up(v, d, T);
        if (lane_in_group >= d) v = o + v;
    }
    return v;
}
#endif

}  // namespace sp
