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
// Opt `kernel` in to `lds_bytes` of dynamic LDS on the current device (once per host thread, kernel and device).
int ensure_dynamic_lds(const void* kernel, int lds_bytes);
// Name -> kernel registry behind sp_kernel_info().
void register_kernel(const char* name, const void* fn, int threads);

// ---- device: wave-level helpers (wave64) ----------------------------------------------------
#ifdef __HIPCC__
constexpr int WAVE = 64;

// Cross-lane move through the DPP data path (VALU speed, no LDS traffic).  CTRL is a DPP control
// word: 0xB1 = quad_perm [1,0,3,2], 0x4E = quad_perm [2,3,0,1], 0x141 = row_half_mirror,
// 0x140 = row_mirror, 0x110 + d = row_shr:d, 0x142 = row_bcast:15, 0x143 = row_bcast:31.
// Lanes without a source (or masked out by ROW_MASK) receive 0.
template <int CTRL, int ROW_MASK = 0xf, typename V>
__device__ __forceinline__ V dpp_move(V v) {
    static_assert(sizeof(V) == 4, "DPP moves 32-bit values");
    return __builtin_bit_cast(V, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}

// The value held by the partner lane of butterfly step D (lane ^ D) for values that are already
// uniform inside aligned groups of D lanes, which is what an all-reduce produces step by step.
template <int D, typename V>
__device__ __forceinline__ V butterfly_partner(V v) {
    if constexpr (D == 1) return dpp_move<0xB1>(v);
    else if constexpr (D == 2) return dpp_move<0x4E>(v);
    else if constexpr (D == 4) return dpp_move<0x141>(v);
    else if constexpr (D == 8) return dpp_move<0x140>(v);
    else return __shfl_xor(v, D, WAVE);
}

// Butterfly all-reduce inside aligned groups of T lanes (T a power of two <= 64).  Every level
// combines the same two partial results in both partner lanes, so for a commutative f all lanes
// of the group end with bit-identical values.
template <int T, typename V, typename F>
__device__ __forceinline__ V group_allreduce(V v, F f) {
    if constexpr (T >= 2) v = f(v, butterfly_partner<1>(v));
    if constexpr (T >= 4) v = f(v, butterfly_partner<2>(v));
    if constexpr (T >= 8) v = f(v, butterfly_partner<4>(v));
    if constexpr (T >= 16) v = f(v, butterfly_partner<8>(v));
    if constexpr (T >= 32) v = f(v, butterfly_partner<16>(v));
    if constexpr (T >= 64) v = f(v, butterfly_partner<32>(v));
    return v;
}

// Inclusive prefix sum inside aligned groups of T lanes.  The association is part of the
// library's contract (the CPU checker restates it to compare cumulative distributions bit for
// bit):
//   1. Hillis-Steele inside rows of min(T, 16) lanes: for d = 1, 2, 4, 8: v_t += v_{t-d} (t >= d);
//   2. T >= 32: every lane of an odd 16-lane row adds the last value of the row before it;
//   3. T == 64: every lane of rows 2 and 3 then adds the value lane 31 holds after step 2.
template <int T, typename V>
__device__ __forceinline__ V group_inclusive_scan(V v, int lane_in_group) {
    constexpr int R = T < 16 ? T : 16;
    if constexpr (R >= 2) { const V o = dpp_move<0x111>(v); if (R == 16 || lane_in_group >= 1) v = o + v; }
    if constexpr (R >= 4) { const V o = dpp_move<0x112>(v); if (R == 16 || lane_in_group >= 2) v = o + v; }
    if constexpr (R >= 8) { const V o = dpp_move<0x114>(v); if (R == 16 || lane_in_group >= 4) v = o + v; }
    if constexpr (R >= 16) { const V o = dpp_move<0x118>(v); v = o + v; }
    if constexpr (T >= 32) v = dpp_move<0x142, 0xa>(v) + v;
    if constexpr (T >= 64) v = dpp_move<0x143, 0xc>(v) + v;
    return v;
}

// A 16-byte store that is written THROUGH the XCD's L2 as it is issued (device scope, `sc1`) instead of being parked
// there until its line is evicted or the kernel ends: for outputs that are written once and not read again in the
// launch (measured: C of a 65536 x 256 x 256 GEMM 20.8 -> 18.0 us, probabilities + scan of the fused row kernel
// 31.4 -> 30.5 us, transpose 20.6 -> 20.4 us).  The compiler has no builtin that sets sc1 on a 16-byte store, so it
// is issued from asm, and the hardware's two wait states between a store of more than 8 bytes and a vector-ALU
// write of its data registers -- which the compiler inserts for its own stores and cannot see here -- are the s_nop
// (without it the next instruction's result reaches memory in place of some lanes' data).
template <typename V>
__device__ __forceinline__ void store16_through(V* p, V v) {
    static_assert(sizeof(V) == 16, "one 16-byte piece per lane");
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}

// All-reduce for one row per wave (T == 64) whose result comes back through a scalar register:
// butterfly inside the 16-lane rows, row_bcast:15 / row_bcast:31 to fold the rows into lane 63,
// v_readlane to broadcast.  Narrower groups use the butterfly.  Masked-out lanes of the row_bcast
// steps keep their own value, so any idempotent-or-not f is safe (only lane 63 is read).
template <int T, typename V, typename F>
__device__ __forceinline__ V group_reduce(V v, F f) {
    if constexpr (T < 64) {
        return group_allreduce<T>(v, f);
    } else {
        v = f(v, butterfly_partner<1>(v));
        v = f(v, butterfly_partner<2>(v));
        v = f(v, butterfly_partner<4>(v));
        v = f(v, butterfly_partner<8>(v));
        const int vi = __builtin_bit_cast(int, v);
        V o = __builtin_bit_cast(V, __builtin_amdgcn_update_dpp(vi, vi, 0x142, 0xa, 0xf, false));
        v = f(v, o);   // rows 1 and 3 fold in the row before them (their own value elsewhere: f(v, v))
        const int vj = __builtin_bit_cast(int, v);
        o = __builtin_bit_cast(V, __builtin_amdgcn_update_dpp(vj, vj, 0x143, 0xc, 0xf, false));
        v = f(v, o);   // rows 2 and 3 fold in lane 31
        return __builtin_bit_cast(V, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    }
}

// Value of lane `src` of the own group (src < T), broadcast to the group.  A 16-lane group is a
// DPP row, whose lanes can all read one lane of the row directly (control 0x150 + lane).
template <int T, typename V>
__device__ __forceinline__ V group_broadcast(V v, int src) {
    if constexpr (T == 64) return __builtin_bit_cast(V, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src));
    else return __shfl(v, src, T);
}
template <int T, typename V>
__device__ __forceinline__ V group_broadcast_last(V v) {
    if constexpr (T == 16) return dpp_move<0x15F>(v);
    else return group_broadcast<T>(v, T - 1);
}

// max(x, y) as the single hardware instruction: fmaxf() first canonicalises operands that come
// straight from memory, which doubles the instruction count of a max over freshly loaded data.
__device__ __forceinline__ float vmax(float x, float y) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}

// One butterfly step of a max all-reduce, the cross-lane read folded into the v_max (the
// compiler does this by itself for add and min, not for max).  The s_nop covers the two wait
// states a DPP read needs after a VALU write of the same register.
template <int D>
__device__ __forceinline__ float max_with_partner(float v) {
    float r;
    if constexpr (D == 1)
        asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));
    else if constexpr (D == 2)
        asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));
    else if constexpr (D == 4)
        asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));
    else
        asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 row_mirror row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(v));
    return r;
}

// Row max for every lane of an aligned group of T lanes.
template <int T>
__device__ __forceinline__ float group_max(float v) {
    if constexpr (T >= 2) v = max_with_partner<1>(v);
    if constexpr (T >= 4) v = max_with_partner<2>(v);
    if constexpr (T >= 8) v = max_with_partner<4>(v);
    if constexpr (T >= 16) v = max_with_partner<8>(v);
    if constexpr (T == 64) {
        const int vi = __builtin_bit_cast(int, v);
        float o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(vi, vi, 0x142, 0xa, 0xf, false));
        v = vmax(v, o);
        const int vj = __builtin_bit_cast(int, v);
        o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(vj, vj, 0x143, 0xc, 0xf, false));
        v = vmax(v, o);
        v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    }
    return v;
}
#endif

}  // namespace sp
