// Elementwise map, full-tensor sum and inner-dimension transpose for gfx950.  All three are
// HBM-bound: 16-byte accesses, grid-stride loops, no MFMA.
//
// Semantics: primitives.map (ml/primitives.spi:115-133), reduce / grid_reduce (:136-197),
// grid_transpose_snd (:36-112).
#include "common.h"

#include <atomic>
#include <cstdlib>
#include <mutex>

namespace sp {

typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int EW_THREADS = 256;
constexpr int REDUCE_MAX_BLOCKS = 1024;
// A reduction's scratch memory: two 64-bit slots per possible block (low and high half of an 8-byte partial result),
// then the give-up counter (and 8 bytes that keep the size a multiple of 16).
constexpr long REDUCE_STATUS_WORD = (long)REDUCE_MAX_BLOCKS * 2;     // index in 64-bit words
constexpr long REDUCE_SLOT_BYTES = (long)REDUCE_MAX_BLOCKS * 2 * 8;
constexpr long REDUCE_SCRATCH_BYTES = REDUCE_SLOT_BYTES + 16;
// Workgroups per compute unit of the grid-stride kernels (tuning constants; a build may override them).
#ifndef SP_MAP_BLOCKS_PER_CU
#define SP_MAP_BLOCKS_PER_CU 4      // (map on 65536 x 256 f32: 19.3 us from 1024 workgroups, 20.4 from 2048, 24.4 from 256)
#endif
#ifndef SP_REDUCE_BLOCKS_PER_CU
#define SP_REDUCE_BLOCKS_PER_CU 2
#endif

template <int OP>
__device__ __forceinline__ float map_op(float x) {
    if constexpr (OP == SP_MAP_RELU) return fmaxf(x, 0.f);
    else if constexpr (OP == SP_MAP_TANH) return tanhf(x);
    else if constexpr (OP == SP_MAP_SIGMOID) return 1.f / (1.f + expf(-x));
    else return x;
}

template <int OP>
__global__ __launch_bounds__(EW_THREADS) void map_kernel(const f32x4* __restrict__ x, f32x4* __restrict__ out, long n4) {
    const long stride = (long)gridDim.x * EW_THREADS;
    for (long i = (long)blockIdx.x * EW_THREADS + threadIdx.x; i < n4; i += stride) {
        f32x4 v = x[i];
        v.x = map_op<OP>(v.x); v.y = map_op<OP>(v.y); v.z = map_op<OP>(v.z); v.w = map_op<OP>(v.w);
        out[i] = v;
    }
}

// The reduction operators of `reduce neutral f` (ml/primitives.spi:136-197) this library names: (0, +), (1, *),
// (-inf, max), (+inf, min) with the neutral elements of corebase/limit.spi.  max / min of floats follow the
// hardware's v_max / v_min: a NaN operand is ignored unless both are NaN.
template <int OP, typename T>
__device__ __forceinline__ T red_neutral() {
    if constexpr (OP == SP_REDUCE_SUM) return T(0);
    else if constexpr (OP == SP_REDUCE_PROD) return T(1);
    else if constexpr (std::is_same<T, float>::value) return OP == SP_REDUCE_MAX ? -__builtin_inff() : __builtin_inff();
    else if constexpr (std::is_same<T, int>::value) return OP == SP_REDUCE_MAX ? (int)0x80000000 : 0x7fffffff;
    else return OP == SP_REDUCE_MAX ? T(0) : ~T(0);
}
template <int OP, typename T>
__device__ __forceinline__ T red_op(T a, T b) {
    if constexpr (OP == SP_REDUCE_SUM) return a + b;
    else if constexpr (OP == SP_REDUCE_PROD) return a * b;
    else if constexpr (std::is_same<T, float>::value) return OP == SP_REDUCE_MAX ? fmaxf(a, b) : fminf(a, b);
    else if constexpr (OP == SP_REDUCE_MAX) return a > b ? a : b;
    else return a < b ? a : b;
}

// Block-wide reduction: lanes -> wave (shuffles) -> LDS (one slot per wave) -> first wave.
template <int OP, typename T>
__device__ __forceinline__ T block_reduce(T v, T* slots) {
    if constexpr (sizeof(T) == 4) {
        v = group_reduce<WAVE>(v, [](T a, T b) { return red_op<OP>(a, b); });    // DPP butterflies, no LDS round trips
    } else {
#pragma unroll
        for (int d = 1; d < WAVE; d <<= 1) v = red_op<OP>(v, __shfl_xor(v, d, WAVE));
    }
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    T r = (threadIdx.x < EW_THREADS / WAVE) ? slots[threadIdx.x] : red_neutral<OP, T>();
    if (wave == 0) {
#pragma unroll
        for (int d = 1; d < EW_THREADS / WAVE; d <<= 1) r = red_op<OP>(r, __shfl_xor(r, d, WAVE));
    }
    __syncthreads();
    return r;  // valid in wave 0
}

// Full-tensor reduction in ONE launch.  Every block folds its share (16-byte loads, U of them in flight per lane
// and U independent running results) and PUBLISHES its partial result as one 64-bit word per 32 bits of value --
// the value below, the launch's MARK above -- with a single device-scope atomic store into slot blockIdx.x (an
// 8-byte result takes two words, REDUCE_MAX_BLOCKS apart).  Block 0 then polls the slots with device-scope atomic
// loads until every one carries the mark, clears each slot, folds the partials in index order and writes the
// result: the order of the operations depends on n and the grid only.
// The value and its mark travel in the same atomic word, so no fence, no counter and no acknowledgement stand
// between a block's last operation and the moment block 0 can see it: the end of the kernel is one store on its way
// out and one load that finds it.  (The form this replaces -- store, wait for its acknowledgement, draw a ticket
// from a counter per 64 blocks, then from a top counter, last block loads the partials -- had four dependent round
// trips to memory past the XCD's private L2 in that place, ~0.5 us each with every memory channel busy.)
// Device-scope atomic accesses go to memory past the L2, so nothing has to be written back or invalidated.
// Block 0's own partial never leaves its registers.
// The mark is a 32-bit number the host draws per launch (never 0): a slot left behind by another launch -- one that
// gave up, or one whose late blocks published after block 0 had given up -- or memory that was never cleared cannot
// pass for this launch's partial.  Block 0 still leaves every slot it polled at zero, so a launch that is replayed
// with the same mark (a captured graph) finds no mark of its previous run either.
// All blocks of the grid are resident at once when the launch has the device to itself (at most
// SP_REDUCE_BLOCKS_PER_CU per compute unit), and a poller that got a unit before the others only holds one block's
// worth of it, so the poll cannot keep a block from running.  It still has a bound: REDUCE_POLL_NS of the constant
// 100 MHz clock (s_memrealtime), a few milliseconds.  A launch that shares the device with enough other work to
// exceed it gives up: the result is a NaN / all-ones word, every slot is cleared, and the give-up counter in the
// last word of the scratch memory goes up by one (sp_reduce_status reads it).
constexpr long REDUCE_POLL_TICKS = 500000;       // 5 ms of the 100 MHz constant clock
static std::atomic<long> reduce_poll_ticks_now{REDUCE_POLL_TICKS};
static long reduce_poll_ticks() { return reduce_poll_ticks_now.load(std::memory_order_relaxed); }

template <typename T, int U, int OP>
__global__ __launch_bounds__(EW_THREADS) void reduce_kernel(const T* __restrict__ x, T* __restrict__ out, long n,
                                                            unsigned long long* slots_mem, unsigned mark, long poll_ticks) {
    __shared__ T slots[EW_THREADS / WAVE];
    constexpr int V = 16 / sizeof(T);
    constexpr int W = sizeof(T) / 4;                            // 64-bit words per published partial result
    typedef T VT __attribute__((ext_vector_type(V)));
    typedef unsigned long long u64;
    const VT* xv = reinterpret_cast<const VT*>(x);
    const long nv = n / V;
    const long stride = (long)gridDim.x * EW_THREADS;
    const long tid = (long)blockIdx.x * EW_THREADS + threadIdx.x;
    const u64 valid = (u64)mark << 32;
    auto vec_op = [](VT a, VT b) {
        if constexpr (OP == SP_REDUCE_SUM) return a + b;
        else if constexpr (OP == SP_REDUCE_PROD) return a * b;
        else {
            VT r;
#pragma unroll
            for (int k = 0; k < V; ++k) r[k] = red_op<OP>(a[k], b[k]);
            return r;
        }
    };
    VT a[U];
#pragma unroll
    for (int k = 0; k < U; ++k) a[k] = VT(red_neutral<OP, T>());
    long i = tid;
    for (; i + (U - 1) * stride < nv; i += U * stride) {
        VT v[U];
#pragma unroll
        for (int k = 0; k < U; ++k) v[k] = xv[i + k * stride];
#pragma unroll
        for (int k = 0; k < U; ++k) a[k] = vec_op(a[k], v[k]);
    }
    for (; i < nv; i += stride) a[0] = vec_op(a[0], xv[i]);
#pragma unroll
    for (int d = 1; d < U; d <<= 1)
#pragma unroll
        for (int k = 0; k + d < U; k += 2 * d) a[k] = vec_op(a[k], a[k + d]);
    T acc = a[0][0];
#pragma unroll
    for (int k = 1; k < V; ++k) acc = red_op<OP>(acc, a[0][k]);
    for (long j = nv * V + tid; j < n; j += stride) acc = red_op<OP>(acc, x[j]);   // the last n % V elements
    acc = block_reduce<OP>(acc, slots);                                          // valid in wave 0

    unsigned bits[W];
    __builtin_memcpy(bits, &acc, sizeof(T));
    if (blockIdx.x != 0) {
        if (threadIdx.x == 0) {
#pragma unroll
            for (int j = 0; j < W; ++j)
                __hip_atomic_store(slots_mem + (long)j * REDUCE_MAX_BLOCKS + blockIdx.x, valid | bits[j],
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    // Block 0: thread t collects slots t, t + EW_THREADS, ...; all of a thread's loads are in flight together.
    // (Every wave polling all slots, the waves a quarter of a poll period apart, measured 1 % slower.)
    constexpr int S = REDUCE_MAX_BLOCKS / EW_THREADS;
    u64 w[S][W] = {};
    bool pending = true;
    const u64 t_start = __builtin_amdgcn_s_memrealtime();
    for (long round = 0; pending; ++round) {
        if (round) {
            __builtin_amdgcn_s_sleep(2);
            if ((long)(__builtin_amdgcn_s_memrealtime() - t_start) > poll_ticks) break;
        } else if (poll_ticks < 0) {
            break;                                   // a bound below zero: do not wait at all
        }
#pragma unroll
        for (int k = 0; k < S; ++k) {
            const unsigned b = threadIdx.x + k * EW_THREADS;
#pragma unroll
            for (int j = 0; j < W; ++j) {
                if (b == 0) w[k][j] = valid | bits[j];
                else if (b < gridDim.x)
                    w[k][j] = __hip_atomic_load(slots_mem + (long)j * REDUCE_MAX_BLOCKS + b, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_AGENT);
                else w[k][j] = valid;
            }
        }
        bool all = true;
#pragma unroll
        for (int k = 0; k < S; ++k)
#pragma unroll
            for (int j = 0; j < W; ++j) all = all && (w[k][j] >> 32) == mark;
        pending = !all;
    }
    T total = red_neutral<OP, T>();
#pragma unroll
    for (int k = 0; k < S; ++k) {
        const unsigned b = threadIdx.x + k * EW_THREADS;
        if (b < gridDim.x) {
            unsigned part[W];
#pragma unroll
            for (int j = 0; j < W; ++j) {
                part[j] = (unsigned)w[k][j];
                if (b != 0)     // every polled slot goes back to zero, whatever it held
                    __hip_atomic_store(slots_mem + (long)j * REDUCE_MAX_BLOCKS + b, 0ull, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            }
            T v;
            __builtin_memcpy(&v, part, sizeof(T));
            total = red_op<OP>(total, v);
        }
    }
    const int gave_up = __syncthreads_or(pending);
    total = block_reduce<OP>(total, slots);
    if (threadIdx.x == 0) {
        if (gave_up) {
            __builtin_memset(&total, 0xff, sizeof(T));   // f32: a NaN; integers: all ones
            __hip_atomic_fetch_add(slots_mem + REDUCE_STATUS_WORD, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        out[0] = total;
    }
}

// Sets `count` 32-bit words to zero (a kernel rather than a memset so that callers may record it into a graph).
__global__ __launch_bounds__(EW_THREADS) void clear_words_kernel(unsigned* p, int count) {
    for (int i = threadIdx.x; i < count; i += EW_THREADS) p[i] = 0u;
}

// to[a][c][b] = from[a][b][c]; 64x64 tiles through LDS, padded by one word per row so that the
// transposed (column) reads hit 64 different banks.  (The reference sizes this tile at run time: `frame_iter`
// doubles a 32 x 32 minimum under its shared-memory budget, ml/primitives.spi:17-33,56-66; here it is fixed at one
// wave-width square, which is what 64 banks and 64 lanes ask for.)
__global__ __launch_bounds__(EW_THREADS) void transpose_kernel(const unsigned* __restrict__ from, unsigned* __restrict__ to,
                                                               long B, long C, long tiles_b, long tiles_c) {
    __shared__ unsigned tile[64][65];
    const long t = blockIdx.x;
    const long a = t / (tiles_b * tiles_c);
    const long tb = (t / tiles_c) % tiles_b, tc = t % tiles_c;
    const unsigned* src = from + a * B * C;
    unsigned* dst = to + a * B * C;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        const long b = tb * 64 + r, c = tc * 64 + tx;
        if (b < B && c < C) tile[r][tx] = src[b * C + c];
    }
    __syncthreads();
    for (int r = ty; r < 64; r += 4) {
        const long c = tc * 64 + r, b = tb * 64 + tx;
        if (b < B && c < C) dst[c * B + b] = tile[tx][r];
    }
}

// The same for B and C multiples of 4: 16-byte reads and writes (a quarter of the memory
// instructions), the transposition happens between four 4-byte LDS writes and four 4-byte LDS
// reads per lane; with rows padded to 65 words both hit 64 different banks per wave.
__global__ __launch_bounds__(EW_THREADS) void transpose_vec4_kernel(const unsigned* __restrict__ from,
                                                                    unsigned* __restrict__ to, long B, long C,
                                                                    long tiles_b, long tiles_c) {
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    __shared__ unsigned tile[64][65];
    const long t = blockIdx.x;
    const long a = t / (tiles_b * tiles_c);
    const long tb = (t / tiles_c) % tiles_b, tc = t % tiles_c;
    const unsigned* src = from + a * B * C;
    unsigned* dst = to + a * B * C;
    const int q = threadIdx.x & 15, r0 = threadIdx.x >> 4;   // 16 lanes per 64-word row, 16 rows per pass
    u32x4 v[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const long b = tb * 64 + 16 * p + r0, c = tc * 64 + 4 * q;
        v[p] = u32x4{0u, 0u, 0u, 0u};
        if (b < B && c < C) v[p] = *reinterpret_cast<const u32x4*>(src + b * C + c);
    }
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int k = 0; k < 4; ++k) tile[16 * p + r0][4 * q + k] = v[p][k];
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int cl = 16 * p + r0;
        const long c = tc * 64 + cl, b = tb * 64 + 4 * q;
        const u32x4 w = {tile[4 * q][cl], tile[4 * q + 1][cl], tile[4 * q + 2][cl], tile[4 * q + 3][cl]};
        if (b < B && c < C) store16_through(reinterpret_cast<u32x4*>(dst + c * B + b), w);
    }
}

template <typename T, int OP>
static int run_reduce(const void* x, void* out, int64_t n, void* scratch_mem, hipStream_t stream, const char* what) {
    // Two workgroups per compute unit: a read-only stream of 256 MiB runs at 6.8 TB/s from 512 workgroups and at
    // 5.8 TB/s from 2048 (more waves in flight make the memory controllers' job harder, not easier).
    long blocks = (n + EW_THREADS * 16 - 1) / (EW_THREADS * 16);   // >= 4 vectors of 16 bytes per lane
    const long cap = (long)device_cu_count() * SP_REDUCE_BLOCKS_PER_CU;
    if (blocks > cap) blocks = cap;
    if (blocks > REDUCE_MAX_BLOCKS) blocks = REDUCE_MAX_BLOCKS;
    if (blocks < 1) blocks = 1;
    static std::atomic<unsigned> launches{0};
    unsigned mark = ++launches;
    if (mark == 0) mark = ++launches;                               // 0 is what a cleared slot holds
    hipLaunchKernelGGL((reduce_kernel<T, 4, OP>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, stream, (const T*)x, (T*)out,
                       (long)n, (unsigned long long*)scratch_mem, mark, reduce_poll_ticks());
    return check_launch(what);
}

template <typename T>
static int run_reduce_op(int op, const void* x, void* out, int64_t n, void* scratch_mem, hipStream_t s, const char* what) {
    switch (op) {
        case SP_REDUCE_SUM: return run_reduce<T, SP_REDUCE_SUM>(x, out, n, scratch_mem, s, what);
        case SP_REDUCE_PROD: return run_reduce<T, SP_REDUCE_PROD>(x, out, n, scratch_mem, s, what);
        case SP_REDUCE_MAX: return run_reduce<T, SP_REDUCE_MAX>(x, out, n, scratch_mem, s, what);
        case SP_REDUCE_MIN: return run_reduce<T, SP_REDUCE_MIN>(x, out, n, scratch_mem, s, what);
    }
    return fail(SP_ERR_ARG, "%s: op must be SP_REDUCE_SUM, _PROD, _MAX or _MIN, got %d", what, op);
}

static int run_reduce_dtype(int op, int dtype, const void* x, void* out, int64_t n, void* scratch_mem, hipStream_t s,
                            const char* what) {
    switch (dtype) {
        case 0: return run_reduce_op<float>(op, x, out, n, scratch_mem, s, what);
        case 1: return run_reduce_op<int>(op, x, out, n, scratch_mem, s, what);
        case 2: return run_reduce_op<unsigned long long>(op, x, out, n, scratch_mem, s, what);
    }
    return fail(SP_ERR_DTYPE, "%s: dtype must be 0 (f32), 1 (i32) or 2 (u64), got %d", what, dtype);
}

}  // namespace sp

using namespace sp;

extern "C" int sp_map_f32(int op, const float* x, float* out, int64_t n, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    if (n <= 0 || n % 4 != 0) return fail(SP_ERR_SHAPE, "sp_map_f32: n must be a positive multiple of 4, got %lld", (long long)n);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const long n4 = n / 4;
    long blocks = (n4 + EW_THREADS - 1) / EW_THREADS;
    const long cap = (long)device_cu_count() * SP_MAP_BLOCKS_PER_CU;
    if (blocks > cap) blocks = cap;
    hipStream_t s = (hipStream_t)stream;
    const f32x4* xi = (const f32x4*)x;
    f32x4* xo = (f32x4*)out;
    switch (op) {
        case SP_MAP_COPY: hipLaunchKernelGGL(map_kernel<SP_MAP_COPY>, dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, xi, xo, n4); break;
        case SP_MAP_RELU: hipLaunchKernelGGL(map_kernel<SP_MAP_RELU>, dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, xi, xo, n4); break;
        case SP_MAP_TANH: hipLaunchKernelGGL(map_kernel<SP_MAP_TANH>, dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, xi, xo, n4); break;
        case SP_MAP_SIGMOID: hipLaunchKernelGGL(map_kernel<SP_MAP_SIGMOID>, dim3((unsigned)blocks), dim3(EW_THREADS), 0, s, xi, xo, n4); break;
        default: return fail(SP_ERR_ARG, "sp_map_f32: unknown op %d", op);
    }
    return check_launch(__func__);
}

extern "C" int64_t sp_reduce_workspace_bytes(void) { return (int64_t)REDUCE_SCRATCH_BYTES; }

extern "C" int sp_reduce(int op, int dtype, const void* x, void* out, int64_t n, void* workspace, int64_t workspace_bytes,
                         void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    SP_REQUIRE_PTR(workspace);
    if (n <= 0) return fail(SP_ERR_SHAPE, "sp_reduce: n must be positive");
    if (op < SP_REDUCE_SUM || op > SP_REDUCE_MIN)
        return fail(SP_ERR_ARG, "sp_reduce: op must be SP_REDUCE_SUM, _PROD, _MAX or _MIN, got %d", op);
    if (dtype < 0 || dtype > 2) return fail(SP_ERR_DTYPE, "sp_reduce: dtype must be 0 (f32), 1 (i32) or 2 (u64), got %d", dtype);
    if (workspace_bytes < sp_reduce_workspace_bytes())
        return fail(SP_ERR_ARG, "sp_reduce: workspace must hold %lld bytes, got %lld",
                    (long long)sp_reduce_workspace_bytes(), (long long)workspace_bytes);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    return run_reduce_dtype(op, dtype, x, out, n, workspace, (hipStream_t)stream, "sp_reduce");
}

extern "C" int sp_reduce_sum(int dtype, const void* x, void* out, int64_t n, void* workspace, int64_t workspace_bytes,
                             void* stream) {
    return sp_reduce(SP_REDUCE_SUM, dtype, x, out, n, workspace, workspace_bytes, stream);
}

extern "C" int sp_reduce_status(const void* workspace, int64_t workspace_bytes, int64_t* give_ups, void* stream) {
    SP_REQUIRE_PTR(workspace);
    if (give_ups == nullptr) return fail(SP_ERR_NULL, "sp_reduce_status: give_ups is NULL");
    if (workspace_bytes < sp_reduce_workspace_bytes())
        return fail(SP_ERR_ARG, "sp_reduce_status: workspace must hold %lld bytes, got %lld",
                    (long long)sp_reduce_workspace_bytes(), (long long)workspace_bytes);
    unsigned long long count = 0;
    hipError_t e = hipMemcpyAsync(&count, (const unsigned long long*)workspace + REDUCE_STATUS_WORD, 8, hipMemcpyDeviceToHost,
                                  (hipStream_t)stream);
    if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "sp_reduce_status: reading the counter failed: %s", hipGetErrorString(e));
    *give_ups = (int64_t)count;
    return SP_OK;
}

extern "C" int sp_reduce_set_poll_limit(int64_t microseconds) {
    if (microseconds > 10000000) return fail(SP_ERR_ARG, "sp_reduce_set_poll_limit: the limit must be at most 10 seconds");
    reduce_poll_ticks_now.store(microseconds == 0 ? REDUCE_POLL_TICKS : microseconds < 0 ? -1 : (long)microseconds * 100,
                                std::memory_order_relaxed);
    return SP_OK;
}

// ---- the sum for callers that cannot allocate: scratch memory inside the library's own image ----
// One copy of this array exists on every GPU the library runs on, for the life of the process.  Host code must not
// use the name as an address (it is a host-side stand-in for the device symbol): the per-device address comes from
// hipGetSymbolAddress, once per device, and everything below uses that pointer.
static __device__ __align__(256) unsigned char scratch[REDUCE_SCRATCH_BYTES];

static int static_scratch(void** out) {
    static std::mutex lock;
    static void* address[64] = {nullptr};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(SP_ERR_DEVICE, "sp_reduce_sum_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> guard(lock);
    if (address[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));   // with device `dev` current: its copy of the array
        if (e != hipSuccess || p == nullptr)
            return fail(SP_ERR_DEVICE, "sp_reduce_sum_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        address[dev] = p;
    }
    *out = address[dev];
    return SP_OK;
}

extern "C" int64_t sp_reduce_sum_static_max_n(void) { return (int64_t)1 << 36; }

extern "C" int sp_reduce_sum_static(int dtype, const void* x, void* out, int64_t n, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    if (n <= 0) return fail(SP_ERR_SHAPE, "sp_reduce_sum_static: n must be positive");
    if (n > sp_reduce_sum_static_max_n())
        return fail(SP_ERR_SHAPE, "sp_reduce_sum_static: n = %lld is beyond the maximum of %lld elements", (long long)n,
                    (long long)sp_reduce_sum_static_max_n());
    if (dtype < 0 || dtype > 2)
        return fail(SP_ERR_DTYPE, "sp_reduce_sum_static: dtype must be 0 (f32), 1 (i32) or 2 (u64), got %d", dtype);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    void* mem = nullptr;
    rc = static_scratch(&mem);
    if (rc != SP_OK) return rc;
    // The array keeps what the last call left in it.  A call that ran to its end leaves its slots at zero and a
    // replayed launch carries the mark of its recording, so the slots are cleared all the same (by a kernel, not a
    // memset, so that the call may be recorded into a graph): this entry point has no caller-owned workspace whose
    // state the caller vouches for.  The give-up counter behind the slots is left alone.
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(EW_THREADS), 0, s, reinterpret_cast<unsigned*>(mem),
                       (int)(REDUCE_SLOT_BYTES / 4));
    rc = check_launch(__func__);
    if (rc != SP_OK) return rc;
    return run_reduce_dtype(SP_REDUCE_SUM, dtype, x, out, n, mem, s, "sp_reduce_sum_static");
}

extern "C" int sp_transpose_inner_b32(const void* from, void* to, int64_t a, int64_t b, int64_t c, void* stream) {
    SP_REQUIRE_PTR(from);
    SP_REQUIRE_PTR(to);
    if (a <= 0 || b <= 0 || c <= 0) return fail(SP_ERR_SHAPE, "sp_transpose_inner_b32: dimensions must be positive");
    if (from == to) return fail(SP_ERR_ARG, "sp_transpose_inner_b32: in-place transpose is not supported");
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const long tiles_b = (b + 63) / 64, tiles_c = (c + 63) / 64;
    const long blocks = a * tiles_b * tiles_c;
    if (blocks > 0x7fffffffL) return fail(SP_ERR_SHAPE, "sp_transpose_inner_b32: too many tiles");
    const bool vec4 = b % 4 == 0 && c % 4 == 0 && ((uintptr_t)from | (uintptr_t)to) % 16 == 0;
    if (vec4)
        hipLaunchKernelGGL(transpose_vec4_kernel, dim3((unsigned)blocks), dim3(EW_THREADS), 0, (hipStream_t)stream,
                           (const unsigned*)from, (unsigned*)to, (long)b, (long)c, tiles_b, tiles_c);
    else
        hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)blocks), dim3(EW_THREADS), 0, (hipStream_t)stream,
                           (const unsigned*)from, (unsigned*)to, (long)b, (long)c, tiles_b, tiles_c);
    return check_launch(__func__);
}
