// Pieces shared by the fused dense-stack kernels (mlp.hip, mlp_packed.hip): argument block, the head of a
// batch row (softmax / regret matching / sampling), packed conversions, the LDS DMA.
#pragma once
#include "common.h"
#include "philox.h"

#pragma clang fp contract(off)

namespace sp {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int MLP_MAX_LAYERS = 8;
constexpr int MLP_MAX_DIM = 256;       // widest layer input / hidden width
constexpr int MLP_MAX_OUT = 64;        // widest head
constexpr int MLP_STAGES = 4;
constexpr int MLP_STAGE_BYTES = MLP_MAX_DIM * 128;   // 256 weight rows x 64 K-columns x 2 bytes
constexpr int MLP_DMA_PER_CHUNK = MLP_MAX_DIM / 8;         // 1 KiB DMA instructions per full chunk
constexpr int INT_MAX_ = 2147483647;

struct MlpArgs {
    const void* x;
    const void* w[MLP_MAX_LAYERS];
    const float* b[MLP_MAX_LAYERS];
    int dims[MLP_MAX_LAYERS + 1];
    int n_layers;
    const float* u;
    float* policy;
    int* action;
    float* logits;
    long batch;
    int head;
    int mask_size;
    int k0, nout;        // dims[0] and dims[n_layers] once more, so that a kernel needs no dependent load for them
    int out_stride;      // floats between two rows of policy / logits (= dims[n_layers]; nout may be smaller, see sp_mlp_forward)
    PhiloxStream ph;     // philox_mode >= 0: the head draws its uniform itself (ml/layers.spi:339-344) and `u` is not read
};

// Arguments of the kernel that keeps a stack's weights in registers and walks over many 64-row tiles per compute
// unit (mlp_resident.hip); both sp_mlp_forward and sp_mlp_forward_packed hand large batches to it.
struct MlpResidentArgs {
    const void* x;
    const void* packed;                  // packed weights (PACKED instantiations)
    const void* w[4];                    // row-major weights (the others)
    const float* b[4];
    const float* u;
    float* policy;
    int* action;
    float* logits;
    long batch;
    int tiles;                           // steps of the walk (filled in by mlp_resident_launch)
    int head, mask_size, k0, nout, out_stride;
    PhiloxStream ph;
};

bool mlp_resident_takes(int n_layers, const int32_t* dims, int nout);
int mlp_resident_launch(int dtype, bool packed, int n_layers, MlpResidentArgs a, hipStream_t stream, const char* what);
// The same for four-layer stacks with at most 4 computed outputs: the two 256 x 256 layers as a two-stage pipeline on
// the two waves of every SIMD (mlp_pipe.hip).  mlp_resident_launch hands such stacks on to it.
bool mlp_pipe_takes(int n_layers, const int32_t* dims, int nout);
int mlp_pipe_launch(int dtype, bool packed, MlpResidentArgs a, hipStream_t stream, const char* what);
// 64-row tiles per compute unit from which the resident kernel is used: its one-time load of all weights has to pay,
// and it walks tiles in pairs, so few tiles per unit leave units idle in the last round.  Measured against the
// per-tile kernels (32 -> 256 -> 256 -> 256 -> 3, us per launch, per-tile / resident): packed weights 65536 rows
// 19.7 / 19.6, 98304 29.1 / 26.7, 131072 39.1 / 33.8, 262144 76.3 / 61.8; row-major weights (which stream in at about
// a quarter of the rate) 98304 31.8 / 32.7, 131072 42.7 / 39.9, 262144 81.7 / 69.3.
#ifndef SP_MLP_RESIDENT_MIN_TILES_PACKED
#define SP_MLP_RESIDENT_MIN_TILES_PACKED 6
#endif
#ifndef SP_MLP_RESIDENT_MIN_TILES_ROWMAJOR
#define SP_MLP_RESIDENT_MIN_TILES_ROWMAJOR 8
#endif

// The same thresholds for the stacks the pipelined kernel takes (it fills faster than the resident one pays back its
// weight load).  Measured, us per launch, per-tile kernels / pipelined, packed weights: 32768 rows 10.3 / 12.4, 49152
// 15.2 / 15.4, 65536 19.9 / 18.2, 81920 25.0 / 24.3, 98304 29.3 / 24.5, 131072 38.5 / 30.7; row-major weights: 65536
// 21.6 / 23.2, 81920 30.9 / 26.6, 98304 31.8 / 29.4, 131072 41.9 / 36.0.  (Resident / pipelined on the stacks both take:
// 98304 rows 26.1 / 24.6, 262144 61.4 / 55.9, 1048576 230.2 / 207.4: the pipelined one wherever it applies.)
#ifndef SP_MLP_PIPE_MIN_TILES_PACKED
#define SP_MLP_PIPE_MIN_TILES_PACKED 4
#endif
#ifndef SP_MLP_PIPE_MIN_TILES_ROWMAJOR
#define SP_MLP_PIPE_MIN_TILES_ROWMAJOR 5
#endif

// The Philox stream of a head that draws its own uniforms: the sampling node of the layer graph works on rows of
// `cols` = the last layer's full width, which the reference's row primitives need to be a multiple of 4.
inline int mlp_set_philox(PhiloxStream& ph, const sp_philox_t* philox, int64_t batch, int cols, const char* fn) {
    ph.philox_mode = -1;
    if (philox == nullptr) return SP_OK;
    if (cols % 4 != 0)
        return fail(SP_ERR_ARG, "%s: a head that draws from a Philox stream needs an output width that is a multiple of 4 (the "
                    "row width of the sampling op whose stream it follows), got %d", fn, cols);
    ph.cols = cols;
    return set_philox(ph, philox, batch, (int64_t)cols, fn);
}

// max(x, 0) and rounding of two f32 values to the 16-bit storage type, packed into one register
// (v_max_f32 + v_cvt_pk_{f16,bf16}_f32: round to nearest even in hardware).  The max is issued from
// assembly because fmaxf() would first canonicalise its operand with a second v_max.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <int DT>
__device__ __forceinline__ unsigned relu_pack2(float a, float b) {
    float ra, rb;
    asm("v_max_f32 %0, 0, %1" : "=v"(ra) : "v"(a));
    asm("v_max_f32 %0, 0, %1" : "=v"(rb) : "v"(b));
    if constexpr (DT == SP_F16) return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{ra, rb}, f16x2));
    else return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{ra, rb}, bf16x2));
}

// One wave-wide DMA: lane i copies 16 bytes from base + lane_offset to LDS byte lds_addr + 16 * i.
// Issued from inline assembly so the chunks in flight do not make the compiler wait before LDS
// reads of the chunk being multiplied; completion is tracked by vmcnt.
__device__ __forceinline__ void mlp_dma(const unsigned char* base, unsigned lane_offset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
}

// Head of one batch row: optional softmax and/or regret matching over the columns j < limit, then
// local_discrete_sampling (ml/primitives.spi:782-798) with sequential prefix sums.  `src` holds the
// row's N last-layer outputs; MAXN bounds N at compile time so that narrow heads stay in registers.
// Columns past `limit` enter the softmax as -inf and leave it as exact zeros, columns past N are zeros
// from the start: sums over all MAXN columns then equal the sums over the valid ones bit for bit, and
// the loops need no per-column conditions.
struct HeadOut {
    float* policy;
    int* action;
    float* logits;
    int head;
    int stride;   // floats between two rows of policy / logits; columns N .. stride - 1 of policy are written as zeros
};
__device__ __forceinline__ HeadOut head_out(const MlpArgs& a) {
    return HeadOut{a.policy, a.action, a.logits, a.head, a.out_stride};
}

template <int MAXN>
__device__ __forceinline__ void head_row(const HeadOut& o, const float* src, long row, int N, int limit, float u,
                                         int fill_end = 1 << 30) {
    float p[MAXN];
#pragma unroll
    for (int n = 0; n < MAXN; ++n) p[n] = n < N ? src[n] : 0.f;
    if (o.logits != nullptr) {
#pragma unroll
        for (int n = 0; n < MAXN; ++n)
            if (n < N) o.logits[row * o.stride + n] = p[n];
    }
    // exp on the hardware exp2 unit and one hardware reciprocal (1 ulp) per normalisation: a 16-lane
    // serial head is otherwise a visible part of a forward pass that takes a few microseconds
    if (o.head == SP_HEAD_SOFTMAX || o.head == SP_HEAD_SOFTMAX_RM) {
        float m = -__builtin_inff();
#pragma unroll
        for (int n = 0; n < MAXN; ++n) {
            p[n] = n < limit ? p[n] : -__builtin_inff();
            m = fmaxf(m, p[n]);
        }
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < MAXN; ++n) {
            p[n] = __builtin_amdgcn_exp2f((p[n] - m) * 1.44269504088896340736f);
            s = s + p[n];
        }
        const float inv = __builtin_amdgcn_rcpf(s);
#pragma unroll
        for (int n = 0; n < MAXN; ++n) p[n] = p[n] * inv;
    }
    if (o.head == SP_HEAD_REGRET_MATCHING || o.head == SP_HEAD_SOFTMAX_RM) {
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < MAXN; ++n) {
            p[n] = n < limit ? fmaxf(p[n], 0.f) : 0.f;
            s = s + p[n];
        }
        const float inv_len = __builtin_amdgcn_rcpf((float)limit);
        const float inv = s != 0.f ? __builtin_amdgcn_rcpf(s) : 0.f;
#pragma unroll
        for (int n = 0; n < MAXN; ++n) p[n] = s != 0.f ? p[n] * inv : (n < limit ? inv_len : 0.f);
    }
#pragma unroll
    for (int n = 0; n < MAXN; ++n)
        if (n < N) o.policy[row * o.stride + n] = p[n];
    if (o.stride > N) {   // a masked head computed for its valid columns only: the rest of the row is exact zeros
        float* tail = o.policy + row * o.stride;   // (up to fill_end: the caller may fill the rest with whole waves)
        const int end = o.stride < fill_end ? o.stride : fill_end;
        int c = N;
        for (; c < end && ((c & 3) != 0 || (o.stride & 3) != 0); ++c) tail[c] = 0.f;
        for (; c + 4 <= end; c += 4) *reinterpret_cast<float4*>(tail + c) = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (o.action != nullptr) {
        float run = 0.f, m = -__builtin_inff();
        float cdf[MAXN];
#pragma unroll
        for (int n = 0; n < MAXN; ++n) {
            run = run + p[n];
            cdf[n] = run;
            if (p[n] > 0.f) m = fmaxf(m, run);
        }
        const float thr = u * m;
        int pick = INT_MAX_;
#pragma unroll
        for (int n = MAXN - 1; n >= 0; --n)
            if (p[n] > 0.f && cdf[n] >= thr) pick = n;
        o.action[row] = pick;
    }
}

// The same for at most 4 outputs with the head kind as a template parameter (the caller switches on it once):
// a short straight line instead of a chain of small blocks, each of which is a jump into code the instruction
// cache has not seen yet.  Same formulas, same order of operations as head_row<4>.
template <int HEAD>
__device__ __forceinline__ void head_row4(const HeadOut& o, const float (&src)[4], long row, int N, int limit, float u,
                                          int fill_end) {
    float p[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) p[n] = n < N ? src[n] : 0.f;
    float* const policy_row = o.policy + row * o.stride;
    if (o.logits != nullptr) {
        float* logits_row = o.logits + row * o.stride;
#pragma unroll
        for (int n = 0; n < 4; ++n)
            if (n < N) logits_row[n] = p[n];
    }
    if constexpr (HEAD == SP_HEAD_SOFTMAX || HEAD == SP_HEAD_SOFTMAX_RM) {
        float m = -__builtin_inff();
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = n < limit ? p[n] : -__builtin_inff();
            m = fmaxf(m, p[n]);
        }
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = __builtin_amdgcn_exp2f((p[n] - m) * 1.44269504088896340736f);
            s = s + p[n];
        }
        const float inv = __builtin_amdgcn_rcpf(s);
#pragma unroll
        for (int n = 0; n < 4; ++n) p[n] = p[n] * inv;
    }
    if constexpr (HEAD == SP_HEAD_REGRET_MATCHING || HEAD == SP_HEAD_SOFTMAX_RM) {
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = n < limit ? fmaxf(p[n], 0.f) : 0.f;
            s = s + p[n];
        }
        const float inv_len = __builtin_amdgcn_rcpf((float)limit);
        const float inv = s != 0.f ? __builtin_amdgcn_rcpf(s) : 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) p[n] = s != 0.f ? p[n] * inv : (n < limit ? inv_len : 0.f);
    }
#pragma unroll
    for (int n = 0; n < 4; ++n)
        if (n < N) policy_row[n] = p[n];
    if (o.stride > N) {   // a masked head computed for its valid columns only: the rest of the row is exact zeros
        const int end = o.stride < fill_end ? o.stride : fill_end;      // (past fill_end the caller fills with whole waves)
        for (int c = N; c < end; ++c) policy_row[c] = 0.f;
    }
    if (o.action != nullptr) {
        float run = 0.f, m = -__builtin_inff();
        float cdf[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            run = run + p[n];
            cdf[n] = run;
            if (p[n] > 0.f) m = fmaxf(m, run);
        }
        const float thr = u * m;
        int pick = INT_MAX_;
#pragma unroll
        for (int n = 3; n >= 0; --n)
            if (p[n] > 0.f && cdf[n] >= thr) pick = n;
        o.action[row] = pick;
    }
}

// The commonest shape of all, as short as it gets (every byte of a head is fetched cold, once per launch, at about a
// cycle per byte): at most 4 outputs packed densely (row stride N), no logits wanted, an action wanted.
template <int HEAD>
__device__ __forceinline__ void head_row4_plain(float* policy, int* action, const float (&src)[4], long row, int N, int limit, float u) {
    float p[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) p[n] = n < N ? src[n] : 0.f;
    if constexpr (HEAD == SP_HEAD_SOFTMAX || HEAD == SP_HEAD_SOFTMAX_RM) {
        float m = -__builtin_inff();
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = n < limit ? p[n] : -__builtin_inff();
            m = fmaxf(m, p[n]);
        }
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = __builtin_amdgcn_exp2f((p[n] - m) * 1.44269504088896340736f);
            s = s + p[n];
        }
        const float inv = __builtin_amdgcn_rcpf(s);
#pragma unroll
        for (int n = 0; n < 4; ++n) p[n] = p[n] * inv;
    }
    if constexpr (HEAD == SP_HEAD_REGRET_MATCHING || HEAD == SP_HEAD_SOFTMAX_RM) {
        float s = 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = n < limit ? fmaxf(p[n], 0.f) : 0.f;
            s = s + p[n];
        }
        const float inv_len = __builtin_amdgcn_rcpf((float)limit);
        const float inv = s != 0.f ? __builtin_amdgcn_rcpf(s) : 0.f;
#pragma unroll
        for (int n = 0; n < 4; ++n) p[n] = s != 0.f ? p[n] * inv : (n < limit ? inv_len : 0.f);
    }
    float* const policy_row = policy + row * N;
    policy_row[0] = p[0];
    if (N > 1) policy_row[1] = p[1];
    if (N > 2) policy_row[2] = p[2];
    if (N > 3) policy_row[3] = p[3];
    float run = 0.f, m = -__builtin_inff();
    float cdf[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
        run = run + p[n];
        cdf[n] = run;
        if (p[n] > 0.f) m = fmaxf(m, run);
    }
    const float thr = u * m;
    int pick = INT_MAX_;
#pragma unroll
    for (int n = 3; n >= 0; --n)
        if (p[n] > 0.f && cdf[n] >= thr) pick = n;
    action[row] = pick;
}

template <typename... A>
__device__ __forceinline__ void head_row4_plain_any(int head, A&&... args) {
    switch (head) {
        case SP_HEAD_SOFTMAX_RM: head_row4_plain<SP_HEAD_SOFTMAX_RM>(args...); break;
        case SP_HEAD_SOFTMAX: head_row4_plain<SP_HEAD_SOFTMAX>(args...); break;
        case SP_HEAD_REGRET_MATCHING: head_row4_plain<SP_HEAD_REGRET_MATCHING>(args...); break;
        default: head_row4_plain<SP_HEAD_NONE>(args...); break;
    }
}

template <typename... A>
__device__ __forceinline__ void head_row4_any(int head, A&&... args) {
    switch (head) {
        case SP_HEAD_SOFTMAX: head_row4<SP_HEAD_SOFTMAX>(args...); break;
        case SP_HEAD_REGRET_MATCHING: head_row4<SP_HEAD_REGRET_MATCHING>(args...); break;
        case SP_HEAD_SOFTMAX_RM: head_row4<SP_HEAD_SOFTMAX_RM>(args...); break;
        default: head_row4<SP_HEAD_NONE>(args...); break;
    }
}

__device__ __forceinline__ int mlp_swz(int row) { return (((row >> 3) & 3) << 1) | ((row >> 1) & 1); }


template <int N>
struct IC { static constexpr int value = N; };

// relu + rounding of four f32 to the 16-bit storage type: round first (v_cvt_pk), then clamp the two
// packed values at zero as signed 16-bit integers -- a negative float of either format has the sign
// bit set, so it is a negative integer, and relu commutes with the sign-symmetric rounding.
template <int DT>
__device__ __forceinline__ unsigned pack_relu2(float a, float b) {
    unsigned p;
    if constexpr (DT == SP_F16) p = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, f16x2));
    else p = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
    unsigned r;
    asm("v_pk_max_i16 %0, %1, 0" : "=v"(r) : "v"(p));
    return r;
}


}  // namespace sp
