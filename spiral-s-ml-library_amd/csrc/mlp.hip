// Fused dense-stack forward for gfx950: every workgroup pushes a tile of 64 batch rows through all
// layers.  Activations stay in LDS as 16-bit values (two ping-pong buffers); each layer's weight
// matrix is streamed from L2 through a double-buffered LDS stage in 64-wide K-chunks; products run
// on v_mfma_f32_32x32x16_{f16,bf16} with f32 accumulation; ReLU (and bias) are applied in
// registers; the head (softmax / regret matching / sampling) runs on the last layer's f32
// outputs without leaving the CU.
//
// Semantics follow the graph interpreter of ml/layers.spi:194-240 (BlockMatmul = x . w^T with w
// stored (out, in), relu = max 0) and the heads of ml/primitives.spi:711-722,748-798.
#include "common.h"

#pragma clang fp contract(off)

namespace sp {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int MLP_MAX_LAYERS = 8;
constexpr int MLP_ROWS = 64;       // batch rows per workgroup
constexpr int MLP_THREADS = 256;   // 4 waves; wave w owns output fragments w, w+4, ...
constexpr int MLP_MAX_DIM = 256;   // widest layer input / hidden width
constexpr int MLP_MAX_OUT = 64;    // widest head
constexpr int W_ROW_BYTES = 144;   // 64 16-bit K values + 16 bytes of padding (odd number of 16-byte slots)
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
    int act_stride_bytes;  // (max width + 8) * 2: odd number of 16-byte slots per row
};

template <int DT>
__device__ __forceinline__ unsigned short to_half_bits(float v) {
    if constexpr (DT == SP_F16) {
        _Float16 h = (_Float16)v;
        return __builtin_bit_cast(unsigned short, h);
    } else {
        unsigned u = __float_as_uint(v);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return (unsigned short)(u >> 16);
    }
}

template <int DT>
__global__ __launch_bounds__(MLP_THREADS) void mlp_forward_kernel(const MlpArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const long row0 = (long)blockIdx.x * MLP_ROWS;
    const int stride = a.act_stride_bytes;
    unsigned char* act0 = lds;
    unsigned char* act1 = lds + MLP_ROWS * stride;
    unsigned char* wst = lds + 2 * MLP_ROWS * stride;      // two weight stages of MLP_MAX_DIM rows
    constexpr int WSTAGE = MLP_MAX_DIM * W_ROW_BYTES;

    // ---- stage the input tile (zero rows past the batch) ----
    {
        const int k0 = a.dims[0];
        const int chunks_per_row = k0 / 8;
        const int total = MLP_ROWS * chunks_per_row;
        for (int id = tid; id < total; id += MLP_THREADS) {
            const int r = id / chunks_per_row, c = id % chunks_per_row;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (row0 + r < a.batch)
                v = *reinterpret_cast<const u32x4*>((const unsigned char*)a.x + ((row0 + r) * k0 + c * 8) * 2);
            *reinterpret_cast<u32x4*>(act0 + r * stride + c * 16) = v;
        }
    }

    unsigned char* act_in = act0;
    unsigned char* act_out = act1;

    for (int layer = 0; layer < a.n_layers; ++layer) {
        const int K = a.dims[layer], N = a.dims[layer + 1];
        const int nf = (N + 31) / 32;              // 32-wide output fragments
        const int wrows = nf * 32;
        const bool last = layer + 1 == a.n_layers;
        const unsigned char* W = (const unsigned char*)a.w[layer];
        const int nchunks = (K + 63) / 64;
        const int loads = wrows * 8 / MLP_THREADS;  // 16-byte pieces per thread and chunk (1..8)

        u32x4 rw[8];
        auto fetch = [&](int kc, u32x4(&dst)[8]) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i < loads) {
                    const int id = i * MLP_THREADS + tid;
                    const int n = id >> 3, c = id & 7;
                    const int k = kc * 64 + c * 8;
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (n < N && k < K) v = *reinterpret_cast<const u32x4*>(W + ((long)n * K + k) * 2);
                    dst[i] = v;
                }
            }
        };
        auto stash = [&](int stage, const u32x4(&src)[8]) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (i < loads) {
                    const int id = i * MLP_THREADS + tid;
                    const int n = id >> 3, c = id & 7;
                    *reinterpret_cast<u32x4*>(wst + stage * WSTAGE + n * W_ROW_BYTES + c * 16) = src[i];
                }
            }
        };

        f32x16 acc[2][2];  // [output fragment slot][batch-row fragment]
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[s][m][r] = 0.f;

        fetch(0, rw);
        __syncthreads();  // previous layer's readers of the weight stages and writers of act_in are done
        stash(0, rw);
        __syncthreads();
        for (int kc = 0; kc < nchunks; ++kc) {
            const bool more = kc + 1 < nchunks;
            if (more) fetch(kc + 1, rw);
            const int ksteps = (K - kc * 64) >= 64 ? 4 : (K - kc * 64) / 16;
            const unsigned char* ws = wst + (kc & 1) * WSTAGE;
            for (int ks = 0; ks < ksteps; ++ks) {
                u32x4 fa[2];
#pragma unroll
                for (int m = 0; m < 2; ++m)
                    fa[m] = *reinterpret_cast<const u32x4*>(act_in + (m * 32 + l32) * stride +
                                                            (kc * 64 + ks * 16 + half * 8) * 2);
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int f = wave + 4 * s;
                    if (f < nf) {
                        const u32x4 fw = *reinterpret_cast<const u32x4*>(ws + (f * 32 + l32) * W_ROW_BYTES +
                                                                         (ks * 16 + half * 8) * 2);
#pragma unroll
                        for (int m = 0; m < 2; ++m) {
                            // weights as the first operand: the result fragment is (n, batch row), so a
                            // lane ends up with 4 consecutive n of one row -> one 8-byte store
                            if constexpr (DT == SP_F16)
                                acc[s][m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                                    __builtin_bit_cast(f16x8, fw), __builtin_bit_cast(f16x8, fa[m]), acc[s][m], 0, 0, 0);
                            else
                                acc[s][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                    __builtin_bit_cast(bf16x8, fw), __builtin_bit_cast(bf16x8, fa[m]), acc[s][m], 0, 0, 0);
                        }
                    }
                }
            }
            if (more) stash((kc + 1) & 1, rw);
            __syncthreads();
        }

        // ---- layer epilogue: lane holds rows m*32 + l32, columns f*32 + 8*g + 4*half + 0..3 ----
        const float* bias = a.b[layer];
        float* lg = reinterpret_cast<float*>(wst);  // f32 staging of the last layer's outputs [64][wrows]
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int f = wave + 4 * s;
            if (f >= nf) continue;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const int r_loc = m * 32 + l32;
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    const int n = f * 32 + gq * 8 + half * 4;
                    float v[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        v[q] = acc[s][m][gq * 4 + q];
                        if (bias != nullptr && n + q < N) v[q] += bias[n + q];
                    }
                    if (!last) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) v[q] = fmaxf(v[q], 0.f);
                        u32x2 packed;
                        packed.x = (unsigned)to_half_bits<DT>(v[0]) | ((unsigned)to_half_bits<DT>(v[1]) << 16);
                        packed.y = (unsigned)to_half_bits<DT>(v[2]) | ((unsigned)to_half_bits<DT>(v[3]) << 16);
                        *reinterpret_cast<u32x2*>(act_out + r_loc * stride + n * 2) = packed;
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; ++q) lg[r_loc * wrows + n + q] = v[q];
                    }
                }
            }
        }
        unsigned char* t = act_in; act_in = act_out; act_out = t;
    }
    __syncthreads();

    // ---- head: one thread per batch row ----
    if (tid < MLP_ROWS && row0 + tid < a.batch) {
        const int N = a.dims[a.n_layers];
        const int wrows = ((N + 31) / 32) * 32;
        float* p = reinterpret_cast<float*>(wst) + tid * wrows;  // this row's outputs, updated in place
        const long row = row0 + tid;
        const int limit = a.mask_size > 0 ? a.mask_size : N;
        if (a.logits != nullptr)
            for (int j = 0; j < N; ++j) a.logits[row * N + j] = p[j];
        if (a.head == SP_HEAD_SOFTMAX || a.head == SP_HEAD_SOFTMAX_RM) {
            float m = -__builtin_inff();
            for (int j = 0; j < limit; ++j) m = fmaxf(m, p[j]);
            float s = 0.f;
            for (int j = 0; j < N; ++j) {
                p[j] = j < limit ? expf(p[j] - m) : 0.f;
                s = s + p[j];
            }
            for (int j = 0; j < N; ++j) p[j] = p[j] / s;
        }
        if (a.head == SP_HEAD_REGRET_MATCHING || a.head == SP_HEAD_SOFTMAX_RM) {
            float s = 0.f;
            for (int j = 0; j < N; ++j) {
                p[j] = j < limit ? fmaxf(p[j], 0.f) : 0.f;
                s = s + p[j];
            }
            const float inv_len = 1.f / (float)limit;
            for (int j = 0; j < N; ++j) p[j] = j < limit ? (s != 0.f ? p[j] / s : inv_len) : 0.f;
        }
        for (int j = 0; j < N; ++j) a.policy[row * N + j] = p[j];
        if (a.action != nullptr) {
            // local_discrete_sampling (ml/primitives.spi:782-798), sequential prefix sums
            float run = 0.f, m = -__builtin_inff();
            for (int j = 0; j < N; ++j) {
                run = run + p[j];
                if (p[j] > 0.f) m = fmaxf(m, run);
            }
            const float thr = a.u[row] * m;
            int pick = INT_MAX_;
            run = 0.f;
            for (int j = 0; j < N; ++j) {
                run = run + p[j];
                if (pick == INT_MAX_ && p[j] > 0.f && run >= thr) pick = j;
            }
            a.action[row] = pick;
        }
    }
}

}  // namespace sp

using namespace sp;

extern "C" int sp_mlp_forward(int dtype, const void* x, int32_t n_layers, const void* const* weights,
                              const float* const* biases, const int32_t* dims, const float* u, float* policy_out,
                              int32_t* action_out, float* logits_out, int64_t batch, int32_t head, int32_t mask_size,
                              void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(policy_out);
    SP_OPTIONAL_PTR(u); SP_OPTIONAL_PTR(action_out); SP_OPTIONAL_PTR(logits_out);
    if (weights == nullptr || dims == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward: weights/dims is NULL");
    if (dtype != SP_F16 && dtype != SP_BF16) return fail(SP_ERR_DTYPE, "sp_mlp_forward: dtype must be f16 or bf16");
    if (n_layers < 1 || n_layers > MLP_MAX_LAYERS)
        return fail(SP_ERR_ARG, "sp_mlp_forward: n_layers must be in [1, %d], got %d", MLP_MAX_LAYERS, n_layers);
    if (batch <= 0) return fail(SP_ERR_SHAPE, "sp_mlp_forward: batch must be positive");
    if (head < SP_HEAD_NONE || head > SP_HEAD_SOFTMAX_RM) return fail(SP_ERR_ARG, "sp_mlp_forward: unknown head %d", head);
    if (action_out != nullptr && u == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward: action requested but u is NULL");
    MlpArgs a{};
    int maxw = 0;
    for (int i = 0; i <= n_layers; ++i) {
        const int d = dims[i];
        if (d <= 0) return fail(SP_ERR_SHAPE, "sp_mlp_forward: dims[%d] must be positive", i);
        if (i < n_layers) {
            if (d % 16 != 0 || d > MLP_MAX_DIM)
                return fail(SP_ERR_SHAPE, "sp_mlp_forward: dims[%d] = %d must be a multiple of 16 and <= %d", i, d,
                            MLP_MAX_DIM);
            if (i > 0 && d % 32 != 0)
                return fail(SP_ERR_SHAPE, "sp_mlp_forward: hidden width dims[%d] = %d must be a multiple of 32", i, d);
            if (d > maxw) maxw = d;
        } else if (d > MLP_MAX_OUT) {
            return fail(SP_ERR_SHAPE, "sp_mlp_forward: output width %d must be <= %d", d, MLP_MAX_OUT);
        }
        a.dims[i] = d;
    }
    if (mask_size < 0 || mask_size > dims[n_layers])
        return fail(SP_ERR_ARG, "sp_mlp_forward: mask_size must be in [0, %d], got %d", dims[n_layers], mask_size);
    for (int i = 0; i < n_layers; ++i) {
        if (weights[i] == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward: weights[%d] is NULL", i);
        if (!aligned16(weights[i])) return fail(SP_ERR_ALIGN, "sp_mlp_forward: weights[%d] is not 16-byte aligned", i);
        a.w[i] = weights[i];
        a.b[i] = biases ? biases[i] : nullptr;
    }
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    a.x = x; a.n_layers = n_layers; a.u = u; a.policy = policy_out; a.action = action_out; a.logits = logits_out;
    a.batch = batch; a.head = head; a.mask_size = mask_size;
    a.act_stride_bytes = (maxw + 8) * 2;
    const int lds_bytes = 2 * MLP_ROWS * a.act_stride_bytes + 2 * MLP_MAX_DIM * W_ROW_BYTES;
    auto kernel = dtype == SP_F16 ? mlp_forward_kernel<SP_F16> : mlp_forward_kernel<SP_BF16>;
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "hipFuncSetAttribute failed: %s", hipGetErrorString(e));
    const long blocks = (batch + MLP_ROWS - 1) / MLP_ROWS;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(MLP_THREADS), lds_bytes, (hipStream_t)stream, a);
    return check_launch(__func__);
}
