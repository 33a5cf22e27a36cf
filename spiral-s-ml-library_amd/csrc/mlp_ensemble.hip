// Fused forward of an ENSEMBLE of small f32 stacks on one shared input: member e of E computes
//     policy[e] = head(relu(x . W1[e]^T) . W2[e]^T)          x: (batch, K0), W1: (E, 64, K0), W2: (E, N, 64), all f32
// in one launch, activations never leaving registers.  This is the graph of the reference's Leduc policy
// (game/leduc/model_cem.spi:55-63: input -> matmul_ensemble_with_adjoint (E, 128, 64) -> relu ->
// matmul_ensemble_with_adjoint (E, 64, 64) -> masked_regret_matching' 3), which the graph interpreter
// (ml/layers.spi:194-240, 336-344) runs member by member, node by node.
//
// One wave per SIMD (four per workgroup, nothing shared between them: no LDS, no barrier).  A wave loads the weights
// of its member once -- 128 registers for the first layer, 32 per computed output for the second -- and walks over
// 32-row tiles of the batch.
//   Layer 1 is v_mfma_f32_32x32x2_f32 with the WEIGHTS as the row operand, so a result tile is (features x batch rows)
// and lane (r, g) -- r = lane % 32 the batch row, g = lane / 32 -- holds features 8 a + 4 g + b (a, b = 0..3) of row
// r in register 4 a + b.  Both operands of an MFMA step take their two K-values from the lane halves g = 0, 1, and
// WHICH K-index a (step, half) pair stands for is free as long as both operands agree: step 4 j + i, half g stands
// for k = 8 j + 4 g + i, so every lane's inputs and weights are 16-byte loads.
//   Layer 2 is computed for at most 4 outputs (a masked head's valid columns, or a head that narrow), which is too
// little for the matrix pipe (a 32 x 32 tile for 3 useful rows costs a quarter of layer 1): every lane multiplies the
// 32 features of its row that it holds (after the relu) with the matching weights -- fused multiply-adds on the
// vector ALU -- and the two halves of a row are added across the lane halves.
// Sums therefore add up in another order than a row-by-row dot product; f32 throughout.  Tiles go through in pairs: the lanes
// with g = 0 run the head for their row of the first tile, the lanes with g = 1 for the second; the zeros behind the
// valid columns of a masked head are written by the whole wave, 16 bytes per lane.
#include "mlp_common.h"

#pragma clang fp contract(off)

namespace sp {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int EN_ROWS = 32;       // batch rows per tile
constexpr int EN_HIDDEN = 64;     // width of the hidden layer
constexpr int EN_THREADS = 256;
constexpr int EN_MAX_OUT = 4;     // computed outputs

struct EnsembleArgs {
    const float* x;
    const float* w1;
    const float* w2;
    const float* u;               // (members, batch) uniforms, or nullptr
    float* policy;                // (members, batch, n)
    int* action;                  // (members, batch), or nullptr
    long batch, tiles;
    int members, k0, n, nout, head, mask_size;
    unsigned* words;              // (members, batch) hash words of the binarize head, or nullptr
    unsigned modulo;
    PhiloxStream ph;
};

// KG: 8-wide groups of the input width the kernel is unrolled for; EXACT: K0 = 8 KG (else K0 < 8 KG and the groups
// past K0 are zeros); ACTION: an action per row is wanted (a uniform per row, from a tensor or a Philox stream)
template <int KG, bool EXACT, bool ACTION>
__global__ __launch_bounds__(EN_THREADS) void mlp_ensemble_kernel(const EnsembleArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int e = blockIdx.y;
    const int K0 = EXACT ? 8 * KG : a.k0;
    const int N = a.n, NOUT = a.nout;
    const int groups = K0 >> 3;
    const long batch = a.batch, tiles = a.tiles;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

    // ---- the member's weights, once ----
    f32x4 w1v[2][KG];             // [feature tile][j]: W1[e][32 t + r][8 j + 4 g .. + 3]
    {
        const float* w1 = a.w1 + (long)e * EN_HIDDEN * K0;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < KG; ++j) {
                const int jj = EXACT || j < groups ? j : 0;
                const f32x4 v = *reinterpret_cast<const f32x4*>(w1 + (long)(32 * t + r) * K0 + 8 * jj + 4 * g);
                w1v[t][j] = EXACT || j < groups ? v : zero4;
            }
    }
    f32x4 w2v[EN_MAX_OUT][2][4];  // [output][t][a]: W2[e][o][32 t + 8 a + 4 g .. + 3]: the features this lane half holds
    {
        const float* w2 = a.w2 + (long)e * N * EN_HIDDEN;
#pragma unroll
        for (int o = 0; o < EN_MAX_OUT; ++o)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int a4 = 0; a4 < 4; ++a4) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(w2 + (long)(o < NOUT ? o : 0) * EN_HIDDEN + 32 * t + 8 * a4 + 4 * g);
                    w2v[o][t][a4] = o < NOUT ? v : zero4;
                }
    }

    // inputs of a tile: lane (r, g) takes x[row0 + r][8 j + 4 g .. + 3]; rows past the batch read the last row (their
    // results are not stored), groups past K0 read group 0 and count as zeros
    auto x_row = [&](long tile) {
        long row = tile * EN_ROWS + r;
        row = row < batch ? row : batch - 1;
        return a.x + row * K0 + 4 * g;
    };
    auto load_piece = [&](const float* xr, int j) { return *reinterpret_cast<const f32x4*>(xr + 8 * (EXACT || j < groups ? j : 0)); };

    const long stride = (long)gridDim.x * 4;
    long tile = (long)blockIdx.x * 4 + wave;
    if (tile >= tiles) return;
    f32x4 xv[KG];
    {
        const float* xr = x_row(tile);
#pragma unroll
        for (int j = 0; j < KG; ++j) xv[j] = load_piece(xr, j);
    }
    const HeadOut out = HeadOut{a.policy, ACTION ? a.action : nullptr, nullptr, a.head, N};
    const int limit = a.mask_size > 0 ? a.mask_size : NOUT;
    const bool wave_fill = N > NOUT && (N & 3) == 0;
    const int s4 = N >> 2, c0 = (NOUT + 3) >> 2;

    // The zeros behind the valid columns of a masked head are written by the whole wave, 16 bytes per lane: lane l takes
    // pieces l, l + 64, ... of a tile's 32 s4 pieces.  64-wide rows (16 pieces): a lane's pieces are 1 KiB apart, all in
    // one column -- eight stores in a straight line; other widths walk (row and column of a piece advance by fixed
    // steps: no division inside the walk).
    const int fill_r0 = wave_fill ? lane / s4 : 0, fill_c0 = wave_fill ? lane - fill_r0 * s4 : 0;
    const int fill_dr = wave_fill ? 64 / s4 : 0, fill_dc = wave_fill ? 64 - fill_dr * s4 : 0;
    auto fill_zeros = [&](long t) {
        const long row0 = t * EN_ROWS;
        float* block = a.policy + ((long)e * batch + row0) * N;
        const int rows_here = batch - row0 < EN_ROWS ? (int)(batch - row0) : EN_ROWS;
        if (s4 == 16 && rows_here == EN_ROWS) {
            if (fill_c0 >= c0) {
                f32x4* mine = reinterpret_cast<f32x4*>(block) + lane;
#pragma unroll
                for (int k = 0; k < 8; ++k) mine[64 * k] = zero4;
            }
        } else {
            int rr = fill_r0, c = fill_c0;
            for (int idx = lane; idx < EN_ROWS * s4; idx += 64) {
                if (c >= c0 && rr < rows_here) *reinterpret_cast<f32x4*>(block + rr * N + 4 * c) = zero4;
                rr += fill_dr;
                c += fill_dc;
                if (c >= s4) {
                    c -= s4;
                    ++rr;
                }
            }
        }
    };

    // Both layers of one tile; the outputs of row r end up in BOTH lanes (r, 0) and (r, 1).
    auto forward = [&](long next_tile, float (&p)[4]) {
        // ---- layer 1: (64 features x 32 rows) += W1 . x^T, two K-values per step.  A register of inputs is asked for
        //      the NEXT tile's values as soon as this tile's MFMAs have read it: they arrive a whole tile ahead. ----
        const float* const xr_next = x_row(next_tile);
        f32x16 acc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
#pragma unroll
        for (int j = 0; j < KG; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(w1v[t][j][i], xv[j][i], acc[t], 0, 0, 0);
            xv[j] = load_piece(xr_next, j);
            __builtin_amdgcn_sched_barrier(0);      // (keeps every load behind the MFMAs that free its register)
        }
        // ---- relu; layer 2: this lane's 32 features of its row against the matching weights, then the other half's ----
#pragma unroll
        for (int o = 0; o < EN_MAX_OUT; ++o) {
            p[o] = 0.f;
            if (o >= NOUT) continue;                           // (uniform)
            float s0 = 0.f, s1 = 0.f;                          // (two chains: an FMA need not wait for the one before)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    s0 = __builtin_fmaf(w2v[o][t][i >> 2][i & 3], fmaxf(acc[t][i], 0.f), s0);
                    s1 = __builtin_fmaf(w2v[o][t][(i + 1) >> 2][(i + 1) & 3], fmaxf(acc[t][i + 1], 0.f), s1);
                }
            const float mine = s0 + s1;
            p[o] = mine + __shfl_xor(mine, 32);
        }
    };

    // Tiles go through in pairs and the heads of a pair run together -- lanes (r, 0) finish row r of the first tile,
    // lanes (r, 1) row r of the second: the head is a chain of dependent instructions that costs the same for 64 lanes
    // as for 32, and vector-ALU work does not hide behind f32 MFMAs.
    for (; tile < tiles; tile += 2 * stride) {
        const long tile_b = tile + stride;
        const bool has_b = tile_b < tiles;                      // (uniform)
        float p[4] = {0.f, 0.f, 0.f, 0.f};                     // of this lane's row: the first tile's for g = 0, the second's for g = 1
#pragma unroll 1
        for (int half = 0; half < (has_b ? 2 : 1); ++half) {
            const long after = tile + (half + 1) * stride;      // the tile whose inputs are requested meanwhile
            float ph[4];
            forward(after < tiles ? after : tile, ph);
#pragma unroll
            for (int n = 0; n < 4; ++n) p[n] = g == half ? ph[n] : p[n];
        }
        int fill_end = 1 << 30;
        if (wave_fill) {
            fill_end = 4 * c0;
            fill_zeros(tile);
            if (has_b) fill_zeros(tile_b);
        }
        const long my_tile = g == 0 ? tile : tile_b;
        const long my_row = my_tile * EN_ROWS + r;
        if ((g == 0 || has_b) && my_row < batch) {
            const long grow = (long)e * batch + my_row;
            float u = 1.f;
            if constexpr (ACTION) u = a.u != nullptr ? a.u[grow] : reference_row_uniform(a.ph, grow);
            head_row4_any(a.head, out, p, grow, NOUT, limit, u, fill_end);
        }
    }
}

// ONE ensemble layer and its head: policy[e] = head(x . W[e]^T) for a head of at most 4 computed outputs, or
// word[e][r] = (OR over j < 32 of (not (y[r][j] <= 0)) << j) mod modulo with y = x . W[e]^T -- the graphs of the
// reference's other agents (game/nl_hu_holdem/model_cem.spi:84-100: matmul_ensemble_with_adjoint -> masked regret
// matching; game/leduc/model_cfr.spi:56-61 and game/nl_hu_holdem/model_cfr.spi:82-88: matmul_ensemble -> binarize,
// ml/primitives.spi:817-821).  Either head needs at most the first 32 output columns, so the layer is ONE 32 x 32
// MFMA tile per 32 batch rows (the weights' rows past the needed columns are zeros) instead of the full product, and the
// (members x batch x outputs) activations are never written.  Same walk, same operand mapping and the same input
// prefetch as the first layer of the kernel above; lane (r, g) ends up with outputs 8 a + 4 g + b of row r.
// MODE 0: policy, 1: policy and action, 2: binarize.
template <int KG, bool EXACT, int MODE>
__global__ __launch_bounds__(EN_THREADS) void ensemble_layer_kernel(const EnsembleArgs a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int e = blockIdx.y;
    const int K0 = EXACT ? 8 * KG : a.k0;
    const int N = a.n, NOUT = a.nout;                        // NOUT: rows of W that are read (<= 32)
    const int groups = K0 >> 3;
    const long batch = a.batch, tiles = a.tiles;
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

    f32x4 wv[KG];                                            // W[e][r][8 j + 4 g .. + 3], rows past NOUT are zeros
    {
        const float* w = a.w1 + ((long)e * N + (r < NOUT ? r : 0)) * K0 + 4 * g;
#pragma unroll
        for (int j = 0; j < KG; ++j) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(w + 8 * (EXACT || j < groups ? j : 0));
            wv[j] = (EXACT || j < groups) && r < NOUT ? v : zero4;
        }
    }
    auto x_row = [&](long tile) {
        long row = tile * EN_ROWS + r;
        row = row < batch ? row : batch - 1;
        return a.x + row * K0 + 4 * g;
    };
    auto load_piece = [&](const float* xr, int j) { return *reinterpret_cast<const f32x4*>(xr + 8 * (EXACT || j < groups ? j : 0)); };

    const long stride = (long)gridDim.x * 4;
    long tile = (long)blockIdx.x * 4 + wave;
    if (tile >= tiles) return;
    f32x4 xv[KG];
    {
        const float* xr = x_row(tile);
#pragma unroll
        for (int j = 0; j < KG; ++j) xv[j] = load_piece(xr, j);
    }
    const HeadOut out = HeadOut{a.policy, MODE == 1 ? a.action : nullptr, nullptr, a.head, N};
    const int limit = a.mask_size > 0 ? a.mask_size : NOUT;
    const bool wave_fill = MODE != 2 && N > NOUT && (N & 3) == 0;
    const int s4 = N >> 2, c0 = (NOUT + 3) >> 2;
    const int fill_r0 = wave_fill ? lane / s4 : 0, fill_c0 = wave_fill ? lane - fill_r0 * s4 : 0;
    const int fill_dr = wave_fill ? 64 / s4 : 0, fill_dc = wave_fill ? 64 - fill_dr * s4 : 0;

    for (; tile < tiles; tile += stride) {
        const long next = tile + stride;
        const float* const xr_next = x_row(next < tiles ? next : tile);
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int j = 0; j < KG; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[j][i], xv[j][i], acc, 0, 0, 0);
            xv[j] = load_piece(xr_next, j);
            __builtin_amdgcn_sched_barrier(0);      // (left alone, the scheduler sinks the loads to the end of the tile,
                                                    //  and the next tile then starts by waiting for all of them)
        }
        const long row0 = tile * EN_ROWS;
        const long first = (long)e * batch + row0;              // row of the stacked (members x batch) outputs
        if constexpr (MODE == 2) {
            unsigned word = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i)
                word |= (acc[i] <= 0.f ? 0u : 1u) << (8 * (i >> 2) + 4 * g + (i & 3));
            word |= (unsigned)__shfl_xor((int)word, 32);
            if (g == 0 && row0 + r < batch) a.words[first + r] = word % a.modulo;
        } else {
            float u = 1.f;
            if constexpr (MODE == 1) {
                const long row = first + (row0 + r < batch ? r : 0);
                u = a.u != nullptr ? a.u[row] : reference_row_uniform(a.ph, row);
            }
            int fill_end = 1 << 30;
            if (wave_fill) {
                fill_end = 4 * c0;
                float* block = a.policy + first * N;
                const int rows_here = batch - row0 < EN_ROWS ? (int)(batch - row0) : EN_ROWS;
                if (s4 == 16 && rows_here == EN_ROWS) {
                    if (fill_c0 >= c0) {
                        f32x4* mine = reinterpret_cast<f32x4*>(block) + lane;
#pragma unroll
                        for (int k = 0; k < 8; ++k) mine[64 * k] = zero4;
                    }
                } else {
                    int rr = fill_r0, c = fill_c0;
                    for (int idx = lane; idx < EN_ROWS * s4; idx += 64) {
                        if (c >= c0 && rr < rows_here) *reinterpret_cast<f32x4*>(block + rr * N + 4 * c) = zero4;
                        rr += fill_dr;
                        c += fill_dc;
                        if (c >= s4) {
                            c -= s4;
                            ++rr;
                        }
                    }
                }
            }
            const float p[4] = {acc[0], acc[1], acc[2], acc[3]};
            if (g == 0 && row0 + r < batch) head_row4_any(a.head, out, p, first + r, NOUT, limit, u, fill_end);
        }
    }
}

}  // namespace sp

using namespace sp;

template <int KG>
static const void* pick_ensemble_kernel_kg(bool exact, bool action) {
    if (exact) return action ? (const void*)mlp_ensemble_kernel<KG, true, true> : (const void*)mlp_ensemble_kernel<KG, true, false>;
    return action ? (const void*)mlp_ensemble_kernel<KG, false, true> : (const void*)mlp_ensemble_kernel<KG, false, false>;
}
static const void* pick_ensemble_kernel(int kg, bool exact, bool action) {
    return kg == 4 ? pick_ensemble_kernel_kg<4>(exact, action) : kg == 8 ? pick_ensemble_kernel_kg<8>(exact, action)
                                                                         : pick_ensemble_kernel_kg<16>(exact, action);
}

template <int KG, int MODE>
static const void* pick_layer_kernel_kg(bool exact) {
    return exact ? (const void*)ensemble_layer_kernel<KG, true, MODE> : (const void*)ensemble_layer_kernel<KG, false, MODE>;
}
template <int MODE>
static const void* pick_layer_kernel(int kg, bool exact) {
    return kg == 4 ? pick_layer_kernel_kg<4, MODE>(exact) : kg == 8 ? pick_layer_kernel_kg<8, MODE>(exact)
         : kg == 16 ? pick_layer_kernel_kg<16, MODE>(exact) : pick_layer_kernel_kg<32, MODE>(exact);
}

// One workgroup (4 waves, one per SIMD) per compute unit while the members leave room for that: a wave then keeps its
// member's weights for all its tiles.
static int ensemble_launch(const void* kernel, EnsembleArgs& a, hipStream_t stream, const char* what) {
    a.tiles = (a.batch + EN_ROWS - 1) / EN_ROWS;
    const long cus = device_cu_count();
    long gx = (cus + a.members - 1) / a.members;
    const long most = (a.tiles + 3) / 4;
    if (gx > most) gx = most;
    if (gx < 1) gx = 1;
    void* args[] = {(void*)&a};
    hipError_t err = hipLaunchKernel(kernel, dim3((unsigned)gx, (unsigned)a.members), dim3(EN_THREADS), args, 0, stream);
    if (err != hipSuccess) return fail(SP_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(err));
    return check_launch(what);
}

// Reference role: the body of `graph_run_host model {ensemble}` (ml/layers.spi:336-344) for a graph of the shape
// input -> matmul_ensemble -> relu -> matmul_ensemble -> head (game/leduc/model_cem.spi:55-63) or
// input -> matmul_ensemble -> head (game/nl_hu_holdem/model_cem.spi:84-100).
extern "C" int sp_mlp_forward_ensemble(int dtype, const void* x, int32_t n_layers, const void* const* weights,
                                       const int32_t* dims, int32_t members, const float* u, const sp_philox_t* philox,
                                       float* policy_out, int32_t* action_out, int64_t batch, int32_t head,
                                       int32_t mask_size, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(policy_out);
    SP_OPTIONAL_PTR(u); SP_OPTIONAL_PTR(action_out);
    if (weights == nullptr || dims == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward_ensemble: weights/dims is NULL");
    if (dtype != SP_F32) return fail(SP_ERR_DTYPE, "sp_mlp_forward_ensemble: dtype must be f32");
    if (n_layers != 1 && n_layers != 2) return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: one or two layers, got %d", n_layers);
    if (members <= 0 || members > 65535) return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: members must be in [1, 65535]");
    if (batch <= 0 || batch > (1ll << 40) / members) return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: batch must be positive (and members x batch below 2^40)");
    if (head < SP_HEAD_NONE || head > SP_HEAD_SOFTMAX_RM) return fail(SP_ERR_ARG, "sp_mlp_forward_ensemble: unknown head %d", head);
    if (action_out != nullptr && u == nullptr && philox == nullptr)
        return fail(SP_ERR_NULL, "sp_mlp_forward_ensemble: action requested but u and philox are NULL");
    if (u != nullptr && philox != nullptr) return fail(SP_ERR_ARG, "sp_mlp_forward_ensemble: at most one of u and philox may be given");
    const int k0 = dims[0], n = dims[n_layers];
    const int k_max = n_layers == 2 ? 128 : 256;
    if (k0 < 8 || k0 % 8 != 0 || k0 > k_max)
        return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: input width %d must be a multiple of 8 in [8, %d]", k0, k_max);
    if (n_layers == 2 && dims[1] != EN_HIDDEN)
        return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: hidden width must be %d, got %d", EN_HIDDEN, dims[1]);
    if (n <= 0 || n > MLP_MAX_OUT) return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: output width %d must be in [1, %d]", n, MLP_MAX_OUT);
    if (mask_size < 0 || mask_size > n) return fail(SP_ERR_ARG, "sp_mlp_forward_ensemble: mask_size must be in [0, %d], got %d", n, mask_size);
    // a masked head gives probability zero to the columns past the mask: only the valid ones are computed
    const int nout = head != SP_HEAD_NONE && mask_size > 0 ? mask_size : n;
    if (nout > EN_MAX_OUT)
        return fail(SP_ERR_SHAPE, "sp_mlp_forward_ensemble: at most 4 computed outputs (the head's width, or its mask), got %d", nout);
    for (int i = 0; i < n_layers; ++i) {
        if (weights[i] == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward_ensemble: weights[%d] is NULL", i);
        if (!aligned16(weights[i])) return fail(SP_ERR_ALIGN, "sp_mlp_forward_ensemble: weights[%d] is not 16-byte aligned", i);
    }
    if (!aligned16(x)) return fail(SP_ERR_ALIGN, "sp_mlp_forward_ensemble: x is not 16-byte aligned");
    if (n % 4 == 0 && !aligned16(policy_out)) return fail(SP_ERR_ALIGN, "sp_mlp_forward_ensemble: policy_out is not 16-byte aligned");
    EnsembleArgs a{};
    a.ph.philox_mode = -1;
    int rc = mlp_set_philox(a.ph, philox, (int64_t)members * batch, n, __func__);
    if (rc != SP_OK) return rc;
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    a.x = (const float*)x; a.w1 = (const float*)weights[0]; a.w2 = n_layers == 2 ? (const float*)weights[1] : nullptr; a.u = u;
    a.policy = policy_out; a.action = action_out; a.batch = batch; a.members = members; a.k0 = k0; a.n = n; a.nout = nout;
    a.head = head; a.mask_size = mask_size;
    const int kg = k0 <= 32 ? 4 : k0 <= 64 ? 8 : k0 <= 128 ? 16 : 32;
    const void* kernel = n_layers == 2 ? pick_ensemble_kernel(kg, k0 == 8 * kg, action_out != nullptr)
                       : action_out != nullptr ? pick_layer_kernel<1>(kg, k0 == 8 * kg) : pick_layer_kernel<0>(kg, k0 == 8 * kg);
    return ensemble_launch(kernel, a, (hipStream_t)stream, __func__);
}

// Reference role: `graph_run_host model {ensemble}` for input -> matmul_ensemble -> binarize' (game/leduc/model_cfr.spi:56-61,
// game/nl_hu_holdem/model_cfr.spi:82-88; ml/layers.spi:439-446, ml/primitives.spi:817-821).
extern "C" int sp_ensemble_binarize(int dtype, const void* x, const void* weights, uint32_t* out, int32_t members,
                                    int64_t batch, int32_t k0, int32_t n, uint32_t modulo, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(weights);
    SP_REQUIRE_PTR(out);
    if (dtype != SP_F32) return fail(SP_ERR_DTYPE, "sp_ensemble_binarize: dtype must be f32");
    if (members <= 0 || members > 65535) return fail(SP_ERR_SHAPE, "sp_ensemble_binarize: members must be in [1, 65535]");
    if (batch <= 0 || batch > (1ll << 40) / members) return fail(SP_ERR_SHAPE, "sp_ensemble_binarize: batch must be positive (and members x batch below 2^40)");
    if (k0 < 8 || k0 % 8 != 0 || k0 > 256)
        return fail(SP_ERR_SHAPE, "sp_ensemble_binarize: input width %d must be a multiple of 8 in [8, 256]", k0);
    if (n <= 0) return fail(SP_ERR_SHAPE, "sp_ensemble_binarize: output width must be positive");
    if (modulo == 0) return fail(SP_ERR_ARG, "sp_ensemble_binarize: modulo must be positive");
    if (!aligned16(x) || !aligned16(weights)) return fail(SP_ERR_ALIGN, "sp_ensemble_binarize: x / weights not 16-byte aligned");
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    EnsembleArgs a{};
    a.ph.philox_mode = -1;
    a.x = (const float*)x; a.w1 = (const float*)weights; a.batch = batch; a.members = members; a.k0 = k0; a.n = n;
    a.nout = n < 32 ? n : 32;          // the device's 32-bit shift drops the columns from 32 on
    a.words = out; a.modulo = modulo;
    const int kg = k0 <= 32 ? 4 : k0 <= 64 ? 8 : k0 <= 128 ? 16 : 32;
    return ensemble_launch(pick_layer_kernel<2>(kg, k0 == 8 * kg), a, (hipStream_t)stream, __func__);
}

namespace {
struct MlpEnsembleKernelNames {
    MlpEnsembleKernelNames() { register_kernel("mlp_forward_ensemble", (const void*)mlp_ensemble_kernel<16, true, false>, EN_THREADS); }
} mlp_ensemble_kernel_names;
}  // namespace
