// Fused dense-stack forward for gfx950.
//
// A workgroup is 4 waves; every wave owns 16 batch rows and pushes them through ALL layers, so
// activations never leave the wave's registers: the f32 accumulator fragment of one layer,
// after bias / ReLU / rounding to 16 bits, is bit-for-bit the MFMA operand fragment of the next
// layer.  (v_mfma_f32_16x16x32_{f16,bf16}: a lane ends up with 4 consecutive rows of the first
// operand.  The weight rows are therefore fed in the order 32 u + 8 (i / 4) + i % 4 for an even
// output tile and + 4 for the odd tile next to it, so that the two quads a lane holds in a pair
// of tiles are the 8 consecutive columns 32 u + 8 q .. + 7: exactly the K-values lane group q
// feeds to the next layer's MFMA.)
//
// Weights are the shared operand.  All layers' weight matrices are cut into chunks of 64 K-columns
// and streamed as one flat sequence through a ring of 4 LDS stages by global_load_lds DMA, three
// chunks ahead of the MFMAs (also across layer boundaries); one barrier per chunk.  Inside a
// stage a chunk is stored as 128-byte rows (one weight row each) whose eight 16-byte pieces are
// XOR-swizzled with swz(row) = 2 * ((row >> 3) & 3) + ((row >> 1) & 1): a DMA instruction then fetches 8 whole 128-byte lines (8
// adjacent lanes per line), and the ds_read_b128 operand fetches of the 16 rows of a tile are
// bank-conflict free.
//
// The head (softmax / regret matching / sampling) runs on the last layer's f32 outputs.
//
// Stacks of 256-wide hidden layers with a narrow head and at most 64 rows per compute unit take another
// route (mlp_split_kernel, described where it is defined): there a wave owns 64 OUTPUT FEATURES of all
// 64 rows of the workgroup and the activations are exchanged through LDS.
//
// Semantics follow the graph interpreter of ml/layers.spi:194-240 (BlockMatmul = x . w^T with w
// stored (out, in), relu = max 0) and the heads of ml/primitives.spi:711-722,748-798.
#include "mlp_common.h"

#pragma clang fp contract(off)

namespace sp {


// NW waves per workgroup, 16 batch rows per wave.
template <int DT, int NW>
__global__ __launch_bounds__(NW * 64) void mlp_forward_kernel(const MlpArgs a) {
    constexpr int MLP_THREADS = NW * 64;
    constexpr int MLP_ROWS = NW * 16;
    constexpr int MLP_DMA_PER_WAVE = MLP_DMA_PER_CHUNK / NW;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15;       // batch row inside the wave's 16-row tile; weight row inside a 16-row tile
    const int q = lane >> 4;       // which 8 of the 32 K-values of an MFMA step this lane feeds
    const long row = (long)blockIdx.x * MLP_ROWS + wave * 16 + j;
    const bool row_ok = row < a.batch;
    const unsigned lds_base = (unsigned)(size_t)lds;
    const unsigned dummy_dst = lds_base + MLP_STAGES * MLP_STAGE_BYTES;

    // ---- weight chunk pipeline: chunk = (layer, 64-column slab c) ----
    int pf_layer = 0, pf_c = 0;    // next chunk to fetch
    int pf_stage = 0;
    auto fetch_next_chunk = [&]() {
        const bool live = pf_layer < a.n_layers;
        const int layer = live ? pf_layer : 0;
        const int K = a.dims[layer], N = a.dims[layer + 1];
        const unsigned char* W = (const unsigned char*)a.w[layer];
        const int n_instr = live ? (N + 7) / 8 : 0;            // 8 weight rows (128 bytes each) per instruction
#pragma unroll
        for (int m = 0; m < MLP_DMA_PER_WAVE; ++m) {
            const int ii = wave + NW * m;
            if (ii < n_instr) {
                int n = ii * 8 + (lane >> 3);
                const int piece = (lane & 7) ^ mlp_swz(n);        // the K piece that belongs in LDS slot lane & 7
                n = n < N ? n : N - 1;                             // rows past N: any valid row, never used
                int k = pf_c * 64 + piece * 8;
                k = k <= K - 8 ? k : K - 8;                        // pieces past K: multiplied by zero activations
                mlp_dma(W, (unsigned)((n * K + k) * 2), lds_base + pf_stage * MLP_STAGE_BYTES + ii * 1024);
            } else {
                mlp_dma((const unsigned char*)a.w[0], 0u, dummy_dst);  // keeps the per-chunk DMA count fixed
            }
        }
        if (live) {
            ++pf_c;
            if (pf_c * 64 >= K) { pf_c = 0; ++pf_layer; }
        }
        pf_stage = (pf_stage + 1) & (MLP_STAGES - 1);
    };
    fetch_next_chunk();
    fetch_next_chunk();
    fetch_next_chunk();

    // ---- the wave's input rows as MFMA operand fragments: for step s (32 K-values) lane (j, q)
    //      holds x[row][32 s + 8 q .. + 7] ----
    u32x4 act[MLP_MAX_DIM / 32];
    {
        const int K0 = a.dims[0];
        const unsigned char* xr = (const unsigned char*)a.x + row * K0 * 2;
#pragma unroll
        for (int s = 0; s < MLP_MAX_DIM / 32; ++s) {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (row_ok && 32 * s + 8 * q < K0) v = *reinterpret_cast<const u32x4*>(xr + (32 * s + 8 * q) * 2);
            act[s] = v;
        }
    }

    f32x4 acc[MLP_MAX_DIM / 16];
    int stage = 0;
    // LDS byte offset of this lane's 16-byte weight piece for the first tile of a chunk: lane j feeds
    // weight row n0 = 8 (j / 4) + j % 4 of the 32-row group, K piece 4 sp + q (sp = which 32-wide step
    // of the chunk).  Tile t adds (t / 2) * 32 + (t % 2) * 4 rows, which leaves swz() unchanged.
    const int n0 = 8 * (j >> 2) + (j & 3);
    unsigned frag_off[2];
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) frag_off[sp] = (unsigned)(n0 * 128 + (((4 * sp + q) ^ mlp_swz(n0)) << 4));
    auto tile_off = [](int t) { return ((t >> 1) * 32 + (t & 1) * 4) * 128; };
    auto tile_col = [&](int t) { return 32 * (t >> 1) + 4 * (t & 1) + 8 * q; };  // first of this lane's 4 columns
    // per-wave f32 staging of the last layer's outputs; it reuses the first weight stage once every
    // wave is done with the weights
    float* head_rows = reinterpret_cast<float*>(lds) + wave * 16 * MLP_MAX_OUT;
    static_assert(NW * 16 * MLP_MAX_OUT * 4 <= MLP_STAGE_BYTES, "head staging must fit one weight stage");

    for (int layer = 0; layer < a.n_layers; ++layer) {
        const int K = a.dims[layer], N = a.dims[layer + 1];
        const int nt = 2 * ((N + 31) / 32);   // output tiles come in pairs covering 32 columns
        const bool last = layer + 1 == a.n_layers;
#pragma unroll
        for (int t = 0; t < MLP_MAX_DIM / 16; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (int c = 0; c < MLP_MAX_DIM / 64; ++c) {
            if (c * 64 < K) {
                // the two newer chunks may still be in flight; everything older has landed
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * MLP_DMA_PER_WAVE) : "memory");
                __syncthreads();
                fetch_next_chunk();   // into the stage every wave finished reading before this barrier
                const unsigned char* st = lds + stage * MLP_STAGE_BYTES;
                // Output tiles are walked in groups of 4 (64 columns) with one uniform branch per
                // group, so that the 8 or 16 LDS reads and the MFMAs of a group form one straight
                // line the scheduler can overlap.  A partly filled last group multiplies whatever
                // the stage holds past row N; those columns are never used.
                const bool two_steps = c * 64 + 32 < K;
                auto mma = [&](int t, int sp, const u32x4& w) {
                    // weights are the first operand: the result fragment is (n, batch row)
                    if constexpr (DT == SP_F16)
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            __builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, act[2 * c + sp]), acc[t], 0, 0, 0);
                    else
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, act[2 * c + sp]), acc[t], 0, 0, 0);
                };
                auto read = [&](int t, int sp) {
                    return *reinterpret_cast<const u32x4*>(st + frag_off[sp] + tile_off(t));
                };
                if (nt == MLP_MAX_DIM / 16 && two_steps) {
                    // full-width chunk: 8 groups of (4 tiles, one 32-wide step), software pipelined by
                    // hand: the weight pieces of group g + 2 are requested before the MFMAs of group g
                    // (with one wave per SIMD nothing else hides the LDS latency)
                    u32x4 w[3][4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) w[0][t] = read(t, 0);
#pragma unroll
                    for (int t = 0; t < 4; ++t) w[1][t] = read(t, 1);
#pragma unroll
                    for (int g = 0; g < 8; ++g) {
                        if (g + 2 < 8) {
#pragma unroll
                            for (int t = 0; t < 4; ++t) w[(g + 2) % 3][t] = read(((g + 2) >> 1) * 4 + t, (g + 2) & 1);
                        }
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int t = 0; t < 4; ++t) mma((g >> 1) * 4 + t, g & 1, w[g % 3][t]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int g4 = 0; g4 < MLP_MAX_DIM / 64; ++g4) {
                        if (g4 * 4 < nt) {
                            u32x4 w0[4], w1[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t) w0[t] = read(g4 * 4 + t, 0);
                            if (two_steps) {
#pragma unroll
                                for (int t = 0; t < 4; ++t) w1[t] = read(g4 * 4 + t, 1);
                            }
#pragma unroll
                            for (int t = 0; t < 4; ++t) mma(g4 * 4 + t, 0, w0[t]);
                            if (two_steps) {
#pragma unroll
                                for (int t = 0; t < 4; ++t) mma(g4 * 4 + t, 1, w1[t]);
                            }
                        }
                    }
                }
                stage = (stage + 1) & (MLP_STAGES - 1);
            }
        }

        // ---- layer epilogue: in tile t lane (j, q) holds columns tile_col(t) + 0..3 of batch row j;
        //      tiles 2 s and 2 s + 1 together give it columns 32 s + 8 q .. + 7 ----
        const float* bias = a.b[layer];
#pragma unroll
        for (int t = 0; t < MLP_MAX_DIM / 16; ++t) {
            if (t < nt && bias != nullptr) {
                const int n = tile_col(t);
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < N) acc[t][r] += bias[n + r];
            }
        }
        if (!last) {
#pragma unroll
            for (int s = 0; s < MLP_MAX_DIM / 32; ++s) {
                u32x4 v = {0u, 0u, 0u, 0u};
                if (32 * s < N) {
                    const f32x4 lo = acc[2 * s], hi = acc[2 * s + 1];
                    v.x = relu_pack2<DT>(lo[0], lo[1]);
                    v.y = relu_pack2<DT>(lo[2], lo[3]);
                    v.z = relu_pack2<DT>(hi[0], hi[1]);
                    v.w = relu_pack2<DT>(hi[2], hi[3]);
                }
                act[s] = v;
            }
        } else {
            __syncthreads();   // all waves have read their last weight chunk: the stage can be reused
#pragma unroll
            for (int t = 0; t < MLP_MAX_OUT / 16; ++t) {
                if (t < nt) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) head_rows[j * MLP_MAX_OUT + tile_col(t) + r] = acc[t][r];
                }
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // drain the dummy DMAs before the LDS is released

    // ---- head: lanes 0..15 of every wave own one batch row each (the staging is wave private) ----
    if (lane < 16 && row_ok) {
        const int N = a.dims[a.n_layers];
        const int limit = a.mask_size > 0 ? a.mask_size : N;
        float* p = head_rows + lane * MLP_MAX_OUT;   // this row's outputs
        const float u = a.ph.philox_mode >= 0 ? reference_row_uniform(a.ph, row) : a.action != nullptr ? a.u[row] : 1.f;
        if (N <= 8) head_row<8>(head_out(a), p, row, N, limit, u);      // narrow heads run in registers
        else head_row<MLP_MAX_OUT>(head_out(a), p, row, N, limit, u);
    }
}


// ---- stacks whose hidden layers are all 256 wide ------------------------------------------------
// Same data flow as mlp_forward_kernel (16 batch rows per wave, activations in registers, weights
// streamed through the LDS ring three chunks ahead), with the hidden width a compile-time 256 and
// NO data-dependent control flow around the register arrays: every 256-row chunk has the same
// shape, all per-lane DMA offsets are computed once, a chunk costs a wave no vector instructions
// besides its 32 MFMAs and 32 LDS reads, and the DMA instructions are issued one by one between
// the MFMA groups.  The first layer always runs C0 whole chunks (1 for K0 <= 64, else 4; K-pieces
// past K0 re-read the last valid piece and meet zero activations), the last layer (at most 64
// outputs) travels as ONE chunk holding its four 64-column slabs at 64-row spacing and always
// computes 4 tiles (rows past the outputs are stale but finite-or-not they only reach unused columns).
template <int DT, int NW, int C0>
__global__ __launch_bounds__(NW * 64) void mlp_h256_kernel(const MlpArgs a) {
    constexpr int H = 256;
    constexpr int PW = 32 / NW;                      // DMA instructions per wave and chunk
    constexpr int ROWS = NW * 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, q = lane >> 4;
    const long row = (long)blockIdx.x * ROWS + wave * 16 + j;
    const unsigned lds_base = (unsigned)(size_t)lds;
    const unsigned dummy_dst = lds_base + MLP_STAGES * MLP_STAGE_BYTES;
    // Every scalar the kernel needs is read from the argument block HERE, in one round trip: a read
    // at the point of use costs a few hundred cycles each time, and the wait for it also drains the
    // LDS reads in flight.  The per-layer pointers, which the layer loop indexes at run time, travel
    // in two registers instead (lane l holds weights[l] and biases[l]) and are picked by v_readlane.
    const int K0 = a.k0, NL = a.n_layers, NOUT = a.nout;
    const unsigned char* const x_ptr = (const unsigned char*)a.x;
    const unsigned char* const w0_ptr = (const unsigned char*)a.w[0];
    const unsigned char* const w1_ptr = (const unsigned char*)a.w[1];
    const float* const b0_ptr = a.b[0];
    const float* const u_ptr = a.u;
    const long batch = a.batch;
    const HeadOut out = head_out(a);
    const int mask_size = a.mask_size;
    const int ph_mode = a.ph.philox_mode;
    asm volatile("" ::"s"(K0), "s"(NL), "s"(NOUT), "s"(x_ptr), "s"(w0_ptr), "s"(w1_ptr), "s"(b0_ptr), "s"(u_ptr), "s"(batch),
                 "s"(out.policy), "s"(out.action), "s"(out.logits), "s"(out.head), "s"(mask_size), "s"(ph_mode));
    const int n_chunks = C0 + 4 * (NL - 2) + 1;
    u32x2 tab_w, tab_b;
    {
        const unsigned char* args = (const unsigned char*)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(tab_w) : "v"((lane & 7) * 8), "s"(args + __builtin_offsetof(MlpArgs, w)) : "memory");
        asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(tab_b) : "v"((lane & 7) * 8), "s"(args + __builtin_offsetof(MlpArgs, b)) : "memory");
    }
    auto table_ptr = [&](const u32x2& tab, int l) {
        const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)tab[0], l);
        const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)tab[1], l);
        return (const unsigned char*)(((unsigned long long)hi << 32) | lo);
    };

    // ---- the wave's input rows, requested before any weight so that they are the oldest loads;
    //      the row's uniform for the sampling head travels with them ----
    constexpr int XS = C0 == 1 ? 2 : H / 32;         // 32-wide k-steps of the input (K0 <= 64 when C0 is 1)
    const bool row_ok = row < batch;
    u32x4 act[H / 32];
    float u_row = 1.f;
    {
        const unsigned char* xr = x_ptr + (row_ok ? row : 0) * K0 * 2;
        // (in operand order a lane touches a cache line of its own, which the texture path serves at a
        //  quarter of its rate: no loads for k-steps the first layer cannot have)
#pragma unroll
        for (int s = 0; s < XS; ++s) {
            const int k = 32 * s + 8 * q;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(act[s]) : "v"(xr + (k < K0 ? k : 0) * 2) : "memory");
        }
        if (u_ptr != nullptr)
            asm volatile("global_load_dword %0, %1, off" : "=v"(u_row) : "v"(u_ptr + (row_ok ? row : 0)) : "memory");
    }

    // ---- per-lane source offsets, once ----
    // 256-row chunks: instruction m of this wave fetches rows 8 * (wave + NW * m) .. + 7; NW is a
    // multiple of 4, so the swizzle of its rows does not depend on m.
    static_assert(NW % 4 == 0, "the K piece of a lane must not depend on the DMA instruction");
    const int piece = (lane & 7) ^ ((2 * (wave & 3)) | ((lane >> 4) & 1));
    unsigned off0[PW], offH[PW], offL[PW];
    unsigned dstL[PW];                               // LDS offsets of the last layer's instructions inside a stage
#pragma unroll
    for (int m = 0; m < PW; ++m) {
        const int n = (wave + NW * m) * 8 + (lane >> 3);
        offH[m] = (unsigned)((n * H + piece * 8) * 2);
        off0[m] = (unsigned)(n * K0 * 2);            // + the K piece, clamped per slab when the chunk is prepared
    }

    int pf = 0, pf_stage = 0;                        // next chunk to fetch and its ring stage
    const unsigned char* pf_base = w0_ptr;
    unsigned pf_dst0 = lds_base;
    bool pf_last = false, pf_none = false;
    unsigned cur[PW];
    // EARLY: one of the three fetches issued before the pointer table has landed; they read the first
    // or the second layer, whose pointers are in scalar registers
    auto prepare = [&](auto EARLY_) {
        constexpr bool early = decltype(EARLY_)::value != 0;
        auto layer_ptr = [&](int l) { return early ? (l == 0 ? w0_ptr : w1_ptr) : table_ptr(tab_w, l); };
        pf_dst0 = lds_base + pf_stage * MLP_STAGE_BYTES;
        pf_last = pf == n_chunks - 1;
        pf_none = pf >= n_chunks;
        if (pf < C0) {
            pf_base = w0_ptr;
            int k = pf * 64 + piece * 8;
            k = k <= K0 - 8 ? k : K0 - 8;
#pragma unroll
            for (int m = 0; m < PW; ++m) cur[m] = off0[m] + (unsigned)(k * 2);
        } else if (pf < n_chunks - 1) {
            const int hl = (pf - C0) >> 2;
            pf_base = layer_ptr(1 + hl) + ((pf - C0) & 3) * 128;
#pragma unroll
            for (int m = 0; m < PW; ++m) cur[m] = offH[m];
        } else {
            pf_base = layer_ptr(NL - 1);
#pragma unroll
            for (int m = 0; m < PW; ++m) cur[m] = offL[m];
        }
        ++pf;
        pf_stage = (pf_stage + 1) & (MLP_STAGES - 1);
    };
    auto issue = [&](int m) {
        const int ii = wave + NW * m;
        unsigned dst = pf_dst0 + ii * 1024;                                        // 256-row chunk: 8 rows per KiB
        if (pf_last) dst = dstL[m] != ~0u ? pf_dst0 + dstL[m] : dummy_dst;
        if (pf_none) dst = dummy_dst;
        mlp_dma(pf_base, cur[m], __builtin_amdgcn_readfirstlane(dst));
    };
    auto fetch = [&]() {
        prepare(IC<1>{});
#pragma unroll
        for (int m = 0; m < PW; ++m) issue(m);
    };
    fetch();   // the first chunk (always of the first layer) is on its way before the remaining setup
    {
        const int rb = (NOUT + 7) / 8;               // 8-row blocks of the last layer (at most 8)
#pragma unroll
        for (int m = 0; m < PW; ++m) {
            // last layer: instruction ii = (slab, 8-row block); no division: ii < 32, rb <= 8
            const int ii = wave + NW * m;
            const int slab = (ii >= rb) + (ii >= 2 * rb) + (ii >= 3 * rb);
            const int blk = ii - slab * rb;
            int nl = blk * 8 + (lane >> 3);
            const int pl = (lane & 7) ^ mlp_swz(nl);
            nl = nl < NOUT ? nl : NOUT - 1;
            offL[m] = (unsigned)((nl * H + slab * 64 + pl * 8) * 2);
            dstL[m] = ii < 4 * rb ? (unsigned)((slab * 64 + blk * 8) * 128) : ~0u;
        }
    }
    fetch();
    fetch();

    int stage = 0;
    const int n0 = 8 * (j >> 2) + (j & 3);
    unsigned frag_off[2];
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) frag_off[sp] = (unsigned)(n0 * 128 + (((4 * sp + q) ^ mlp_swz(n0)) << 4));
    auto tile_off = [](int t) { return ((t >> 1) * 32 + (t & 1) * 4) * 128; };
    auto tile_col = [&](int t) { return 32 * (t >> 1) + 4 * (t & 1) + 8 * q; };
    auto mfma = [&](const f32x4& c, const u32x4& w, const u32x4& x) {
        if constexpr (DT == SP_F16)
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, x), c, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), c, 0, 0, 0);
    };
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 acc[H / 16];
    // ---- the MFMA pipeline ----
    // A chunk is 8 groups (output-tile quad g / 2, 32-wide k-step g % 2) of 4 operand reads + 4 MFMAs.
    // The reads run D = RING - 1 groups ahead of the MFMAs, across chunk boundaries: with four waves on
    // a compute unit an LDS read comes back after 250 cycles or more and a group's MFMAs take 64, so a
    // short look-ahead leaves the matrix pipe waiting for every group.  (Seven groups ahead need 128
    // registers, which 8-wave workgroups do not have; they look three ahead.)  Group g of a chunk lives
    // in slot g % RING; when it starts, slot (g + D) % RING is free and receives group g + D of this
    // chunk or, from g = 8 - D on, group g + D - 8 of the next one.  The next chunk must therefore have
    // landed when group 8 - D starts: that is where the wave waits for its DMA, meets the others at the
    // barrier (which also frees the stage of the previous chunk for the fetch three chunks ahead) and
    // prepares that fetch.
    constexpr int RING = NW == 4 ? 8 : 4;
    constexpr int D = RING - 1;
    constexpr int GSYNC = 8 - D;
    u32x4 w[RING][4];
    const unsigned char* st_cur = lds;
    auto read_group = [&](const unsigned char* st, int g) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            w[g % RING][t] = *reinterpret_cast<const u32x4*>(st + frag_off[g & 1] + tile_off((g >> 1) * 4 + t));
    };
    // the first chunk: it has landed when only the two younger fetches are outstanding
    auto first_sync = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PW) : "memory");
        __syncthreads();
        st_cur = lds;
        stage = 1;
#pragma unroll
        for (int g = 0; g < D; ++g) read_group(st_cur, g);
    };
    // KIND 0..3: chunk KIND of a layer, i.e. K-columns 64 KIND .. + 63 for all 16 output tiles (chunk 0
    // starts the accumulators from zero); KIND 4: the last layer, whose chunk holds the K-columns
    // 64 s .. + 63 of all its (at most 64) outputs in slab s = g / 2 and accumulates into tiles 0..3.
    // FIRST: the chunk behind first_sync (no earlier fetch is waiting for its last DMA instructions).
    auto run_chunk = [&](auto KIND_, auto FIRST_) {
        constexpr int kind = decltype(KIND_)::value;
        constexpr bool first = decltype(FIRST_)::value != 0;
        constexpr bool last = kind == 4;
        const unsigned char* st_next = st_cur;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g + D < 8) {
                read_group(st_cur, g + D);
            } else if (!last) {
                if (g == GSYNC) {
                    // a bare s_barrier: __syncthreads() would first wait for the LDS reads in flight, which
                    // is the pipeline this loop exists to keep full.  Nothing needs that wait: the DMA data is
                    // covered by vmcnt, and a stage is only overwritten after its reads have fed MFMAs
                    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(PW) : "memory");
                    prepare(IC<0>{});
                    st_next = lds + stage * MLP_STAGE_BYTES;
                    stage = (stage + 1) & (MLP_STAGES - 1);
                }
                read_group(st_next, g + D - 8);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                if constexpr (last) {
                    acc[t] = mfma(g == 0 ? zero4 : acc[t], w[g % RING][t], act[g]);
                } else {
                    f32x4& d = acc[(g >> 1) * 4 + t];
                    d = mfma((kind == 0 && (g & 1) == 0) ? zero4 : d, w[g % RING][t], act[2 * kind + (g & 1)]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!last && !(first && g < GSYNC)) {
                // the DMA instructions of the fetch prepared at group GSYNC go out one by one behind the
                // groups from there to group GSYNC - 1 of the next chunk
                const int gi = (g + 8 - GSYNC) & 7;
#pragma unroll
                for (int m = gi * PW / 8; m < (gi + 1) * PW / 8; ++m) issue(m);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        st_cur = st_next;
    };
    // (the bias test is uniform and made once per layer, not once per register pair)
    auto next_activations = [&](const float* bias) {
        auto convert = [&](auto HAS_BIAS_) {
#pragma unroll
            for (int s = 0; s < H / 32; ++s) {
                f32x4 lo = acc[2 * s], hi = acc[2 * s + 1];
                if constexpr (decltype(HAS_BIAS_)::value != 0) {
                    // (a pointer that came out of a register table must be told that it points to global memory)
                    typedef const __attribute__((address_space(1))) f32x4* gptr;
                    lo += *(gptr)(unsigned long long)(bias + tile_col(2 * s));
                    hi += *(gptr)(unsigned long long)(bias + tile_col(2 * s + 1));
                }
                act[s] = u32x4{pack_relu2<DT>(lo[0], lo[1]), pack_relu2<DT>(lo[2], lo[3]), pack_relu2<DT>(hi[0], hi[1]),
                               pack_relu2<DT>(hi[2], hi[3])};
            }
        };
        if (bias != nullptr) convert(IC<1>{});
        else convert(IC<0>{});
    };

    // ---- first layer: K0 -> 256.  The inputs are older than every weight DMA, so they have landed
    //      with the first chunk; lanes past K0 (and rows past the batch) feed zeros ----
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PW) : "memory");
#pragma unroll
    for (int s = 0; s < H / 32; ++s) {
        if (s < XS) {
            asm volatile("" : "+v"(act[s]));
            const bool live = row_ok && 32 * s + 8 * q < K0;
            act[s] = live ? act[s] : u32x4{0u, 0u, 0u, 0u};
        } else {
            act[s] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    asm volatile("" : "+v"(u_row), "+v"(tab_w), "+v"(tab_b));
    if (ph_mode >= 0) u_row = reference_row_uniform(a.ph, row_ok ? row : 0);   // the head draws its own uniform
    first_sync();
    run_chunk(IC<0>{}, IC<1>{});
    if constexpr (C0 > 1) {
        run_chunk(IC<1>{}, IC<0>{});
        run_chunk(IC<2>{}, IC<0>{});
        run_chunk(IC<3>{}, IC<0>{});
    }
    next_activations(b0_ptr);

    // ---- hidden layers: 256 -> 256 ----
    for (int layer = 1; layer + 1 < NL; ++layer) {
        run_chunk(IC<0>{}, IC<0>{});
        run_chunk(IC<1>{}, IC<0>{});
        run_chunk(IC<2>{}, IC<0>{});
        run_chunk(IC<3>{}, IC<0>{});
        next_activations((const float*)table_ptr(tab_b, layer));
    }

    // ---- last layer: 256 -> NOUT <= 64, one chunk, 4 tiles ----
    run_chunk(IC<4>{}, IC<0>{});
    // the dummy DMAs (they land in their own KiB) must be done before the LDS is released; they are
    // long done, and waiting here rather than at the end keeps the outputs' stores out of the wait
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // (a pointer that came out of a register table must be told that it points to global memory)
    const __attribute__((address_space(1))) float* bias = (const __attribute__((address_space(1))) float*)(unsigned long long)table_ptr(tab_b, NL - 1);
    const int limit = mask_size > 0 ? mask_size : NOUT;
    if (NOUT <= 8) {
        // narrow heads never leave the registers: in tiles 0 and 1 lane (j, q = 0) holds columns 0..3 and
        // 4..7 of batch row j, and those lanes are lanes 0..15 of the wave
        float p[8];
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            p[n] = acc[n >> 2][n & 3];
            if (bias != nullptr && n < NOUT) p[n] += bias[n];
        }
        if (lane < 16 && row_ok) {
            if (NOUT <= 4) head_row<4>(out, p, row, NOUT, limit, u_row);
            else head_row<8>(out, p, row, NOUT, limit, u_row);
        }
    } else {
        __syncthreads();                                    // every wave has read its last weights: reuse stage 0
        float* head_rows = reinterpret_cast<float*>(lds) + wave * 16 * MLP_MAX_OUT;
#pragma unroll
        for (int t = 0; t < MLP_MAX_OUT / 16; ++t) {
            f32x4 v = acc[t];
            if (bias != nullptr) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (tile_col(t) + r < NOUT) v[r] += bias[tile_col(t) + r];
            }
            *reinterpret_cast<f32x4*>(head_rows + j * MLP_MAX_OUT + tile_col(t)) = v;
        }
        // lanes 0..15 of every wave own one batch row each (the staging is wave private)
        if (lane < 16 && row_ok) head_row<MLP_MAX_OUT>(out, head_rows + lane * MLP_MAX_OUT, row, NOUT, limit, u_row);
    }
}

// ---- stacks of three or more layers, all hidden layers 256 wide, at most 16 outputs, one 64-row
//      workgroup per compute unit ----
// With 16 batch rows per wave every wave reads ALL weights from LDS: 32 KiB per 64-column chunk, and a
// SIMD's registers take operands from LDS at little more than 47 bytes per cycle -- 700 cycles for a
// chunk whose MFMAs need 512.  This kernel splits a hidden layer by OUTPUT FEATURES instead: wave w
// computes features 64 w .. 64 w + 63 for all 64 batch rows of the workgroup.  It streams only its own
// quarter of the weights (8 KiB per chunk: 64 rows x 64 K-columns) through a ring of four LDS stages
// that no other wave touches -- weights need no barrier, only the wave's own vmcnt -- and reads the
// activations of all 64 rows from a shared 32 KiB buffer ([row][feature], the 16-byte pieces of a row
// XOR-swizzled with the row number, so that the 16 rows of an operand fetch fall into different banks).
// Per layer a SIMD takes 64 KiB from LDS instead of 128.  A layer ends with: barrier, the outputs (bias,
// relu, rounded to 16 bits) written over the activations, barrier.
// Tile (p, h) of a wave's 64 features feeds MFMA row i with feature 32 p + 8 (i / 4) + 4 h + i % 4: the
// two quads a lane holds in tiles (p, 0) and (p, 1) are then 8 consecutive features, one 16-byte write.
// The last layer (at most 16 outputs, one MFMA tile) is split by batch rows: wave w multiplies rows
// 16 w .. 16 w + 15 with all outputs (every wave streams the whole last matrix, one chunk of four
// 64-column slabs), and lanes 0..15 run the head.
// Every global load is issued from assembly and counted by hand: the counter of outstanding loads is in
// order and the schedule is static, so each wait names the exact number of younger loads.  Chunk c + 3
// is requested behind the first k-step of chunk c; chunk c + 1 is awaited before the second.
constexpr int SPLIT_ROWS = 64;
constexpr int SPLIT_ACT_BYTES = SPLIT_ROWS * 2 * MLP_MAX_DIM;      // 32 KiB
constexpr int SPLIT_STAGE_BYTES = 64 * 128;                        // 64 weight rows x 64 K-columns
constexpr int SPLIT_STAGES = 4;
constexpr int SPLIT_RING_BYTES = SPLIT_STAGES * SPLIT_STAGE_BYTES;
constexpr int SPLIT_LDS_BYTES = SPLIT_ACT_BYTES + 4 * SPLIT_RING_BYTES;

template <int DT, int KS0>
__global__ __launch_bounds__(256) void mlp_split_kernel(const void* x_first, const void* w0_first, const void* w1_first,
                                                        const float* b0_first, const float* u_first, int batch_first,
                                                        unsigned k0_nl_nout, const MlpArgs a) {
    // (the leading parameters repeat fields of `a`: the library is built with kernel-argument preloading, which hands
    //  the first dwords of scalar parameters to a wave in registers when it starts, so the first loads do not wait
    //  for a scalar load from the argument block; k0_nl_nout = k0 | n_layers << 16 | nout << 24)
    constexpr int ARGS_OFFSET = 48;                  // of `a` inside the kernel's argument block: 5 pointers, 2 ints
    constexpr int C0 = (KS0 + 1) / 2;                // chunks of the first layer
    constexpr bool HALF0 = KS0 == 1;                 // ... which is half a chunk when K0 <= 32
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, q = lane >> 4;
    const long row0 = (long)blockIdx.x * SPLIT_ROWS;
    const u32x4 zero_u4 = {0u, 0u, 0u, 0u};
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    // every scalar argument in one round trip; the per-layer pointers in a register table (lane l holds
    // weights[l] and biases[l], picked by v_readlane)
    const int K0 = (int)(k0_nl_nout & 0xffffu), NL = (int)((k0_nl_nout >> 16) & 0xffu), NOUT = (int)(k0_nl_nout >> 24);
    const unsigned char* const x_ptr = (const unsigned char*)x_first;
    const unsigned char* const w0_ptr = (const unsigned char*)w0_first;
    const unsigned char* const w1_ptr = (const unsigned char*)w1_first;
    const unsigned char* const b0_ptr = (const unsigned char*)b0_first;
    const float* const u_ptr = u_first;
    const long batch = batch_first;
    const HeadOut out = head_out(a);
    const int mask_size = a.mask_size;
    const int ph_mode = a.ph.philox_mode;
    u32x2 tab_w, tab_b;
    {
        const unsigned char* args = (const unsigned char*)__builtin_amdgcn_kernarg_segment_ptr() + ARGS_OFFSET;
        asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(tab_w) : "v"((lane & 7) * 8), "s"(args + __builtin_offsetof(MlpArgs, w)) : "memory");
        asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(tab_b) : "v"((lane & 7) * 8), "s"(args + __builtin_offsetof(MlpArgs, b)) : "memory");
    }
    auto table_ptr = [&](const u32x2& tab, int l) {
        const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)tab[0], l);
        const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)tab[1], l);
        return (const unsigned char*)(((unsigned long long)hi << 32) | lo);
    };

    // ---- the workgroup's input rows (16-byte pieces, 4 KS0 per row) and the uniform of the row this
    //      lane will finish ----
    u32x4 xin[KS0];
    bool x_ok[KS0];
#pragma unroll
    for (int i = 0; i < KS0; ++i) {
        const int idx = tid + 256 * i;
        const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
        x_ok[i] = row0 + r < batch && pc * 8 < K0;
        const long off = x_ok[i] ? ((row0 + r) * K0 + pc * 8) * 2 : 0;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xin[i]) : "v"(x_ptr + off) : "memory");
    }
    const long head_row_idx = row0 + wave * 16 + j;          // the row lanes 0..15 finish
    const bool head_ok = lane < 16 && head_row_idx < batch;
    float u_row = 1.f;
    {
        const unsigned char* up = u_ptr != nullptr ? (const unsigned char*)(u_ptr + (head_ok ? head_row_idx : 0)) : x_ptr;
        asm volatile("global_load_dword %0, %1, off" : "=v"(u_row) : "v"(up) : "memory");
    }
    // ---- a layer's 64 bias values of this wave, always four loads: a missing bias reads the layer's
    //      weights instead (and is not added), so that the number of loads never depends on the arguments ----
    f32x4 bias_r[4];                                         // [2 p + h]: features 64 wave + 32 p + 8 q + 4 h ..+ 3
    bool has_bias = false;
    auto load_bias = [&](const unsigned char* bias, const unsigned char* valid) {
        has_bias = bias != nullptr;
        const unsigned char* src = (has_bias ? bias : valid) + (64 * wave + 8 * q) * 4;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(bias_r[0]) : "v"(src) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(bias_r[1]) : "v"(src) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:128" : "=v"(bias_r[2]) : "v"(src) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off offset:144" : "=v"(bias_r[3]) : "v"(src) : "memory");
    };
    load_bias(b0_ptr, w0_ptr);

    // ---- the weight stream of this wave: chunk after chunk, 8 DMA instructions each ----
    // Instruction m fills stage rows 8 m .. 8 m + 7: lane l fetches, for row R = 8 m + l / 8, the 16-byte
    // piece (l % 8) ^ swz(R), swz(R) = 2 ((R >> 3) & 3) + ((R >> 1) & 1) = 2 (m & 3) + ((l >> 4) & 1).
    const unsigned ring_base = (unsigned)(size_t)lds + SPLIT_ACT_BYTES + wave * SPLIT_RING_BYTES;
    const int dr = lane >> 3, dc = lane & 7, db = (lane >> 4) & 1;
    int f_layer = 0, f_kc = 0, f_stage = 0;
    auto issue_chunk = [&](auto EARLY_) {
        constexpr bool early = decltype(EARLY_)::value != 0;   // before the table has landed: layers 0 and 1 only
        const unsigned dst0 = ring_base + f_stage * SPLIT_STAGE_BYTES;
        if (f_layer == 0) {
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                int k = f_kc * 64 + (dc ^ (2 * (m & 3) + db)) * 8;
                k = k <= K0 - 8 ? k : K0 - 8;                  // pieces past K0 meet zero activations
                mlp_dma(w0_ptr, (unsigned)(((64 * wave + 8 * m + dr) * K0 + k) * 2), dst0 + m * 1024);
            }
        } else if (f_layer < NL - 1) {
            const unsigned char* base = (early ? w1_ptr : table_ptr(tab_w, f_layer)) + f_kc * 128;
#pragma unroll
            for (int m = 0; m < 8; ++m)
                mlp_dma(base, (unsigned)(((64 * wave + 8 * m + dr) * 256 + (dc ^ (2 * (m & 3) + db)) * 8) * 2), dst0 + m * 1024);
        } else {
            const unsigned char* base = table_ptr(tab_w, NL - 1);
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                // one chunk: slab s = R / 16 holds K-columns 64 s .. of outputs R % 16 (outputs past NOUT repeat
                // the last one and only reach accumulator rows nobody reads)
                const int R = 8 * m + dr;
                int o = R & 15;
                o = o < NOUT ? o : NOUT - 1;
                const int kcol = (R >> 4) * 64 + (dc ^ (2 * (m & 3) + db)) * 8;
                mlp_dma(base, (unsigned)((o * 256 + kcol) * 2), dst0 + m * 1024);
            }
        }
        const int count = f_layer == 0 ? C0 : (f_layer < NL - 1 ? 4 : 1);
        ++f_kc;
        if (f_kc == count) { f_kc = 0; ++f_layer; }
        f_stage = (f_stage + 1) & (SPLIT_STAGES - 1);
    };
    issue_chunk(IC<1>{});
    issue_chunk(IC<1>{});
    issue_chunk(IC<1>{});
    // every other scalar argument is waited for HERE, once, behind the first loads (a read at the point of use costs
    // a few hundred cycles, and the wait for it also drains the LDS reads in flight)
    asm volatile("" ::"s"(out.policy), "s"(out.action), "s"(out.logits), "s"(out.head), "s"(out.stride), "s"(mask_size));

    // ---- operand addresses ----
    // weights: tile (p, h), MFMA row j -> stage row R = 32 p + 4 h + R0, R0 = 8 (j / 4) + j % 4; swz(R) does not
    // depend on p and h
    const int R0 = 8 * (j >> 2) + (j & 3);
    const int swzR = 2 * ((j >> 2) & 3) + ((j >> 1) & 1);
    unsigned fragW[2];
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) fragW[sp] = (unsigned)(SPLIT_ACT_BYTES + wave * SPLIT_RING_BYTES + R0 * 128 + (((4 * sp + q) ^ swzR) << 4));
    auto read_w = [&](int stage, int sp, int t) {
        return *reinterpret_cast<const u32x4*>(lds + fragW[sp] + stage * SPLIT_STAGE_BYTES + (32 * (t >> 1) + 4 * (t & 1)) * 128);
    };
    // activations: row r, piece P (of 32) lives in slot (P & 16) | ((P ^ r) & 15)
    unsigned aoff[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) aoff[k4] = (unsigned)(j * 512 + (((4 * k4 + q) ^ j) << 4));
    auto read_a = [&](int bt_bytes, int ks) {               // bt_bytes = 8192 * batch tile
        return *reinterpret_cast<const u32x4*>(lds + aoff[ks & 3] + bt_bytes + (ks >> 2) * 256);
    };
    unsigned pw[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) pw[p] = (unsigned)(j * 512 + (wave >> 1) * 256 + (((8 * (wave & 1) + 4 * p + q) ^ j) << 4));

    // ---- everything older than the second chunk has landed: inputs into the activation buffer ----
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
#pragma unroll
    for (int i = 0; i < KS0; ++i) asm volatile("" : "+v"(xin[i]));
    asm volatile("" : "+v"(u_row), "+v"(tab_w), "+v"(tab_b), "+v"(bias_r[0]), "+v"(bias_r[1]), "+v"(bias_r[2]), "+v"(bias_r[3]));
    if (ph_mode >= 0) u_row = reference_row_uniform(a.ph, head_ok ? head_row_idx : 0);   // the head draws its own uniform
#pragma unroll
    for (int i = 0; i < KS0; ++i) {
        const int idx = tid + 256 * i;
        const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
        *reinterpret_cast<u32x4*>(lds + r * 512 + (pc & 16) * 16 + (((pc ^ r) & 15) << 4)) = x_ok[i] ? xin[i] : zero_u4;
    }
    __syncthreads();

    auto mfma = [&](const f32x4& c, const u32x4& w, const u32x4& x) {
        if constexpr (DT == SP_F16)
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, x), c, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), c, 0, 0, 0);
    };
    // The feature-split layers accumulate in architected registers, MFMAs issued from assembly: the conversion after
    // a layer then reads the sums directly instead of copying 64 registers out of the accumulation file (with one
    // wave per SIMD every instruction costs matrix-pipe time).  publish() supplies the wait states that the
    // compiler would otherwise insert between the last MFMA and the first read of its result.
    auto mfma_v = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first) {
        if (first) {
            if constexpr (DT == SP_F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=v"(c) : "v"(w), "v"(x));
            else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=v"(c) : "v"(w), "v"(x));
        } else {
            if constexpr (DT == SP_F16) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(w), "v"(x));
            else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(w), "v"(x));
        }
    };
    f32x4 acc[4][4];                                         // [batch tile][feature tile]
    u32x4 wf[2][4], bf[2][4];                                // operands of k-step parity 0 / 1
    int r_stage = 0;                                         // ring stage of the chunk being multiplied
#pragma unroll
    for (int t = 0; t < 4; ++t) wf[0][t] = read_w(0, 0, t);

    // One chunk of a feature-split layer.  KC: its place in the layer (activation k-steps 2 KC, 2 KC + 1);
    // FIRSTK / LASTK: first / last chunk of the layer; HALF: only the first k-step exists; ISSUE: request chunk
    // c + 3 behind the first k-step; BIAS: then request this layer's bias; WAITN: loads younger than chunk c + 1
    // at that point; NEXTW: chunk c + 1 is of the same kind, fetch its first operands.
    auto chunk = [&](auto KC_, auto FIRSTK_, auto LASTK_, auto HALF_, auto ISSUE_, auto BIAS_, auto WAITN_, auto NEXTW_,
                     const unsigned char* bias, const unsigned char* valid) {
        constexpr int KC = decltype(KC_)::value;
        constexpr bool firstk = decltype(FIRSTK_)::value != 0, lastk = decltype(LASTK_)::value != 0;
        constexpr bool half = decltype(HALF_)::value != 0, issue = decltype(ISSUE_)::value != 0;
        constexpr bool want_bias = decltype(BIAS_)::value != 0, nextw = decltype(NEXTW_)::value != 0;
        constexpr int WAITN = decltype(WAITN_)::value;
        if constexpr (firstk) {
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) bf[0][bt] = read_a(bt * 8192, 2 * KC);
        }
        // operand reads of the other k-step go out one at a time behind the first MFMAs, in the order of their use
        auto read1 = [&](int m) {
            if (m == 0) wf[1][0] = read_w(r_stage, 1, 0);
            else if (m < 5) bf[1][m - 1] = read_a((m - 1) * 8192, 2 * KC + 1);
            else wf[1][m - 4] = read_w(r_stage, 1, m - 4);
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) {
                mfma_v(acc[bt][t], wf[0][t], bf[0][bt], KC == 0);
                if (!half && 4 * t + bt < 8) read1(4 * t + bt);
                __builtin_amdgcn_sched_barrier(0);
            }
        if constexpr (issue) issue_chunk(IC<0>{});
        if constexpr (want_bias) load_bias(bias, valid);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WAITN) : "memory");
        const int next_stage = (r_stage + 1) & (SPLIT_STAGES - 1);
        auto read0 = [&](int m) {
            if (m == 0) { if constexpr (nextw) wf[0][0] = read_w(next_stage, 0, 0); }
            else if (m < 5) { if constexpr (!lastk) bf[0][m - 1] = read_a((m - 1) * 8192, 2 * KC + 2); }
            else { if constexpr (nextw) wf[0][m - 4] = read_w(next_stage, 0, m - 4); }
        };
        if constexpr (half) {
#pragma unroll
            for (int m = 0; m < 8; ++m) read0(m);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!half) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) {
                    mfma_v(acc[bt][t], wf[1][t], bf[1][bt], false);
                    if (4 * t + bt < 8) read0(4 * t + bt);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
        r_stage = next_stage;
    };
    // the layer's outputs replace its inputs: barrier (every wave is done reading), bias, relu, rounding,
    // 16 bytes per (batch tile, tile pair), barrier
    auto publish = [&]() {
        asm volatile("s_nop 15\n\ts_nop 3\n\ts_barrier" ::: "memory");   // the last MFMAs have written their results
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(bias_r[i]));
        auto convert = [&](auto HAS_BIAS_) {
#pragma unroll
            for (int bt = 0; bt < 4; ++bt)
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    f32x4 lo = acc[bt][2 * p], hi = acc[bt][2 * p + 1];
                    if constexpr (decltype(HAS_BIAS_)::value != 0) {
                        lo += bias_r[2 * p];
                        hi += bias_r[2 * p + 1];
                    }
                    const u32x4 v = {pack_relu2<DT>(lo[0], lo[1]), pack_relu2<DT>(lo[2], lo[3]), pack_relu2<DT>(hi[0], hi[1]),
                                     pack_relu2<DT>(hi[2], hi[3])};
                    *reinterpret_cast<u32x4*>(lds + pw[p] + bt * 8192) = v;
                }
        };
        if (has_bias) convert(IC<1>{});                      // uniform, once per layer
        else convert(IC<0>{});
        __syncthreads();
    };

    // ---- first layer: K0 -> 256 (its bias was requested with the inputs) ----
    if constexpr (C0 == 1) {
        chunk(IC<0>{}, IC<1>{}, IC<1>{}, IC<HALF0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
    } else {
        chunk(IC<0>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<2>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<3>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
    }
    publish();
    // ---- hidden layers but the last one ----
    for (int layer = 1; layer + 2 < NL; ++layer) {
        const unsigned char* bias = table_ptr(tab_b, layer);
        const unsigned char* valid = table_ptr(tab_w, layer);
        chunk(IC<0>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, IC<20>{}, IC<1>{}, bias, valid);
        chunk(IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<20>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<2>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<20>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<3>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<16>{}, IC<1>{}, nullptr, nullptr);
        publish();
    }
    // ---- the last hidden layer: the stream ends with the output layer's chunk ----
    {
        const unsigned char* bias = table_ptr(tab_b, NL - 2);
        const unsigned char* valid = table_ptr(tab_w, NL - 2);
        chunk(IC<0>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, IC<20>{}, IC<1>{}, bias, valid);
        chunk(IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<20>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<2>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<12>{}, IC<1>{}, nullptr, nullptr);
        chunk(IC<3>{}, IC<0>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nullptr, nullptr);
        publish();
    }
    // ---- output layer: rows 16 wave .. + 15 of the workgroup; MFMA row i is output i, stage row 16 s + i
    //      in slab s ----
    f32x4 d;
    {
        u32x4 al[8], wl[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            al[ks] = read_a(wave * 8192, ks);
            const int R = 16 * (ks >> 1) + j;
            const int sw = 2 * ((R >> 3) & 3) + ((R >> 1) & 1);
            wl[ks] = *reinterpret_cast<const u32x4*>(lds + SPLIT_ACT_BYTES + wave * SPLIT_RING_BYTES + r_stage * SPLIT_STAGE_BYTES + R * 128 +
                                                     (((4 * (ks & 1) + q) ^ sw) << 4));
        }
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) d = mfma(ks == 0 ? zero4 : d, wl[ks], al[ks]);
    }
    // (a pointer that came out of a register table must be told that it points to global memory)
    const __attribute__((address_space(1))) float* bias =
        (const __attribute__((address_space(1))) float*)(unsigned long long)table_ptr(tab_b, NL - 1);
    const int limit = mask_size > 0 ? mask_size : NOUT;
    // A masked head that was computed for its valid columns only: the wave's 16 policy rows are one contiguous
    // block, and whole waves write its zeros (16 bytes per lane) instead of 16 lanes writing a row each.
    int fill_end = 1 << 30;
    if (out.stride > NOUT && (out.stride & 3) == 0) {
        const int s4 = out.stride >> 2, c0 = (NOUT + 3) >> 2;    // float4 groups per row; the first one that is all zeros
        fill_end = 4 * c0;
        const long first_row = row0 + wave * 16;
        float* block = out.policy + first_row * out.stride;
        for (int idx = lane; idx < 16 * s4; idx += 64) {
            const int r = idx / s4, c = idx - r * s4;
            if (c >= c0 && first_row + r < batch)
                *reinterpret_cast<float4*>(block + (long)r * out.stride + 4 * c) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    if (NOUT <= 4) {
        // lane (j, q = 0) holds outputs 0..3 of batch row j; those are lanes 0..15 of the wave
        float p[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            p[n] = d[n];
            if (bias != nullptr && n < NOUT) p[n] += bias[n];
        }
        if (head_ok) head_row<4>(out, p, head_row_idx, NOUT, limit, u_row, fill_end);
    } else {
        // every chunk of this wave's ring has been consumed: its first stage stages the 16 x NOUT outputs
        float* head_rows = reinterpret_cast<float*>(lds + SPLIT_ACT_BYTES + wave * SPLIT_RING_BYTES);
        f32x4 v = d;
        if (bias != nullptr) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (4 * q + r < NOUT) v[r] += bias[4 * q + r];
        }
        *reinterpret_cast<f32x4*>(head_rows + j * 16 + 4 * q) = v;
        if (head_ok) head_row<16>(out, head_rows + lane * 16, head_row_idx, NOUT, limit, u_row, fill_end);
    }
}

namespace {
struct MlpKernelNames {
    MlpKernelNames() {
        register_kernel("mlp_forward", (const void*)mlp_forward_kernel<SP_F16, 4>, 256);
        register_kernel("mlp_forward_wide", (const void*)mlp_forward_kernel<SP_F16, 8>, 512);
    }
} mlp_kernel_names;
}  // namespace

}  // namespace sp

using namespace sp;

static const void* pick_split_kernel(int dtype, int ks0) {
    if (dtype == SP_F16) {
        if (ks0 == 1) return (const void*)mlp_split_kernel<SP_F16, 1>;
        if (ks0 == 2) return (const void*)mlp_split_kernel<SP_F16, 2>;
        return (const void*)mlp_split_kernel<SP_F16, 8>;
    }
    if (ks0 == 1) return (const void*)mlp_split_kernel<SP_BF16, 1>;
    if (ks0 == 2) return (const void*)mlp_split_kernel<SP_BF16, 2>;
    return (const void*)mlp_split_kernel<SP_BF16, 8>;
}

extern "C" int sp_mlp_forward(int dtype, const void* x, int32_t n_layers, const void* const* weights,
                              const float* const* biases, const int32_t* dims, const float* u, const sp_philox_t* philox,
                              float* policy_out, int32_t* action_out, float* logits_out, int64_t batch, int32_t head,
                              int32_t mask_size, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(policy_out);
    SP_OPTIONAL_PTR(u); SP_OPTIONAL_PTR(action_out); SP_OPTIONAL_PTR(logits_out);
    if (weights == nullptr || dims == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward: weights/dims is NULL");
    if (dtype != SP_F16 && dtype != SP_BF16) return fail(SP_ERR_DTYPE, "sp_mlp_forward: dtype must be f16 or bf16");
    if (n_layers < 1 || n_layers > MLP_MAX_LAYERS)
        return fail(SP_ERR_ARG, "sp_mlp_forward: n_layers must be in [1, %d], got %d", MLP_MAX_LAYERS, n_layers);
    if (batch <= 0) return fail(SP_ERR_SHAPE, "sp_mlp_forward: batch must be positive");
    if (head < SP_HEAD_NONE || head > SP_HEAD_SOFTMAX_RM) return fail(SP_ERR_ARG, "sp_mlp_forward: unknown head %d", head);
    if (action_out != nullptr && u == nullptr && philox == nullptr)
        return fail(SP_ERR_NULL, "sp_mlp_forward: action requested but u and philox are NULL");
    if (u != nullptr && philox != nullptr) return fail(SP_ERR_ARG, "sp_mlp_forward: at most one of u and philox may be given");
    MlpArgs a{};
    a.ph.philox_mode = -1;
    for (int i = 0; i <= n_layers; ++i) {
        const int d = dims[i];
        if (d <= 0) return fail(SP_ERR_SHAPE, "sp_mlp_forward: dims[%d] must be positive", i);
        if (i < n_layers) {
            if (d % 16 != 0 || d > MLP_MAX_DIM)
                return fail(SP_ERR_SHAPE, "sp_mlp_forward: dims[%d] = %d must be a multiple of 16 and <= %d", i, d,
                            MLP_MAX_DIM);
            if (i > 0 && d % 32 != 0)
                return fail(SP_ERR_SHAPE, "sp_mlp_forward: hidden width dims[%d] = %d must be a multiple of 32", i, d);
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
    int rc = mlp_set_philox(a.ph, philox, batch, dims[n_layers], __func__);
    if (rc != SP_OK) return rc;
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    a.x = x; a.n_layers = n_layers; a.u = u; a.policy = policy_out; a.action = action_out; a.logits = logits_out;
    a.batch = batch; a.head = head; a.mask_size = mask_size; a.k0 = dims[0]; a.nout = dims[n_layers];
    a.out_stride = dims[n_layers];
    // 4 waves (64 rows) per workgroup while such workgroups fit the compute units in one round: every
    // wave reads all weights from LDS, so 8 waves on a unit are LDS-bandwidth bound (2048 cycles per
    // 32 KiB chunk) where 4 are not; beyond one round, 8 waves (128 rows) halve the rounds
    const int cus = device_cu_count();
    const bool wide = (batch + 63) / 64 > cus;
    const int nw = wide ? 8 : 4;
    bool h256 = n_layers >= 2;   // all hidden layers 256 wide: the lean kernel
    for (int i = 1; i < n_layers; ++i) h256 = h256 && dims[i] == 256;
    // A masked head gives probability zero to the columns past the mask whatever their logits are: when the logits
    // themselves are not asked for, the last layer is computed for the valid columns only (the first rows of its
    // weight matrix) and the head fills the rest of each policy row with zeros.  A 64-wide layer with 3 valid
    // columns, the shape the reference's 16-byte row primitives force on a 3-action game, then runs on the
    // narrow-head kernels.
    if (h256 && head != SP_HEAD_NONE && logits_out == nullptr && mask_size > 0 && mask_size <= 16 &&
        mask_size < dims[n_layers])
        a.nout = mask_size;
    if (h256 && mlp_resident_takes(n_layers, dims, a.nout) &&
        (batch + 63) / 64 >= (long)(mlp_pipe_takes(n_layers, dims, a.nout) ? SP_MLP_PIPE_MIN_TILES_ROWMAJOR
                                                                           : SP_MLP_RESIDENT_MIN_TILES_ROWMAJOR) * cus) {
        // many tiles per compute unit: the kernel that loads the weights once and keeps them in registers
        MlpResidentArgs r{};
        r.x = x; r.u = u; r.policy = policy_out; r.action = action_out; r.logits = logits_out;
        r.batch = batch; r.head = head; r.mask_size = mask_size; r.k0 = a.k0; r.nout = a.nout; r.out_stride = a.out_stride;
        r.ph = a.ph;
        for (int i = 0; i < n_layers; ++i) {
            r.w[i] = a.w[i];
            r.b[i] = a.b[i];
        }
        return mlp_resident_launch(dtype, false, n_layers, r, (hipStream_t)stream, __func__);
    }
    const void* kernel;
    int lds_bytes = MLP_STAGES * MLP_STAGE_BYTES + 1024;   // weight ring + the dummy DMA target
    int rows_per_block = nw * 16;
    int threads = nw * 64;
    // at most one 64-row workgroup per compute unit and a narrow head: hidden layers split by output features
    const bool split = h256 && n_layers >= 3 && !wide && a.nout <= 16;
    if (split) {
        const int ks0 = dims[0] <= 32 ? 1 : dims[0] <= 64 ? 2 : 8;
        kernel = pick_split_kernel(dtype, ks0);
        lds_bytes = SPLIT_LDS_BYTES;
        rows_per_block = SPLIT_ROWS;
        threads = 256;
    } else if (h256) {
        const bool small_k = dims[0] <= 64;
        if (dtype == SP_F16)
            kernel = wide ? (small_k ? (const void*)mlp_h256_kernel<SP_F16, 8, 1> : (const void*)mlp_h256_kernel<SP_F16, 8, 4>)
                          : (small_k ? (const void*)mlp_h256_kernel<SP_F16, 4, 1> : (const void*)mlp_h256_kernel<SP_F16, 4, 4>);
        else
            kernel = wide ? (small_k ? (const void*)mlp_h256_kernel<SP_BF16, 8, 1> : (const void*)mlp_h256_kernel<SP_BF16, 8, 4>)
                          : (small_k ? (const void*)mlp_h256_kernel<SP_BF16, 4, 1> : (const void*)mlp_h256_kernel<SP_BF16, 4, 4>);
    } else if (dtype == SP_F16) {
        kernel = wide ? (const void*)mlp_forward_kernel<SP_F16, 8> : (const void*)mlp_forward_kernel<SP_F16, 4>;
    } else {
        kernel = wide ? (const void*)mlp_forward_kernel<SP_BF16, 8> : (const void*)mlp_forward_kernel<SP_BF16, 4>;
    }
    rc = ensure_dynamic_lds(kernel, lds_bytes);
    if (rc != SP_OK) return rc;
    const long blocks = (batch + rows_per_block - 1) / rows_per_block;
    hipError_t e;
    if (split) {
        if (batch > 0x7fffffffll) return fail(SP_ERR_SHAPE, "sp_mlp_forward: batch must be below 2^31");
        int batch32 = (int)batch;
        unsigned k0_nl_nout = (unsigned)a.k0 | ((unsigned)a.n_layers << 16) | ((unsigned)a.nout << 24);
        void* args[] = {(void*)&a.x, (void*)&a.w[0], (void*)&a.w[1], (void*)&a.b[0], (void*)&a.u, (void*)&batch32,
                        (void*)&k0_nl_nout, (void*)&a};
        e = hipLaunchKernel(kernel, dim3((unsigned)blocks), dim3(threads), args, lds_bytes, (hipStream_t)stream);
    } else {
        void* args[] = {(void*)&a};
        e = hipLaunchKernel(kernel, dim3((unsigned)blocks), dim3(threads), args, lds_bytes, (hipStream_t)stream);
    }
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "sp_mlp_forward: launch failed: %s", hipGetErrorString(e));
    return check_launch(__func__);
}
