// Fused dense-stack forward with the weights RESIDENT in registers, for batches of several 64-row tiles per compute unit.
//
// One launch of the per-tile kernels (mlp.hip, mlp_packed.hip) spends most of its time streaming every layer's
// weights into every compute unit: 274 KiB per unit for 32 -> 256 -> 256 -> 256 -> 3 at the texture path's 64 bytes
// per cycle is as long as the 4.5 k cycles of MFMA work of a 64-row tile, and a workgroup that starts cold pays
// the latency of its first loads on top.  When a unit has more than one tile to do, none of that needs repeating:
// a workgroup of EIGHT waves, two per SIMD with 256 registers each, holds all the 256 x 256 weights of a stack with
// up to two such layers -- wave v keeps output features 32 v .. 32 v + 31 of each (64 + 64 registers, in MFMA operand
// order); the few KiB of the first and the last layer sit in LDS -- and walks over the tiles blockIdx.x,
// blockIdx.x + gridDim.x, ...  A tile then costs its MFMAs, the exchange of activations through LDS (one barrier
// per layer), the head, and 4 KiB of input.  Tiles are walked in PAIRS: every layer is done for both tiles of a pair
// (128 rows) between two barriers, so the start-up and the drain of a layer -- first fragments on their way, last
// conversion and write, the barrier -- are paid once per 128 rows, a wave's head finishes 16 rows at once, and the
// two waves of a SIMD, which drift apart between barriers, fill each other's gaps.
// Two waves per SIMD, not one with twice the features: a wave cannot issue anything else in the shadow of its own
// MFMAs (every LDS read, conversion or wait of a lone wave costs the matrix pipe 4-5 cycles; measured on the
// four-wave form of this kernel: 3.0-3.2 k cycles per 256 x 256 layer for 2 k cycles of MFMA), its neighbour on the
// SIMD can.
//
// The weights come either packed (sp_mlp_pack_weights: one contiguous KiB per wave-wide load) or straight from the
// row-major matrices of sp_mlp_forward: in operand order a lane then touches half a cache line of a row of its
// own, which the texture path serves at a fraction of its rate -- paid once per launch, not once per tile.
//
// Layer by layer the arithmetic is that of mlp_packed_kernel (same operand layout, same k-order of the sums, same
// head), so results are bit-identical to sp_mlp_forward_packed's per-tile kernel.
//
// Semantics follow the graph interpreter of ml/layers.spi:194-240 and the heads of ml/primitives.spi:711-722,748-798.
#include "mlp_common.h"

#pragma clang fp contract(off)

namespace sp {

constexpr int RS_ROWS = 64;                              // batch rows per tile
constexpr int RS_PAIR_ROWS = 2 * RS_ROWS;                // ... per step of a workgroup's walk
constexpr int RS_WAVES = 8;
constexpr int RS_THREADS = RS_WAVES * 64;
constexpr int RS_TILE_BYTES = RS_ROWS * 512;             // activations of one tile: 64 rows x 256 features x 2 bytes
constexpr int RS_ACT_BYTES = 2 * RS_TILE_BYTES;          // ... of a pair
constexpr int RS_X_OFF = 2 * RS_ACT_BYTES;               // two activation buffers, then the inputs of a pair: 128 rows x 128 bytes
constexpr int RS_HEAD_OFF = RS_X_OFF + RS_PAIR_ROWS * 128;   // a KiB per wave: the outputs of a head wider than 4
constexpr int RS_WL_OFF = RS_HEAD_OFF + RS_WAVES * 1024;     // the output layer's weights: 8 k-steps x 1 KiB
constexpr int RS_LDS_TOTAL = RS_WL_OFF + 8 * 1024;           // = 160 KiB, all of a compute unit's LDS
static_assert(RS_LDS_TOTAL <= 160 * 1024, "fits the LDS of one compute unit");

#ifdef SP_RS_TIMELINE
__device__ unsigned long long sp_rs_timeline[256 * 8 * 16 * 8];
#endif

template <int FROM, int TO, typename F>
__device__ __forceinline__ void rs_static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(IC<FROM>{});
        rs_static_for<FROM + 1, TO>(f);
    }
}

// KS0: 32-wide k-steps of the first layer (1 or 2); NL: layers (3 or 4); PLAIN: at most 4 dense policy columns and an
// action, no logits, no bias on the output layer; PACKED: the weights are in the layout of sp_mlp_pack_weights.
template <int DT, int KS0, int NL, bool PLAIN, bool PACKED>
__global__ __launch_bounds__(RS_THREADS) void mlp_resident_kernel(const MlpResidentArgs a) {
    constexpr int S = NL - 1;                                // feature-split layers 0 .. S - 1
    static_assert(S == 2 || S == 3, "one or two 256 x 256 layers fit the registers");
    static_assert(KS0 == 1 || KS0 == 2, "a first layer of at most 64 inputs");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);      // 0..7: features 32 wave .. 32 wave + 31
    const int w4 = wave >> 1, wp = wave & 1;                        // ... = tile pair wp of the 64-feature slice w4
    const int j = lane & 15, q = lane >> 4;
    const u32x4 zero_u4 = {0u, 0u, 0u, 0u};
    const int K0 = a.k0, NOUT = a.nout;
    const unsigned char* const x_ptr = (const unsigned char*)a.x;
    const long batch = a.batch;
    const int pairs = a.tiles;                               // steps of the walk: pairs of tiles
    const HeadOut out = HeadOut{a.policy, a.action, a.logits, a.head, a.out_stride};
    const int mask_size = a.mask_size;
    const float* const u_ptr = a.u;
    const float* const last_bias = a.b[S];
    const int ph_mode = a.ph.philox_mode;
    unsigned has_bias = 0;                                   // bit l: layer l has a bias (uniform)
#pragma unroll
    for (int l = 0; l < S; ++l)
        if (a.b[l] != nullptr) has_bias |= 1u << l;

    // ---- the weights of the 256 x 256 layers, once: into the accumulation registers, where they stay (block (k-step,
    //      feature tile) = 4 registers: lane (i, q) holds the 8 K-values 32 ks + 8 q .. of feature row i of the
    //      tile; this wave's tiles are 2 wp and 2 wp + 1 of the four that make up slice w4).  The output layer's
    //      eight blocks (everybody's) go to LDS in the same order; the first layer's few blocks are fetched per
    //      pair of tiles (they are a KiB or two per wave, and the L2 has them) ----
    // (The second 256 x 256 layer keeps its last k-step in ordinary registers: a file that is spoken for to the last
    //  register makes the allocator park a block elsewhere and copy it in front of every use.)
    u32x4 W1[8][2], W2[S == 3 ? 7 : 1][2], W2v[2];
    const int i16 = lane & 15;
    // feature row of lane i in tile t of slice w4: 64 w4 + 32 (t / 2) + 8 (i / 4) + 4 (t % 2) + i % 4
    const unsigned lane_row = (unsigned)(8 * (i16 >> 2) + (i16 & 3));
    const long tile_row = 64 * w4 + 32 * wp;                 // first feature row of this wave's tile 0 (tile 1: + 4)
    {
        unsigned char* const wl_lds = lds + RS_WL_OFF + lane * 16;
        if constexpr (PACKED) {
            const unsigned char* const packed = (const unsigned char*)a.packed;
            const unsigned voff = (unsigned)lane * 16u;
            const long first_bytes = 4l * KS0 * 4096;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W1[ks][h]) : "v"(voff), "s"(packed + first_bytes + ((long)(w4 * 8 + ks) * 4 + 2 * wp + h) * 1024) : "memory");
            if constexpr (S == 3) {
#pragma unroll
                for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W2[ks][h]) : "v"(voff), "s"(packed + first_bytes + 131072 + ((long)(w4 * 8 + ks) * 4 + 2 * wp + h) * 1024) : "memory");
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(W2v[h]) : "v"(voff), "s"(packed + first_bytes + 131072 + ((long)(w4 * 8 + 7) * 4 + 2 * wp + h) * 1024) : "memory");
            }
            *reinterpret_cast<u32x4*>(wl_lds + wave * 1024) =
                *reinterpret_cast<const u32x4*>(packed + first_bytes + (long)(S - 1) * 131072 + wave * 1024 + voff);
        } else {
            // row-major: k-step ks = 64 bytes further per step; the lane adds its row inside the tile and its quarter
            const unsigned char* const w1 = (const unsigned char*)a.w[1];
            const unsigned char* const w2 = (const unsigned char*)a.w[S == 3 ? 2 : 1];
            const unsigned char* const wl = (const unsigned char*)a.w[S];
            const unsigned vo_h = (unsigned)((lane_row * 256 + 8 * q) * 2);
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W1[ks][h]) : "v"(vo_h), "s"(w1 + (tile_row + 4 * h) * 512 + ks * 64) : "memory");
            if constexpr (S == 3) {
#pragma unroll
                for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W2[ks][h]) : "v"(vo_h), "s"(w2 + (tile_row + 4 * h) * 512 + ks * 64) : "memory");
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(W2v[h]) : "v"(vo_h), "s"(w2 + (tile_row + 4 * h) * 512 + 7 * 64) : "memory");
            }
            // output layer: MFMA row i is output i; rows past the computed outputs are zeros
            u32x4 v = zero_u4;
            if (i16 < NOUT) v = *reinterpret_cast<const u32x4*>(wl + ((long)i16 * 256 + 32 * wave + 8 * q) * 2);
            *reinterpret_cast<u32x4*>(wl_lds + wave * 1024) = v;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    // the first layer's blocks of this wave (KS0 k-steps x 2 tiles), as the MFMAs read them; k-values past K0 are zeros
    auto load_w0 = [&](u32x4 (&w)[KS0][2]) {
#pragma unroll
        for (int ks = 0; ks < KS0; ++ks)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if constexpr (PACKED) {
                    w[ks][h] = *reinterpret_cast<const u32x4*>((const unsigned char*)a.packed + ((long)(w4 * KS0 + ks) * 4 + 2 * wp + h) * 1024 + lane * 16);
                } else {
                    const bool ok = 32 * ks + 8 * q < K0;
                    const u32x4 v = *reinterpret_cast<const u32x4*>((const unsigned char*)a.w[0] + ((tile_row + 4 * h + lane_row) * K0 + (ok ? 32 * ks + 8 * q : 0)) * 2);
                    w[ks][h] = ok ? v : zero_u4;
                }
            }
    };

    // ---- operand addresses ----
    // activations: row r, 16-byte piece P (of 32) lives in slot (P & 16) | ((P ^ r) & 15) of the row's 512 bytes;
    // rows 64 g + 16 bt + j: tile g of the pair, batch tile bt
    unsigned aoff[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) aoff[k4] = (unsigned)(j * 512 + (((4 * k4 + q) ^ j) << 4));
    auto read_at = [&](int base, int g, int bt, int ks) {
        return *reinterpret_cast<const u32x4*>(lds + base + aoff[ks & 3] + g * RS_TILE_BYTES + bt * 8192 + (ks >> 2) * 256);
    };
    // outputs: this wave's two tiles give lane (j, q) the features 64 w4 + 32 wp + 8 q .. + 7 of batch row j
    const unsigned pw = (unsigned)(j * 512 + (w4 >> 1) * 256 + (((8 * (w4 & 1) + 4 * wp + q) ^ j) << 4));

    // the 16-byte pieces of a pair's input rows this thread moves: 4 KS0 pieces per row, 512 KS0 in all, KS0 per thread.
    // (The loads are unconditional -- a piece outside the batch or past K0 reads the tensor's first bytes and is replaced
    //  by zeros when it is stored: a load under a condition would be waited for where the branches meet.)
    auto x_valid = [&](int pair, int i) {
        const int idx = tid + RS_THREADS * i;
        const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
        return (long)pair * RS_PAIR_ROWS + r < batch && pc * 8 < K0;
    };
    auto load_x = [&](int pair, u32x4 (&v)[KS0]) {
#pragma unroll
        for (int i = 0; i < KS0; ++i) {
            const int idx = tid + RS_THREADS * i;
            const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
            const long off = x_valid(pair, i) ? (((long)pair * RS_PAIR_ROWS + r) * K0 + pc * 8) * 2 : 0;
            v[i] = *reinterpret_cast<const u32x4*>(x_ptr + off);
        }
    };
    // inputs: row r, piece pc (of at most 8) lives in slot (pc ^ r) & 7 of the row's 128 bytes
    auto store_x = [&](int pair, const u32x4 (&v)[KS0]) {
#pragma unroll
        for (int i = 0; i < KS0; ++i) {
            const int idx = tid + RS_THREADS * i;
            const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
            *reinterpret_cast<u32x4*>(lds + RS_X_OFF + r * 128 + (((pc ^ r) & 7) << 4)) = x_valid(pair, i) ? v[i] : zero_u4;
        }
    };
    unsigned xoff[KS0];
#pragma unroll
    for (int ks = 0; ks < KS0; ++ks) xoff[ks] = (unsigned)(RS_X_OFF + j * 128 + ((((4 * ks + q) ^ j) & 7) << 4));

    f32x4 acc[4][2];                                         // [batch tile][feature tile of this wave]
    // The MFMAs are asm: their weight operand lives in registers the asm loads above filled, which the compiler must
    // neither move nor copy.  It therefore cannot see the wait states an MFMA needs after a vector-ALU write of a
    // register it reads; WAIT puts two in front (used where the compiler's own vector-ALU work is interleaved; the
    // build scans the generated code for the pattern everywhere else).
#define SP_RS_MFMA(PRE, T, C, CONSTRAINT, WC) asm volatile(PRE "v_mfma_f32_16x16x32_" T " %0, %1, %2, " C : CONSTRAINT(c) : WC(w), "v"(x))
#define SP_RS_MFMA_ALL(WC)                                                                   \
        if (first) {                                                                         \
            if constexpr (DT == SP_F16 && wait) SP_RS_MFMA("s_nop 1\n\t", "f16", "0", "=v", WC);      \
            else if constexpr (DT == SP_F16) SP_RS_MFMA("", "f16", "0", "=v", WC);                    \
            else if constexpr (wait) SP_RS_MFMA("s_nop 1\n\t", "bf16", "0", "=v", WC);                \
            else SP_RS_MFMA("", "bf16", "0", "=v", WC);                                               \
        } else {                                                                             \
            if constexpr (DT == SP_F16 && wait) SP_RS_MFMA("s_nop 1\n\t", "f16", "%0", "+v", WC);     \
            else if constexpr (DT == SP_F16) SP_RS_MFMA("", "f16", "%0", "+v", WC);                   \
            else if constexpr (wait) SP_RS_MFMA("s_nop 1\n\t", "bf16", "%0", "+v", WC);               \
            else SP_RS_MFMA("", "bf16", "%0", "+v", WC);                                              \
        }
    auto mfma_v = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first, auto WAIT_) {
        constexpr bool wait = decltype(WAIT_)::value != 0;
        SP_RS_MFMA_ALL("v")
    };
    auto mfma_a = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first, auto WAIT_) {
        constexpr bool wait = decltype(WAIT_)::value != 0;
        SP_RS_MFMA_ALL("a")
    };
#undef SP_RS_MFMA_ALL
#undef SP_RS_MFMA


    u32x4 W0[KS0][2];                                        // the first layer's blocks, fetched anew for every pair of tiles

    // One feature-split layer L for both tiles of the pair, reading the activations at LDS offset `in_base` and
    // writing its outputs (bias, relu, rounding) to `out_base`.  Per tile: k-steps in order, the activation fragments
    // of the next k-step read one at a time behind the first MFMAs.  The LAST two k-steps (the last one, of a layer
    // that has only one) are walked batch tile by batch tile instead: batch tile bt's sums are then complete while
    // tiles bt + 1 .. 3 are still being multiplied, and its outputs are converted and written one packed word per
    // MFMA; only the last batch tile's conversion stands alone.  `before_barrier` runs in front of the barrier that
    // makes the outputs everyone's inputs.
    auto layer = [&](auto L_, int in_base, int out_base, auto&& before_barrier) {
        constexpr int L = decltype(L_)::value;
        constexpr int KS = L == 0 ? KS0 : 8;
        constexpr int TAILK = KS >= 2 ? 2 : 1;                // k-steps walked batch tile by batch tile
        constexpr int HEADK = KS - TAILK;
        const bool with_bias = (has_bias & (1u << L)) != 0;   // uniform
        auto mm = [&](f32x4& c, int ks, int h, const u32x4& x, bool first, auto WAIT_) {
            if constexpr (L == 0) mfma_v(c, W0[ks][h], x, first, WAIT_);
            else if constexpr (L == 1) mfma_a(c, W1[ks][h], x, first, WAIT_);
            else if (ks < 7) mfma_a(c, W2[ks < 7 ? ks : 0][h], x, first, WAIT_);
            else mfma_v(c, W2v[h], x, first, WAIT_);
        };
        // (two copies, with and without a bias: the test is uniform and made once per layer)
        auto both_tiles = [&](auto HAS_BIAS_) {
        constexpr bool has_b = decltype(HAS_BIAS_)::value != 0;
        f32x4 bias_r[2];                                      // [h]: features 64 w4 + 32 wp + 8 q + 4 h .. + 3
        if constexpr (has_b) {
#pragma unroll
            for (int h = 0; h < 2; ++h) bias_r[h] = *reinterpret_cast<const f32x4*>(a.b[L] + 64 * w4 + 32 * wp + 8 * q + 4 * h);
        }
        rs_static_for<0, 2>([&](auto G_) {
            constexpr int g = decltype(G_)::value;            // tile of the pair
            // activation fragment (batch tile bt, k-step ks) of this layer's input
            auto read_in = [&](int bt, int ks) {
                if constexpr (L == 0) return *reinterpret_cast<const u32x4*>(lds + xoff[ks] + g * (RS_ROWS * 128) + bt * 2048);
                else return read_at(in_base, g, bt, ks);
            };
            u32x4 bf[2][4];
#pragma unroll
            for (int bt = 0; bt < 4; ++bt) bf[0][bt] = read_in(bt, 0);
            rs_static_for<0, HEADK>([&](auto KS_) {
                constexpr int ks = decltype(KS_)::value;
                rs_static_for<0, 2>([&](auto H_) {
                    constexpr int h = decltype(H_)::value;
#pragma unroll
                    for (int bt = 0; bt < 4; ++bt) {
                        mm(acc[bt][h], ks, h, bf[ks & 1][bt], ks == 0, IC<0>{});
                        if (h == 0) bf[(ks + 1) & 1][bt] = read_in(bt, ks + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            });
            // ---- the end of the tile's layer, batch tile by batch tile ----
            if constexpr (TAILK == 2) {
                // fragments of k-step KS - 1 (those of KS - 2 were read behind the MFMAs of the k-step before it, or above)
                if constexpr (HEADK == 0) {
#pragma unroll
                    for (int bt = 0; bt < 4; ++bt) bf[1][bt] = read_in(bt, 1);
                } else {
#pragma unroll
                    for (int bt = 0; bt < 4; ++bt) bf[(KS - 1) & 1][bt] = read_in(bt, KS - 1);
                }
            }
            {
                // word E (0..3) of batch tile BT's outputs: tile E / 2, accumulator rows 2 (E % 2) and + 1; one 16-byte write
                u32x4 cv;
                auto convert_word = [&](auto BT_, auto E_) {
                    constexpr int bt = decltype(BT_)::value, e = decltype(E_)::value;
                    constexpr int h = e >> 1, r = 2 * (e & 1);
                    float a0 = acc[bt][h][r], a1 = acc[bt][h][r + 1];
                    if constexpr (has_b) {
                        a0 += bias_r[h][r];
                        a1 += bias_r[h][r + 1];
                    }
                    cv[e] = pack_relu2<DT>(a0, a1);
                    if constexpr (e == 3) *reinterpret_cast<u32x4*>(lds + out_base + pw + g * RS_TILE_BYTES + bt * 8192) = cv;
                };
                rs_static_for<0, 4>([&](auto BT_) {
                    constexpr int bt = decltype(BT_)::value;
                    rs_static_for<0, 2 * TAILK>([&](auto M_) {
                        constexpr int m = decltype(M_)::value;
                        constexpr int ks = HEADK + m / 2, h = m % 2;
                        // (wait states in front of the MFMA where the bias additions' register traffic surrounds it; the
                        //  copy without a bias has none of it, and the build's scan of the generated code holds it to that)
                        mm(acc[bt][h], ks, h, bf[ks & 1][bt], ks == 0, IC<has_b ? 1 : 0>{});
                        __builtin_amdgcn_sched_barrier(0);
                        if constexpr (bt > 0) {               // the batch tile before this one is complete: 4 words over these MFMAs
                            constexpr int per = 4 / (2 * TAILK);
                            rs_static_for<0, per>([&](auto I_) { convert_word(IC<bt - 1>{}, IC<per * m + decltype(I_)::value>{}); });
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    });
                });
                // the last batch tile: the s_nops are the wait states between the last MFMA and the first read of its
                // result, which the compiler does not know about (the accumulators are operands so that it cannot
                // move their conversion in front of the wait)
                asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc[3][0]), "+v"(acc[3][1]) : : "memory");
                rs_static_for<0, 4>([&](auto E_) { convert_word(IC<3>{}, E_); });
            }
        });
        };
        if (with_bias) both_tiles(IC<1>{});
        else both_tiles(IC<0>{});
        before_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    // ---- the first pair's inputs and first-layer weights ----
    int pair = blockIdx.x;
    {
        u32x4 xin[KS0];
        load_x(pair, xin);
        store_x(pair, xin);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");          // inputs and the output layer's weights are in LDS

#ifdef SP_RS_TIMELINE
    // measurement build: per wave and step of the walk, the cycle counter at every phase boundary (8 words per step)
    int tl_n = 0;
#define SP_RS_STAMP(K) do { if (lane == 0 && tl_n < 16) sp_rs_timeline[(((long)blockIdx.x * 8 + wave) * 16 + tl_n) * 8 + (K)] = (K) == 7 ? __builtin_amdgcn_s_memrealtime() : __builtin_amdgcn_s_memtime(); } while (0)
#else
#define SP_RS_STAMP(K) do {} while (0)
#endif
    // Two activation buffers P and Q.  Three feature-split layers: inputs -> P -> Q -> P, and the output layer reads P,
    // which the next pair's first layer writes again: a barrier behind the output layer's reads keeps the two apart.
    // Two: inputs -> P -> Q, the output layer reads Q, and nothing of the next pair touches Q before its second barrier.
    constexpr int BUF_P = 0, BUF_Q = RS_ACT_BYTES;
    for (;;) {
        SP_RS_STAMP(0);
        load_w0(W0);                                         // (a KiB or two from the L2, first in line)
        const int next = pair + (int)gridDim.x;
        const bool has_next = next < pairs;
        float u_row = 1.f;                                   // of the row lanes 0..15 finish
        {
            const long r = (long)pair * RS_PAIR_ROWS + wave * 16 + j;
            const long r_ok = lane < 16 && r < batch ? r : 0;
            if (ph_mode >= 0) u_row = reference_row_uniform(a.ph, r_ok);
            else if (u_ptr != nullptr) u_row = u_ptr[r_ok];                        // (unconditional per lane, as above)
        }
        // the next pair's inputs are requested now (they come from HBM and take a microsecond) and written over this
        // pair's in front of the last feature-split layer's barrier (a pair past the end is a pair of zeros)
        u32x4 xnext[KS0];
        load_x(has_next ? next : pairs, xnext);
        __builtin_amdgcn_sched_barrier(0);
        auto nothing = [] {};
        auto publish_next = [&] { store_x(has_next ? next : pairs, xnext); };

        layer(IC<0>{}, 0, BUF_P, nothing);
        SP_RS_STAMP(1);
        if constexpr (S == 2) {
            layer(IC<1>{}, BUF_P, BUF_Q, publish_next);
            SP_RS_STAMP(2);
        } else {
            layer(IC<1>{}, BUF_P, BUF_Q, nothing);
            SP_RS_STAMP(2);
            layer(IC<2>{}, BUF_Q, BUF_P, publish_next);
        }
        SP_RS_STAMP(3);

        // ---- output layer: rows 16 wave .. + 15 of the pair; MFMA row i is output i ----
        constexpr int last_in = S == 3 ? BUF_P : BUF_Q;
        f32x4 d;
        {
            u32x4 al[8], WL[8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) al[ks] = read_at(last_in, wave >> 2, wave & 3, ks);     // (tile wave / 4 of the pair, batch tile wave % 4)
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) WL[ks] = *reinterpret_cast<const u32x4*>(lds + RS_WL_OFF + ks * 1024 + lane * 16);
            if constexpr (S == 3) {
                // the next pair's first layer writes the buffer these reads come from: nobody goes on before everybody
                // has them
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
            // even and odd k-steps add up separately: two chains of four dependent MFMAs instead of one of eight
            f32x4 dd[2];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const f32x4 c = ks < 2 ? f32x4{0.f, 0.f, 0.f, 0.f} : dd[ks & 1];
                if constexpr (DT == SP_F16)
                    dd[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, WL[ks]), __builtin_bit_cast(f16x8, al[ks]), c, 0, 0, 0);
                else
                    dd[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, WL[ks]), __builtin_bit_cast(bf16x8, al[ks]), c, 0, 0, 0);
            }
            d = dd[0] + dd[1];
        }
        SP_RS_STAMP(4);
        // (the row numbers are worked out here rather than carried through the layers in registers)
        const long row0 = (long)pair * RS_PAIR_ROWS;
        const long head_row_idx = row0 + wave * 16 + j;
        const bool head_ok = lane < 16 && head_row_idx < batch;
        const float* bias = last_bias;
        const int limit = mask_size > 0 ? mask_size : NOUT;
        if constexpr (PLAIN) {
            const float p[4] = {d[0], d[1], d[2], d[3]};
            if (head_ok) head_row4_plain_any(out.head, out.policy, out.action, p, head_row_idx, NOUT, limit, u_row);
        } else {
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
                        store16_through(reinterpret_cast<f32x4*>(block + (long)r * out.stride + 4 * c), f32x4{0.f, 0.f, 0.f, 0.f});
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
                if (head_ok) head_row4_any(out.head, out, p, head_row_idx, NOUT, limit, u_row, fill_end);
            } else {
                // the wave's 16 x NOUT outputs staged in its own KiB of LDS
                float* head_rows = reinterpret_cast<float*>(lds + RS_HEAD_OFF + wave * 1024);
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
        SP_RS_STAMP(5);
        SP_RS_STAMP(7);
#ifdef SP_RS_TIMELINE
        ++tl_n;
#endif
        if (!has_next) break;
        pair = next;
    }
#undef SP_RS_STAMP
}

template <int DT, int KS0, int NL, bool PACKED>
static const void* pick_resident_plain(bool plain) {
    return plain ? (const void*)mlp_resident_kernel<DT, KS0, NL, true, PACKED> : (const void*)mlp_resident_kernel<DT, KS0, NL, false, PACKED>;
}
template <int DT, bool PACKED>
static const void* pick_resident(int ks0, int n_layers, bool plain) {
    if (n_layers == 3) return ks0 == 1 ? pick_resident_plain<DT, 1, 3, PACKED>(plain) : pick_resident_plain<DT, 2, 3, PACKED>(plain);
    return ks0 == 1 ? pick_resident_plain<DT, 1, 4, PACKED>(plain) : pick_resident_plain<DT, 2, 4, PACKED>(plain);
}

// Stacks the resident kernel takes: 3 or 4 layers, hidden widths 256, at most 64 inputs, at most 16 computed outputs.
bool mlp_resident_takes(int n_layers, const int32_t* dims, int nout) {
    if (n_layers != 3 && n_layers != 4) return false;
    if (dims[0] <= 0 || dims[0] % 16 != 0 || dims[0] > 64) return false;
    for (int i = 1; i < n_layers; ++i)
        if (dims[i] != 256) return false;
    return nout >= 1 && nout <= 16;
}

// Launches the resident kernel on `a` (every field but `tiles` filled in by the caller, who has checked the stack with
// mlp_resident_takes): one workgroup per compute unit, fewer when there are fewer tiles.
int mlp_resident_launch(int dtype, bool packed, int n_layers, MlpResidentArgs a, hipStream_t stream, const char* what) {
    if (n_layers == 4 && a.k0 <= 64 && a.nout <= 4) return mlp_pipe_launch(dtype, packed, a, stream, what);
    const long pairs = (a.batch + RS_PAIR_ROWS - 1) / RS_PAIR_ROWS;
    if (pairs > 0x7fffffffl - 4096) return fail(SP_ERR_SHAPE, "%s: batch too large", what);
    a.tiles = (int)pairs;                                  // the kernel walks pairs of tiles
    const int ks0 = a.k0 <= 32 ? 1 : 2;
    const bool plain = a.nout <= 4 && a.out_stride == a.nout && a.logits == nullptr && a.action != nullptr && a.b[n_layers - 1] == nullptr;
    const void* kernel = dtype == SP_F16 ? (packed ? pick_resident<SP_F16, true>(ks0, n_layers, plain) : pick_resident<SP_F16, false>(ks0, n_layers, plain))
                                         : (packed ? pick_resident<SP_BF16, true>(ks0, n_layers, plain) : pick_resident<SP_BF16, false>(ks0, n_layers, plain));
    const int lds_bytes = RS_LDS_TOTAL;
    int rc = ensure_dynamic_lds(kernel, lds_bytes);
    if (rc != SP_OK) return rc;
    const long cus = device_cu_count();
    const unsigned blocks = (unsigned)(pairs < cus ? pairs : cus);
    void* args[] = {(void*)&a};
    hipError_t e = hipLaunchKernel(kernel, dim3(blocks), dim3(RS_THREADS), args, lds_bytes, stream);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return check_launch(what);
}

namespace {
struct MlpResidentKernelNames {
    MlpResidentKernelNames() { register_kernel("mlp_forward_resident", (const void*)mlp_resident_kernel<SP_F16, 1, 4, true, true>, RS_THREADS); }
} mlp_resident_kernel_names;
}  // namespace

}  // namespace sp

#ifdef SP_RS_TIMELINE
extern "C" int sp_debug_resident_timeline(unsigned long long* host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(sp::sp_rs_timeline), sizeof(unsigned long long) * 256 * 8 * 16 * 8);
}
#endif
