// Fused dense-stack forward with the weights RESIDENT in registers, for batches of several 64-row tiles per compute unit.
//
// One launch of the per-tile kernels (mlp.hip, mlp_packed.hip) spends most of its time streaming every layer's
// weights into every compute unit: 274 KiB per unit for 32 -> 256 -> 256 -> 256 -> 3 at the texture path's 64 bytes
// per cycle is as long as the 4.5 k cycles of MFMA work of a 64-row tile, and a workgroup that starts cold pays
// the latency of its first loads on top.  When a unit has more than one tile to do, none of that needs repeating:
// a workgroup of four waves, one per SIMD with 512 registers each, holds ALL the weights of a stack with up to two
// 256 x 256 layers -- wave w keeps output features 64 w .. 64 w + 63 of every feature-split layer (16 or 32 + 128 +
// 128 registers) and the at most 16 rows of the output layer (32 registers), in MFMA operand order -- and walks over
// the tiles blockIdx.x, blockIdx.x + gridDim.x, ...  A tile then costs its MFMAs, the exchange of activations
// through LDS (one barrier per layer), the head, and 4 KiB of input.
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
constexpr int RS_ACT_BYTES = RS_ROWS * 512;              // one activation buffer: 64 rows x 256 features x 2 bytes
constexpr int RS_X_OFF = 2 * RS_ACT_BYTES;               // two input buffers, 64 rows x 128 bytes (a tile's inputs are
constexpr int RS_X_BYTES = RS_ROWS * 128;                //   written while the tile before it is still computed)
constexpr int RS_BIAS_OFF = RS_X_OFF + 2 * RS_X_BYTES;   // the biases of the feature-split layers, 256 f32 each
constexpr int RS_HEAD_OFF = RS_BIAS_OFF + 3 * 1024;      // a KiB per wave: the outputs of a head wider than 4
constexpr int RS_WL_OFF = RS_HEAD_OFF + 4 * 1024;        // the output layer's weights: 8 k-steps x 1 KiB
constexpr int RS_W0_OFF = RS_WL_OFF + 8 * 1024;          // the first layer's: per wave KS0 k-steps x 4 tiles x 1 KiB
constexpr int RS_LDS_TOTAL = RS_W0_OFF + 4 * 2 * 4096;

#ifdef SP_RS_TIMELINE
__device__ unsigned long long sp_rs_timeline[256 * 4 * 16 * 8];
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
__global__ __launch_bounds__(256) void mlp_resident_kernel(const MlpResidentArgs a) {
    constexpr int S = NL - 1;                                // feature-split layers 0 .. S - 1
    static_assert(S == 2 || S == 3, "one or two 256 x 256 layers fit the registers next to the first and the last layer");
    static_assert(KS0 == 1 || KS0 == 2, "a first layer of at most 64 inputs");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, q = lane >> 4;
    const u32x4 zero_u4 = {0u, 0u, 0u, 0u};
    const int K0 = a.k0, NOUT = a.nout;
    const unsigned char* const x_ptr = (const unsigned char*)a.x;
    const long batch = a.batch;
    const int tiles = a.tiles;
    const HeadOut out = HeadOut{a.policy, a.action, a.logits, a.head, a.out_stride};
    const int mask_size = a.mask_size;
    const float* const u_ptr = a.u;
    const float* const last_bias = a.b[S];
    const int ph_mode = a.ph.philox_mode;

    // ---- the biases of the feature-split layers into their LDS table (feature tid of each) ----
    unsigned has_bias = 0;                                   // bit l: layer l has a bias (uniform)
#pragma unroll
    for (int l = 0; l < S; ++l) {
        const float* b = a.b[l];
        if (b != nullptr) {
            has_bias |= 1u << l;
            *reinterpret_cast<float*>(lds + RS_BIAS_OFF + l * 1024 + tid * 4) = b[tid];
        }
    }

    // ---- the weights, once.  The 256 x 256 layers go into the accumulation registers and stay there (block (k-step,
    //      feature tile) = 4 registers: lane (i, q) holds the 8 K-values 32 ks + 8 q .. of feature row i of the
    //      tile); the first layer's few blocks (this wave's) and the output layer's eight (everybody's) go to LDS in
    //      the same order, from where a tile reads them back with one ds_read_b128 each ----
    // (The second 256 x 256 layer keeps its last k-step in ordinary registers: with all 256 accumulation registers
    //  spoken for the register allocator parks one block elsewhere and copies it in front of every use.)
    u32x4 W1[8][4], W2[S == 3 ? 7 : 1][4], W2v[4];
    {
        const int i16 = lane & 15;
        // feature row of lane i in tile t of this wave: 64 w + 32 (t / 2) + 8 (i / 4) + 4 (t % 2) + i % 4
        const unsigned lane_row = (unsigned)(8 * (i16 >> 2) + (i16 & 3));
        unsigned char* const w0_lds = lds + RS_W0_OFF + wave * (KS0 * 4096) + lane * 16;
        unsigned char* const wl_lds = lds + RS_WL_OFF + lane * 16;
        if constexpr (PACKED) {
            const unsigned char* const packed = (const unsigned char*)a.packed;
            const unsigned voff = (unsigned)lane * 16u;
            const long first_bytes = 4l * KS0 * 4096;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W1[ks][t]) : "v"(voff), "s"(packed + first_bytes + ((long)(wave * 8 + ks) * 4 + t) * 1024) : "memory");
            if constexpr (S == 3) {
#pragma unroll
                for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W2[ks][t]) : "v"(voff), "s"(packed + first_bytes + 131072 + ((long)(wave * 8 + ks) * 4 + t) * 1024) : "memory");
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(W2v[t]) : "v"(voff), "s"(packed + first_bytes + 131072 + ((long)(wave * 8 + 7) * 4 + t) * 1024) : "memory");
            }
#pragma unroll
            for (int b = 0; b < 4 * KS0; ++b)
                *reinterpret_cast<u32x4*>(w0_lds + b * 1024) = *reinterpret_cast<const u32x4*>(packed + ((long)wave * KS0 * 4 + b) * 1024 + voff);
#pragma unroll
            for (int h = 0; h < 2; ++h)
                *reinterpret_cast<u32x4*>(wl_lds + (2 * wave + h) * 1024) =
                    *reinterpret_cast<const u32x4*>(packed + first_bytes + (long)(S - 1) * 131072 + (2 * wave + h) * 1024 + voff);
        } else {
            // row-major: base of (tile t) = row 64 w + 32 (t / 2) + 4 (t % 2), k-step ks = 64 bytes further per step;
            // the lane adds its row inside the tile and its quarter of the k-step
            const unsigned char* const w0 = (const unsigned char*)a.w[0];
            const unsigned char* const w1 = (const unsigned char*)a.w[1];
            const unsigned char* const w2 = (const unsigned char*)a.w[S == 3 ? 2 : 1];
            const unsigned char* const wl = (const unsigned char*)a.w[S];
            const unsigned vo_h = (unsigned)((lane_row * 256 + 8 * q) * 2);
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W1[ks][t]) : "v"(vo_h), "s"(w1 + (long)(64 * wave + 32 * (t >> 1) + 4 * (t & 1)) * 512 + ks * 64) : "memory");
            if constexpr (S == 3) {
#pragma unroll
                for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W2[ks][t]) : "v"(vo_h), "s"(w2 + (long)(64 * wave + 32 * (t >> 1) + 4 * (t & 1)) * 512 + ks * 64) : "memory");
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(W2v[t]) : "v"(vo_h), "s"(w2 + (long)(64 * wave + 32 * (t >> 1) + 4 * (t & 1)) * 512 + 7 * 64) : "memory");
            }
            // layer 0: rows of K0 values; k-values past K0 are zeros
#pragma unroll
            for (int ks = 0; ks < KS0; ++ks) {
                const bool ok = 32 * ks + 8 * q < K0;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    u32x4 v = zero_u4;
                    if (ok) v = *reinterpret_cast<const u32x4*>(w0 + ((long)(64 * wave + 32 * (t >> 1) + 4 * (t & 1) + lane_row) * K0 + 32 * ks + 8 * q) * 2);
                    *reinterpret_cast<u32x4*>(w0_lds + (ks * 4 + t) * 1024) = v;
                }
            }
            // output layer: MFMA row i is output i; rows past the computed outputs are zeros
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                u32x4 v = zero_u4;
                if (i16 < NOUT) v = *reinterpret_cast<const u32x4*>(wl + ((long)i16 * 256 + 32 * (2 * wave + h) + 8 * q) * 2);
                *reinterpret_cast<u32x4*>(wl_lds + (2 * wave + h) * 1024) = v;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }

    // ---- operand addresses ----
    // activations: row r, 16-byte piece P (of 32) lives in slot (P & 16) | ((P ^ r) & 15) of the row's 512 bytes
    unsigned aoff[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) aoff[k4] = (unsigned)(j * 512 + (((4 * k4 + q) ^ j) << 4));
    auto read_at = [&](int base, int bt, int ks) {
        return *reinterpret_cast<const u32x4*>(lds + base + aoff[ks & 3] + bt * 8192 + (ks >> 2) * 256);
    };
    // outputs: tiles (p, 0) and (p, 1) give lane (j, q) the features 64 w + 32 p + 8 q .. + 7 of batch row j
    unsigned pw[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) pw[p] = (unsigned)(j * 512 + (wave >> 1) * 256 + (((8 * (wave & 1) + 4 * p + q) ^ j) << 4));

    // the 16-byte pieces of a tile's input rows this thread moves: piece idx = tid + 256 i, 4 KS0 pieces per row
    auto load_x = [&](int tile, u32x4 (&xin)[KS0]) {
        const long row0 = (long)tile * RS_ROWS;
#pragma unroll
        for (int i = 0; i < KS0; ++i) {
            const int idx = tid + 256 * i;
            const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
            const bool ok = row0 + r < batch && pc * 8 < K0;
            xin[i] = zero_u4;
            if (ok) xin[i] = *reinterpret_cast<const u32x4*>(x_ptr + ((row0 + r) * K0 + pc * 8) * 2);
        }
    };
    // inputs: row r, piece pc (of at most 8) lives in slot (pc ^ r) & 7 of the row's 128 bytes
    auto store_x = [&](int buf, const u32x4 (&xin)[KS0]) {
#pragma unroll
        for (int i = 0; i < KS0; ++i) {
            const int idx = tid + 256 * i;
            const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
            *reinterpret_cast<u32x4*>(lds + RS_X_OFF + buf * RS_X_BYTES + r * 128 + (((pc ^ r) & 7) << 4)) = xin[i];
        }
    };
    unsigned xoff[KS0];
#pragma unroll
    for (int ks = 0; ks < KS0; ++ks) xoff[ks] = (unsigned)(RS_X_OFF + j * 128 + ((((4 * ks + q) ^ j) & 7) << 4));

    f32x4 acc[4][4];                                         // [batch tile][feature tile]
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

    // One feature-split layer L reading the activations at LDS offset `in_base` and writing its outputs (bias, relu,
    // rounding) to `out_base`.  K-steps in order, the activation fragments of the next k-step read one at a time behind
    // the first MFMAs.  The LAST two k-steps (the last one, of a layer that has only one) are walked batch tile by
    // batch tile instead: tile bt's sums are then complete while tiles bt + 1 .. 3 are still being multiplied, and
    // its outputs are converted and written one packed word per MFMA, in the matrix pipe's shadow; only the last
    // tile's conversion stands alone.  `before_barrier` runs in front of the barrier that makes the outputs
    // everyone's inputs.
    auto layer = [&](auto L_, int in_base, int out_base, auto&& before_barrier) {
        constexpr int L = decltype(L_)::value;
        constexpr int KS = L == 0 ? KS0 : 8;
        constexpr int TAILK = KS >= 2 ? 2 : 1;                // k-steps walked batch tile by batch tile
        constexpr int HEADK = KS - TAILK;
        const bool with_bias = (has_bias & (1u << L)) != 0;   // uniform
        u32x4 W0[L == 0 ? KS0 : 1][4];                        // the first layer's weights come back from LDS
        if constexpr (L == 0) {
#pragma unroll
            for (int ks = 0; ks < KS0; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    W0[ks][t] = *reinterpret_cast<const u32x4*>(lds + RS_W0_OFF + wave * (KS0 * 4096) + (ks * 4 + t) * 1024 + lane * 16);
        }
        auto mm = [&](f32x4& c, int ks, int t, const u32x4& x, bool first, auto WAIT_) {
            if constexpr (L == 0) mfma_v(c, W0[ks][t], x, first, WAIT_);
            else if constexpr (L == 1) mfma_a(c, W1[ks][t], x, first, WAIT_);
            else if (ks < 7) mfma_a(c, W2[ks < 7 ? ks : 0][t], x, first, WAIT_);
            else mfma_v(c, W2v[t], x, first, WAIT_);
        };
        // activation fragment (batch tile bt, k-step ks) of this layer's input
        auto read_in = [&](int bt, int ks) {
            if constexpr (L == 0) return *reinterpret_cast<const u32x4*>(lds + in_base + xoff[ks] + bt * 2048);
            else return read_at(in_base, bt, ks);
        };
        u32x4 bf[2][4];
#pragma unroll
        for (int bt = 0; bt < 4; ++bt) bf[0][bt] = read_in(bt, 0);
        rs_static_for<0, HEADK>([&](auto KS_) {
            constexpr int ks = decltype(KS_)::value;
            rs_static_for<0, 4>([&](auto T_) {
                constexpr int t = decltype(T_)::value;
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) {
                    mm(acc[bt][t], ks, t, bf[ks & 1][bt], ks == 0, IC<0>{});
                    if (t == 0) bf[(ks + 1) & 1][bt] = read_in(bt, ks + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
        });
        // ---- the end of the layer, batch tile by batch tile ----
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
        // (two copies, with and without a bias: the test is uniform and made once per layer)
        auto end_of_layer = [&](auto HAS_BIAS_) {
            constexpr bool has_b = decltype(HAS_BIAS_)::value != 0;
            f32x4 bias_r[4];                                  // [2 p + h]: features 64 w + 32 p + 8 q + 4 h .. + 3
            if constexpr (has_b) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    bias_r[i] = *reinterpret_cast<const f32x4*>(lds + RS_BIAS_OFF + L * 1024 + (64 * wave + 32 * (i >> 1) + 8 * q + 4 * (i & 1)) * 4);
            }
            // word E (0..7) of batch tile BT's outputs: group p = E / 4 is the tile pair (2 p, 2 p + 1), one 16-byte write
            u32x4 cv;
            auto convert_word = [&](auto BT_, auto E_) {
                constexpr int bt = decltype(BT_)::value, e = decltype(E_)::value;
                constexpr int p = e >> 2, tile = 2 * p + ((e >> 1) & 1), r = 2 * (e & 1);
                float a0 = acc[bt][tile][r], a1 = acc[bt][tile][r + 1];
                if constexpr (has_b) {
                    a0 += bias_r[tile][r];
                    a1 += bias_r[tile][r + 1];
                }
                cv[e & 3] = pack_relu2<DT>(a0, a1);
                if constexpr ((e & 3) == 3) *reinterpret_cast<u32x4*>(lds + out_base + pw[p] + bt * 8192) = cv;
            };
            rs_static_for<0, 4>([&](auto BT_) {
                constexpr int bt = decltype(BT_)::value;
                rs_static_for<0, 4 * TAILK>([&](auto M_) {
                    constexpr int m = decltype(M_)::value;
                    constexpr int ks = HEADK + m / 4, t = m % 4;
                    mm(acc[bt][t], ks, t, bf[ks & 1][bt], ks == 0, IC<1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (bt > 0) {                   // the tile before this one is complete: 8 words over these MFMAs
                        constexpr int per = 8 / (4 * TAILK);
                        rs_static_for<0, per>([&](auto I_) { convert_word(IC<bt - 1>{}, IC<per * m + decltype(I_)::value>{}); });
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            });
            // the last tile: the s_nops are the wait states between the last MFMA and the first read of its result,
            // which the compiler does not know about
            asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
            rs_static_for<0, 8>([&](auto E_) { convert_word(IC<3>{}, E_); });
        };
        if (with_bias) end_of_layer(IC<1>{});
        else end_of_layer(IC<0>{});
        before_barrier();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    // ---- the first tile's inputs ----
    int tile = blockIdx.x;
    int xbuf = 0;
    {
        u32x4 xin[KS0];
        load_x(tile, xin);
        store_x(0, xin);
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");          // inputs and biases are in LDS

#ifdef SP_RS_TIMELINE
    // measurement build: per wave and tile walked, the cycle counter at every phase boundary (8 words per tile)
    int tl_n = 0;
#define SP_RS_STAMP(K) do { if (lane == 0 && tl_n < 16) sp_rs_timeline[(((long)blockIdx.x * 4 + wave) * 16 + tl_n) * 8 + (K)] = (K) == 7 ? __builtin_amdgcn_s_memrealtime() : __builtin_amdgcn_s_memtime(); } while (0)
#else
#define SP_RS_STAMP(K) do {} while (0)
#endif
    for (;;) {
        SP_RS_STAMP(0);
        const int next = tile + (int)gridDim.x;
        const bool has_next = next < tiles;
        const long row0 = (long)tile * RS_ROWS;
        const long head_row_idx = row0 + wave * 16 + j;      // the row lanes 0..15 finish
        const bool head_ok = lane < 16 && head_row_idx < batch;
        float u_row = 1.f;
        if (ph_mode >= 0) u_row = reference_row_uniform(a.ph, head_ok ? head_row_idx : 0);
        else if (u_ptr != nullptr && head_ok) u_row = u_ptr[head_row_idx];
        __builtin_amdgcn_sched_barrier(0);

        // the next tile's inputs are requested in front of the last feature-split layer and written to the other input
        // buffer in front of its barrier (a tile past the end is a tile of zeros)
        u32x4 xnext[KS0];
        auto nothing = [] {};
        auto fetch_next = [&] { load_x(has_next ? next : tiles, xnext); };
        auto publish_next = [&] { store_x(xbuf ^ 1, xnext); };

        layer(IC<0>{}, xbuf * RS_X_BYTES, RS_ACT_BYTES, nothing);
        SP_RS_STAMP(1);
        if constexpr (S == 2) {
            fetch_next();
            __builtin_amdgcn_sched_barrier(0);
            layer(IC<1>{}, RS_ACT_BYTES, 0, publish_next);
            SP_RS_STAMP(2);
        } else {
            layer(IC<1>{}, RS_ACT_BYTES, 0, nothing);
            SP_RS_STAMP(2);
            fetch_next();
            __builtin_amdgcn_sched_barrier(0);
            layer(IC<2>{}, 0, RS_ACT_BYTES, publish_next);
        }
        SP_RS_STAMP(3);

        // ---- output layer: rows 16 wave .. + 15 of the tile; MFMA row i is output i ----
        constexpr int last_in = (S & 1) ? RS_ACT_BYTES : 0;
        f32x4 d;
        {
            u32x4 al[8], WL[8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) al[ks] = read_at(last_in, wave, ks);
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) WL[ks] = *reinterpret_cast<const u32x4*>(lds + RS_WL_OFF + ks * 1024 + lane * 16);
            if constexpr (S == 3) {
                // the next tile's first layer writes the buffer these reads come from: nobody goes on before
                // everybody has them
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
        tile = next;
        xbuf ^= 1;
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
    const long tiles = (a.batch + RS_ROWS - 1) / RS_ROWS;
    if (tiles > 0x7fffffffl - 4096) return fail(SP_ERR_SHAPE, "%s: batch too large", what);
    a.tiles = (int)tiles;
    const int ks0 = a.k0 <= 32 ? 1 : 2;
    const bool plain = a.nout <= 4 && a.out_stride == a.nout && a.logits == nullptr && a.action != nullptr && a.b[n_layers - 1] == nullptr;
    const void* kernel = dtype == SP_F16 ? (packed ? pick_resident<SP_F16, true>(ks0, n_layers, plain) : pick_resident<SP_F16, false>(ks0, n_layers, plain))
                                         : (packed ? pick_resident<SP_BF16, true>(ks0, n_layers, plain) : pick_resident<SP_BF16, false>(ks0, n_layers, plain));
    int rc = ensure_dynamic_lds(kernel, RS_LDS_TOTAL);
    if (rc != SP_OK) return rc;
    const long cus = device_cu_count();
    const unsigned blocks = (unsigned)(tiles < cus ? tiles : cus);
    void* args[] = {(void*)&a};
    hipError_t e = hipLaunchKernel(kernel, dim3(blocks), dim3(256), args, RS_LDS_TOTAL, stream);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return check_launch(what);
}

namespace {
struct MlpResidentKernelNames {
    MlpResidentKernelNames() { register_kernel("mlp_forward_resident", (const void*)mlp_resident_kernel<SP_F16, 1, 4, true, true>, 256); }
} mlp_resident_kernel_names;
}  // namespace

}  // namespace sp

#ifdef SP_RS_TIMELINE
extern "C" int sp_debug_resident_timeline(unsigned long long* host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(sp::sp_rs_timeline), sizeof(unsigned long long) * 256 * 4 * 16 * 8);
}
#endif
