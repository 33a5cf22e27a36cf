// Fused forward of a four-layer stack (K0 -> 256 -> 256 -> 256 -> at most 4 outputs) for batches of many tiles per
// compute unit: weights resident in registers, and the two 256 x 256 layers run as a two-stage PIPELINE on the two
// waves of every SIMD.
//
// mlp_resident.hip keeps the weights in registers and walks over tiles; what it cannot do is keep the matrix pipe busy
// while a tile passes through the parts that are chains of latencies -- first fragments on their way from LDS, the
// last conversion and write of a layer, the barrier, the first layer's 16 MFMAs, the head's hundred dependent
// instructions on a handful of lanes: all eight waves reach them together (measured: 2.6 k cycles for a 256 x 256
// layer's 2.07 k of MFMA, 3.4 k more per tile in first layer, output layer and head), and with every wave reading all
// of a layer's activations the LDS is as busy as the matrix pipe.  Here the two waves of a SIMD have different jobs:
//   wave A (w4 = its number, 0..3) holds features 64 w4 .. + 63 of layer 1 (128 registers) and, per step t of the
//          walk, multiplies layer 1 of tile t and then the first layer of tile t + 1;
//   wave B (same SIMD) holds the same features of layer 2 and, per step, multiplies layer 2 of tile t - 1, feeds its
//          own 64 features of the result -- which, rounded, are in the output layer's operand order already -- to the
//          output layer's weights for those features, and leaves the partial sums of the (at most 4) outputs in LDS;
//          every eighth step it finishes the eight tiles before that (sum of the partial results, head, sampling: a
//          few hundred dependent instructions that cost the same for 64 lanes as for 8).
// One barrier per step.  While one wave waits or converts, its neighbour multiplies; an activation fragment read from
// LDS feeds four MFMAs instead of two, and the second layer's outputs never go to LDS at all.  Every buffer that is
// written and read in the same step exists twice (tiles are 32 rows so that all of them fit).
//
// The sums of the three feature-split layers add up in the same order as in the other kernels of this family; the
// output layer adds its k-steps per 64-feature slice and then the four slices in order, so logits agree with the
// other kernels to rounding, not bit for bit.
//
// Semantics follow the graph interpreter of ml/layers.spi:194-240 and the heads of ml/primitives.spi:711-722,748-798.
#include "mlp_common.h"

#pragma clang fp contract(off)

namespace sp {

constexpr int PP_ROWS = 32;                              // batch rows per tile
constexpr int PP_THREADS = 512;
constexpr int PP_ACT_BYTES = PP_ROWS * 512;              // activations of one tile: 32 rows x 256 features x 2 bytes
constexpr int PP_X_BYTES = PP_ROWS * 128;                // inputs of one tile: 32 rows x (at most) 64 features x 2 bytes
constexpr int PP_X_OFF = 0;                              // two input buffers
constexpr int PP_H0_OFF = PP_X_OFF + 2 * PP_X_BYTES;     // two buffers of first-layer outputs
constexpr int PP_H1_OFF = PP_H0_OFF + 2 * PP_ACT_BYTES;  // two buffers of layer-1 outputs
constexpr int PP_PO_OFF = PP_H1_OFF + 2 * PP_ACT_BYTES;  // a ring of 16 tiles' output-layer partial sums: 4 slices x 32 rows x 4 f32
constexpr int PP_PO_BYTES = 4 * 32 * 16;
constexpr int PP_PO_RING = 16;
constexpr int PP_HEAD_TILES = 8;                         // tiles finished per head pass: 8 rows of each per B wave = 64 lanes
constexpr int PP_BIAS_OFF = PP_PO_OFF + PP_PO_RING * PP_PO_BYTES; // the biases of the three feature-split layers, 256 f32 each
constexpr int PP_W0_OFF = PP_BIAS_OFF + 3 * 1024;        // the first layer's weights: per A wave KS0 k-steps x 4 tiles x 1 KiB
constexpr int pp_lds_total(int ks0) { return PP_W0_OFF + 4 * ks0 * 4096; }

#ifdef SP_PP_TIMELINE
__device__ unsigned long long sp_pp_timeline[256 * 8 * 8 * 4];
#endif

template <int FROM, int TO, typename F>
__device__ __forceinline__ void pp_static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(IC<FROM>{});
        pp_static_for<FROM + 1, TO>(f);
    }
}

// KS0: 32-wide k-steps of the first layer (1 or 2); PLAIN: a dense policy and an action, no logits, no bias on the
// output layer; PACKED: the weights are in the layout of sp_mlp_pack_weights.
template <int DT, int KS0, bool PLAIN, bool PACKED>
__global__ __launch_bounds__(PP_THREADS) void mlp_pipe_kernel(const MlpResidentArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int role = wave >> 2;                              // 0: wave A (layers 0 and 1), 1: wave B (layer 2, output layer, head)
    const int w4 = wave & 3;                                 // features 64 w4 .. + 63; waves w4 and w4 + 4 share a SIMD
    const int j = lane & 15, q = lane >> 4;
    const u32x4 zero_u4 = {0u, 0u, 0u, 0u};
    const int K0 = a.k0, NOUT = a.nout;
    const unsigned char* const x_ptr = (const unsigned char*)a.x;
    const long batch = a.batch;
    const long tiles_all = a.tiles;
    const HeadOut out = HeadOut{a.policy, a.action, a.logits, a.head, a.out_stride};
    const int mask_size = a.mask_size;
    const float* const u_ptr = a.u;
    const float* const last_bias = a.b[3];
    const int ph_mode = a.ph.philox_mode;
    // tiles of this workgroup: blockIdx.x, blockIdx.x + gridDim.x, ...
    const int T = (int)((tiles_all - blockIdx.x + gridDim.x - 1) / gridDim.x);
    auto tile_of = [&](int t) { return (long)blockIdx.x + (long)t * gridDim.x; };

    unsigned has_bias = 0;                                   // bit l: layer l has a bias (uniform)
#pragma unroll
    for (int l = 0; l < 3; ++l) {
        const float* b = a.b[l];
        if (b != nullptr) {
            has_bias |= 1u << l;
            if (tid < 256) *reinterpret_cast<float*>(lds + PP_BIAS_OFF + l * 1024 + tid * 4) = b[tid];
        }
    }

    // ---- the weights, once.  Wave A: layer 1, wave B: layer 2 -- the same code on another matrix: 8 k-steps x 4
    //      feature tiles of 4 registers (lane (i, q) holds the 8 K-values 32 ks + 8 q .. of feature row i of the
    //      tile), in the accumulation registers but for the last k-step (a register file that is spoken for to the last
    //      register makes the allocator park a block elsewhere and copy it in front of every use).  Wave A also puts
    //      its blocks of the first layer into LDS, wave B keeps the output layer's blocks for its own 64 features
    //      (k-steps 2 w4 and 2 w4 + 1) in registers. ----
    u32x4 W[7][4], Wv[4], WLr[2];
    const int i16 = lane & 15;
    // feature row of lane i in tile t of slice w4: 64 w4 + 32 (t / 2) + 8 (i / 4) + 4 (t % 2) + i % 4
    const unsigned lane_row = (unsigned)(8 * (i16 >> 2) + (i16 & 3));
    {
        unsigned char* const w0_lds = lds + PP_W0_OFF + w4 * (KS0 * 4096) + lane * 16;
        if constexpr (PACKED) {
            const unsigned char* const packed = (const unsigned char*)a.packed;
            const unsigned voff = (unsigned)lane * 16u;
            const long first_bytes = 4l * KS0 * 4096;
            const unsigned char* const mine = packed + first_bytes + (long)role * 131072 + (long)w4 * 32768;
#pragma unroll
            for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W[ks][t]) : "v"(voff), "s"(mine + (ks * 4 + t) * 1024) : "memory");
#pragma unroll
            for (int t = 0; t < 4; ++t)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(Wv[t]) : "v"(voff), "s"(mine + (7 * 4 + t) * 1024) : "memory");
            if (role == 0) {
#pragma unroll
                for (int b = 0; b < 4 * KS0; ++b)
                    *reinterpret_cast<u32x4*>(w0_lds + b * 1024) = *reinterpret_cast<const u32x4*>(packed + ((long)w4 * KS0 * 4 + b) * 1024 + voff);
            }
#pragma unroll
            for (int p = 0; p < 2; ++p)
                WLr[p] = *reinterpret_cast<const u32x4*>(packed + first_bytes + 2 * 131072 + (2 * w4 + p) * 1024 + voff);
        } else {
            const unsigned char* const wm = (const unsigned char*)a.w[1 + role];
            const unsigned char* const w0 = (const unsigned char*)a.w[0];
            const unsigned char* const wl = (const unsigned char*)a.w[3];
            const unsigned vo_h = (unsigned)((lane_row * 256 + 8 * q) * 2);
#pragma unroll
            for (int ks = 0; ks < 7; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=a"(W[ks][t]) : "v"(vo_h), "s"(wm + (long)(64 * w4 + 32 * (t >> 1) + 4 * (t & 1)) * 512 + ks * 64) : "memory");
#pragma unroll
            for (int t = 0; t < 4; ++t)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(Wv[t]) : "v"(vo_h), "s"(wm + (long)(64 * w4 + 32 * (t >> 1) + 4 * (t & 1)) * 512 + 7 * 64) : "memory");
            if (role == 0) {
                // layer 0: rows of K0 values; k-values past K0 are zeros
#pragma unroll
                for (int ks = 0; ks < KS0; ++ks) {
                    const bool ok = 32 * ks + 8 * q < K0;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        u32x4 v = zero_u4;
                        if (ok) v = *reinterpret_cast<const u32x4*>(w0 + ((long)(64 * w4 + 32 * (t >> 1) + 4 * (t & 1) + lane_row) * K0 + 32 * ks + 8 * q) * 2);
                        *reinterpret_cast<u32x4*>(w0_lds + (ks * 4 + t) * 1024) = v;
                    }
                }
            }
            // output layer: MFMA row i is output i; rows past the computed outputs are zeros
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                WLr[p] = zero_u4;
                if (i16 < NOUT) WLr[p] = *reinterpret_cast<const u32x4*>(wl + ((long)i16 * 256 + 32 * (2 * w4 + p) + 8 * q) * 2);
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
    // outputs: tiles (p, 0) and (p, 1) give lane (j, q) the features 64 w4 + 32 p + 8 q .. + 7 of batch row j
    unsigned pw[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) pw[p] = (unsigned)(j * 512 + (w4 >> 1) * 256 + (((8 * (w4 & 1) + 4 * p + q) ^ j) << 4));
    // inputs: row r, piece pc (of at most 8) lives in slot (pc ^ r) & 7 of the row's 128 bytes
    unsigned xoff[KS0];
#pragma unroll
    for (int ks = 0; ks < KS0; ++ks) xoff[ks] = (unsigned)(j * 128 + ((((4 * ks + q) ^ j) & 7) << 4));
    // the 16-byte piece of a tile's input rows this thread moves (4 KS0 pieces per row, 128 KS0 in all; the threads of
    // the A waves).  The load is unconditional -- a piece outside the batch or past K0 reads the tensor's first bytes and
    // is replaced by zeros when it is stored: a load under a condition would be waited for where the branches meet.
    const int x_r = tid / (4 * KS0), x_pc = tid % (4 * KS0);
    const bool x_mine = tid < 128 * KS0;
    auto x_valid = [&](int t) { return x_mine && t < T && tile_of(t) * PP_ROWS + x_r < batch && x_pc * 8 < K0; };
    auto load_x = [&](int t) {
        const long off = x_valid(t) ? ((tile_of(t) * PP_ROWS + x_r) * K0 + x_pc * 8) * 2 : 0;
        return *reinterpret_cast<const u32x4*>(x_ptr + off);
    };
    auto store_x = [&](int buf, const u32x4& v, bool valid) {
        if (x_mine) *reinterpret_cast<u32x4*>(lds + PP_X_OFF + buf * PP_X_BYTES + x_r * 128 + (((x_pc ^ x_r) & 7) << 4)) = valid ? v : zero_u4;
    };

    f32x4 acc[2][4];                                         // [batch tile][feature tile]
    // The MFMAs are asm: their weight operand lives in registers the asm loads above filled, which the compiler must
    // neither move nor copy.  It therefore cannot see the wait states an MFMA needs after a vector-ALU write of a
    // register it reads; WAIT puts two in front (used where the compiler's own vector-ALU work is interleaved; the
    // build scans the generated code for the pattern everywhere else).
#define SP_PP_MFMA(PRE, T, C, CONSTRAINT, WC) asm volatile(PRE "v_mfma_f32_16x16x32_" T " %0, %1, %2, " C : CONSTRAINT(c) : WC(w), "v"(x))
#define SP_PP_MFMA_ALL(WC)                                                                   \
        if (first) {                                                                         \
            if constexpr (DT == SP_F16 && wait) SP_PP_MFMA("s_nop 1\n\t", "f16", "0", "=v", WC);      \
            else if constexpr (DT == SP_F16) SP_PP_MFMA("", "f16", "0", "=v", WC);                    \
            else if constexpr (wait) SP_PP_MFMA("s_nop 1\n\t", "bf16", "0", "=v", WC);                \
            else SP_PP_MFMA("", "bf16", "0", "=v", WC);                                               \
        } else {                                                                             \
            if constexpr (DT == SP_F16 && wait) SP_PP_MFMA("s_nop 1\n\t", "f16", "%0", "+v", WC);     \
            else if constexpr (DT == SP_F16) SP_PP_MFMA("", "f16", "%0", "+v", WC);                   \
            else if constexpr (wait) SP_PP_MFMA("s_nop 1\n\t", "bf16", "%0", "+v", WC);               \
            else SP_PP_MFMA("", "bf16", "%0", "+v", WC);                                              \
        }
    auto mfma_v = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first, auto WAIT_) {
        constexpr bool wait = decltype(WAIT_)::value != 0;
        SP_PP_MFMA_ALL("v")
    };
    auto mfma_a = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first, auto WAIT_) {
        constexpr bool wait = decltype(WAIT_)::value != 0;
        SP_PP_MFMA_ALL("a")
    };
#undef SP_PP_MFMA_ALL
#undef SP_PP_MFMA

    // One feature-split layer of one tile.  FIRST: the first layer (weights from LDS, inputs from an input buffer at
    // `in_base`), else a 256 x 256 layer on this wave's resident weights.  TO_LDS: outputs (bias, relu, rounding) go to
    // the activation buffer at `out_base`; else they stay in registers as the output layer's operand and the partial
    // sums of the outputs go to `out_base`.  K-steps in order, the two activation fragments of the next k-step read
    // behind the first MFMAs; the LAST two k-steps (the last one, of a layer that has only one) run batch tile by batch
    // tile, so that batch tile 0 is converted among the MFMAs of batch tile 1.
    auto layer = [&](auto FIRST_, auto TO_LDS_, int bias_layer, int in_base, int out_base) {
        constexpr bool FIRST = decltype(FIRST_)::value != 0, TO_LDS = decltype(TO_LDS_)::value != 0;
        constexpr int KS = FIRST ? KS0 : 8;
        constexpr int TAILK = KS >= 2 ? 2 : 1;
        constexpr int HEADK = KS - TAILK;
        const bool with_bias = (has_bias & (1u << bias_layer)) != 0;   // uniform
        u32x4 W0[FIRST ? KS0 : 1][4];
        if constexpr (FIRST) {
#pragma unroll
            for (int ks = 0; ks < KS0; ++ks)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    W0[ks][t] = *reinterpret_cast<const u32x4*>(lds + PP_W0_OFF + w4 * (KS0 * 4096) + (ks * 4 + t) * 1024 + lane * 16);
        }
        auto mm = [&](f32x4& c, int ks, int t, const u32x4& x, bool first, auto WAIT_) {
            if constexpr (FIRST) mfma_v(c, W0[ks][t], x, first, WAIT_);
            else if (ks < 7) mfma_a(c, W[ks < 7 ? ks : 0][t], x, first, WAIT_);
            else mfma_v(c, Wv[t], x, first, WAIT_);
        };
        auto read_in = [&](int bt, int ks) {
            if constexpr (FIRST) return *reinterpret_cast<const u32x4*>(lds + in_base + xoff[ks] + bt * 2048);
            else return read_at(in_base, bt, ks);
        };
        f32x4 po[2];                                          // (TO_LDS == false) partial sums of the outputs, per batch tile
        // (two copies, with and without a bias: the test is uniform and made once per layer)
        auto body = [&](auto HAS_BIAS_) {
            constexpr bool has_b = decltype(HAS_BIAS_)::value != 0;
            f32x4 bias_r[4];                                  // [2 p + h]: features 64 w4 + 32 p + 8 q + 4 h .. + 3
            if constexpr (has_b) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    bias_r[i] = *reinterpret_cast<const f32x4*>(lds + PP_BIAS_OFF + bias_layer * 1024 + (64 * w4 + 32 * (i >> 1) + 8 * q + 4 * (i & 1)) * 4);
            }
            // the fragments of a k-step are requested TWO k-steps ahead: eight MFMAs are 130 cycles, less than an LDS
            // read takes once the neighbouring wave reads too
            u32x4 bf[3][2];
#pragma unroll
            for (int bt = 0; bt < 2; ++bt) bf[0][bt] = read_in(bt, 0);
            if constexpr (KS >= 2) {
#pragma unroll
                for (int bt = 0; bt < 2; ++bt) bf[1][bt] = read_in(bt, 1);
            }
            pp_static_for<0, HEADK>([&](auto KS_) {
                constexpr int ks = decltype(KS_)::value;
                pp_static_for<0, 4>([&](auto T_) {
                    constexpr int t = decltype(T_)::value;
#pragma unroll
                    for (int bt = 0; bt < 2; ++bt) {
                        mm(acc[bt][t], ks, t, bf[ks % 3][bt], ks == 0, IC<0>{});
                        if (t == 0 && ks + 2 < KS) bf[(ks + 2) % 3][bt] = read_in(bt, ks + 2);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            });
            // word E (0..7) of batch tile BT's outputs: group p = E / 4 is the tile pair (2 p, 2 p + 1): four words = the 8
            // features 64 w4 + 32 p + 8 q .. + 7 of batch row j, one 16-byte piece of the next layer's operand
            u32x4 cv[2];                                      // (one per group: an MFMA may still be reading the other)
            auto convert_word = [&](auto BT_, auto E_) {
                constexpr int bt = decltype(BT_)::value, e = decltype(E_)::value;
                constexpr int p = e >> 2, tile = 2 * p + ((e >> 1) & 1), r = 2 * (e & 1);
                float a0 = acc[bt][tile][r], a1 = acc[bt][tile][r + 1];
                if constexpr (has_b) {
                    a0 += bias_r[tile][r];
                    a1 += bias_r[tile][r + 1];
                }
                cv[p][e & 3] = pack_relu2<DT>(a0, a1);
                if constexpr ((e & 3) == 3) {
                    if constexpr (TO_LDS) *reinterpret_cast<u32x4*>(lds + out_base + pw[p] + bt * 8192) = cv[p];
                    else mfma_v(po[bt], WLr[p], cv[p], p == 0, IC<1>{});       // k-step 2 w4 + p of the output layer
                }
            };
            pp_static_for<0, 2>([&](auto BT_) {
                constexpr int bt = decltype(BT_)::value;
                pp_static_for<0, 4 * TAILK>([&](auto M_) {
                    constexpr int m = decltype(M_)::value;
                    constexpr int ks = HEADK + m / 4, t = m % 4;
                    mm(acc[bt][t], ks, t, bf[ks % 3][bt], ks == 0, IC<1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (bt > 0) {                   // batch tile 0 is complete: its 8 words over these MFMAs
                        constexpr int per = 8 / (4 * TAILK);
                        pp_static_for<0, per>([&](auto I_) { convert_word(IC<bt - 1>{}, IC<per * m + decltype(I_)::value>{}); });
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            });
            // the last batch tile: the s_nops are the wait states between the last MFMA and the first read of its
            // result, which the compiler does not know about (the accumulators are operands so that it cannot move
            // their conversion in front of the wait)
            asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc[1][0]), "+v"(acc[1][1]), "+v"(acc[1][2]), "+v"(acc[1][3]) : : "memory");
            pp_static_for<0, 8>([&](auto E_) { convert_word(IC<1>{}, E_); });
        };
        if (with_bias) body(IC<1>{});
        else body(IC<0>{});
        if constexpr (!TO_LDS) {
            // the partial sums of this slice: lane (j, q) holds outputs 4 q .. 4 q + 3 of batch row 16 bt + j
            asm volatile("s_nop 15\n\ts_nop 3" : "+v"(po[0]), "+v"(po[1]) : : "memory");
            if (q == 0) {
#pragma unroll
                for (int bt = 0; bt < 2; ++bt)
                    *reinterpret_cast<f32x4*>(lds + out_base + ((w4 * 2 + bt) * 16 + j) * 16) = po[bt];
            }
        }
    };

    // ---- prologue: inputs of tiles 0 and 1, the first layer of tile 0 ----
    store_x(0, load_x(0), x_valid(0));
    store_x(1, load_x(1), x_valid(1));
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");          // inputs, biases and first-layer weights are in LDS
    if (role == 0) layer(IC<1>{}, IC<1>{}, 0, PP_X_OFF, PP_H0_OFF);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // A head pass finishes the tiles whose partial sums are complete and not yet used -- tiles `done` .. s - 2 in step s
    // -- once there are PP_HEAD_TILES of them, or in the last step: lane 8 g + i of B wave w4 finishes row 8 w4 + i of
    // tile done + g.  The row's uniform is requested at the start of the step before, so that it has long arrived.
    // Always a load (from the inputs when there is no tensor of uniforms): a load under a condition would be waited for
    // where the branches meet.
    int done = 0;                                            // tiles finished so far (uniform)
    auto pass_due = [&](int s_pass, int done_then) { return s_pass - 1 - done_then == PP_HEAD_TILES || (s_pass == T + 1 && done_then < T); };
    auto head_row_of = [&](int t) { return tile_of(t) * PP_ROWS + w4 * 8 + (lane & 7); };
    const unsigned char* const u_or_x = u_ptr != nullptr ? (const unsigned char*)u_ptr : x_ptr;
    auto fetch_u = [&](int s_pass, int done_then) {
        const int t = done_then + (lane >> 3);
        const bool ok = t < s_pass - 1 && t < T;
        const long r = head_row_of(ok ? t : 0);
        const long r_ok = u_ptr != nullptr && ok && r < batch ? r : 0;
        float u = *reinterpret_cast<const float*>(u_or_x + r_ok * 4);
        if (ph_mode >= 0) u = reference_row_uniform(a.ph, ok && r < batch ? r : 0);
        return u;
    };
    float u_next = 1.f;

#ifdef SP_PP_TIMELINE
    // measurement build: per wave and step, the cycle counter at the step's start, between its two parts, in front of and
    // behind its barrier
#define SP_PP_STAMP(K) do { if (lane == 0 && s >= 4 && s < 12) sp_pp_timeline[(((long)blockIdx.x * 8 + wave) * 8 + (s - 4)) * 4 + (K)] = __builtin_amdgcn_s_memtime(); } while (0)
#else
#define SP_PP_STAMP(K) do {} while (0)
#endif
    for (int s = 0; s < T + 2; ++s) {
        SP_PP_STAMP(0);
        const bool due = pass_due(s, done);
        const int done_after = due ? s - 1 : done;
        if (role == 0) {
            // ---- wave A: layer 1 of tile s, the first layer of tile s + 1; the inputs of tile s + 2 on their way ----
            const u32x4 xnext = load_x(s + 2);
            const bool xnext_valid = x_valid(s + 2);
            __builtin_amdgcn_sched_barrier(0);
            if (s < T) layer(IC<0>{}, IC<1>{}, 1, PP_H0_OFF + (s & 1) * PP_ACT_BYTES, PP_H1_OFF + (s & 1) * PP_ACT_BYTES);
            SP_PP_STAMP(1);
            if (s + 1 < T) layer(IC<1>{}, IC<1>{}, 0, PP_X_OFF + ((s + 1) & 1) * PP_X_BYTES, PP_H0_OFF + ((s + 1) & 1) * PP_ACT_BYTES);
            store_x(s & 1, xnext, xnext_valid);
        } else {
            // ---- wave B: a head pass when one is due; layer 2 + its share of the output layer of tile s - 1 ----
            const float u_row = u_next;
            if (pass_due(s + 1, done_after)) u_next = fetch_u(s + 1, done_after);
            __builtin_amdgcn_sched_barrier(0);
            if (due) {
                const int count = s - 1 - done;               // 1 .. PP_HEAD_TILES tiles
                const int t = done + (lane >> 3);
                const bool t_ok = (lane >> 3) < count;
                const int tt = t_ok ? t : done;
                const int r = 8 * w4 + (lane & 7);            // row of the tile: batch tile r / 16, accumulator lane r % 16
                const unsigned char* po_base = lds + PP_PO_OFF + (tt & (PP_PO_RING - 1)) * PP_PO_BYTES + r * 16;
                f32x4 d = *reinterpret_cast<const f32x4*>(po_base);
#pragma unroll
                for (int sl = 1; sl < 4; ++sl) d = d + *reinterpret_cast<const f32x4*>(po_base + sl * 512);
                const long head_row_idx = head_row_of(tt);
                const bool head_ok = t_ok && head_row_idx < batch;
                const int limit = mask_size > 0 ? mask_size : NOUT;
                if constexpr (PLAIN) {
                    const float p[4] = {d[0], d[1], d[2], d[3]};
                    if (head_ok) head_row4_plain_any(out.head, out.policy, out.action, p, head_row_idx, NOUT, limit, u_row);
                } else {
                    // A masked head that was computed for its valid columns only: the wave's 8 policy rows of a tile are
                    // one contiguous block, whose zeros the wave writes 16 bytes per lane.
                    int fill_end = 1 << 30;
                    if (out.stride > NOUT && (out.stride & 3) == 0) {
                        const int s4 = out.stride >> 2, c0 = (NOUT + 3) >> 2;
                        fill_end = 4 * c0;
                        for (int g = 0; g < count; ++g) {
                            const long first_row = tile_of(done + g) * PP_ROWS + w4 * 8;
                            float* block = out.policy + first_row * out.stride;
                            for (int idx = lane; idx < 8 * s4; idx += 64) {
                                const int rr = idx / s4, c = idx - rr * s4;
                                if (c >= c0 && first_row + rr < batch)
                                    store16_through(reinterpret_cast<f32x4*>(block + (long)rr * out.stride + 4 * c), f32x4{0.f, 0.f, 0.f, 0.f});
                            }
                        }
                    }
                    float p[4];
#pragma unroll
                    for (int n = 0; n < 4; ++n) {
                        p[n] = d[n];
                        if (last_bias != nullptr && n < NOUT) p[n] += last_bias[n];
                    }
                    if (head_ok) head_row4_any(out.head, out, p, head_row_idx, NOUT, limit, u_row, fill_end);
                }
            }
            SP_PP_STAMP(1);
            if (s >= 1 && s - 1 < T)
                layer(IC<0>{}, IC<0>{}, 2, PP_H1_OFF + ((s - 1) & 1) * PP_ACT_BYTES, PP_PO_OFF + ((s - 1) & (PP_PO_RING - 1)) * PP_PO_BYTES);
        }
        done = done_after;
        SP_PP_STAMP(2);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        SP_PP_STAMP(3);
    }
#undef SP_PP_STAMP
}

template <int DT, int KS0, bool PACKED>
static const void* pick_pipe_plain(bool plain) {
    return plain ? (const void*)mlp_pipe_kernel<DT, KS0, true, PACKED> : (const void*)mlp_pipe_kernel<DT, KS0, false, PACKED>;
}
template <int DT, bool PACKED>
static const void* pick_pipe(int ks0, bool plain) {
    return ks0 == 1 ? pick_pipe_plain<DT, 1, PACKED>(plain) : pick_pipe_plain<DT, 2, PACKED>(plain);
}

// Stacks the pipelined kernel takes: K0 <= 64 -> 256 -> 256 -> 256 -> at most 4 computed outputs.
bool mlp_pipe_takes(int n_layers, const int32_t* dims, int nout) {
    if (n_layers != 4) return false;
    if (dims[0] <= 0 || dims[0] % 16 != 0 || dims[0] > 64) return false;
    for (int i = 1; i < n_layers; ++i)
        if (dims[i] != 256) return false;
    return nout >= 1 && nout <= 4;
}

// Launches the pipelined kernel on `a` (every field but `tiles` filled in by the caller, who has checked the stack with
// mlp_pipe_takes): one workgroup per compute unit, fewer when there are fewer tiles.
int mlp_pipe_launch(int dtype, bool packed, MlpResidentArgs a, hipStream_t stream, const char* what) {
    const long tiles = (a.batch + PP_ROWS - 1) / PP_ROWS;
    if (tiles > 0x7fffffffl - 4096) return fail(SP_ERR_SHAPE, "%s: batch too large", what);
    a.tiles = (int)tiles;
    const int ks0 = a.k0 <= 32 ? 1 : 2;
    const bool plain = a.out_stride == a.nout && a.logits == nullptr && a.action != nullptr && a.b[3] == nullptr;
    const void* kernel = dtype == SP_F16 ? (packed ? pick_pipe<SP_F16, true>(ks0, plain) : pick_pipe<SP_F16, false>(ks0, plain))
                                         : (packed ? pick_pipe<SP_BF16, true>(ks0, plain) : pick_pipe<SP_BF16, false>(ks0, plain));
    const int lds_bytes = pp_lds_total(ks0);
    int rc = ensure_dynamic_lds(kernel, lds_bytes);
    if (rc != SP_OK) return rc;
    const long cus = device_cu_count();
    const unsigned blocks = (unsigned)(tiles < cus ? tiles : cus);
    void* args[] = {(void*)&a};
    hipError_t e = hipLaunchKernel(kernel, dim3(blocks), dim3(PP_THREADS), args, lds_bytes, stream);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "%s: launch failed: %s", what, hipGetErrorString(e));
    return check_launch(what);
}

namespace {
struct MlpPipeKernelNames {
    MlpPipeKernelNames() { register_kernel("mlp_forward_pipelined", (const void*)mlp_pipe_kernel<SP_F16, 1, true, true>, PP_THREADS); }
} mlp_pipe_kernel_names;
}  // namespace

}  // namespace sp

#ifdef SP_PP_TIMELINE
extern "C" int sp_debug_pipe_timeline(unsigned long long* host_out) {
    return (int)hipMemcpyFromSymbol(host_out, HIP_SYMBOL(sp::sp_pp_timeline), sizeof(unsigned long long) * 256 * 8 * 8 * 4);
}
#endif
