// Fused dense-stack forward over PRE-PACKED weights for gfx950: the weights never touch the LDS.
//
// Stacks of 256-wide hidden layers with a narrow head (the policy networks of the reference's agents) are bound by
// how fast every compute unit can pull all the weights out of the L2 -- 274 KiB per unit and launch for
// 32 -> 256 -> 256 -> 256 -> 3, against 4.5 k cycles of MFMA work for 64 batch rows.  Measured on all 256 units at
// once, that stream runs at the texture path's 64 bytes per cycle and unit when every load is in flight from the
// start, and at half of that when it is fed through an LDS ring that compute has to drain first.  So this kernel
// asks for everything at once and lets the register file be the buffer: a workgroup is four waves, one per SIMD,
// each with 512 registers; wave w owns output features 64 w .. 64 w + 63 of every hidden layer for all 64 batch
// rows of the workgroup and holds its 32 KiB slice of a layer's weights in 128 accumulation registers, two such
// sets (layer l in set l % 2), loaded straight from global memory as MFMA operands.  That needs the weights in
// operand order (one contiguous KiB per wave-wide load: lane (i, q) holds the 8 K-values 32 ks + 8 q .. of feature
// row i of a 16-row tile), which is what sp_mlp_pack_weights writes once per set of weights.
// Layer l + 2 is requested into set l % 2 k-step by k-step, as layer l's MFMAs release the registers.
// Activations are exchanged through two LDS buffers of 64 rows x 256 features (16-byte pieces of a row XOR-swizzled
// with the row number), layer l reading one and writing the other: one barrier per layer.
// The output layer (at most 16 outputs) is split by batch rows: wave w multiplies rows 16 w .. 16 w + 15, and lanes
// 0..15 run the head.
// All weight loads are issued from assembly and counted by hand (the counter of outstanding loads runs in order
// and the schedule is static): every wait names the exact number of younger loads.
//
// Semantics follow the graph interpreter of ml/layers.spi:194-240 and the heads of ml/primitives.spi:711-722,748-798,
// like sp_mlp_forward.
#include "mlp_common.h"

#pragma clang fp contract(off)

namespace sp {

constexpr int PK_ROWS = 64;                              // batch rows per workgroup
constexpr int PK_ACT_BYTES = PK_ROWS * 512;              // one activation buffer: 64 rows x 256 features x 2 bytes
constexpr int PK_BIAS_OFF = 2 * PK_ACT_BYTES;            // then the biases of the feature-split layers, 256 f32 each
constexpr int PK_LDS_BYTES = PK_BIAS_OFF + (MLP_MAX_LAYERS - 1) * 1024;
constexpr int PK_HIDDEN_BYTES = 256 * 256 * 2;           // a packed hidden layer
constexpr int PK_LAST_BYTES = 8 * 1024;                  // the packed output layer: 8 k-steps x one 16-row tile

__host__ __device__ constexpr int pk_ks0(int k0) { return k0 <= 32 ? 1 : (k0 <= 64 ? 2 : 8); }
__host__ __device__ constexpr long pk_first_bytes(int ks0) { return 4l * ks0 * 4096; }
__host__ __device__ constexpr long pk_total_bytes(int ks0, int n_layers) {
    return pk_first_bytes(ks0) + (long)(n_layers - 2) * PK_HIDDEN_BYTES + PK_LAST_BYTES;
}

struct MlpPackedArgs {
    const void* x;
    const void* packed;
    const float* b[MLP_MAX_LAYERS];
    const float* u;
    float* policy;
    int* action;
    float* logits;
    long batch;
    int head, mask_size, k0, nout, out_stride;
    PhiloxStream ph;     // philox_mode >= 0: the head draws its uniform itself and `u` is not read
};

// Where feature-split layer `layer` (0: the first layer with ks0 k-steps, else a hidden layer) keeps the block of
// (wave, k-step, feature tile): one KiB, 16 bytes per lane.
__host__ __device__ constexpr long pk_block_offset(int ks0, int layer, int wave, int ks, int t) {
    return layer == 0 ? ((long)(wave * ks0 + ks) * 4 + t) * 1024
                      : pk_first_bytes(ks0) + (long)(layer - 1) * PK_HIDDEN_BYTES + ((long)(wave * 8 + ks) * 4 + t) * 1024;
}

// One thread per 16-byte piece of the packed buffer.
template <int DT>
__global__ __launch_bounds__(256) void mlp_pack_kernel(const MlpArgs a, unsigned char* packed, int ks0, long pieces) {
    const long g = (long)blockIdx.x * 256 + threadIdx.x;
    if (g >= pieces) return;
    const int NL = a.n_layers;
    const long first = pk_first_bytes(ks0) / 16, hidden = PK_HIDDEN_BYTES / 16;
    int layer, ksn;
    long rel;
    if (g < first) { layer = 0; rel = g; ksn = ks0; }
    else if (g < first + (long)(NL - 2) * hidden) { layer = 1 + (int)((g - first) / hidden); rel = (g - first) % hidden; ksn = 8; }
    else { layer = NL - 1; rel = g - first - (long)(NL - 2) * hidden; ksn = 8; }
    const int lane = (int)(rel & 63);
    const int block = (int)(rel >> 6);
    const int i = lane & 15, q = lane >> 4;
    const int K = a.dims[layer], N = a.dims[layer + 1];
    int row, ks;
    if (layer < NL - 1) {
        const int t = block & 3;
        ks = (block >> 2) % ksn;
        const int wave = (block >> 2) / ksn;
        // tile (p, h) = (t / 2, t % 2) feeds MFMA row i with feature 32 p + 8 (i / 4) + 4 h + i % 4 of the wave's 64
        row = 64 * wave + 32 * (t >> 1) + 8 * (i >> 2) + 4 * (t & 1) + (i & 3);
    } else {
        ks = block;
        row = i;       // the first 16 outputs: a wider layer is only ever run under a mask of at most 16 columns
    }
    const int k = 32 * ks + 8 * q;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < N && k < K) v = *reinterpret_cast<const u32x4*>((const unsigned char*)a.w[layer] + ((long)row * K + k) * 2);
    *reinterpret_cast<u32x4*>(packed + g * 16) = v;
}

// f(IC<I>{}) for I = FROM .. TO - 1: loop indices that have to be constant expressions (asm immediates).
template <int FROM, int TO, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(IC<FROM>{});
        static_for<FROM + 1, TO>(f);
    }
}

// ---- the schedule of the weight loads (all compile time) ----
// A load instruction is not fire-and-forget: the texture path takes one wave-wide 1 KiB load per ~16 cycles per
// compute unit and its queue is short, so a wave that issues loads back to back stands still for as long as the
// data takes to stream (asking for all 274 KiB up front kept every wave at its load instructions for 4 k cycles).
// The loads are therefore dealt out over the whole kernel, one at a time between other work, in the order the
// layers need them:
//   program order: G = KS0 + 1 + S per-thread loads (inputs, uniform, biases), layer 0's 4 KS0 blocks, then the
//   queue q = 0 .. QN - 1: layers 1 .. S - 1 (32 blocks each, k-step by k-step), the output layer's 8 blocks;
//   issue slots:   phase 0 (start-up, while the first data is on its way): PK_SLOTS_START; phase 2 L + 1 (the MFMAs
//   of layer L): one behind every fourth MFMA and PK_SLOTS_TAIL more at its end; phase 2 L + 2 (the last of layer
//   L's outputs are converted and written): none.  (Measured: a load among MFMAs costs the wave ~6 cycles, among
//   the conversions ~40.)
// A block of layer l lands in the registers layer l - 2 multiplied from, so it may go out from phase 2 l - 2 on.
// Every wait names the exact number of loads issued after the one it needs (the counter runs in order).
#ifndef SP_PK_SLOTS_START
#define SP_PK_SLOTS_START 8
#endif
constexpr int PK_SLOTS_START = SP_PK_SLOTS_START;
#ifndef SP_PK_SLOTS_TAIL
#define SP_PK_SLOTS_TAIL 4
#endif
constexpr int PK_SLOTS_TAIL = SP_PK_SLOTS_TAIL;      // extra slots in the batch-tile-major end of a layer

template <int KS0, int NL>
struct PkSched {
    static constexpr int S = NL - 1;                    // feature-split layers 0 .. S - 1
    static constexpr int G = KS0 + 1 + S;
    static constexpr int QN = 32 * (S - 1) + 8;
    static constexpr int PHASES = 2 * S + 1;
    static constexpr int slots(int p) { return p == 0 ? PK_SLOTS_START : (p & 1) ? 4 * (p == 1 ? KS0 : 8) + PK_SLOTS_TAIL : 0; }
    static constexpr int allowed(int p) {               // queue entries that may have gone out by the end of phase p
        const int lmax = (p + 2) / 2 < S - 1 ? (p + 2) / 2 : S - 1;
        return lmax == S - 1 ? QN : 32 * lmax;
    }
    static constexpr int first_q(int p) {               // queue entries issued before phase p
        if (p == 0) return 0;
        const int n = first_q(p - 1) + slots(p - 1);
        return n < allowed(p - 1) ? n : allowed(p - 1);
    }
    static constexpr int issued_at(int p, int s) {      // ... before slot s of phase p
        return first_q(p) + s < first_q(p + 1) ? first_q(p) + s : first_q(p + 1);
    }
    // loads younger than the blocks of k-step ks of layer L at the wait in front of slot `at` of that layer's phase
    static constexpr int younger(int L, int ks, int at) {
        const int issued = G + 4 * KS0 + issued_at(2 * L + 1, at);
        const int pos_end = L == 0 ? G + 4 * (ks + 1) : G + 4 * KS0 + 32 * (L - 1) + 4 * ks + 4;
        return issued - pos_end;
    }
    static constexpr int clamp63(int n) { return n > 63 ? 63 : n; }   // the wait's operand has 6 bits; waiting for more is safe
    static constexpr int inputs_landed = 4 * KS0 + first_q(1);
    static constexpr bool all_issued = first_q(PHASES) == QN;
};

// PLAIN: the commonest call -- a dense policy of at most 4 columns and an action, no logits, no bias on the output
// layer -- gets an instantiation that ends in nothing but that head: what follows the last MFMA is fetched cold,
// once per launch, and every jump over code that does not run is another round trip to the instruction cache.
// The leading parameters repeat fields of `a`: this file is built with kernel-argument preloading, which hands the
// first 14 dwords of scalar parameters to a wave in registers when it starts (a struct is not preloaded), so the
// addresses the first loads need are there without the ~900-cycle round trip of a scalar load from the argument
// block; everything else is read from `a` while those loads are in flight.  (`k0_nout`: k0 | nout << 16; stacks with
// more than three feature-split layers read all their bias pointers from `a` instead, up front as before.)
template <int DT, int KS0, int NL, bool PLAIN>
__global__ __launch_bounds__(256) void mlp_packed_kernel(const void* x_first, const void* packed_first, const float* u_first,
                                                         const float* b0_first, const float* b1_first, const float* b2_first,
                                                         int batch_first, unsigned k0_nout, const MlpPackedArgs a) {
    typedef PkSched<KS0, NL> SCH;
    constexpr int S = SCH::S;
    static_assert(SCH::all_issued, "every weight block has an issue slot");
    static_assert(S >= 2 && NL <= MLP_MAX_LAYERS, "three to eight layers");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, q = lane >> 4;
    const long row0 = (long)blockIdx.x * PK_ROWS;
    const u32x4 zero_u4 = {0u, 0u, 0u, 0u};
    const int K0 = (int)(k0_nout & 0xffffu), NOUT = (int)(k0_nout >> 16);
    const unsigned char* const x_ptr = (const unsigned char*)x_first;
    const unsigned char* const packed = (const unsigned char*)packed_first;
    const long batch = batch_first;
    const HeadOut out = HeadOut{a.policy, a.action, a.logits, a.head, a.out_stride};
    const int mask_size = a.mask_size;
    const float* const u_ptr = u_first;
    const float* const last_bias = a.b[S];
    const int ph_mode = a.ph.philox_mode;

    // ---- per-thread loads: the workgroup's input rows (16-byte pieces, 4 KS0 per row), the uniform of the row
    //      this lane will finish, one bias value per feature-split layer (feature tid) ----
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
    float u_row;
    {
        const unsigned char* up = u_ptr != nullptr ? (const unsigned char*)(u_ptr + (head_ok ? head_row_idx : 0)) : x_ptr;
        asm volatile("global_load_dword %0, %1, off" : "=v"(u_row) : "v"(up) : "memory");
    }
    float bias_in[S];
    unsigned has_bias = 0;                                   // bit l: layer l has a bias (uniform)
#pragma unroll
    for (int l = 0; l < S; ++l) {
        const float* b = S > 3 ? a.b[l] : l == 0 ? b0_first : l == 1 ? b1_first : b2_first;
        if (b != nullptr) has_bias |= 1u << l;
        const unsigned char* bp = b != nullptr ? (const unsigned char*)(b + tid) : x_ptr;   // always a load: fixed count
        asm volatile("global_load_dword %0, %1, off" : "=v"(bias_in[l]) : "v"(bp) : "memory");
    }

    // ---- the weights: two sets of 8 k-steps x 4 feature tiles in the accumulation registers, the output layer's
    //      8 blocks in ordinary registers ----
    u32x4 WA[8][4], WB[8][4], WL[8];
    const unsigned voff = (unsigned)lane * 16u;
    auto load_acc = [voff](u32x4& dst, const unsigned char* base, auto IMM_) {   // (a name used only as an asm operand is not captured implicitly)
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=a"(dst) : "v"(voff), "s"(base), "n"(decltype(IMM_)::value) : "memory");
    };
    auto load_reg = [voff](u32x4& dst, const unsigned char* base) {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(base) : "memory");
    };
    auto layer_base = [&](int l) {      // this wave's first block of feature-split layer l
        return packed + (l == 0 ? (long)wave * (KS0 * 4096) : pk_first_bytes(KS0) + (long)(l - 1) * PK_HIDDEN_BYTES + (long)wave * 32768);
    };
    auto wreg = [&](auto SET_, int ks, int t) -> u32x4& {
        if constexpr (decltype(SET_)::value == 0) return WA[ks][t];
        else return WB[ks][t];
    };
    auto load_kstep = [&](auto SET_, int l, int ks) {         // the four blocks of k-step ks of layer l
        const unsigned char* base = layer_base(l) + ks * 4096;
        load_acc(wreg(SET_, ks, 0), base, IC<0>{});
        load_acc(wreg(SET_, ks, 1), base, IC<1024>{});
        load_acc(wreg(SET_, ks, 2), base, IC<2048>{});
        load_acc(wreg(SET_, ks, 3), base, IC<3072>{});
    };
#pragma unroll
    for (int ks = 0; ks < KS0; ++ks) load_kstep(IC<0>{}, 0, ks);
    // entry Q of the queue: block (k-step, tile) of layer 1 + Q / 32, or block Q - 32 (S - 1) of the output layer
    auto issue = [&](auto Q_) {
        constexpr int Q = decltype(Q_)::value;
        if constexpr (Q < 32 * (S - 1)) {
            constexpr int l = 1 + Q / 32, ks = (Q % 32) / 4, t = Q % 4;
            load_acc(wreg(IC<(l & 1)>{}, ks, t), layer_base(l) + ks * 4096, IC<1024 * t>{});
        } else if constexpr (Q < SCH::QN) {
            load_reg(WL[Q - 32 * (S - 1)], packed + pk_first_bytes(KS0) + (long)(S - 1) * PK_HIDDEN_BYTES + (Q - 32 * (S - 1)) * 1024);
        }
    };
    // slot s of phase P
    auto slot = [&](auto P_, auto S_) {
        constexpr int P = decltype(P_)::value, s_ = decltype(S_)::value;
        if constexpr (SCH::first_q(P) + s_ < SCH::first_q(P + 1)) issue(IC<SCH::first_q(P) + s_>{});
    };
    static_for<0, PK_SLOTS_START>([&](auto S_) { slot(IC<0>{}, S_); });
    // every other scalar argument is waited for HERE, once, behind the first loads: a read at the point of use costs
    // a few hundred cycles, and the wait for it also drains the LDS reads in flight
    asm volatile("" ::"s"(out.policy), "s"(out.action), "s"(out.logits), "s"(out.head), "s"(out.stride), "s"(mask_size), "s"(last_bias),
                 "s"(ph_mode));
    // a head that draws its own uniform does so here, while the first loads are on their way
    float u_ph = 0.f;
    if (ph_mode >= 0) u_ph = reference_row_uniform(a.ph, head_ok ? head_row_idx : 0);

    // ---- operand addresses ----
    // activations: row r, 16-byte piece P (of 32) lives in slot (P & 16) | ((P ^ r) & 15) of the row's 512 bytes
    unsigned aoff[4];
#pragma unroll
    for (int k4 = 0; k4 < 4; ++k4) aoff[k4] = (unsigned)(j * 512 + (((4 * k4 + q) ^ j) << 4));
    auto read_a = [&](int buf, int bt, int ks) {
        return *reinterpret_cast<const u32x4*>(lds + buf * PK_ACT_BYTES + aoff[ks & 3] + bt * 8192 + (ks >> 2) * 256);
    };
    // outputs: tiles (p, 0) and (p, 1) give lane (j, q) the features 64 w + 32 p + 8 q .. + 7 of batch row j
    unsigned pw[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) pw[p] = (unsigned)(j * 512 + (wave >> 1) * 256 + (((8 * (wave & 1) + 4 * p + q) ^ j) << 4));

    // ---- the per-thread loads have landed: inputs into activation buffer 0, biases into their LDS table ----
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SCH::clamp63(SCH::inputs_landed)) : "memory");
#pragma unroll
    for (int i = 0; i < KS0; ++i) asm volatile("" : "+v"(xin[i]));
    asm volatile("" : "+v"(u_row));
    if (ph_mode >= 0) u_row = u_ph;
#pragma unroll
    for (int l = 0; l < S; ++l) asm volatile("" : "+v"(bias_in[l]));
#pragma unroll
    for (int i = 0; i < KS0; ++i) {
        const int idx = tid + 256 * i;
        const int r = idx / (4 * KS0), pc = idx % (4 * KS0);
        *reinterpret_cast<u32x4*>(lds + r * 512 + (pc & 16) * 16 + (((pc ^ r) & 15) << 4)) = x_ok[i] ? xin[i] : zero_u4;
    }
#pragma unroll
    for (int l = 0; l < S; ++l)
        if (has_bias & (1u << l)) *reinterpret_cast<float*>(lds + PK_BIAS_OFF + l * 1024 + tid * 4) = bias_in[l];
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    f32x4 acc[4][4];                                         // [batch tile][feature tile]
    // The MFMAs are asm (their weight operand is filled by asm loads the compiler must not move or copy), so the
    // compiler cannot see the wait states one needs after a vector-ALU write of a register it reads: where the
    // register allocator moves an accumulator with v_mov right in front of the MFMA, the matrix pipe reads the old
    // value.  WAIT puts two wait states in front (used where the compiler's own vector-ALU work is interleaved; the
    // build scans the generated code for the pattern everywhere else).
    auto mfma_acc = [&](f32x4& c, const u32x4& w, const u32x4& x, bool first, auto WAIT_) {
        constexpr bool wait = decltype(WAIT_)::value != 0;   // (the s_nop has to sit in the MFMA's own asm statement:
                                                             //  the moves are placed right in front of the statement)
#define SP_PK_MFMA(PRE, T, C, CONSTRAINT) asm volatile(PRE "v_mfma_f32_16x16x32_" T " %0, %1, %2, " C : CONSTRAINT(c) : "a"(w), "v"(x))
        if (first) {
            if constexpr (DT == SP_F16 && wait) SP_PK_MFMA("s_nop 1\n\t", "f16", "0", "=v");
            else if constexpr (DT == SP_F16) SP_PK_MFMA("", "f16", "0", "=v");
            else if constexpr (wait) SP_PK_MFMA("s_nop 1\n\t", "bf16", "0", "=v");
            else SP_PK_MFMA("", "bf16", "0", "=v");
        } else {
            if constexpr (DT == SP_F16 && wait) SP_PK_MFMA("s_nop 1\n\t", "f16", "%0", "+v");
            else if constexpr (DT == SP_F16) SP_PK_MFMA("", "f16", "%0", "+v");
            else if constexpr (wait) SP_PK_MFMA("s_nop 1\n\t", "bf16", "%0", "+v");
            else SP_PK_MFMA("", "bf16", "%0", "+v");
        }
#undef SP_PK_MFMA
    };

    // One feature-split layer L.  K-steps in order, the activation fragments of the next k-step read one at a time
    // behind the first MFMAs, a weight block of the queue requested behind every fourth MFMA.  The LAST two k-steps
    // (the last one, of a layer that has only one) are walked batch tile by batch tile instead: tile bt's sums are
    // then complete while tiles bt + 1 .. 3 are still being multiplied, and its outputs (bias, relu, rounding) are
    // converted and written to the other activation buffer one packed word per MFMA, in the matrix pipe's shadow;
    // only the last tile's conversion stands alone.  The barrier makes the outputs everyone's inputs.
    auto layer = [&](auto L_) {
        constexpr int L = decltype(L_)::value;
        constexpr int KS = L == 0 ? KS0 : 8;
        constexpr int TAILK = KS >= 2 ? 2 : 1;                // k-steps walked batch tile by batch tile
        constexpr int HEADK = KS - TAILK;
        constexpr int in_buf = L & 1;
        constexpr int PHASE = 2 * L + 1;
        const bool with_bias = (has_bias & (1u << L)) != 0;   // uniform
        u32x4 bf[2][4];
#pragma unroll
        for (int bt = 0; bt < 4; ++bt) bf[0][bt] = read_a(in_buf, bt, 0);
        static_for<0, HEADK>([&](auto KS_) {
            constexpr int ks = decltype(KS_)::value;
            static_assert(SCH::younger(L, ks, 4 * ks) >= 0, "a block is requested before the k-step that multiplies it");
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SCH::clamp63(SCH::younger(L, ks, 4 * ks))) : "memory");
            static_for<0, 4>([&](auto T_) {
                constexpr int t = decltype(T_)::value;
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) {
                    mfma_acc(acc[bt][t], wreg(IC<(L & 1)>{}, ks, t), bf[ks & 1][bt], ks == 0, IC<0>{});
                    if (t == 0) bf[(ks + 1) & 1][bt] = read_a(in_buf, bt, ks + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                slot(IC<PHASE>{}, IC<4 * ks + t>{});
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        // ---- the end of the layer, batch tile by batch tile ----
        if constexpr (TAILK == 2) {
            // fragments of k-step KS - 1 (those of KS - 2 were read behind the MFMAs of the k-step before it, or above)
            if constexpr (HEADK == 0) {
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) bf[1][bt] = read_a(in_buf, bt, 1);
            } else {
#pragma unroll
                for (int bt = 0; bt < 4; ++bt) bf[(KS - 1) & 1][bt] = read_a(in_buf, bt, KS - 1);
            }
        }
        static_assert(SCH::younger(L, KS - 1, 4 * HEADK) >= 0, "a block is requested before the k-step that multiplies it");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SCH::clamp63(SCH::younger(L, KS - 1, 4 * HEADK))) : "memory");
        // (two copies, with and without a bias: the test is uniform and made once per layer)
        auto end_of_layer = [&](auto HAS_BIAS_) {
            constexpr bool has_b = decltype(HAS_BIAS_)::value != 0;
            f32x4 bias_r[4];                                  // [2 p + h]: features 64 w + 32 p + 8 q + 4 h .. + 3
            if constexpr (has_b) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    bias_r[i] = *reinterpret_cast<const f32x4*>(lds + PK_BIAS_OFF + L * 1024 + (64 * wave + 32 * (i >> 1) + 8 * q + 4 * (i & 1)) * 4);
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
                if constexpr ((e & 3) == 3) *reinterpret_cast<u32x4*>(lds + (in_buf ^ 1) * PK_ACT_BYTES + pw[p] + bt * 8192) = cv;
            };
            static_for<0, 4>([&](auto BT_) {
                constexpr int bt = decltype(BT_)::value;
                static_for<0, 4 * TAILK>([&](auto M_) {
                    constexpr int m = decltype(M_)::value;
                    constexpr int ks = HEADK + m / 4, t = m % 4;
                    mfma_acc(acc[bt][t], wreg(IC<(L & 1)>{}, ks, t), bf[ks & 1][bt], ks == 0, IC<1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (bt > 0) {                   // the tile before this one is complete: 8 words over these MFMAs
                        constexpr int per = 8 / (4 * TAILK);
                        static_for<0, per>([&](auto I_) { convert_word(IC<bt - 1>{}, IC<per * m + decltype(I_)::value>{}); });
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    // TAILK + 1 slots per batch tile, numbered in program order (the waits count on it): behind the
                    // second MFMA, then behind every fourth
                    if constexpr (m == 1) slot(IC<PHASE>{}, IC<4 * HEADK + bt * (TAILK + 1)>{});
                    if constexpr (m % 4 == 3) slot(IC<PHASE>{}, IC<4 * HEADK + bt * (TAILK + 1) + 1 + m / 4>{});
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
            // the last tile: the s_nops are the wait states between the last MFMA and the first read of its result,
            // which the compiler does not know about
            asm volatile("s_nop 15\n\ts_nop 3" ::: "memory");
            static_for<0, 8>([&](auto E_) { convert_word(IC<3>{}, E_); });
        };
        if (with_bias) end_of_layer(IC<1>{});
        else end_of_layer(IC<0>{});
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    layer(IC<0>{});
    layer(IC<1>{});
    if constexpr (S >= 3) layer(IC<2>{});
    if constexpr (S >= 4) layer(IC<3>{});
    if constexpr (S >= 5) layer(IC<4>{});
    if constexpr (S >= 6) layer(IC<5>{});
    if constexpr (S >= 7) layer(IC<6>{});

    // ---- output layer: rows 16 wave .. + 15 of the workgroup; MFMA row i is output i ----
    f32x4 d;
    {
        u32x4 al[8];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) al[ks] = read_a(S & 1, wave, ks);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // even and odd k-steps add up separately: two chains of four dependent MFMAs instead of one of eight
        f32x4 dd[2];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            asm volatile("" : "+v"(WL[ks]));
            const f32x4 c = ks < 2 ? f32x4{0.f, 0.f, 0.f, 0.f} : dd[ks & 1];
            if constexpr (DT == SP_F16)
                dd[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, WL[ks]), __builtin_bit_cast(f16x8, al[ks]), c, 0, 0, 0);
            else
                dd[ks & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, WL[ks]), __builtin_bit_cast(bf16x8, al[ks]), c, 0, 0, 0);
        }
        d = dd[0] + dd[1];
    }
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
        // the activation buffer nobody reads any more stages the wave's 16 x NOUT outputs
        float* head_rows = reinterpret_cast<float*>(lds + ((S & 1) ^ 1) * PK_ACT_BYTES + wave * 1024);
        f32x4 v = d;
        if (bias != nullptr) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (4 * q + r < NOUT) v[r] += bias[4 * q + r];
        }
        *reinterpret_cast<f32x4*>(head_rows + j * 16 + 4 * q) = v;
        if (head_ok) head_row<16>(out, head_rows + lane * 16, head_row_idx, NOUT, limit, u_row, fill_end);
    }
    }   // (the general tail)
}

template <int DT, int KS0, bool PLAIN>
static const void* pick_packed_kernel_nl(int n_layers) {
    switch (n_layers) {
        case 3: return (const void*)mlp_packed_kernel<DT, KS0, 3, PLAIN>;
        case 4: return (const void*)mlp_packed_kernel<DT, KS0, 4, PLAIN>;
        case 5: return (const void*)mlp_packed_kernel<DT, KS0, 5, PLAIN>;
    }
    return nullptr;
}

template <int DT, bool PLAIN>
static const void* pick_packed_kernel_ks(int ks0, int n_layers) {
    if (ks0 == 1) return pick_packed_kernel_nl<DT, 1, PLAIN>(n_layers);
    if (ks0 == 2) return pick_packed_kernel_nl<DT, 2, PLAIN>(n_layers);
    return pick_packed_kernel_nl<DT, 8, PLAIN>(n_layers);
}

template <int DT>
static const void* pick_packed_kernel(int ks0, int n_layers, bool plain) {
    return plain ? pick_packed_kernel_ks<DT, true>(ks0, n_layers) : pick_packed_kernel_ks<DT, false>(ks0, n_layers);
}

constexpr int PK_MIN_LAYERS = 3, PK_MAX_LAYERS = 5;

// The stacks the packed kernel runs: 3..5 layers, every hidden width 256, first width a multiple of 16, head <= 16.
static bool packed_shape_ok(int n_layers, const int32_t* dims) {
    if (n_layers < PK_MIN_LAYERS || n_layers > PK_MAX_LAYERS) return false;
    if (dims[0] <= 0 || dims[0] % 16 != 0 || dims[0] > 256) return false;
    for (int i = 1; i < n_layers; ++i)
        if (dims[i] != 256) return false;
    return dims[n_layers] >= 1 && dims[n_layers] <= 64;
}

namespace {
struct MlpPackedKernelNames {
    MlpPackedKernelNames() { register_kernel("mlp_forward_packed", (const void*)mlp_packed_kernel<SP_F16, 1, 4, true>, 256); }
} mlp_packed_kernel_names;
}  // namespace

}  // namespace sp

using namespace sp;

extern "C" int64_t sp_mlp_packed_bytes(int32_t n_layers, const int32_t* dims) {
    if (dims == nullptr || !packed_shape_ok(n_layers, dims)) return 0;
    return pk_total_bytes(pk_ks0(dims[0]), n_layers);
}

extern "C" int sp_mlp_pack_weights(int dtype, int32_t n_layers, const void* const* weights, const int32_t* dims, void* packed,
                                   int64_t packed_bytes, void* stream) {
    SP_REQUIRE_PTR(packed);
    if (weights == nullptr || dims == nullptr) return fail(SP_ERR_NULL, "sp_mlp_pack_weights: weights/dims is NULL");
    if (dtype != SP_F16 && dtype != SP_BF16) return fail(SP_ERR_DTYPE, "sp_mlp_pack_weights: dtype must be f16 or bf16");
    if (n_layers < 1 || n_layers > MLP_MAX_LAYERS)
        return fail(SP_ERR_ARG, "sp_mlp_pack_weights: n_layers must be in [1, %d], got %d", MLP_MAX_LAYERS, n_layers);
    if (!packed_shape_ok(n_layers, dims))
        return fail(SP_ERR_UNSUPPORTED, "sp_mlp_pack_weights: the packed kernel takes %d to %d layers, hidden widths of 256, "
                    "a first width that is a multiple of 16 and an output width of at most 64 (of which it uses the first 16 rows)",
                    PK_MIN_LAYERS, PK_MAX_LAYERS);
    const int ks0 = pk_ks0(dims[0]);
    const long need = pk_total_bytes(ks0, n_layers);
    if (packed_bytes < need)
        return fail(SP_ERR_ARG, "sp_mlp_pack_weights: the packed buffer must hold %lld bytes, got %lld", (long long)need,
                    (long long)packed_bytes);
    MlpArgs a{};
    for (int i = 0; i < n_layers; ++i) {
        if (weights[i] == nullptr) return fail(SP_ERR_NULL, "sp_mlp_pack_weights: weights[%d] is NULL", i);
        if (!aligned16(weights[i])) return fail(SP_ERR_ALIGN, "sp_mlp_pack_weights: weights[%d] is not 16-byte aligned", i);
        a.w[i] = weights[i];
    }
    for (int i = 0; i <= n_layers; ++i) a.dims[i] = dims[i];
    a.n_layers = n_layers;
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const long pieces = need / 16;
    const unsigned blocks = (unsigned)((pieces + 255) / 256);
    if (dtype == SP_F16)
        hipLaunchKernelGGL(mlp_pack_kernel<SP_F16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a, (unsigned char*)packed, ks0, pieces);
    else
        hipLaunchKernelGGL(mlp_pack_kernel<SP_BF16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a, (unsigned char*)packed, ks0, pieces);
    return check_launch(__func__);
}

extern "C" int sp_mlp_forward_packed(int dtype, const void* x, int32_t n_layers, const void* packed, int64_t packed_bytes,
                                     const float* const* biases, const int32_t* dims, const float* u, const sp_philox_t* philox,
                                     float* policy_out, int32_t* action_out, float* logits_out, int64_t batch, int32_t head,
                                     int32_t mask_size, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(packed);
    SP_REQUIRE_PTR(policy_out);
    SP_OPTIONAL_PTR(u); SP_OPTIONAL_PTR(action_out); SP_OPTIONAL_PTR(logits_out);
    if (dims == nullptr) return fail(SP_ERR_NULL, "sp_mlp_forward_packed: dims is NULL");
    if (dtype != SP_F16 && dtype != SP_BF16) return fail(SP_ERR_DTYPE, "sp_mlp_forward_packed: dtype must be f16 or bf16");
    if (n_layers < 1 || n_layers > MLP_MAX_LAYERS)
        return fail(SP_ERR_ARG, "sp_mlp_forward_packed: n_layers must be in [1, %d], got %d", MLP_MAX_LAYERS, n_layers);
    if (batch <= 0) return fail(SP_ERR_SHAPE, "sp_mlp_forward_packed: batch must be positive");
    if (head < SP_HEAD_NONE || head > SP_HEAD_SOFTMAX_RM) return fail(SP_ERR_ARG, "sp_mlp_forward_packed: unknown head %d", head);
    if (action_out != nullptr && u == nullptr && philox == nullptr)
        return fail(SP_ERR_NULL, "sp_mlp_forward_packed: action requested but u and philox are NULL");
    if (u != nullptr && philox != nullptr) return fail(SP_ERR_ARG, "sp_mlp_forward_packed: at most one of u and philox may be given");
    if (!packed_shape_ok(n_layers, dims))
        return fail(SP_ERR_UNSUPPORTED, "sp_mlp_forward_packed: the packed kernel takes %d to %d layers, hidden widths of 256 and "
                    "a first width that is a multiple of 16", PK_MIN_LAYERS, PK_MAX_LAYERS);
    if (mask_size < 0 || mask_size > dims[n_layers])
        return fail(SP_ERR_ARG, "sp_mlp_forward_packed: mask_size must be in [0, %d], got %d", dims[n_layers], mask_size);
    // the size names the layout: it depends on the layer count and on how many k-steps the first layer has
    if (packed_bytes != pk_total_bytes(pk_ks0(dims[0]), n_layers))
        return fail(SP_ERR_ARG, "sp_mlp_forward_packed: a packed buffer for this stack holds %lld bytes (sp_mlp_packed_bytes), got "
                    "%lld: it was packed for another stack", (long long)pk_total_bytes(pk_ks0(dims[0]), n_layers), (long long)packed_bytes);
    MlpPackedArgs a{};
    a.nout = dims[n_layers];
    // a masked head whose logits are not asked for is computed for its valid columns only (see sp_mlp_forward)
    if (head != SP_HEAD_NONE && logits_out == nullptr && mask_size > 0 && mask_size <= 16 && mask_size < dims[n_layers])
        a.nout = mask_size;
    if (a.nout > 16)
        return fail(SP_ERR_UNSUPPORTED, "sp_mlp_forward_packed: at most 16 outputs (or a mask of at most 16 columns without "
                    "logits_out), got %d", a.nout);
    for (int i = 0; i < n_layers; ++i) {
        a.b[i] = biases ? biases[i] : nullptr;
        if (a.b[i] != nullptr && !aligned16(a.b[i]))
            return fail(SP_ERR_ALIGN, "sp_mlp_forward_packed: biases[%d] is not 16-byte aligned", i);
    }
    int rc = mlp_set_philox(a.ph, philox, batch, dims[n_layers], __func__);
    if (rc != SP_OK) return rc;
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    a.x = x; a.packed = packed; a.u = u; a.policy = policy_out; a.action = action_out; a.logits = logits_out;
    a.batch = batch; a.head = head; a.mask_size = mask_size; a.k0 = dims[0]; a.out_stride = dims[n_layers];
    if (mlp_resident_takes(n_layers, dims, a.nout) &&
        (batch + PK_ROWS - 1) / PK_ROWS >= (long)(mlp_pipe_takes(n_layers, dims, a.nout) ? SP_MLP_PIPE_MIN_TILES_PACKED
                                                                                         : SP_MLP_RESIDENT_MIN_TILES_PACKED) * device_cu_count()) {
        // several tiles per compute unit: the kernel that loads the weights once and keeps them in registers
        MlpResidentArgs r{};
        r.x = x; r.packed = packed; r.u = u; r.policy = policy_out; r.action = action_out; r.logits = logits_out;
        r.batch = batch; r.head = head; r.mask_size = mask_size; r.k0 = a.k0; r.nout = a.nout; r.out_stride = a.out_stride;
        r.ph = a.ph;
        for (int i = 0; i < n_layers; ++i) r.b[i] = a.b[i];
        return mlp_resident_launch(dtype, true, n_layers, r, (hipStream_t)stream, __func__);
    }
    const int ks0 = pk_ks0(dims[0]);
    const bool plain = a.nout <= 4 && a.out_stride == a.nout && logits_out == nullptr && action_out != nullptr && a.b[n_layers - 1] == nullptr;
    const void* kernel = dtype == SP_F16 ? pick_packed_kernel<SP_F16>(ks0, n_layers, plain) : pick_packed_kernel<SP_BF16>(ks0, n_layers, plain);
    rc = ensure_dynamic_lds(kernel, PK_LDS_BYTES);
    if (rc != SP_OK) return rc;
    const long blocks = (batch + PK_ROWS - 1) / PK_ROWS;
    if (batch > 0x7fffffffll) return fail(SP_ERR_SHAPE, "sp_mlp_forward_packed: batch must be below 2^31");
    int batch32 = (int)batch;
    unsigned k0_nout = (unsigned)a.k0 | ((unsigned)a.nout << 16);
    void* args[] = {(void*)&a.x, (void*)&a.packed, (void*)&a.u, (void*)&a.b[0], (void*)&a.b[1], (void*)&a.b[2], (void*)&batch32,
                    (void*)&k0_nout, (void*)&a};
    hipError_t e = hipLaunchKernel(kernel, dim3((unsigned)blocks), dim3(256), args, PK_LDS_BYTES, (hipStream_t)stream);
    if (e != hipSuccess) return fail(SP_ERR_DEVICE, "sp_mlp_forward_packed: launch failed: %s", hipGetErrorString(e));
    return check_launch(__func__);
}
