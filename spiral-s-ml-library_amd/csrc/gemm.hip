// C = alpha * A . B^T + beta * C [+ bias] [ReLU] for gfx950 (CDNA4) with MFMA.
//
// A (M,K) and B (N,K) are both K-contiguous, so neither operand needs a transposing read: a
// 32x32 MFMA fragment of either one is "32 rows x one 16-byte K-chunk per lane".
//
// Two tiled kernels: gemm_abt_w4_kernel (four waves, 16x16x32 MFMAs; large 16-bit shapes) and gemm_abt_kernel (eight or
// four waves, 32x32 MFMAs; f32, small tiles, single-column outputs).
//
// Data movement per workgroup and K-tile (128 bytes of K per row: 64 bf16/f16 or 32 f32):
//   global --global_load_lds_dwordx4 (DMA, no registers)--> LDS (double buffered, XOR-swizzled
//   16-byte chunks) --ds_read_b128--> MFMA operands.  One barrier per K-tile; the DMA of tile k+1
//   runs while tile k is multiplied.  A wave-wide DMA instruction fills 1 KiB of LDS linearly
//   (lane i -> byte 16*i), i.e. 8 tile rows; the swizzle is applied by choosing which global
//   16-byte chunk each lane fetches.
//
// Semantics follow matmul_tf32_template (ml/matmul/kernel.spi:25-240) with a_trans=false,
// b_trans=true; the f32 path multiplies in full f32 (v_mfma_f32_32x32x2_f32), not TF32.
#include "common.h"
#include <type_traits>

namespace sp {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

struct GemmArgs {
    const void* A;
    const void* B;
    void* C;
    const float* bias;
    long M, N, K;
    float alpha, beta;
    int relu;
    int out_dtype;
    int tiles_m, tiles_n;
    long stride_a, stride_b, stride_c;   // bytes between the matrices of a batch (0: shared)
    int batch;
    int group_m;   // tile rows per group of the block -> tile walk (4: an XCD's 32 concurrent tiles form a 4 x 8 patch)
    int ragged;    // M or N is not a multiple of the tile: tiles_m / tiles_n are rounded up
    int k_rotate;  // workgroup t starts its K loop at K-tile (t * k_rotate) % nk and wraps around (0: everyone at 0)
    int store_policy;   // ST_THROUGH or ST_STREAM for the stores of C when beta == 0 (with beta != 0 C is read here: ST_PLAIN)
    int phase_groups;   // persistent four-wave kernel: workgroup w starts ((w / 8) % phase_groups) * phase_skew
    int phase_skew;     // sleeps of ~2048 cycles late (0 / 1 groups: everybody at once)
};

// The tiled kernels take the fields their first fetches need (operand addresses, K, batch strides, the tile grid) once
// more as leading scalar parameters: the library is built with kernel-argument preloading, which hands the first
// dwords of scalar parameters to a wave in registers when it starts (a struct is not preloaded), so the first
// fetches do not wait for a scalar load from the argument block (~900 cycles).
#define SP_GEMM_PRELOADED const void *A_first, const void *B_first, long K_first, long stride_a_first, long stride_b_first, \
                          int tiles_m_first, int tiles_n_first, int group_m_first
#define SP_GEMM_PRELOADED_ARGS(g) (g).A, (g).B, (g).K, (g).stride_a, (g).stride_b, (g).tiles_m, (g).tiles_n, (g).group_m
__device__ __forceinline__ GemmArgs with_preloaded(const GemmArgs& g0, SP_GEMM_PRELOADED) {
    GemmArgs g = g0;
    g.A = A_first; g.B = B_first; g.K = K_first; g.stride_a = stride_a_first; g.stride_b = stride_b_first;
    g.tiles_m = tiles_m_first; g.tiles_n = tiles_n_first; g.group_m = group_m_first;
    return g;
}
#define SP_GEMM_TAKE_PRELOADED                                                                                          \
    const GemmArgs g = with_preloaded(g_rest, A_first, B_first, K_first, stride_a_first, stride_b_first, tiles_m_first, \
                                      tiles_n_first, group_m_first)

constexpr int ROW_BYTES = 128;  // bytes of K per LDS row and K-tile
constexpr int CHUNKS = 8;       // 16-byte chunks per LDS row

// 16-byte chunk `kc` of LDS row `row` lives at chunk slot kc ^ swz(row): any 8 consecutive rows
// read at the same kc touch 8 different slots, and rows r, r+8 land in different 128-byte halves.
__device__ __forceinline__ int lds_offset(int row, int kc) {
    return row * ROW_BYTES + (((kc ^ row ^ (row >> 3)) & 7) << 4);
}

template <int T>
__device__ __forceinline__ float half_bits_to_f32(unsigned bits) {
    if constexpr (T == SP_BF16) return __uint_as_float(bits << 16);
    else return (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

__device__ __forceinline__ unsigned short f32_to_bf16_rne(float x) {
    unsigned u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// Two f32 values rounded to nearest even and packed into one register (v_cvt_pk_{f16,bf16}_f32).
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <int T>
__device__ __forceinline__ unsigned pack_halves(float a, float b) {
    if constexpr (T == SP_BF16) return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
    else return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, f16x2));
}

// Map the linear workgroup id to an output tile.  Workgroups are dealt round-robin to the 8 XCDs
// (each with a private L2), so id % 8 selects the XCD; each XCD gets a contiguous range of the
// tile sequence, and the sequence walks the tile grid in column-major groups of GROUP_M tile rows
// so that an XCD's concurrent tiles share A and B panels.
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int GROUP_M, int& tm, int& tn) {
    constexpr int XCDS = 8;
    const int n = tiles_m * tiles_n;
    const int xcd = pid % XCDS;
    const int idx = pid / XCDS;
    const int base = n / XCDS, rem = n % XCDS;
    const int t = xcd * base + (xcd < rem ? xcd : rem) + idx;
    const int group_size = GROUP_M * tiles_n;
    const int g = t / group_size;
    const int first_m = g * GROUP_M;
    const int gsz = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_group = t % group_size;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// A store of C with a cache policy.  ST_PLAIN: the compiler's store (write-back in the XCD's L2).  ST_THROUGH
// (sc1): written through the L2 as it is issued, instead of leaving the L2 in bursts when lines are evicted or the
// kernel ends -- the C of a GEMM is written once and read by nobody in this launch.  ST_STREAM (nt): streaming, for
// outputs that should not take room in the caches from operands that are read again.  The host picks one per launch
// (`store_policy`).  Measured (bf16, f32 C, us, plain / through / stream): 65536 x 256 x 256 20.8 / 18.0 / 20.7;
// 131072 x 256 x 256 36.5 / 33.3 / 37.3; 65536 x 256 x 2048 76.0 / 75.2 / 65.0; 8192^3 731 / 730 / 689;
// 16384 x 4096 x 4096 383 / 390 / 364; 65536 x 2048 x 512 178 / 177 / 158; 65536 x 1024 x 512 91 / 91 / 96;
// 8192 x 8192 x 1024 123 / 128 / 132; 4096^3 92.6 / 91.8 / 92.2.
enum { ST_PLAIN = 0, ST_THROUGH = 1, ST_STREAM = 2 };
template <int POLICY, typename V>
__device__ __forceinline__ void store_c(V* p, V v) {
    static_assert(sizeof(V) == 16 || sizeof(V) == 8, "16- or 8-byte pieces of C");
    if constexpr (POLICY == ST_STREAM) __builtin_nontemporal_store(v, p);
    else if constexpr (POLICY == ST_PLAIN) *p = v;
    else if constexpr (sizeof(V) == 16) store16_through(p, v);
    else asm volatile("global_store_dwordx2 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}

// One wave-wide DMA: every lane copies 16 bytes from global memory (uniform base + per-lane
// 32-bit offset) to LDS byte m0 + 16 * lane.  Completion is tracked by vmcnt; the instruction is
// issued from inline assembly so that the tile in flight does not make the compiler wait before
// LDS reads of the tile being multiplied (it cannot tell the two buffers apart).
__device__ __forceinline__ void dma_to_lds(const unsigned char* base, unsigned lane_offset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_addr)
                 : "memory", "m0");
}

// The same with a full address per lane (the last, partial K-tile of a ragged K: chunks past the end of a row
// are fetched from a block of zeros instead).
__device__ __forceinline__ void dma_to_lds_addr(const unsigned char* addr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(addr), "s"(lds_addr) : "memory", "m0");
}
__device__ __attribute__((aligned(16))) const unsigned kZeroChunk[4] = {0u, 0u, 0u, 0u};

__device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const unsigned char*)(((unsigned long long)hi << 32) | lo);
}

// RAGGED: M, N and K need not be multiples of the tile (N a multiple of 4, K of 16 bytes).  Rows past the end are
// fetched as copies of the last row and the chunks of the last K-tile that lie past the end of a row as zeros, so
// every load stays inside the matrices, and the epilogue skips what lies outside C.
template <int DT, int OT, int BM, int BN, int WM, int WN, int NS = 2, int NSA = NS, bool RAGGED = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_abt_kernel(SP_GEMM_PRELOADED, const GemmArgs g_rest) {
    SP_GEMM_TAKE_PRELOADED;
    constexpr int NT = WM * WN * 64;
    static_assert(NS >= 2, "at least two LDS stages");
    // NSA != NS: the A tiles have a ring of their own, longer than B's (which then has two stages).  A is what
    // comes from HBM when B is a single tile column that every workgroup shares through the L2.
    constexpr bool SPLIT_RING = NSA != NS;
    static_assert(!SPLIT_RING || (NS == 2 && NSA > NS), "a separate A ring goes with a two-stage B ring");
    constexpr int ABYTES = BM * ROW_BYTES, BBYTES = BN * ROW_BYTES;
    constexpr int B_BASE = SPLIT_RING ? NSA * ABYTES : ABYTES;   // where the B tile of stage 0 starts
    constexpr int ES = (DT == SP_F32) ? 4 : 2;          // element size
    constexpr int BK = ROW_BYTES / ES;                   // elements of K per tile
    constexpr int WTM = BM / WM, WTN = BN / WN;          // wave tile
    constexpr int TM = WTM / 32, TN = WTN / 32;          // 32x32 fragments per wave
    static_assert(TM >= 1 && TN >= 1, "wave tile too small");
    constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    int tm, tn;
    tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, g.group_m, tm, tn);
    const long m0 = (long)tm * BM, n0 = (long)tn * BN;
    const long K = g.K;
    // batch member blockIdx.y (strided-batched launches; a plain GEMM has one member and zero strides)
    const unsigned char* const Ab = (const unsigned char*)g.A + (long)blockIdx.y * g.stride_a;
    const unsigned char* const Bb = (const unsigned char*)g.B + (long)blockIdx.y * g.stride_b;
    unsigned char* const Cb = (unsigned char*)g.C + (long)blockIdx.y * g.stride_c;

    // ---- loader: DMA instruction q of wave w fills the 8 rows of row block q * NW + w of the
    //      stacked (A rows, then B rows) tile ----
    constexpr int NW = WM * WN;
    constexpr int NI = (BM + BN) / 8 / NW;      // DMA instructions per wave and K-tile
    constexpr int NIA = BM / 8 / NW;            // the first NIA of them fetch A
    static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "row blocks must split evenly over the waves");
    const unsigned lds_base = (unsigned)(size_t)lds;
    const unsigned char* src[NI];
    unsigned lane_off[NI];
    unsigned dst[NI];
    const int nk = RAGGED ? (int)((K + BK - 1) / BK) : (int)(K / BK);
    const bool k_tail = RAGGED && K % BK != 0;   // the last K-tile is partial
    unsigned tail_in = 0;                        // bit q: this lane's chunk of the last K-tile lies inside the row
#pragma unroll
    for (int q = 0; q < NI; ++q) {
        const bool is_a = q < NIA;
        const int blk = (is_a ? q : q - NIA) * NW + wave;           // row block inside the A (or B) tile
        const int r = lane >> 3;                                    // row inside the block
        const int kc = (lane & 7) ^ ((r ^ blk) & 7);                // global chunk that belongs in slot lane & 7
        long first = (is_a ? m0 : n0) + blk * 8, mine = first + r;      // first row of the block, this lane's row
        if constexpr (RAGGED) {
            const long last = (is_a ? g.M : g.N) - 1;
            first = first < last ? first : last;
            mine = first + r < last ? first + r : last;
        }
        const unsigned char* origin = (is_a ? Ab : Bb) + first * K * ES;
        src[q] = uniform_ptr(origin);
        lane_off[q] = (unsigned)((mine - first) * K * ES + kc * 16);
        if ((long)(nk - 1) * CHUNKS + kc < K * ES / 16) tail_in |= 1u << q;
        dst[q] = __builtin_amdgcn_readfirstlane(lds_base + (is_a ? 0 : B_BASE) + blk * 8 * ROW_BYTES);
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int frag_row = lane & 31, frag_half = lane >> 5;

    // Per-lane LDS byte offsets of the fragments.  For fragment 0 the chunk of k-step t sits at
    // va[t]; fragment i (32 rows further down) has the same low row bits and (row >> 3) + 4 * i, so
    // its swizzle differs by bit 2 for odd i: its chunk for step ks sits at va[ks ^ 2 * (i & 1)] plus
    // the constant i * 32 rows.  Only 8 address registers are live and the per-fragment part is an
    // instruction immediate.  The stage (double buffer) is toggled into the registers once per tile.
    int va[4], vb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        va[t] = lds_offset(wm * WTM + frag_row, 2 * t + frag_half);
        vb[t] = B_BASE + lds_offset(wn * WTN + frag_row, 2 * t + frag_half);
    }
    auto load_frags = [&](int ks, u32x4(&fa)[TM], u32x4(&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
            fa[i] = *reinterpret_cast<const u32x4*>(lds + va[ks ^ (2 * (i & 1))] + i * 32 * ROW_BYTES);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[j] = *reinterpret_cast<const u32x4*>(lds + vb[ks ^ (2 * (j & 1))] + j * 32 * ROW_BYTES);
    };
    // NS stages form a ring; `cur` is the one being multiplied (two stages: a sign flip does it).
    int cur = 0;
    int stage_delta = STAGE_BYTES;
    auto next_stage = [&](int kt) {
        int released, delta;
        if constexpr (SPLIT_RING) {
            released = cur;                                   // the A stage; B's is kt & 1
            cur = (cur + 1 == NSA) ? 0 : cur + 1;
            const int da = (cur == 0) ? -(NSA - 1) * ABYTES : ABYTES;
            const int db = (kt & 1) ? -BBYTES : BBYTES;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                va[t] += da;
                vb[t] += db;
            }
            return released;
        } else if constexpr (NS == 2) {
            released = kt & 1;
            delta = stage_delta;
            stage_delta = -stage_delta;
        } else {
            released = cur;
            cur = (cur + 1 == NS) ? 0 : cur + 1;
            delta = (cur == 0) ? -(NS - 1) * STAGE_BYTES : STAGE_BYTES;
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            va[t] += delta;
            vb[t] += delta;
        }
        return released;
    };
    // The B fragment is the MFMA's first operand, so the result fragment is (n, m): register r of
    // lane l holds C[m = l % 32][n = 8 * (r / 4) + 4 * (l / 32) + r % 4], 4 consecutive columns per
    // register quad.
    auto mma = [&](const u32x4(&fa)[TM], const u32x4(&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (DT == SP_BF16) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, fb[j]), __builtin_bit_cast(bf16x8, fa[i]), acc[i][j], 0, 0, 0);
                } else if constexpr (DT == SP_F16) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                        __builtin_bit_cast(f16x8, fb[j]), __builtin_bit_cast(f16x8, fa[i]), acc[i][j], 0, 0, 0);
                } else {
                    // the chunk holds 4 consecutive k for this half-wave; A and B use the same
                    // k for the same (half, step), which is all the MFMA needs
                    const f32x4 pa = __builtin_bit_cast(f32x4, fa[i]);
                    const f32x4 pb = __builtin_bit_cast(f32x4, fb[j]);
#pragma unroll
                    for (int s = 0; s < 4; ++s)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pb[s], pa[s], acc[i][j], 0, 0, 0);
                }
            }
    };
    // Main loop: a continuous stream of k-steps (4 per K-tile).  Before the MFMAs of a step are
    // issued, the fragments of the next step are requested from LDS, so LDS latency hides behind
    // 8 * TM * TN / 8 MFMAs.  The K-tile boundary sits in front of the LAST step of a tile: wait
    // for the next tile's DMA, barrier (every wave has finished reading this tile and everyone's
    // share of the next tile has landed), request the next tile's first fragments, run the last
    // step's MFMAs under that latency, then start the DMA of the tile after next into the stage
    // that was just released.
    u32x4 fa[2][TM], fb[2][TN];
    // The next K-tile of every DMA instruction of this wave (src[] is advanced to it first) into the stage at
    // byte offset `stage_off`; one branch per tile, not per instruction.
    auto fetch_tile = [&](int tile, unsigned stage_off, bool advance) {
        if (k_tail && tile == nk - 1) {
#pragma unroll
            for (int q = 0; q < NI; ++q) {
                if (advance) src[q] += ROW_BYTES;
                const unsigned char* inside = src[q] + lane_off[q];
                dma_to_lds_addr((tail_in >> q) & 1u ? inside : (const unsigned char*)kZeroChunk, dst[q] + stage_off);
            }
        } else {
#pragma unroll
            for (int q = 0; q < NI; ++q) {
                if (advance) src[q] += ROW_BYTES;
                dma_to_lds(src[q], lane_off[q], dst[q] + stage_off);
            }
        }
    };
    // Where this workgroup's K loop starts (split ring only): all workgroups walking K in step would ask the
    // memory system for the same column offsets of 256 different rows each at the same time.
    int left_a = nk, left_b = nk;      // tiles until the walk wraps around to K-tile 0
    if constexpr (SPLIT_RING) {
        const int kt0 = (int)(((long)blockIdx.x * g.k_rotate) % nk);
#pragma unroll
        for (int q = 0; q < NI; ++q) src[q] += (long)kt0 * ROW_BYTES;
        left_a = left_b = nk - kt0;
    }
    auto next_a = [&]() { return --left_a == 0 ? -(long)(nk - 1) * ROW_BYTES : (long)ROW_BYTES; };
    auto next_b = [&]() { return --left_b == 0 ? -(long)(nk - 1) * ROW_BYTES : (long)ROW_BYTES; };
    if constexpr (SPLIT_RING) {
        // Issue order, here and in the loop: B tile j + 2, then A tile j + NSA, for j = -NSA, -NSA + 1, ...  The
        // counter of outstanding loads runs in order; with B ahead of A in every pair, "B tile kt + 1 has landed"
        // leaves exactly the NIA instructions of the A tile issued behind it outstanding.
#pragma unroll
        for (int j = -NSA; j < 0; ++j) {
            if (j + 2 >= 0 && j + 2 < nk) {
                const long step = j + 2 > 0 ? next_b() : 0;
#pragma unroll
                for (int q = NIA; q < NI; ++q) {
                    src[q] += step;
                    dma_to_lds(src[q], lane_off[q], dst[q] + (j + 2) * BBYTES);
                }
            }
            if (j + NSA < nk) {
                const long step = j + NSA > 0 ? next_a() : 0;
#pragma unroll
                for (int q = 0; q < NIA; ++q) {
                    src[q] += step;
                    dma_to_lds(src[q], lane_off[q], dst[q] + (j + NSA) * ABYTES);
                }
            }
        }
        if (nk >= NSA) {   // behind B tile 0: A tile NSA - 2, B tile 1, A tile NSA - 1
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NIA + NI) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    } else {
    // Prologue: the first NS K-tiles (as many as there are) go out at once, one per stage.
#pragma unroll
    for (int st = 0; st < NS; ++st) {
        if (st < nk) fetch_tile(st, st * STAGE_BYTES, st > 0);
    }
    if (nk >= NS) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 1) * NI) : "memory");  // tile 0 landed, NS - 1 tiles may be in flight
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    }
    __syncthreads();
    load_frags(0, fa[0], fb[0]);
    auto first_three_steps = [&]() {
#pragma unroll
        for (int ks = 0; ks < 3; ++ks) {
            load_frags(ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);  // keep these reads ahead of the MFMAs below
            mma(fa[ks & 1], fb[ks & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // waves w and w + NW / 2 share a SIMD when there are 8 of them; with 4 this splits the SIMDs into two groups
    const bool dma_first = __builtin_amdgcn_readfirstlane(wave) < NW / 2;
    for (int kt = 0; kt + 1 < nk; ++kt) {
        first_three_steps();
        // Tile kt + 1 must have landed.  While every stage behind it is still being filled that is
        // "at most NS - 2 tiles outstanding" (the counter runs in order); near the end fewer tiles
        // are in flight and only "none outstanding" says it.
        if (SPLIT_RING && kt + NSA <= nk) {
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NIA) : "memory");
        } else if (!SPLIT_RING && NS > 2 && kt + NS <= nk) {
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NS - 2) * NI) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        }
        __syncthreads();
        const int released = next_stage(kt);
        // The two waves of a SIMD take turns: a wave issuing its DMA instructions waits at the texture
        // path's queue (one 1 KiB instruction per ~16 cycles, 8 waves x NI of them per tile: measured
        // ~600 cycles per wave and tile) and issues no MFMA meanwhile, so one wave of each pair fetches
        // before the last k-step's MFMAs and the other one after them.  Only the DMA issue sits in the
        // (wave-uniform) branches: MFMAs in both arms would make the compiler copy the accumulators.
        auto issue_dma = [&]() {
            if constexpr (SPLIT_RING) {
                if (kt + 2 < nk) {
                    const unsigned stage_off = (unsigned)(kt & 1) * BBYTES;
                    const long step = next_b();
#pragma unroll
                    for (int q = NIA; q < NI; ++q) {
                        src[q] += step;
                        dma_to_lds(src[q], lane_off[q], dst[q] + stage_off);
                    }
                }
                if (kt + NSA < nk) {
                    const unsigned stage_off = (unsigned)released * ABYTES;
                    const long step = next_a();
#pragma unroll
                    for (int q = 0; q < NIA; ++q) {
                        src[q] += step;
                        dma_to_lds(src[q], lane_off[q], dst[q] + stage_off);
                    }
                }
            } else if (kt + NS < nk) {
                fetch_tile(kt + NS, (unsigned)released * STAGE_BYTES, true);
            }
        };
        if (dma_first) issue_dma();
        __builtin_amdgcn_sched_barrier(0);
        load_frags(0, fa[0], fb[0]);
        __builtin_amdgcn_sched_barrier(0);
        mma(fa[1], fb[1]);
        __builtin_amdgcn_sched_barrier(0);
        if (!dma_first) issue_dma();
    }
    first_three_steps();
    mma(fa[1], fb[1]);

    // ---- epilogue: each wave transposes its accumulators through a private LDS strip of 32 rows x
    //      up to 64 columns, so that C is written (and, for beta != 0, read) as whole row segments:
    //      16 bytes per lane, up to 256 contiguous bytes per row ----
    constexpr int SW = WTN < 64 ? WTN : 64;        // columns per strip
    constexpr int SF = SW / 32;                    // fragments per strip
    constexpr int EPI_STRIDE = SW * 4 + 16;        // bytes; the pad keeps the 16-byte column writes conflict free
    constexpr int LPR = SW / 4;                    // lanes per output row
    constexpr int RPP = 64 / LPR;                  // rows per pass
    static_assert(NW * 32 * EPI_STRIDE <= 2 * STAGE_BYTES, "epilogue staging must fit the tile buffers");
    __syncthreads();                               // every wave is done reading the tile buffers
    unsigned char* stg = lds + wave * (32 * EPI_STRIDE);
    const int er = lane / LPR, ec = (lane % LPR) * 4;
    const float alpha = g.alpha, beta = g.beta;
    const long row_step = (long)RPP * g.N;
    // The options are compile-time inside the loops: a branch per output row would split them into blocks of one
    // LDS read -> one store each, with every latency exposed.
    auto write_tile = [&](auto BETA_, auto RELU_, auto POLICY_) {
        constexpr bool HAS_BETA = decltype(BETA_)::value, RELU = decltype(RELU_)::value;
        constexpr int POLICY = decltype(POLICY_)::value;
        auto finish = [&](f32x4 v, const f32x4& old, const f32x4& bias) {
            v = v * alpha;
            if constexpr (HAS_BETA) v += beta * old;
            v += bias;
            if constexpr (RELU) { v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f); v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f); }
            return v;
        };
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int js = 0; js < TN / SF; ++js) {
                const long col = n0 + wn * WTN + js * SW + ec;
                const bool col_ok = !RAGGED || col < g.N;
                f32x4 bias4 = {0.f, 0.f, 0.f, 0.f};
                if (g.bias && col_ok) bias4 = *reinterpret_cast<const f32x4*>(g.bias + col);
#pragma unroll
                for (int jj = 0; jj < SF; ++jj)
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const f32x16& c16 = acc[i][js * SF + jj];
                        f32x4 v = {c16[4 * gq], c16[4 * gq + 1], c16[4 * gq + 2], c16[4 * gq + 3]};
                        *reinterpret_cast<f32x4*>(stg + frag_row * EPI_STRIDE + (jj * 32 + gq * 8 + frag_half * 4) * 4) = v;
                    }
                const long row_first = m0 + wm * WTM + i * 32 + er;
                long idx = row_first * g.N + col;     // advanced by RPP rows per pass
#pragma unroll
                for (int p = 0; p < 32 / RPP; ++p, idx += row_step) {
                    const int rl = p * RPP + er;
                    const f32x4 v = *reinterpret_cast<const f32x4*>(stg + rl * EPI_STRIDE + ec * 4);
                    if (RAGGED && !(col_ok && row_first + p * RPP < g.M)) continue;
                    f32x4 old = {0.f, 0.f, 0.f, 0.f};
                    if constexpr (OT == SP_F32) {
                        f32x4* c = reinterpret_cast<f32x4*>((float*)Cb + idx);
                        if constexpr (HAS_BETA) old = *c;
                        store_c<POLICY>(c, finish(v, old, bias4));
                    } else {
                        u32x2* c = reinterpret_cast<u32x2*>((unsigned short*)Cb + idx);
                        if constexpr (HAS_BETA) {
                            const u32x2 o = *c;
                            old = f32x4{half_bits_to_f32<OT>(o.x & 0xffffu), half_bits_to_f32<OT>(o.x >> 16),
                                        half_bits_to_f32<OT>(o.y & 0xffffu), half_bits_to_f32<OT>(o.y >> 16)};
                        }
                        const f32x4 r = finish(v, old, bias4);
                        u32x2 o;
                        o.x = pack_halves<OT>(r.x, r.y);
                        o.y = pack_halves<OT>(r.z, r.w);
                        store_c<POLICY>(c, o);
                    }
                }
            }
        }
    };
    typedef std::integral_constant<int, ST_PLAIN> plain_t;
    typedef std::integral_constant<int, ST_THROUGH> through_t;
    typedef std::integral_constant<int, ST_STREAM> stream_t;
    if (beta != 0.f) {
        if (g.relu) write_tile(std::true_type{}, std::true_type{}, plain_t{});
        else write_tile(std::true_type{}, std::false_type{}, plain_t{});
    } else if (g.store_policy == ST_STREAM) {
        if (g.relu) write_tile(std::false_type{}, std::true_type{}, stream_t{});
        else write_tile(std::false_type{}, std::false_type{}, stream_t{});
    } else {
        if (g.relu) write_tile(std::false_type{}, std::true_type{}, through_t{});
        else write_tile(std::false_type{}, std::false_type{}, through_t{});
    }
}

// ---- 256 x 256 x 64 tiles on FOUR waves (one per SIMD), 16x16x32 MFMAs: the kernel for large 16-bit GEMMs ----
// Same data movement as gemm_abt_kernel (DMA into two swizzled LDS stages, one barrier per K-tile), but a wave owns a
// 128 x 128 quarter of the tile: 64 accumulator tiles of 16 x 16 = 256 registers in the accumulation file (the wave
// has all 512 registers of its SIMD).  Operands of a 32-wide k-step are 8 + 8 fragments of "16 rows x one 16-byte
// chunk per lane": 32 KiB of LDS reads per wave and K-tile against 24 KiB for each of eight waves, a third less
// per compute unit, and v_mfma_f32_16x16x32 draws less power per flop than the 32x32x16 form, which is what the
// clock of a power-limited GEMM is made of.
// What makes a lone wave per SIMD work: every instruction it issues costs the matrix pipe ~4-5 cycles (there is no
// second wave to issue in the shadow of its MFMAs), and two memory instructions back to back cost more than that.
// So the loop body is straight-line code for two K-tiles (stage addresses are immediates), carries no address
// arithmetic (one scalar base per matrix, per-lane offsets in registers, fragment addresses in registers), and puts
// every LDS read and every DMA alone between two MFMAs: 128 MFMAs + ~76 other instructions per K-tile.
// The fragment of the B matrix is the MFMA's first operand: register r of lane l of accumulator tile
// (tm, tn) holds C[m = 16 tm + l % 16][n = 16 tn + 4 (l / 16) + r].
// NSA = 3: a ring of three stages for the A tiles next to the two for B -- all 160 KiB of LDS.  The A tile of K-tile
// kt + 3 is requested in the second half of K-tile kt, so it has two K-tiles to arrive instead of one; B (re-read by
// every tile row, served by the caches) keeps its lead of one.  For tall shapes whose A panels come straight from
// HBM (65536 x 1024 x 512: 99.7 -> 97.5 us; most of what that main loop waits for is contention with the other
// units' stores, which a longer lead does not cure).  The A stage of a K-tile is then a run-time offset (three
// stages against a loop body of two K-tiles): the eight fragment addresses of A are re-based once per K-tile (8
// vector adds; the square GEMMs, whose loop does not wait, lose 0.5-2 % to them and stay on NSA = 2).  Within a K-tile the B fetches go out before the A fetches, so that at the boundary
// "everything but the 8 youngest fetches has landed" is exactly "tile kt + 1 is complete".
// PERSIST (beta = 0, one batch member): one workgroup per compute unit walks tiles blockIdx.x,
// blockIdx.x + gridDim.x, ... (the same tile -> XCD map as one workgroup per tile), and the fetch stream runs on into
// the NEXT tile: where the last K-tiles of a tile would re-fetch the last tile into dead stages, they fetch A tiles
// 0-2 and B tile 0 of the next tile (the A ring keeps rotating across tiles; B tile 0 lands in B stage 0 because nk
// is even).  The epilogue's staging strips move to the second B stage (XOR-swizzled instead of padded, so that they
// fit), and B tile 1 follows once the strips are free.  What a tile's first fetches take to arrive -- 6-8 k cycles
// when every unit asks at once -- and the 2-4 k cycles between a workgroup's end and its successor's start are then
// spent multiplying and storing.  With NSA = 2 (long K, where the three-stage loop's extra instructions cost more than
// its lead returns) the same: the last two K-tiles fetch K-tiles 0 and 1 of the next tile into the two stages as they
// are released, and the strips live in the 32 KiB of LDS that two stages of 64 KiB leave free, so nothing waits for
// the epilogue's stores either.
template <int DT, int OT, int NSA = 2, bool PERSIST = false>
__global__ __launch_bounds__(256) void gemm_abt_w4_kernel(SP_GEMM_PRELOADED, const GemmArgs g_rest) {
    SP_GEMM_TAKE_PRELOADED;
    static_assert(DT != SP_F32, "16-bit inputs only");
    static_assert(NSA == 2 || NSA == 3, "two stages [A][B], or three A stages followed by two B stages");
    static_assert(NSA == 2 || NSA == 3, "two combined stages, or three A stages next to two B stages");
    constexpr int BM = 256, BN = 256, NW = 4, ES = 2;
    constexpr int BK = ROW_BYTES / ES;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
    constexpr int B_BASE3 = 3 * A_BYTES;         // NSA = 3: where the B stages start
    constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
    constexpr int NI = (BM + BN) / 8 / NW;      // 16 DMA instructions per wave and K-tile
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    int vblock = blockIdx.x;                     // the tile's number in the launch order of one workgroup per tile
    int tm_, tn_;
    tile_of_block(vblock, g.tiles_m, g.tiles_n, g.group_m, tm_, tn_);
    long m0 = (long)tm_ * BM, n0 = (long)tn_ * BN;
    if constexpr (PERSIST) {
        // Phase groups: all units walking their tiles in step means every unit's 256 KiB of C leave at the same
        // moment, with the matrix pipes idle, and then nobody stores for a whole main loop.  Half of the units of
        // every XCD (blockIdx.x / 8 is the unit's number within its XCD) start about half a tile period late, so one
        // half stores while the other multiplies.  This pays together with STREAMED stores only: written back or
        // through the L2, the stores of one half queue in front of the other half's fetches (measured: 105 us
        // against 90 without groups, 77 with streamed stores, 65536 x 1024 x 512).
        const int late = g.phase_groups > 1 ? ((int)(blockIdx.x >> 3) % g.phase_groups) * g.phase_skew : 0;
        for (int i = 0; i < late; ++i) __builtin_amdgcn_s_sleep(32);
    }
    const long K = g.K;
    const unsigned char* const Ab = (const unsigned char*)g.A + (long)blockIdx.y * g.stride_a;
    const unsigned char* const Bb = (const unsigned char*)g.B + (long)blockIdx.y * g.stride_b;
    unsigned char* const Cb = (unsigned char*)g.C + (long)blockIdx.y * g.stride_c;

    // loader: DMA instruction q of wave w fills the 8 rows of row block (q % 8) * NW + w of the A (q < 8) or B tile.
    // One scalar base per matrix (row block `wave` of the tile, advanced by one K-tile at a time) and one per-lane
    // offset per q % 8, shared by A and B (same row pitch): a lone wave per SIMD pays ~4 cycles of matrix-pipe time
    // for EVERY instruction it issues, so the loop carries no per-instruction address arithmetic.
    const unsigned lds_base = (unsigned)(size_t)lds;
    const unsigned char* sA = uniform_ptr(Ab + (m0 + wave * 8) * K * ES);
    const unsigned char* sB = uniform_ptr(Bb + (n0 + wave * 8) * K * ES);
    unsigned dstw = __builtin_amdgcn_readfirstlane(lds_base + wave * 8 * ROW_BYTES);
    unsigned voff[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int r = lane >> 3;
        // chunk fetched by a lane: (lane & 7) ^ swz(row), row = 8 blk + r, blk & 7 = (4 q + wave) & 7
        const unsigned chunk = (unsigned)((((lane & 7) ^ r ^ ((4 * q + wave) & 7)) & 7) << 4);
        voff[q] = (unsigned)((q * 8 * NW + r) * K * ES) + chunk;
    }
    auto dma_plain = [&](int q, int stage) {
        unsigned d = dstw + (q & 7) * NW * 8 * ROW_BYTES;
        if constexpr (NSA == 3) d += q < 8 ? stage * A_BYTES : B_BASE3 + stage * B_BYTES;
        else d += (q < 8 ? 0 : BM * ROW_BYTES) + stage * STAGE_BYTES;
        dma_to_lds(q < 8 ? sA : sB, voff[q & 7], d);
    };

    f32x4 acc[8][8];
    const int fi = lane & 15, fq = lane >> 4;
    // fragment addresses: row = R0 + 16 t + fi, chunk 4 ks + fq; its slot is (4 ks + fq) ^ fi ^ (fi >> 3) ^ 2 (t & 3)
    // (R0 is a multiple of 128): per stage 2 k-steps x 4 values of t & 3 = 8 registers per operand, the rest immediates
    int va[2][2][4], vb[2][2][4];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                // Which 16-byte chunk of the K-tile lane group fq multiplies in k-step ks is free as long as A and B
                // agree.  With 4 * ks + fq (lanes l and l + 32 two chunks apart) half of the LDS cycles of these reads
                // were bank conflicts (SQ_LDS_BANK_CONFLICT 8.5 M per 4096^3 launch); with 2 * fq + ks there are none.
                const int kc = 2 * fq + ks;
                if constexpr (NSA == 3) {       // A: relative to its stage (st is not used); B: its own two stages
                    va[st][ks][t] = lds_offset(wm * 128 + 16 * t + fi, kc);
                    vb[st][ks][t] = B_BASE3 + st * B_BYTES + lds_offset(wn * 128 + 16 * t + fi, kc);
                } else {
                    va[st][ks][t] = st * STAGE_BYTES + lds_offset(wm * 128 + 16 * t + fi, kc);
                    vb[st][ks][t] = st * STAGE_BYTES + BM * ROW_BYTES + lds_offset(wn * 128 + 16 * t + fi, kc);
                }
                // opaque to the compiler, or it keeps one of them and re-derives the others inside the loop
                asm volatile("" : "+v"(va[st][ks][t]), "+v"(vb[st][ks][t]));
            }
    // NSA = 3: the A fragment addresses of the K-tile being read, re-based once per K-tile: [1] (k-step 1 of the
    // K-tile being multiplied) at the start of a K-tile, [0] (k-step 0 of the next one) at its boundary
    int vaa[2][4] = {};
    unsigned a_cur = 0;                          // byte offset of the A stage of the K-tile being multiplied
    auto rebase_a = [&](int ks, unsigned stage_bytes) {
#pragma unroll
        for (int t = 0; t < 4; ++t) vaa[ks][t] = va[0][ks][t] + (int)stage_bytes;
    };
    auto load_a = [&](int st, int ks, int t, u32x4(&fa)[8]) {
        if constexpr (NSA == 3) fa[t] = *reinterpret_cast<const u32x4*>(lds + vaa[ks][t & 3] + (t >> 2) * 64 * ROW_BYTES);
        else fa[t] = *reinterpret_cast<const u32x4*>(lds + va[st][ks][t & 3] + (t >> 2) * 64 * ROW_BYTES);
    };
    auto load_b = [&](int st, int ks, int t, u32x4(&fb)[8]) {
        fb[t] = *reinterpret_cast<const u32x4*>(lds + vb[st][ks][t & 3] + (t >> 2) * 64 * ROW_BYTES);
    };
    // operand read h (0 or 1) of row i: rows 0..3 fetch the B-matrix fragments (the next step's first row needs all
    // of them), rows 4..7 the A-matrix fragments
    auto load_one = [&](int st, int ks, int i, int h, u32x4(&fa)[8], u32x4(&fb)[8]) {
        if (i < 4) load_b(st, ks, 2 * i + h, fb);
        else load_a(st, ks, 2 * (i - 4) + h, fa);
    };
    // The MFMAs are issued from assembly with the accumulator pinned to the accumulation registers: left to
    // itself the register allocator moves parts of the 256-register accumulator between the two register
    // files around the loop.  (Tiles are revisited 64 MFMAs later, so no wait states are needed in between.)
    auto mfma_acc = [&](f32x4& c, const u32x4& b, const u32x4& a) {
        if constexpr (DT == SP_BF16)
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(b), "v"(a));
        else
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(b), "v"(a));
    };
    // MFMAs 4..7 of a row with two DMA instructions among them, as one block: each write of M0 has an MFMA between
    // itself and the DMA that reads it (the wait state it needs), and nothing else can be scheduled in between
    auto mfma4_dma2 = [&](f32x4& c4, f32x4& c5, f32x4& c6, f32x4& c7, const u32x4& b4, const u32x4& b5, const u32x4& b6,
                          const u32x4& b7, const u32x4& a, unsigned vo0, unsigned vo1, const unsigned char* base, unsigned dw,
                          auto D0_, auto D1_) {
        constexpr unsigned D0 = decltype(D0_)::value, D1 = decltype(D1_)::value;
#define SP_W4_BLOCK(T)                                                                                                   \
        asm volatile("s_add_u32 m0, %12, %13\n\t"                                                                      \
                     "v_mfma_f32_16x16x32_" T " %0, %4, %8, %0\n\t"                                                    \
                     "global_load_lds_dwordx4 %9, %11\n\t"                                                             \
                     "v_mfma_f32_16x16x32_" T " %1, %5, %8, %1\n\t"                                                    \
                     "v_mfma_f32_16x16x32_" T " %2, %6, %8, %2\n\t"                                                    \
                     "s_add_u32 m0, %12, %14\n\t"                                                                      \
                     "v_mfma_f32_16x16x32_" T " %3, %7, %8, %3\n\t"                                                    \
                     "global_load_lds_dwordx4 %10, %11"                                                                  \
                     : "+a"(c4), "+a"(c5), "+a"(c6), "+a"(c7)                                                            \
                     : "v"(b4), "v"(b5), "v"(b6), "v"(b7), "v"(a), "v"(vo0), "v"(vo1), "s"(base), "s"(dw), "n"(D0), "n"(D1) \
                     : "memory", "scc", "m0")
        if constexpr (DT == SP_BF16) SP_W4_BLOCK("bf16");
        else SP_W4_BLOCK("f16");
#undef SP_W4_BLOCK
    };
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};

    const int nk = (int)(K / BK);     // even (the launcher checks K % 128 == 0)
    u32x4 fa[2][8], fb[2][8];
    // prologue: tiles 0 and 1 into stages 0 and 1 (NSA = 3: and the A tile 2 into the third A stage; sA then
    // points at tile 2 and sB at tile 1, what the first boundary expects)
#pragma unroll
    for (int q = 0; q < NI; ++q) dma_plain(q, 0);
    sA += ROW_BYTES;
    sB += ROW_BYTES;
#pragma unroll
    for (int q = 0; q < NI; ++q) dma_plain(q, 1);
    if constexpr (NSA == 3) {
        sA += ROW_BYTES;
#pragma unroll
        for (int q = 0; q < 8; ++q) dma_plain(q, 2);
        rebase_a(0, 0);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NSA == 3 ? NI + 8 : NI) : "memory");   // tile 0 has landed
    __syncthreads();
    bool prefetched = false;          // PERSIST: this tile's first fetches went out during the previous tile
    for (;;) {                        // (one pass unless PERSIST)
    // PERSIST: where the next tile's operands start (this wave's rows), for the fetches of the last K-tiles
    int next_block = 0;
    long next_m0 = 0, next_n0 = 0;
    bool has_next = false;
    const unsigned char *next_a = nullptr, *next_b = nullptr;
    if constexpr (PERSIST) {
        next_block = vblock + (int)gridDim.x;
        has_next = next_block < g.tiles_m * g.tiles_n;
        if (has_next) {
            int ntm, ntn;
            tile_of_block(next_block, g.tiles_m, g.tiles_n, g.group_m, ntm, ntn);
            next_m0 = (long)ntm * BM;
            next_n0 = (long)ntn * BN;
            next_a = uniform_ptr(Ab + (next_m0 + wave * 8) * K * ES);
            next_b = uniform_ptr(Bb + (next_n0 + wave * 8) * K * ES);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = zero4;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        load_a(0, 0, t, fa[0]);
        load_b(0, 0, t, fb[0]);
    }
    // row I of k-step 1 of a tile in stage ST: fetches 2 I and 2 I + 1 of the tile after the next go into stage ST
    auto row1 = [&](auto ST_, auto I_) {
        constexpr int ST = decltype(ST_)::value, i = decltype(I_)::value;
        // 0..7: A, 8..15: B; NSA = 3 sends B first (rows 0..3), then A (rows 4..7)
        constexpr int q0 = NSA == 3 ? (2 * i + 8) % 16 : 2 * i, q1 = q0 + 1;
        constexpr unsigned D0 = NSA == 3 ? (q0 < 8 ? 0 : B_BASE3 + ST * B_BYTES) + (q0 & 7) * NW * 8 * ROW_BYTES
                                         : (q0 < 8 ? 0 : BM * ROW_BYTES) + (q0 & 7) * NW * 8 * ROW_BYTES + ST * STAGE_BYTES;
        constexpr unsigned D1 = NSA == 3 ? (q1 < 8 ? 0 : B_BASE3 + ST * B_BYTES) + (q1 & 7) * NW * 8 * ROW_BYTES
                                         : (q1 < 8 ? 0 : BM * ROW_BYTES) + (q1 & 7) * NW * 8 * ROW_BYTES + ST * STAGE_BYTES;
        const unsigned char* base = q0 < 8 ? sA : sB;
        // NSA = 3: the A tile of K-tile kt + 3 goes into the A stage K-tile kt has just released (a_cur)
        const unsigned dw = NSA == 3 && q0 < 8 ? dstw + a_cur : dstw;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            mfma_acc(acc[i][j], fb[1][j], fa[1][i]);
            if (j == 1) load_one(ST ^ 1, 0, i, 0, fa[0], fb[0]);
            if (j == 3) load_one(ST ^ 1, 0, i, 1, fa[0], fb[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
        mfma4_dma2(acc[i][4], acc[i][5], acc[i][6], acc[i][7], fb[1][4], fb[1][5], fb[1][6], fb[1][7], fa[1][i], voff[q0 & 7],
                   voff[q1 & 7], base, dw, std::integral_constant<unsigned, D0>{}, std::integral_constant<unsigned, D1>{});
        __builtin_amdgcn_sched_barrier(0);
    };
    // One K-tile in stage ST.  k-step 0 multiplies fragments taken before it and takes those of k-step 1; the
    // boundary in the middle waits for tile kt + 1 (fetched during the previous tile) and releases stage ST, all
    // of whose fragments are in registers by then; k-step 1 takes the first fragments of tile kt + 1 and sends
    // all 16 fetches of tile kt + 2 into stage ST, two per row of 8 MFMAs, so the last one has a whole k-step plus
    // what the first ones needed to land.  Every memory instruction stands alone between two MFMAs.  Fetches past
    // the last tile repeat the last tile into a stage nobody reads any more: no branch in the loop.
    auto tile = [&](int kt, auto ST_) {
        constexpr int ST = decltype(ST_)::value;
        const unsigned a_next = a_cur == 2 * A_BYTES ? 0 : a_cur + A_BYTES;
        if constexpr (NSA == 3) rebase_a(1, a_cur);
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): one wait for all fragments of this k-step instead of one per row
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                mfma_acc(acc[i][j], fb[0][j], fa[0][i]);
                if (j == 1) load_one(ST, 1, i, 0, fa[1], fb[1]);
                if (j == 3) load_one(ST, 1, i, 1, fa[1], fb[1]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (NSA == 3) {
            // all but the A tile of K-tile kt + 2 (after a prefetch only B tile 1 is in flight at the first boundary)
            if (PERSIST && prefetched && kt == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            __syncthreads();
            if (PERSIST && has_next) {       // past this tile's last K-tile the stream goes on with the next tile's first
                sA = kt + 3 == nk ? next_a : sA + ROW_BYTES;
                sB = kt + 2 < nk ? sB + ROW_BYTES : kt + 2 == nk ? next_b : sB;   // (B tile 1 waits for the strips' stage)
            } else {
                sA += kt + 3 < nk ? ROW_BYTES : 0;
                sB += kt + 2 < nk ? ROW_BYTES : 0;
            }
            rebase_a(0, a_next);
        } else {
            // (PERSIST, first K-tile of a tile whose first two K-tiles came in during the previous tile: both have
            //  landed, and what is outstanding are the previous epilogue's stores, which nobody has to wait for)
            if (!(PERSIST && prefetched && kt == 0)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (PERSIST && has_next && kt + 2 >= nk) {       // the stream goes on with the next tile's K-tiles 0 and 1
                sA = kt + 2 == nk ? next_a : sA + ROW_BYTES;
                sB = kt + 2 == nk ? next_b : sB + ROW_BYTES;
            } else {
                const int adv = kt + 2 < nk ? ROW_BYTES : 0;
                sA += adv;
                sB += adv;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        row1(ST_, std::integral_constant<int, 0>{});
        row1(ST_, std::integral_constant<int, 1>{});
        row1(ST_, std::integral_constant<int, 2>{});
        row1(ST_, std::integral_constant<int, 3>{});
        row1(ST_, std::integral_constant<int, 4>{});
        row1(ST_, std::integral_constant<int, 5>{});
        row1(ST_, std::integral_constant<int, 6>{});
        row1(ST_, std::integral_constant<int, 7>{});
        a_cur = a_next;
    };
    for (int kt = 0; kt < nk; kt += 2) {
        tile(kt, std::integral_constant<int, 0>{});
        tile(kt + 1, std::integral_constant<int, 1>{});
    }
    // the fetches past the end must be done before the stages are reused; the last MFMAs must have written
    // their results before the accumulators are read (18 wait states, which the compiler cannot know about)
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    // ---- epilogue: per 16-row accumulator row, the wave transposes 16 x 128 values through a private LDS strip
    //      and writes C (and, for beta != 0, reads it) 16 bytes per lane: 512-byte row segments, two rows per
    //      instruction for f32 output, 256-byte segments, four rows per instruction for 16-bit output ----
    // (PERSIST: rows of 512 bytes without padding, 16-byte chunk c of row r in slot c ^ r -- in the second B stage
    //  with three A stages, in the 32 KiB that two combined stages leave free otherwise)
    constexpr int EPI_STRIDE = PERSIST ? 128 * 4 : 128 * 4 + 16;
    static_assert(NW * 16 * EPI_STRIDE <= 2 * STAGE_BYTES, "epilogue staging must fit the tile buffers");
    static_assert(!PERSIST || NW * 16 * EPI_STRIDE <= B_BYTES, "epilogue staging must fit one B stage");
    __syncthreads();
    unsigned char* strip = lds + (!PERSIST ? 0 : NSA == 3 ? B_BASE3 + B_BYTES : 2 * STAGE_BYTES) + wave * (16 * EPI_STRIDE);
    auto strip_at = [&](int row, int chunk) {        // byte offset of 16-byte chunk `chunk` of strip row `row`
        return row * EPI_STRIDE + ((PERSIST ? chunk ^ (row & 15) : chunk) << 4);
    };
    constexpr int PER = OT == SP_F32 ? 4 : 8;                 // columns per lane
    constexpr int LPR = 128 / PER;                            // lanes per row
    constexpr int RPP = 64 / LPR;                             // rows per pass
    const int er = lane / LPR, ec = (lane % LPR) * PER;
    const float alpha = g.alpha, beta = g.beta;
    const long col = n0 + wn * 128 + ec;
    f32x4 bias4[PER / 4];
#pragma unroll
    for (int h = 0; h < PER / 4; ++h) {
        bias4[h] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (g.bias) bias4[h] = *reinterpret_cast<const f32x4*>(g.bias + col + 4 * h);
    }
    // The options are compile-time inside the loops: a branch per output row would split them into blocks of one
    // LDS read -> one store each, with every latency exposed.
    auto write_tile = [&](auto BETA_, auto RELU_, auto POLICY_) {
        constexpr bool HAS_BETA = decltype(BETA_)::value, RELU = decltype(RELU_)::value;
        constexpr int POLICY = decltype(POLICY_)::value;
        auto finish = [&](f32x4 v, const f32x4& old, const f32x4& bias) {
            v = v * alpha;
            if constexpr (HAS_BETA) v += beta * old;
            v += bias;
            if constexpr (RELU) { v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f); v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f); }
            return v;
        };
        long idx = (m0 + wm * 128 + er) * g.N + col;      // advanced by RPP rows per pass
        const long row_step = (long)RPP * g.N;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                *reinterpret_cast<f32x4*>(strip + strip_at(fi, 4 * j + fq)) = acc[i][j];
#pragma unroll
            for (int p = 0; p < 16 / RPP; ++p, idx += row_step) {
                const int rl = RPP * p + er;
                f32x4 old0 = {0.f, 0.f, 0.f, 0.f}, old1 = {0.f, 0.f, 0.f, 0.f};
                if constexpr (OT == SP_F32) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(strip + strip_at(rl, ec / 4));
                    f32x4* c = reinterpret_cast<f32x4*>((float*)Cb + idx);
                    if constexpr (HAS_BETA) old0 = *c;
                    store_c<POLICY>(c, finish(v, old0, bias4[0]));
                } else {
                    const f32x4 v0 = *reinterpret_cast<const f32x4*>(strip + strip_at(rl, ec / 4));
                    const f32x4 v1 = *reinterpret_cast<const f32x4*>(strip + strip_at(rl, ec / 4 + 1));
                    u32x4* c = reinterpret_cast<u32x4*>((unsigned short*)Cb + idx);
                    if constexpr (HAS_BETA) {
                        const u32x4 o = *c;
                        old0 = f32x4{half_bits_to_f32<OT>(o.x & 0xffffu), half_bits_to_f32<OT>(o.x >> 16),
                                     half_bits_to_f32<OT>(o.y & 0xffffu), half_bits_to_f32<OT>(o.y >> 16)};
                        old1 = f32x4{half_bits_to_f32<OT>(o.z & 0xffffu), half_bits_to_f32<OT>(o.z >> 16),
                                     half_bits_to_f32<OT>(o.w & 0xffffu), half_bits_to_f32<OT>(o.w >> 16)};
                    }
                    const f32x4 r0 = finish(v0, old0, bias4[0]), r1 = finish(v1, old1, bias4[PER / 4 - 1]);
                    u32x4 o;
                    o.x = pack_halves<OT>(r0.x, r0.y);
                    o.y = pack_halves<OT>(r0.z, r0.w);
                    o.z = pack_halves<OT>(r1.x, r1.y);
                    o.w = pack_halves<OT>(r1.z, r1.w);
                    store_c<POLICY>(c, o);
                }
            }
        }
    };
    typedef std::integral_constant<int, ST_PLAIN> plain_t;
    typedef std::integral_constant<int, ST_THROUGH> through_t;
    typedef std::integral_constant<int, ST_STREAM> stream_t;
    if (beta != 0.f) {
        if (g.relu) write_tile(std::true_type{}, std::true_type{}, plain_t{});
        else write_tile(std::true_type{}, std::false_type{}, plain_t{});
    } else if (g.store_policy == ST_STREAM) {
        if (g.relu) write_tile(std::false_type{}, std::true_type{}, stream_t{});
        else write_tile(std::false_type{}, std::false_type{}, stream_t{});
    } else {
        if (g.relu) write_tile(std::false_type{}, std::true_type{}, through_t{});
        else write_tile(std::false_type{}, std::false_type{}, through_t{});
    }
    if (!PERSIST || !has_next) break;
    if constexpr (NSA == 3) {
        // the stores are acknowledged (the next tile's first fetches landed before the epilogue), here and (barrier)
        // everywhere; the strips are free: B tile 1 goes into the stage they occupied.  The A ring rotates on: a_cur
        // is the stage of the next tile's K-tile 0, and its fragment addresses were re-based at the last boundary.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        sB += ROW_BYTES;
#pragma unroll
        for (int q = 8; q < NI; ++q) dma_plain(q, 1);
    }
    // (two combined stages: K-tiles 0 and 1 of the next tile are in their stages since the wait behind the main
    //  loop, sA and sB point at K-tile 1 as after a prologue, and the strips have a place of their own)
    vblock = next_block;
    m0 = next_m0;
    n0 = next_n0;
    prefetched = true;
    }
}

// Shape-agnostic kernel: one thread per output element, 16-byte loads along K.  Used for shapes
// the tiled kernels do not divide (the MLP's K = 32 or N = 3 for instance).
template <int DT>
__global__ __launch_bounds__(256) void gemm_abt_generic_kernel(const GemmArgs g) {
    constexpr int ES = (DT == SP_F32) ? 4 : 2;
    constexpr int PER = 16 / ES;
    // blocks of 16 x 16 outputs, numbered row by row in blockIdx.x (a grid's y extent stops at 65535)
    const long nb_n = (g.N + 15) / 16;
    const long n = ((long)blockIdx.x % nb_n) * 16 + (threadIdx.x & 15);
    const long m = ((long)blockIdx.x / nb_n) * 16 + (threadIdx.x >> 4);
    if (m >= g.M || n >= g.N) return;
    const unsigned char* a = (const unsigned char*)g.A + (long)blockIdx.y * g.stride_a + m * g.K * ES;
    const unsigned char* b = (const unsigned char*)g.B + (long)blockIdx.y * g.stride_b + n * g.K * ES;
    unsigned char* const Cb = (unsigned char*)g.C + (long)blockIdx.y * g.stride_c;
    float s = 0.f;
    for (long k = 0; k < g.K; k += PER) {
        const u32x4 va = *reinterpret_cast<const u32x4*>(a + k * ES);
        const u32x4 vb = *reinterpret_cast<const u32x4*>(b + k * ES);
        if constexpr (DT == SP_F32) {
            const float* fa = reinterpret_cast<const float*>(&va);
            const float* fb = reinterpret_cast<const float*>(&vb);
#pragma unroll
            for (int i = 0; i < 4; ++i) s += fa[i] * fb[i];
        } else if constexpr (DT == SP_F16) {
            const _Float16* fa = reinterpret_cast<const _Float16*>(&va);
            const _Float16* fb = reinterpret_cast<const _Float16*>(&vb);
#pragma unroll
            for (int i = 0; i < 8; ++i) s += (float)fa[i] * (float)fb[i];
        } else {
            const unsigned short* fa = reinterpret_cast<const unsigned short*>(&va);
            const unsigned short* fb = reinterpret_cast<const unsigned short*>(&vb);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                s += __uint_as_float((unsigned)fa[i] << 16) * __uint_as_float((unsigned)fb[i] << 16);
        }
    }
    const long idx = m * g.N + n;
    float v = g.alpha * s;
    const float bias = g.bias ? g.bias[n] : 0.f;
    if (g.out_dtype == SP_F32) {
        float* c = (float*)Cb;
        if (g.beta != 0.f) v += g.beta * c[idx];
        v += bias;
        if (g.relu) v = fmaxf(v, 0.f);
        c[idx] = v;
    } else if (g.out_dtype == SP_BF16) {
        unsigned short* c = (unsigned short*)Cb;
        if (g.beta != 0.f) v += g.beta * __uint_as_float((unsigned)c[idx] << 16);
        v += bias;
        if (g.relu) v = fmaxf(v, 0.f);
        c[idx] = f32_to_bf16_rne(v);
    } else {
        _Float16* c = (_Float16*)Cb;
        if (g.beta != 0.f) v += g.beta * (float)c[idx];
        v += bias;
        if (g.relu) v = fmaxf(v, 0.f);
        c[idx] = (_Float16)v;
    }
}

// ---- host side: tile choice and launch -------------------------------------------------------

struct TileCfg {
    int bm, bn, wm, wn;
};
static const TileCfg kTileCfgs[] = {{256, 256, 2, 4}, {128, 128, 2, 2}, {64, 64, 2, 2}};
constexpr int kNumCfgs = 3;

// The four-wave kernel takes the 256 x 256 tiles of 16-bit GEMMs whose K is a whole number of K-tile pairs and whose
// B matrix spans more than one tile column; with a single column every A panel is read once, straight from HBM, and
// two waves per SIMD hide that latency better (65536 x 256 x 2048: 85 us against 89-93 us).
static bool use_four_waves(int dtype_in, long N, long K) {
    return dtype_in != SP_F32 && K % 128 == 0 && K <= (1l << 22) && N >= 512;
}

// The counterpart of the reference's tile search (`frame` / `frame_iter`, ml/primitives.spi:17-33, as used by
// matmul_config_tf32, ml/matmul/run.spi:8-19: tiles doubled from 16 x 16 under the shared-memory budget): a fixed menu
// of three tiles.  Largest tile whose grid still fills the chip; otherwise the smallest tile that divides the shape.  "Fills" is 80 %
// of the compute units, except for the four-wave kernel, which does per unit so much more than the 128 x 128 tiles
// that 9/16 of the units are enough (3072^3 bf16: 144 tiles of 256 x 256 take 56 us, 576 tiles of 128 x 128 76 us; at
// 128 tiles the two are level, below that the smaller tiles win).
static int choose_cfg(int dtype_in, long M, long N, long K, long batch = 1) {
    const int bk = dtype_in == SP_F32 ? 32 : 64;
    if (K % bk != 0) return -1;
    const int cus = device_cu_count();
    int smallest = -1;
    for (int i = 0; i < kNumCfgs; ++i) {
        const TileCfg& c = kTileCfgs[i];
        if (M % c.bm != 0 || N % c.bn != 0) continue;
        smallest = i;
        const long tiles = (M / c.bm) * (N / c.bn) * batch;
        const bool four_waves = i == 0 && use_four_waves(dtype_in, N, K);
        if (four_waves ? tiles * 16 >= (long)cus * 9 : tiles * 5 >= (long)cus * 4) return i;
    }
    return smallest;
}

// Shapes no tile divides: the same tiled kernels with rows clamped in the loader, zeros for the missing part of the
// last K-tile and a masked epilogue, provided N is a multiple of 4 (16-byte accesses to C and the bias).  Tile choice
// as above, on tile counts rounded up.
static int choose_cfg_ragged(int dtype_in, long M, long N, long K, long batch) {
    (void)K;   // any K that passed validation (a multiple of 16 bytes)
    if (N % 4 != 0) return -1;
    const int cus = device_cu_count();
    for (int i = 0; i < kNumCfgs; ++i) {
        const TileCfg& c = kTileCfgs[i];
        const long tiles = ((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn) * batch;
        if (tiles * 5 >= (long)cus * 4) return i;
    }
    return kNumCfgs - 1;
}

template <int DT, int OT, int BM, int BN, int WM, int WN, int NS, int NSA = NS, bool RAGGED = false>
static int launch_tiled_stages(const GemmArgs& g, hipStream_t stream) {
    auto kernel = gemm_abt_kernel<DT, OT, BM, BN, WM, WN, NS, NSA, RAGGED>;
    const int lds_bytes = (NSA * BM + NS * BN) * ROW_BYTES;
    const int rc = ensure_dynamic_lds((const void*)kernel, lds_bytes);
    if (rc != SP_OK) return rc;
    const long tiles = (long)g.tiles_m * g.tiles_n;
    hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)g.batch), dim3(WM * WN * 64), lds_bytes, stream,
                       SP_GEMM_PRELOADED_ARGS(g), g);
    return check_launch("sp_gemm_abt");
}

// Two LDS stages keep several small workgroups on a compute unit.  When the grid has at most one
// workgroup per unit anyway, 16-bit GEMMs with a long K give the whole LDS to one deep ring instead
// (128 KiB: 4 stages of a 128 x 128 tile, 8 of a 64 x 64 tile): a K-tile of a small 16-bit tile is
// multiplied in far less time than a load takes to arrive, and with two stages every tile waits
// for its data (1024 x 1024 x 8192 bf16: 51.7 -> 34.2 us).  Measured and left on two stages: f32
// (its K-tile takes 1024 cycles of MFMA and the deep ring was 5-9 % slower) and short K (the burst
// of the prologue delays the first tile: 2048 x 2048 x 512 bf16 9.7 -> 10.4 us).
template <int DT, int OT, int BM, int BN, int WM, int WN>
static int launch_tiled(const GemmArgs& g, hipStream_t stream) {
    if (g.ragged) return launch_tiled_stages<DT, OT, BM, BN, WM, WN, 2, 2, true>(g, stream);
    constexpr int DEEP = (128 * 1024) / ((BM + BN) * ROW_BYTES);
    if constexpr (BM == 256 && BN == 256 && DT != SP_F32) {
        // B is a single tile column: every A panel comes straight from HBM, once, and one 32 KiB stage of it in
        // flight per compute unit is too little to cover that latency (8 MiB over the chip).  The 32 KiB of LDS that
        // two 64 KiB stages leave over become a third A stage.
        if (g.tiles_n == 1 && g.K / (ROW_BYTES / 2) >= 8) return launch_tiled_stages<DT, OT, BM, BN, WM, WN, 2, 3>(g, stream);
    }
    if constexpr (DEEP > 2 && DT != SP_F32) {
        constexpr int BK = ROW_BYTES / 2;
        if ((long)g.tiles_m * g.tiles_n * g.batch <= (long)device_cu_count() && g.K / BK >= 32)
            return launch_tiled_stages<DT, OT, BM, BN, WM, WN, DEEP>(g, stream);
    }
    return launch_tiled_stages<DT, OT, BM, BN, WM, WN, 2>(g, stream);
}

// The four-wave kernel with a third A stage (see the kernel): when the A panels are not shared enough to come from
// the caches.
#ifndef SP_W4_PERSIST
#define SP_W4_PERSIST 1
#endif
#ifndef SP_W4_PERSIST2
#define SP_W4_PERSIST2 1
#endif
#ifndef SP_W4_NSA3_MODE
#define SP_W4_NSA3_MODE 2      // 0: never, 1: always (for tests of the variant), 2: tall shapes
#endif
static bool three_a_stages(const GemmArgs& g) {
    if (g.K / 64 < 4) return false;
    if (SP_W4_NSA3_MODE == 0) return false;
    if (SP_W4_NSA3_MODE == 1) return true;
    return g.tiles_n <= 8 && g.tiles_m >= 4 * g.tiles_n;
}

template <int DT, int OT>
static int launch_four_waves(const GemmArgs& g, hipStream_t stream) {
    if constexpr (DT == SP_F32) {
        return fail(SP_ERR_DTYPE, "sp_gemm_abt: the four-wave kernel takes 16-bit inputs");
    } else {
        const long tiles = (long)g.tiles_m * g.tiles_n;
        const int cus = device_cu_count();
        // (also short-K problems of any aspect with three or more tiles per unit, for the phase groups below:
        //  8192 x 8192 x 512 89 -> 82 us, 16384 x 16384 x 512 351 -> 324; from 16 K-tiles up it no longer pays)
        const bool short_k = g.K / 64 >= 4 && g.K / 64 <= 8 && tiles >= 3l * cus;
        if (SP_W4_PERSIST && (three_a_stages(g) || short_k) && g.batch == 1 && g.beta == 0.f && cus % 8 == 0 &&
            tiles >= 2l * cus) {
            // several tiles per compute unit: one workgroup per unit walks them and fetches ahead across the epilogue
            auto kernel = gemm_abt_w4_kernel<DT, OT, 3, true>;
            const int lds_bytes = (3 * 256 + 2 * 256) * ROW_BYTES;
            const int rc = ensure_dynamic_lds((const void*)kernel, lds_bytes);
            if (rc != SP_OK) return rc;
            GemmArgs gp = g;
            // Two phase groups half a tile period apart + streamed stores, where the epilogue is a large part of a
            // tile (f32 output, at most 16 K-tiles) and there are enough tiles per unit to win back the late start
            // (us, in step / in two groups: 65536 x 1024 x 256 71.9 / 60.2, x 512 90.4 / 77.3, x 1024 139 / 130,
            // x 2048 228 / 235; 65536 x 2048 x 512 164 / 145; 131072 x 1024 x 512 167 / 151; 49152 x 1024 x 512
            // 62.4 / 57.8; two tiles per unit 43.7 / 43.5; bf16 output 65.0 / 65.4).  A tile period is ~2800 cycles
            // per K-tile + ~9000 for the epilogue.
            const int nk = (int)(g.K / 64);
            if (OT == SP_F32 && nk <= 16 && tiles >= 3l * cus) {
                gp.phase_groups = 2;
                gp.phase_skew = 3 + nk / 2;
                gp.store_policy = ST_STREAM;
            }
            hipLaunchKernelGGL(kernel, dim3((unsigned)cus, 1), dim3(256), lds_bytes, stream, SP_GEMM_PRELOADED_ARGS(gp), gp);
            return check_launch("sp_gemm_abt");
        }
        if (SP_W4_PERSIST2 && !three_a_stages(g) && g.K / 64 <= 32 && g.batch == 1 && g.beta == 0.f && cus % 8 == 0 &&
            tiles >= 3l * cus) {
            // medium K, three or more tiles per compute unit: the two-stage loop walking tiles without a prologue per
            // tile, in two phase groups with streamed stores for f32 output (us, one workgroup per tile / this form:
            // 8192 x 8192 x 1024 127.6 / 122; 8192 x 8192 x 2048 214 / 206; 12288 x 4096 x 1024 94.4 / 90.4).  From 64
            // K-tiles up the epilogue is too small a part of a tile: 8192^3 697 / 705-713, with or without groups.
            auto kernel = gemm_abt_w4_kernel<DT, OT, 2, true>;
            const int lds_bytes = (2 * (256 + 256) + 256) * ROW_BYTES;
            const int rc = ensure_dynamic_lds((const void*)kernel, lds_bytes);
            if (rc != SP_OK) return rc;
            GemmArgs gp = g;
            if (OT == SP_F32) {
                gp.phase_groups = 2;
                gp.phase_skew = 5;
                gp.store_policy = ST_STREAM;
            }
            hipLaunchKernelGGL(kernel, dim3((unsigned)cus, 1), dim3(256), lds_bytes, stream, SP_GEMM_PRELOADED_ARGS(gp), gp);
            return check_launch("sp_gemm_abt");
        }
        if (three_a_stages(g)) {
            auto kernel = gemm_abt_w4_kernel<DT, OT, 3>;
            const int lds_bytes = (3 * 256 + 2 * 256) * ROW_BYTES;
            const int rc = ensure_dynamic_lds((const void*)kernel, lds_bytes);
            if (rc != SP_OK) return rc;
            hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)g.batch), dim3(256), lds_bytes, stream,
                               SP_GEMM_PRELOADED_ARGS(g), g);
            return check_launch("sp_gemm_abt");
        }
        auto kernel = gemm_abt_w4_kernel<DT, OT>;
        const int lds_bytes = 2 * (256 + 256) * ROW_BYTES;
        const int rc = ensure_dynamic_lds((const void*)kernel, lds_bytes);
        if (rc != SP_OK) return rc;
        hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)g.batch), dim3(256), lds_bytes, stream,
                           SP_GEMM_PRELOADED_ARGS(g), g);
        return check_launch("sp_gemm_abt");
    }
}

template <int DT, int OT>
static int launch_dtype(int cfg, const GemmArgs& g, hipStream_t stream) {
    switch (cfg) {
        case 0:
            if (!g.ragged && use_four_waves(DT, g.N, g.K)) return launch_four_waves<DT, OT>(g, stream);
            return launch_tiled<DT, OT, 256, 256, 2, 4>(g, stream);
        case 1: return launch_tiled<DT, OT, 128, 128, 2, 2>(g, stream);
        case 2: return launch_tiled<DT, OT, 64, 64, 2, 2>(g, stream);
    }
    dim3 grid((unsigned)(((g.N + 15) / 16) * ((g.M + 15) / 16)), (unsigned)g.batch);
    hipLaunchKernelGGL(gemm_abt_generic_kernel<DT>, grid, dim3(256), 0, stream, g);
    return check_launch("sp_gemm_abt(generic)");
}

static int validate_gemm(int dtype_in, int dtype_out, int64_t M, int64_t N, int64_t K) {
    if (dtype_in != SP_F32 && dtype_in != SP_F16 && dtype_in != SP_BF16)
        return fail(SP_ERR_DTYPE, "sp_gemm_abt: unknown input dtype %d", dtype_in);
    if (dtype_out != SP_F32 && dtype_out != dtype_in)
        return fail(SP_ERR_DTYPE, "sp_gemm_abt: output dtype must be f32 or the input dtype (in %d, out %d)", dtype_in,
                    dtype_out);
    if (M <= 0 || N <= 0 || K <= 0)
        return fail(SP_ERR_SHAPE, "sp_gemm_abt: M, N, K must be positive (got %lld, %lld, %lld)", (long long)M,
                    (long long)N, (long long)K);
    const int per = dtype_in == SP_F32 ? 4 : 8;
    if (K % per != 0)
        return fail(SP_ERR_SHAPE, "sp_gemm_abt: K must be a multiple of %d (16-byte rows), got %lld", per, (long long)K);
    // What the kernels can address: the loaders keep per-lane byte offsets of up to 7 rows (231 in the four-wave
    // kernel, which has a K limit of its own) in 32 bits, and a launch numbers its workgroups with an int.
    const int es = dtype_in == SP_F32 ? 4 : 2;
    if (M > (1ll << 31) || N > (1ll << 31) || K * es > (1ll << 29))
        return fail(SP_ERR_SHAPE, "sp_gemm_abt: dimension too large (M, N <= 2^31, rows of A and B <= 512 MiB)");
    if (((M + 15) / 16) * ((N + 15) / 16) > 2147483647ll)
        return fail(SP_ERR_SHAPE, "sp_gemm_abt: M x N too large (more than 2^31 - 1 blocks of 16 x 16 outputs)");
    return SP_OK;
}

namespace {
struct GemmKernelNames {
    GemmKernelNames() {
        register_kernel("gemm_bf16_256x256", (const void*)gemm_abt_kernel<SP_BF16, SP_F32, 256, 256, 2, 4>, 512);
        register_kernel("gemm_f16_256x256", (const void*)gemm_abt_kernel<SP_F16, SP_F32, 256, 256, 2, 4>, 512);
        register_kernel("gemm_bf16_128x128", (const void*)gemm_abt_kernel<SP_BF16, SP_F32, 128, 128, 2, 2>, 256);
        register_kernel("gemm_f32_64x64", (const void*)gemm_abt_kernel<SP_F32, SP_F32, 64, 64, 2, 2>, 256);
        register_kernel("gemm_bf16_256x256_4w", (const void*)gemm_abt_w4_kernel<SP_BF16, SP_F32>, 256);
        register_kernel("gemm_f16_256x256_4w", (const void*)gemm_abt_w4_kernel<SP_F16, SP_F32>, 256);
        register_kernel("gemm_bf16_256x256_4w_3a", (const void*)gemm_abt_w4_kernel<SP_BF16, SP_F32, 3>, 256);
        register_kernel("gemm_bf16_256x256_4w_3a_persistent", (const void*)gemm_abt_w4_kernel<SP_BF16, SP_F32, 3, true>, 256);
    }
} gemm_kernel_names;
}  // namespace

}  // namespace sp

using namespace sp;

extern "C" int sp_gemm_config(int dtype_in, int64_t M, int64_t N, int64_t K, int32_t* tile_m, int32_t* tile_n,
                              int32_t* tile_k, int32_t* threads) {
    if (!tile_m || !tile_n || !tile_k || !threads) return fail(SP_ERR_NULL, "sp_gemm_config: NULL output");
    int rc = validate_gemm(dtype_in, SP_F32, M, N, K);
    if (rc != SP_OK) return rc;
    int cfg = choose_cfg(dtype_in, M, N, K);
    bool ragged = false;
    if (cfg < 0) {
        cfg = choose_cfg_ragged(dtype_in, M, N, K, 1);
        ragged = cfg >= 0;
    }
    if (cfg < 0) {
        *tile_m = 0; *tile_n = 0; *tile_k = 0; *threads = 256;
    } else {
        *tile_m = kTileCfgs[cfg].bm; *tile_n = kTileCfgs[cfg].bn; *tile_k = dtype_in == SP_F32 ? 32 : 64;
        *threads = kTileCfgs[cfg].wm * kTileCfgs[cfg].wn * 64;
        if (cfg == 0 && !ragged && use_four_waves(dtype_in, N, K)) *threads = 256;
    }
    return SP_OK;
}

static int gemm_entry(const char* fn, int dtype_in, int dtype_out, const void* A, const void* B, void* C,
                      const float* bias, int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a,
                      int64_t stride_b, int64_t stride_c, float alpha, float beta, uint32_t flags, void* stream) {
    int rc = validate_gemm(dtype_in, dtype_out, M, N, K);
    if (rc != SP_OK) return rc;
    if (alpha == 0.f) return fail(SP_ERR_ARG, "%s: The alpha must not be zero.", fn);
    if (batch < 1 || batch > 65535) return fail(SP_ERR_SHAPE, "%s: batch must be in [1, 65535], got %lld", fn, (long long)batch);
    const int es_in = dtype_in == SP_F32 ? 4 : 2, es_out = dtype_out == SP_F32 ? 4 : 2;
    if (stride_a < 0 || stride_b < 0 || stride_c < 0 || (stride_a * es_in) % 16 != 0 || (stride_b * es_in) % 16 != 0 ||
        (stride_c * es_out) % 16 != 0)
        return fail(SP_ERR_ALIGN, "%s: batch strides must be non-negative and keep every matrix 16-byte aligned", fn);
    if (batch > 1 && stride_c < M * N) return fail(SP_ERR_ARG, "%s: the outputs of a batch must not overlap", fn);
    rc = require_gfx950(fn);
    if (rc != SP_OK) return rc;
    int cfg = (flags & SP_GEMM_FORCE_GENERIC) ? -1 : choose_cfg(dtype_in, M, N, K, batch);
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.bias = bias; g.M = M; g.N = N; g.K = K; g.alpha = alpha; g.beta = beta;
    g.relu = (flags & SP_GEMM_RELU) ? 1 : 0;
    g.out_dtype = dtype_out;
    g.group_m = 4;
    g.k_rotate = 7;   // odd: coprime with the power-of-two K-tile counts of the usual shapes (measured: 1, 3, ..., 13 all within 1 %)
    g.batch = (int)batch;
    {
        // Outputs that cannot stay in the 256 MiB memory-side cache anyway, or that would push operands out of it
        // (operands of more than half its size), are streamed; everything else is written through the L2.
        const double MiB = 1048576.0;
        const double in_bytes = (double)es_in * K * ((double)M * (stride_a ? batch : 1) + (double)N * (stride_b ? batch : 1));
        const double out_bytes = (double)es_out * M * N * batch;
        g.store_policy = (in_bytes >= 140 * MiB || out_bytes >= 384 * MiB) ? ST_STREAM : ST_THROUGH;
    }
    g.stride_a = stride_a * es_in; g.stride_b = stride_b * es_in; g.stride_c = stride_c * es_out;
    if (cfg < 0 && !(flags & SP_GEMM_FORCE_GENERIC)) {
        cfg = choose_cfg_ragged(dtype_in, M, N, K, batch);
        g.ragged = cfg >= 0;
    }
    if (cfg >= 0) {
        g.tiles_m = (int)((M + kTileCfgs[cfg].bm - 1) / kTileCfgs[cfg].bm);
        g.tiles_n = (int)((N + kTileCfgs[cfg].bn - 1) / kTileCfgs[cfg].bn);
    }
    hipStream_t s = (hipStream_t)stream;
    switch (dtype_in) {
        case SP_F32: return launch_dtype<SP_F32, SP_F32>(cfg, g, s);
        case SP_F16:
            return dtype_out == SP_F32 ? launch_dtype<SP_F16, SP_F32>(cfg, g, s) : launch_dtype<SP_F16, SP_F16>(cfg, g, s);
        default:
            return dtype_out == SP_F32 ? launch_dtype<SP_BF16, SP_F32>(cfg, g, s) : launch_dtype<SP_BF16, SP_BF16>(cfg, g, s);
    }
}

extern "C" int sp_gemm_abt(int dtype_in, int dtype_out, const void* A, const void* B, void* C, const float* bias,
                           int64_t M, int64_t N, int64_t K, float alpha, float beta, uint32_t flags, void* stream) {
    SP_REQUIRE_PTR(A);
    SP_REQUIRE_PTR(B);
    SP_REQUIRE_PTR(C);
    SP_OPTIONAL_PTR(bias);
    return gemm_entry(__func__, dtype_in, dtype_out, A, B, C, bias, M, N, K, 1, 0, 0, 0, alpha, beta, flags, stream);
}

extern "C" int sp_gemm_abt_batched(int dtype_in, int dtype_out, const void* A, const void* B, void* C, const float* bias,
                                   int64_t M, int64_t N, int64_t K, int64_t batch, int64_t stride_a, int64_t stride_b,
                                   int64_t stride_c, float alpha, float beta, uint32_t flags, void* stream) {
    SP_REQUIRE_PTR(A);
    SP_REQUIRE_PTR(B);
    SP_REQUIRE_PTR(C);
    SP_OPTIONAL_PTR(bias);
    return gemm_entry(__func__, dtype_in, dtype_out, A, B, C, bias, M, N, K, batch, stride_a, stride_b, stride_c, alpha,
                      beta, flags, stream);
}
