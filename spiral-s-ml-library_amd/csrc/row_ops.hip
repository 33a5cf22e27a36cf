// Row primitives for gfx950: one group of T lanes (T = cols/4 rounded up to a power of two, at
// most one wave64) owns a row and keeps it in registers, 4 contiguous columns per lane and chunk,
// so every fused pipeline is a single pass over HBM: one 16-byte load per lane and chunk, shuffles
// for the cross-lane reductions/scans, 16-byte stores.  Bandwidth-bound; no LDS, no MFMA.
//
// Semantics follow ml/primitives.spi (row_ :423-512, local_* :295-348 and :701-814).
#include "common.h"
#include "philox.h"

// The scan/sampling results are compared bit for bit with a CPU restatement, so no operation in
// this file may be fused or re-associated.
#pragma clang fp contract(off)

namespace sp {

typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int ROW_THREADS = 256;
constexpr int INT_MAX_ = 2147483647;

struct RowArgs {
    const float* x;
    const float* u;        // per-row uniforms, or nullptr -> philox (if sample requested)
    float* rowmax;
    float* rowsum;
    float* out;            // mapped output (probabilities / op result)
    float* cdf;
    float* u_out;
    int* argmax;
    int* sample;
    const int* action;     // get_prob: the column whose mapped value goes to prob_out (nullptr: the sampled one)
    float* prob_out;
    unsigned* bits_out;    // binarize
    unsigned modulo;
    long rows;
    int cols;
    int op;                // sp_row_op
    int mask_size;         // columns j < mask_size are valid for the masked ops
    int want_stats;        // rowmax/rowsum are of softmax(x) regardless of op (fused pipeline)
    float threshold;       // l1_normalize: the norm a row is clamped to
    // philox
    unsigned long long seed;
    int philox_mode;       // -1: none
    int tpb;
    int blocks;
    int rows_per_block;
    unsigned long long draw_offset;
    long member_rows;                  // 0: one run; else the rows are stacked runs of member_rows rows each
    unsigned long long member_draws;   // extra draw offset per run
};

// Two standard normals from two 32-bit draws, the Box-Muller form of curand_normal (corecuda/random.spi:85):
// u = x 2^-32 + 2^-33, v = 2 pi (y 2^-32 + 2^-33), (sqrt(-2 ln u) sin v, sqrt(-2 ln u) cos v).  The library's own
// logf / sincosf: the low bits differ from the fast intrinsics of the reference's platform.
__device__ __forceinline__ void box_muller(unsigned x, unsigned y, float& n0, float& n1) {
    const float u = (float)x * 2.3283064e-10f + 1.1641532e-10f;
    const float v = (float)y * (2.3283064e-10f * 6.2831855f) + (2.3283064e-10f * 6.2831855f * 0.5f);
    const float s = sqrtf(-2.0f * logf(u));
    float sn, cs;
    sincosf(v, &sn, &cs);
    n0 = s * sn;
    n1 = s * cs;
}

// exp(x) = 2^(x * log2 e) on the hardware exp2 unit; relative error about 1e-6 for |x| < 20.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

__device__ __forceinline__ float sum4(const float (&v)[4]) { return ((v[0] + v[1]) + v[2]) + v[3]; }

// x / s for many x and one s as x * scale * (1 / (s * scale)): one division per row, and `scale` (a power of two, so
// both products by it are exact) keeps the reciprocal finite when s lies below 2^-126, where 1 / s alone would be
// +inf and every quotient inf or NaN.  The quotients differ from a correctly rounded x / s by at most one unit in
// the last place.
struct RowDivisor {
    float scale, inv;
    __device__ __forceinline__ explicit RowDivisor(float s) {
        scale = fabsf(s) < 4.7019774e-38f ? 1.8446744e19f : 1.f;     // below 2^-124: times 2^64
        inv = 1.f / (s * scale);
    }
    __device__ __forceinline__ float operator()(float x) const { return (x * scale) * inv; }
};

template <int T, int C>
__global__ __launch_bounds__(ROW_THREADS) void row_kernel(const RowArgs a) {
    constexpr int ROWS_PER_WAVE = WAVE / T;
    const int lane = threadIdx.x & (WAVE - 1);
    const int l = lane % T;          // lane inside the row group
    const int sub = lane / T;        // which of the wave's rows
    const long wave_id = (long)blockIdx.x * (ROW_THREADS / WAVE) + (threadIdx.x / WAVE);
    const long n_waves = (long)gridDim.x * (ROW_THREADS / WAVE);
    const float NEG_INF = -__builtin_inff();
    const int cols = a.cols;
    const int op = a.op;
    const bool masked = (op == SP_ROW_MASKED_SOFTMAX || op == SP_ROW_MASKED_REGRET_MATCHING);
    const int limit = masked ? a.mask_size : cols;
    const bool want_stats = a.want_stats;

    for (long row0 = wave_id * ROWS_PER_WAVE; row0 < a.rows; row0 += n_waves * ROWS_PER_WAVE) {
        const long row = row0 + sub;
        const bool row_ok = row < a.rows;
        const float* xr = a.x + row * (long)cols;

        float v[C][4];
        bool ok[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = c * 4 * T + 4 * l;
            ok[c] = row_ok && col < cols;
            if (ok[c]) {
                const float4 t4 = *reinterpret_cast<const float4*>(xr + col);
                v[c][0] = t4.x; v[c][1] = t4.y; v[c][2] = t4.z; v[c][3] = t4.w;
            } else {
                v[c][0] = v[c][1] = v[c][2] = v[c][3] = 0.f;
            }
        }

        // The row's uniform is requested (or computed) while the row itself is on its way: the
        // counter of outstanding loads runs in order, so a load issued in mid-work is waited for
        // with nothing else to do.
        float uu = 0.f;
        if (a.sample != nullptr && row_ok) uu = a.u != nullptr ? a.u[row] : reference_row_uniform(a, row);

        // ---- row max of the raw input, then argmax = lowest index holding it ----
        float bv = NEG_INF;
        int bi = INT_MAX_;
        if (a.argmax != nullptr || a.rowmax != nullptr || want_stats) {
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (ok[c]) bv = fmaxf(bv, v[c][k]);
            bv = group_reduce<T>(bv, [](float x, float y) { return fmaxf(x, y); });
            if (a.argmax != nullptr) {
#pragma unroll
                for (int c = C - 1; c >= 0; --c)
#pragma unroll
                    for (int k = 3; k >= 0; --k)
                        if (ok[c] && v[c][k] == bv) bi = c * 4 * T + 4 * l + k;
                bi = group_reduce<T>(bi, [](int x, int y) { return x < y ? x : y; });
                if (bi == INT_MAX_) bi = 0;   // a row of NaNs: no element equals the max
            }
        }

        // ---- the row map ----
        float p[C][4];
        float stat_sum = 0.f;
        if (op == SP_ROW_SOFTMAX || op == SP_ROW_MASKED_SOFTMAX) {
            float m = NEG_INF;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int j = c * 4 * T + 4 * l + k;
                    const float xv = (ok[c] && j < limit) ? v[c][k] : NEG_INF;
                    p[c][k] = xv;
                    m = fmaxf(m, xv);
                }
            if (op == SP_ROW_SOFTMAX && want_stats) m = bv;   // same reduction as the row max above
            else m = group_reduce<T>(m, [](float x, float y) { return fmaxf(x, y); });
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = (p[c][k] == NEG_INF) ? 0.f : fast_exp(p[c][k] - m);
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            stat_sum = s;
            const float inv = 1.f / s;   // one correctly rounded reciprocal per row, then multiplies
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = p[c][k] * inv;
        } else if (op == SP_ROW_REGRET_MATCHING || op == SP_ROW_MASKED_REGRET_MATCHING) {
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int j = c * 4 * T + 4 * l + k;
                    p[c][k] = (ok[c] && j < limit) ? fmaxf(v[c][k], 0.f) : 0.f;
                }
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            // one division per row, then a multiplication per element (a correctly rounded division is ten
            // instructions; the quotients differ from p / s by at most one unit in the last place)
            const float inv_len = 1.f / (float)limit;
            const RowDivisor over_s(s);
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int j = c * 4 * T + 4 * l + k;
                    p[c][k] = (j < limit) ? (s != 0.f ? over_s(p[c][k]) : inv_len) : 0.f;
                }
        } else if (op == SP_ROW_L1_NORMALIZE) {
            // local_l1_normalize (ml/primitives.spi:725-729): |x|, scaled down to norm `threshold` when its sum is above it
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = fabsf(v[c][k]);
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            const float f = s > a.threshold ? a.threshold / s : 1.f;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = f * p[c][k];
        } else if (op == SP_ROW_LN_L2) {
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                float q[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) q[k] = v[c][k] * v[c][k];
                s = (c == 0) ? sum4(q) : s + sum4(q);
            }
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            const RowDivisor over_s(s);
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = (s != 0.f) ? over_s(v[c][k]) : 0.f;
        } else {  // identity and the scans act on the raw input
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = v[c][k];
        }

        // ---- prefix sums of p (needed by the scans and by sampling) ----
        const bool want_sample = a.sample != nullptr;
        const bool is_scan = (op == SP_ROW_INCLUSIVE_SCAN || op == SP_ROW_EXCLUSIVE_SCAN);
        float cdf[C][4];
        if (want_sample || a.cdf != nullptr || is_scan) {
            float carry = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float s = sum4(p[c]);
                const float incl = group_inclusive_scan<T>(s, l);
                float prev = dpp_move<0x138>(incl);   // wave_shr:1 = the lane before
                if (l == 0) prev = 0.f;
                float run = carry + prev;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (op == SP_ROW_EXCLUSIVE_SCAN) {
                        cdf[c][k] = run;
                        run = run + p[c][k];
                    } else {
                        run = run + p[c][k];
                        cdf[c][k] = run;
                    }
                }
                if (C > 1) carry = carry + group_broadcast<T>(incl, T - 1);
            }
        }

        // ---- inverse-CDF sampling (local_discrete_sampling, ml/primitives.spi:782-798) ----
        int pick = INT_MAX_;
        if (want_sample) {
            float m = NEG_INF;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (p[c][k] > 0.f) m = fmaxf(m, cdf[c][k]);
            m = group_reduce<T>(m, [](float x, float y) { return fmaxf(x, y); });
            const float thr = uu * m;
#pragma unroll
            for (int c = C - 1; c >= 0; --c)
#pragma unroll
                for (int k = 3; k >= 0; --k)
                    if (p[c][k] > 0.f && cdf[c][k] >= thr) pick = c * 4 * T + 4 * l + k;
            pick = group_reduce<T>(pick, [](int x, int y) { return x < y ? x : y; });
        }

        // ---- local_get_prob (ml/primitives.spi:824-830): the mapped value at one column ----
        float got = 0.f;
        if (a.prob_out != nullptr) {
            const int id = a.action != nullptr ? (row_ok ? a.action[row] : 0) : pick;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (ok[c] && c * 4 * T + 4 * l + k == id) got = p[c][k];
            got = group_reduce<T>(got, [](float x, float y) { return x + y; });   // one non-zero term: exact
        }

        // ---- local_binarize (ml/primitives.spi:817-821) ----
        unsigned bits = 0;
        if (a.bits_out != nullptr) {
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int j = c * 4 * T + 4 * l + k;
                    if (ok[c] && j < 32 && !(v[c][k] <= 0.f)) bits |= 1u << j;   // the reference's test: a NaN sets its bit
                }
            bits = group_reduce<T>(bits, [](unsigned x, unsigned y) { return x | y; });
        }

        // ---- stores ----
        float* out_ptr = is_scan ? nullptr : a.out;
        float* cdf_ptr = is_scan ? a.out : a.cdf;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = c * 4 * T + 4 * l;
            if (ok[c]) {
                if (out_ptr != nullptr)
                    store16_through(reinterpret_cast<f32x4*>(out_ptr + row * (long)cols + col),
                                    f32x4{p[c][0], p[c][1], p[c][2], p[c][3]});
                if (cdf_ptr != nullptr)
                    store16_through(reinterpret_cast<f32x4*>(cdf_ptr + row * (long)cols + col),
                                    f32x4{cdf[c][0], cdf[c][1], cdf[c][2], cdf[c][3]});
            }
        }
        if (row_ok && l == 0) {
            if (a.rowmax != nullptr) a.rowmax[row] = bv;
            if (a.rowsum != nullptr) a.rowsum[row] = stat_sum;
            if (a.argmax != nullptr) a.argmax[row] = bi;
            if (a.sample != nullptr) a.sample[row] = pick;
            if (a.u_out != nullptr) a.u_out[row] = uu;
            if (a.prob_out != nullptr) a.prob_out[row] = got;
            if (a.bits_out != nullptr) a.bits_out[row] = bits % a.modulo;
        }
    }
}

// The fused pipeline behind sp_row_ops: softmax of every row plus, each optional, the row max and
// argmax of the input, the sum of exponentials, the probabilities, their running sums and one
// inverse-CDF sample per row.  Same results as row_kernel (the probabilities and running sums
// are computed by the same operations in the same order); what differs is the instruction count:
// padding lanes hold -inf, whose exponential is 0, so no per-element validity tests remain, full
// waves load and store without predicates, and the max reductions are single DPP instructions.
// OPK: the operation, an instantiation each -- 0 plain softmax (sp_row_ops and the plain softmax ops), 1 masked
// softmax, 2 regret matching (masked or not: the mask is the row length then).
template <int T, int C, bool MAT, int OPK>
__device__ __forceinline__ void row_softmax_body(const RowArgs& a) {
    constexpr int ROWS_PER_WAVE = WAVE / T;
    const int lane = threadIdx.x & (WAVE - 1);
    const int l = lane % T;
    const int sub = lane / T;
    const long wave_id = (long)blockIdx.x * (ROW_THREADS / WAVE) + (threadIdx.x / WAVE);
    const long stride = (long)gridDim.x * (ROW_THREADS / WAVE) * ROWS_PER_WAVE;
    const float NEG_INF = -__builtin_inff();
    const int cols = a.cols;
    const bool full_cols = cols == C * 4 * T;

    // Everything that happens to one group of ROWS_PER_WAVE rows once it is in registers.
    auto work = [&](const f32x4 (&v)[C], const float uu, const long row0) {
        const long row = row0 + sub;
        const bool row_ok = row < a.rows;
        const bool full = full_cols && row0 + ROWS_PER_WAVE <= a.rows;   // wave-uniform
        const long base = row * (long)cols + 4 * l;

        float bv = vmax(vmax(v[0][0], v[0][1]), vmax(v[0][2], v[0][3]));
#pragma unroll
        for (int c = 1; c < C; ++c) bv = vmax(bv, vmax(vmax(v[c][0], v[c][1]), vmax(v[c][2], v[c][3])));
        bv = group_max<T>(bv);

        int bi = INT_MAX_;
        if (a.argmax != nullptr) {
#pragma unroll
            for (int c = C - 1; c >= 0; --c)
#pragma unroll
                for (int k = 3; k >= 0; --k)
                    if (v[c][k] == bv) bi = c * 4 * T + 4 * l + k;
            bi = group_reduce<T>(bi, [](int x, int y) { return x < y ? x : y; });
            if (bi == INT_MAX_) bi = 0;   // a row of NaNs: no element equals the max
        }

        float p[C][4];
        float s = 0.f;
        if (OPK == 1) {
            // columns past the mask enter as -inf (their exponential is an exact 0) and the shift is the max of
            // the columns inside the mask, as in row_kernel
            float m = NEG_INF;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    p[c][k] = (c * 4 * T + 4 * l + k < a.mask_size) ? v[c][k] : NEG_INF;
                    m = vmax(m, p[c][k]);
                }
            m = group_max<T>(m);
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = fast_exp(p[c][k] - m);
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
        } else if (OPK == 2) {
            // local_regret_matching (ml/primitives.spi:718-722, masked :761-780), operation for operation as in
            // row_kernel: positive parts over their sum, the uniform distribution over the mask when that sum is 0
            const int limit = a.mask_size;
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = (c * 4 * T + 4 * l + k < limit) ? fmaxf(v[c][k], 0.f) : 0.f;
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            const float inv_len = 1.f / (float)limit;
            const RowDivisor over_s(s);                                  // as in row_kernel: one division per row
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    p[c][k] = (c * 4 * T + 4 * l + k < limit) ? (s != 0.f ? over_s(p[c][k]) : inv_len) : 0.f;
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) {
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = fast_exp(v[c][k] - bv);
                s = (c == 0) ? sum4(p[c]) : s + sum4(p[c]);
            }
        }
        if (OPK != 2) {
            s = group_reduce<T>(s, [](float x, float y) { return x + y; });
            const float inv = 1.f / s;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k) p[c][k] = p[c][k] * inv;
        }

        // Results that are rows themselves leave as soon as they exist, so that neither the
        // probabilities' copy for the store nor the running sums stay in registers.
        if (MAT && a.out != nullptr) {
#pragma unroll
            for (int c = 0; c < C; ++c)
                if (full || (row_ok && c * 4 * T + 4 * l < cols))
                    store16_through(reinterpret_cast<f32x4*>(a.out + base + c * 4 * T), f32x4{p[c][0], p[c][1], p[c][2], p[c][3]});
        }

        const bool want_sample = a.sample != nullptr;
        float first[C], last[C];   // running sum in front of / at the end of this lane's piece of chunk c
        int pick = INT_MAX_;
        if (want_sample || (MAT && a.cdf != nullptr)) {
            float carry = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float incl = group_inclusive_scan<T>(sum4(p[c]), l);
                float prev = dpp_move<0x138>(incl);   // wave_shr:1 = the lane before
                if (l == 0) prev = 0.f;
                float run = carry + prev;
                first[c] = run;
                float r[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    run = run + p[c][k];
                    r[k] = run;
                }
                last[c] = run;
                if (MAT && a.cdf != nullptr && (full || (row_ok && c * 4 * T + 4 * l < cols)))
                    store16_through(reinterpret_cast<f32x4*>(a.cdf + base + c * 4 * T), f32x4{r[0], r[1], r[2], r[3]});
                if (C > 1) carry = carry + group_broadcast_last<T>(incl);
            }
            if (want_sample) {
                // local_discrete_sampling (ml/primitives.spi:782-798): the first index with p > 0 whose
                // running sum reaches u * (largest running sum over p > 0).  Inside one lane and chunk
                // the four running sums never decrease and are > 0 only if some p is (p >= 0), so
                // the largest of them over p > 0 is the last one, provided the chunk's sum is positive.
                float m = NEG_INF;
#pragma unroll
                for (int c = 0; c < C; ++c) m = vmax(m, sum4(p[c]) > 0.f ? last[c] : NEG_INF);
                m = group_max<T>(m);
                const float thr = uu * m;
#pragma unroll
                for (int c = C - 1; c >= 0; --c) {
                    // The running sums are not kept: the same additions in the same order give
                    // the same bits again.
                    float r[4];
                    float run = first[c];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        run = run + p[c][k];
                        r[k] = run;
                    }
#pragma unroll
                    for (int k = 3; k >= 0; --k)
                        if (p[c][k] > 0.f && r[k] >= thr) pick = c * 4 * T + 4 * l + k;
                }
                pick = group_reduce<T>(pick, [](int x, int y) { return x < y ? x : y; });
            }
        }

        // local_get_prob of the sampled column (ml/primitives.spi:824-830): one non-zero term, so the sum is exact
        float got = 0.f;
        if (a.prob_out != nullptr) {
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (c * 4 * T + 4 * l + k == pick) got = p[c][k];
            got = group_reduce<T>(got, [](float x, float y) { return x + y; });
        }
        if (row_ok && l == 0) {
            if (a.rowmax != nullptr) a.rowmax[row] = bv;
            if (a.rowsum != nullptr) a.rowsum[row] = s;
            if (a.argmax != nullptr) a.argmax[row] = bi;
            if (a.sample != nullptr) a.sample[row] = pick;
            if (a.u_out != nullptr) a.u_out[row] = uu;
            if (a.prob_out != nullptr) a.prob_out[row] = got;
        }
    };

    // Whole groups of complete rows: as many 16-byte loads as chunks, none of them predicated.
    auto load_full = [&](long r0, f32x4 (&w)[C], float& uu) {
        const long r = r0 + sub;
        const long b = r * (long)cols + 4 * l;
        // first: whoever waits for a piece of the row then has the uniform too
        // (no uniform tensor and no generator: nothing samples, and no load is issued for it)
        uu = a.philox_mode >= 0 ? reference_row_uniform(a, r) : (a.u != nullptr ? a.u[r] : 1.f);
#pragma unroll
        for (int c = 0; c < C; ++c) w[c] = *reinterpret_cast<const f32x4*>(a.x + b + c * 4 * T);
    };
    // Any group: -inf where the row or the tensor ends.
    auto load_any = [&](long r0, f32x4 (&w)[C], float& uu) {
        const long r = r0 + sub;
        const long b = r * (long)cols + 4 * l;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            w[c] = f32x4{NEG_INF, NEG_INF, NEG_INF, NEG_INF};
            if (r < a.rows && c * 4 * T + 4 * l < cols) w[c] = *reinterpret_cast<const f32x4*>(a.x + b + c * 4 * T);
        }
        uu = r < a.rows ? (a.philox_mode >= 0 ? reference_row_uniform(a, r) : (a.u != nullptr ? a.u[r] : 1.f)) : 1.f;
    };

    // The uniform is requested together with the row: the counter of outstanding loads runs in
    // order, so a load issued in the middle of the work would be waited for with nothing to do.
    const long full_rows = full_cols ? a.rows - a.rows % ROWS_PER_WAVE : 0;
    for (long row0 = wave_id * ROWS_PER_WAVE; row0 < a.rows; row0 += stride) {
        f32x4 v[C];
        float uu;
        // Two copies of the work, so that the common case stays a straight line: merged, the
        // compiler orders the loads of both cases as row, wait, uniform, wait.
        if (row0 < full_rows) {
            load_full(row0, v, uu);
            __builtin_amdgcn_sched_barrier(0);
            work(v, uu, row0);
        } else {
            load_any(row0, v, uu);
            work(v, uu, row0);
        }
    }
}

// The leading scalar parameters of the row kernels repeat fields of `a`: the library is built with kernel-argument
// preloading, which hands the first dwords of scalar parameters to a wave in registers when it starts (a struct is not
// preloaded), so the row's address does not wait for a scalar load from the argument block (~900 cycles).
__device__ __forceinline__ RowArgs with_preloaded(const RowArgs& a, const float* x, const float* u, long rows, int cols) {
    RowArgs b = a;
    b.x = x;
    b.u = u;
    b.rows = rows;
    b.cols = cols;
    return b;
}

// MAT = true: probabilities and/or running sums are written out.
template <int T, int C, int OPK = 0>
__global__ __launch_bounds__(ROW_THREADS) void row_softmax_kernel(const float* x, const float* u, long rows, int cols, const RowArgs a) {
    row_softmax_body<T, C, true, OPK>(with_preloaded(a, x, u, rows, cols));
}

// MAT = false: per-row results only; nothing of the row is written back.
template <int T, int C, int OPK = 0>
__global__ __launch_bounds__(ROW_THREADS) void row_softmax_scalars_kernel(const float* x, const float* u, long rows, int cols,
                                                                         const RowArgs a) {
    row_softmax_body<T, C, false, OPK>(with_preloaded(a, x, u, rows, cols));
}

// Integer rows: identity and exact scans (two's complement wrap-around).
template <int T, int C>
__global__ __launch_bounds__(ROW_THREADS) void row_kernel_i32(const int* __restrict__ x, int* __restrict__ out,
                                                              long rows, int cols, int op) {
    constexpr int ROWS_PER_WAVE = WAVE / T;
    const int lane = threadIdx.x & (WAVE - 1);
    const int l = lane % T;
    const int sub = lane / T;
    const long wave_id = (long)blockIdx.x * (ROW_THREADS / WAVE) + (threadIdx.x / WAVE);
    const long n_waves = (long)gridDim.x * (ROW_THREADS / WAVE);
    for (long row0 = wave_id * ROWS_PER_WAVE; row0 < rows; row0 += n_waves * ROWS_PER_WAVE) {
        const long row = row0 + sub;
        const bool row_ok = row < rows;
        int carry = 0;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = c * 4 * T + 4 * l;
            const bool ok = row_ok && col < cols;
            int4 v = make_int4(0, 0, 0, 0);
            if (ok) v = *reinterpret_cast<const int4*>(x + row * (long)cols + col);
            const int s = ((v.x + v.y) + v.z) + v.w;
            const int incl = group_inclusive_scan<T>(s, l);
            int prev = dpp_move<0x138>(incl);
            if (l == 0) prev = 0;
            const int start = carry + prev;
            int4 r;
            if (op == SP_ROW_EXCLUSIVE_SCAN) {
                r.x = start; r.y = r.x + v.x; r.z = r.y + v.y; r.w = r.z + v.z;
            } else if (op == SP_ROW_INCLUSIVE_SCAN) {
                r.x = start + v.x; r.y = r.x + v.y; r.z = r.y + v.z; r.w = r.z + v.w;
            } else {
                r = v;
            }
            if (ok) *reinterpret_cast<int4*>(out + row * (long)cols + col) = r;
            if (C > 1) carry = carry + group_broadcast<T>(incl, T - 1);
        }
    }
}

// One thread per row: just the uniform the row would draw.
__global__ __launch_bounds__(ROW_THREADS) void philox_uniforms_kernel(const RowArgs a) {
    const long r = (long)blockIdx.x * ROW_THREADS + threadIdx.x;
    if (r < a.rows) a.u_out[r] = reference_row_uniform(a, r);
}

// Cross-entropy-method resampling of one weight position across the ensemble (ml/cem.spi:99-117):
// the row holds that weight for every ensemble member; winners (mask != 0) keep their value, the
// others are redrawn from N(mean, max(std, noise)) of the winners' values, times `decay`.
// z == nullptr: the normals are drawn here -- row r takes the sequence curand_normal yields for (seed, subsequence r)
// from 4-draw group `group0` on, so columns 4 g .. 4 g + 3 come from group group0 + g.
template <int T, int C>
__global__ __launch_bounds__(ROW_THREADS) void cem_kernel(const float* __restrict__ x, const int* __restrict__ mask,
                                                          const float* __restrict__ z, float* __restrict__ out, long rows,
                                                          int cols, float noise, float decay, unsigned long long seed,
                                                          unsigned long long group0) {
    constexpr int ROWS_PER_WAVE = WAVE / T;
    const int lane = threadIdx.x & (WAVE - 1);
    const int l = lane % T;
    const int sub = lane / T;
    const long wave_id = (long)blockIdx.x * (ROW_THREADS / WAVE) + (threadIdx.x / WAVE);
    const long n_waves = (long)gridDim.x * (ROW_THREADS / WAVE);
    for (long row0 = wave_id * ROWS_PER_WAVE; row0 < rows; row0 += n_waves * ROWS_PER_WAVE) {
        const long row = row0 + sub;
        const bool row_ok = row < rows;
        float v[C][4], g[C][4];
        bool win[C][4], ok[C];
        int cnt = 0;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const int col = c * 4 * T + 4 * l;
            ok[c] = row_ok && col < cols;
            f32x4 xv = {0.f, 0.f, 0.f, 0.f}, zv = {0.f, 0.f, 0.f, 0.f};
            int4 mv = make_int4(0, 0, 0, 0);
            if (ok[c]) {
                xv = *reinterpret_cast<const f32x4*>(x + row * (long)cols + col);
                mv = *reinterpret_cast<const int4*>(mask + col);
                if (z != nullptr) {
                    zv = *reinterpret_cast<const f32x4*>(z + row * (long)cols + col);
                } else {
                    unsigned w[4];
                    philox_words(seed, (unsigned long long)row, group0 + (unsigned long long)(col / 4), w);
                    float n0, n1, n2, n3;
                    box_muller(w[0], w[1], n0, n1);
                    box_muller(w[2], w[3], n2, n3);
                    zv = f32x4{n0, n1, n2, n3};
                }
            }
            const int m4[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                v[c][k] = xv[k];
                g[c][k] = zv[k];
                win[c][k] = m4[k] != 0;
                cnt += win[c][k] ? 1 : 0;
            }
        }
        cnt = group_reduce<T>(cnt, [](int a, int b) { return a + b; });
        const float winner_count = (float)cnt;
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int k = 0; k < 4; ++k) s = s + (win[c][k] ? v[c][k] : 0.f);
        s = group_reduce<T>(s, [](float a, float b) { return a + b; });
        const float winner_mean = s / winner_count;
        float q = 0.f;
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float r = v[c][k] - winner_mean;
                q = q + (win[c][k] ? r * r : 0.f);
            }
        q = group_reduce<T>(q, [](float a, float b) { return a + b; });
        const float biased_std = sqrtf(q / winner_count);
        const float winner_std = cnt > 1 ? biased_std * winner_count / (winner_count - 1.f) : 0.f;
        const float scale = fmaxf(winner_std, noise);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (ok[c]) {
                f32x4 o;
#pragma unroll
                for (int k = 0; k < 4; ++k) o[k] = win[c][k] ? v[c][k] : (g[c][k] * scale + winner_mean) * decay;
                *reinterpret_cast<f32x4*>(out + row * (long)cols + c * 4 * T + 4 * l) = o;
            }
        }
    }
}

// grid_update_rewards_mask (ml/cem.spi:92-96) for up to a few thousand ensemble members: one
// workgroup; the average is a sequential f32 sum like the reference's fold.
__global__ __launch_bounds__(ROW_THREADS) void cem_mask_kernel(float* __restrict__ rewards, int* __restrict__ mask, int n) {
    __shared__ float average;
    if (threadIdx.x == 0) {
        float s = 0.f;
        for (int e = 0; e < n; ++e) {
            const float r = rewards[2 * e], c = rewards[2 * e + 1];
            s = s + (c != 0.f ? r / c : 0.f);
        }
        average = s / (float)n;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n; e += ROW_THREADS) {
        const float r = rewards[2 * e], c = rewards[2 * e + 1];
        mask[e] = (c != 0.f ? r / c : 0.f) >= average ? 1 : 0;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 2 * n; e += ROW_THREADS) rewards[e] = 0.f;
}

// Lanes that share a row.  Up to 64 columns: one lane per 4 columns (rounded up to a power of two).
// Up to 256 columns: 16 lanes (one DPP row), each holding one 4-column piece of every 64-column
// chunk, so a wave works on 4 rows at once and no reduction leaves its DPP row.  Wider rows: the
// whole wave, one 4-column piece per 256-column chunk.
static int lanes_per_row(long cols) {
    if (cols > 256) return 64;
    int t = 1;
    while (t * 4 < cols && t < 16) t *= 2;
    return t;
}

#ifndef SP_ROW_BLOCKS_PER_CU
#define SP_ROW_BLOCKS_PER_CU 32     // workgroups per compute unit of the row kernels (a build may override it)
#endif
static int row_grid(long rows, int t) {
    const long rows_per_block = (long)(WAVE / t) * (ROW_THREADS / WAVE);
    long blocks = (rows + rows_per_block - 1) / rows_per_block;
    const long cap = (long)device_cu_count() * SP_ROW_BLOCKS_PER_CU;  // several rounds of short workgroups: the dispatcher evens out the tail
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

template <typename F>
static int dispatch_tc(int t, int c, F&& f) {
    switch (t) {
        case 1: f(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}); return SP_OK;
        case 2: f(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{}); return SP_OK;
        case 4: f(std::integral_constant<int, 4>{}, std::integral_constant<int, 1>{}); return SP_OK;
        case 8: f(std::integral_constant<int, 8>{}, std::integral_constant<int, 1>{}); return SP_OK;
        case 16:
            switch (c) {
                case 1: f(std::integral_constant<int, 16>{}, std::integral_constant<int, 1>{}); return SP_OK;
                case 2: f(std::integral_constant<int, 16>{}, std::integral_constant<int, 2>{}); return SP_OK;
                case 3: f(std::integral_constant<int, 16>{}, std::integral_constant<int, 3>{}); return SP_OK;
                case 4: f(std::integral_constant<int, 16>{}, std::integral_constant<int, 4>{}); return SP_OK;
            }
            break;
        case 64:
            switch (c) {
                case 1: f(std::integral_constant<int, 64>{}, std::integral_constant<int, 1>{}); return SP_OK;
                case 2: f(std::integral_constant<int, 64>{}, std::integral_constant<int, 2>{}); return SP_OK;
                case 3: f(std::integral_constant<int, 64>{}, std::integral_constant<int, 3>{}); return SP_OK;
                case 4: f(std::integral_constant<int, 64>{}, std::integral_constant<int, 4>{}); return SP_OK;
            }
            break;
    }
    return fail(SP_ERR_SHAPE, "row kernels: unsupported lanes/chunks %d/%d", t, c);
}

static int check_rows_cols(const char* fn, int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return fail(SP_ERR_SHAPE, "%s: rows and cols must be positive (got %lld, %lld)", fn,
                                            (long long)rows, (long long)cols);
    if (cols % 4 != 0) return fail(SP_ERR_SHAPE, "%s: cols must be a multiple of 4 (16-byte rows), got %lld", fn,
                                   (long long)cols);
    if (cols > 1024) return fail(SP_ERR_SHAPE, "%s: cols must be <= 1024, got %lld", fn, (long long)cols);
    if (rows > (int64_t)1 << 40) return fail(SP_ERR_SHAPE, "%s: rows too large", fn);
    return SP_OK;
}

template <bool FUSED>
static int launch_row(const RowArgs& args, hipStream_t stream, const char* fn) {
    int rc = require_gfx950(fn);
    if (rc != SP_OK) return rc;
    const RowArgs& a = args;
    const int t = lanes_per_row(a.cols);
    const int c = (int)((a.cols + 4 * t - 1) / (4 * t));
    const int grid = row_grid(a.rows, t);
    rc = dispatch_tc(t, c, [&](auto T_, auto C_) {
        const bool rows_out = a.out != nullptr || a.cdf != nullptr;
        auto fused = [&](auto OPK_) {
            constexpr int OPK = decltype(OPK_)::value;
            if (rows_out)
                hipLaunchKernelGGL((row_softmax_kernel<decltype(T_)::value, decltype(C_)::value, OPK>), dim3(grid),
                                   dim3(ROW_THREADS), 0, stream, a.x, a.u, a.rows, a.cols, a);
            else   // per-row results only: nothing of the row itself is written back
                hipLaunchKernelGGL((row_softmax_scalars_kernel<decltype(T_)::value, decltype(C_)::value, OPK>), dim3(grid),
                                   dim3(ROW_THREADS), 0, stream, a.x, a.u, a.rows, a.cols, a);
        };
        if (FUSED && a.op == SP_ROW_SOFTMAX) fused(std::integral_constant<int, 0>{});
        else if (FUSED && a.op == SP_ROW_MASKED_SOFTMAX) fused(std::integral_constant<int, 1>{});
        else if (FUSED) fused(std::integral_constant<int, 2>{});
        else
            hipLaunchKernelGGL((row_kernel<decltype(T_)::value, decltype(C_)::value>), dim3(grid), dim3(ROW_THREADS), 0,
                               stream, a);
    });
    if (rc != SP_OK) return rc;
    return check_launch(fn);
}

namespace {
struct RowKernelNames {
    RowKernelNames() {
        register_kernel("row_ops", (const void*)row_softmax_kernel<16, 4>, ROW_THREADS);
        register_kernel("row_ops_scalars", (const void*)row_softmax_scalars_kernel<16, 4>, ROW_THREADS);
        register_kernel("row_map", (const void*)row_kernel<16, 4>, ROW_THREADS);
    }
} row_kernel_names;
}  // namespace

}  // namespace sp

using namespace sp;

extern "C" int sp_philox_uniforms(const sp_philox_t* philox, float* u_out, int64_t rows, int64_t cols, void* stream) {
    SP_REQUIRE_PTR(u_out);
    if (philox == nullptr) return fail(SP_ERR_NULL, "sp_philox_uniforms: philox is NULL");
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    RowArgs a{};
    a.rows = rows; a.cols = (int)cols; a.u_out = u_out;
    rc = set_philox(a, philox, rows, cols, __func__);
    if (rc != SP_OK) return rc;
    const long blocks = (rows + ROW_THREADS - 1) / ROW_THREADS;
    if (blocks > 0x7fffffffL) return fail(SP_ERR_SHAPE, "sp_philox_uniforms: rows too large");
    hipLaunchKernelGGL(philox_uniforms_kernel, dim3((unsigned)blocks), dim3(ROW_THREADS), 0, (hipStream_t)stream, a);
    return check_launch(__func__);
}

extern "C" int sp_row_ops(const float* logits, const float* u, float* rowmax, float* rowsum, float* probs, float* cdf,
                          int32_t* argmax, int32_t* sample, int64_t rows, int64_t cols, uint32_t flags, void* stream) {
    if (flags != 0) return fail(SP_ERR_ARG, "sp_row_ops: flags is reserved and must be 0, got %u", flags);
    SP_REQUIRE_PTR(logits);
    SP_OPTIONAL_PTR(rowmax); SP_OPTIONAL_PTR(rowsum); SP_OPTIONAL_PTR(probs); SP_OPTIONAL_PTR(cdf);
    SP_OPTIONAL_PTR(argmax); SP_OPTIONAL_PTR(sample); SP_OPTIONAL_PTR(u);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (sample != nullptr && u == nullptr) return fail(SP_ERR_NULL, "sp_row_ops: sample requested but u is NULL");
    RowArgs a{};
    a.x = logits; a.u = u; a.rowmax = rowmax; a.rowsum = rowsum; a.out = probs; a.cdf = cdf; a.argmax = argmax;
    a.sample = sample; a.rows = rows; a.cols = (int)cols; a.op = SP_ROW_SOFTMAX; a.mask_size = (int)cols;
    a.want_stats = 1; a.philox_mode = -1;
    return launch_row<true>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_row_map_f32(int op, const float* x, float* out, int64_t rows, int64_t cols, int32_t mask_size,
                              void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (op < SP_ROW_IDENTITY || op > SP_ROW_EXCLUSIVE_SCAN) return fail(SP_ERR_ARG, "sp_row_map_f32: unknown op %d", op);
    const bool masked = (op == SP_ROW_MASKED_SOFTMAX || op == SP_ROW_MASKED_REGRET_MATCHING);
    if (masked && (mask_size < 1 || mask_size > cols))
        return fail(SP_ERR_ARG, "sp_row_map_f32: mask_size must be in [1, cols], got %d", mask_size);
    RowArgs a{};
    a.x = x; a.out = out; a.rows = rows; a.cols = (int)cols; a.op = op; a.mask_size = masked ? mask_size : (int)cols;
    a.philox_mode = -1;
    if (op == SP_ROW_SOFTMAX) return launch_row<true>(a, (hipStream_t)stream, __func__);   // the fused kernel's first half
    return launch_row<false>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_row_l1_normalize(const float* x, float* out, int64_t rows, int64_t cols, float threshold, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (!(threshold > 0.f)) return fail(SP_ERR_ARG, "sp_row_l1_normalize: threshold must be positive, got %g", (double)threshold);
    RowArgs a{};
    a.x = x; a.out = out; a.rows = rows; a.cols = (int)cols; a.op = SP_ROW_L1_NORMALIZE; a.mask_size = (int)cols;
    a.threshold = threshold; a.philox_mode = -1;
    return launch_row<false>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_row_sample(int op, const float* x, const float* u, const sp_philox_t* philox, float* probs_out,
                             float* cdf_out, float* u_out, int32_t* sample_out, float* prob_out, int64_t rows,
                             int64_t cols, int32_t mask_size, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(sample_out);
    SP_OPTIONAL_PTR(u); SP_OPTIONAL_PTR(probs_out); SP_OPTIONAL_PTR(cdf_out); SP_OPTIONAL_PTR(u_out);
    SP_OPTIONAL_PTR(prob_out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (!(op == SP_ROW_IDENTITY || op == SP_ROW_SOFTMAX || op == SP_ROW_MASKED_SOFTMAX ||
          op == SP_ROW_REGRET_MATCHING || op == SP_ROW_MASKED_REGRET_MATCHING))
        return fail(SP_ERR_ARG, "sp_row_sample: op %d cannot feed a sampler", op);
    const bool masked = (op == SP_ROW_MASKED_SOFTMAX || op == SP_ROW_MASKED_REGRET_MATCHING);
    if (masked && (mask_size < 1 || mask_size > cols))
        return fail(SP_ERR_ARG, "sp_row_sample: mask_size must be in [1, cols], got %d", mask_size);
    if ((u == nullptr) == (philox == nullptr))
        return fail(SP_ERR_ARG, "sp_row_sample: exactly one of u and philox must be given");
    RowArgs a{};
    a.x = x; a.u = u; a.out = probs_out; a.cdf = cdf_out; a.u_out = u_out; a.sample = sample_out; a.rows = rows;
    a.prob_out = prob_out;
    a.cols = (int)cols; a.op = op; a.mask_size = masked ? mask_size : (int)cols; a.philox_mode = -1;
    if (philox != nullptr) {
        rc = set_philox(a, philox, rows, cols, __func__);
        if (rc != SP_OK) return rc;
    }
    // Softmax and regret-matching sampling, masked or not, is what the fused pipeline does (same operations, same
    // order, same bits as the general kernel).
    if (op != SP_ROW_IDENTITY) return launch_row<true>(a, (hipStream_t)stream, __func__);
    return launch_row<false>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_row_map_i32(int op, const int32_t* x, int32_t* out, int64_t rows, int64_t cols, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (!(op == SP_ROW_IDENTITY || op == SP_ROW_INCLUSIVE_SCAN || op == SP_ROW_EXCLUSIVE_SCAN))
        return fail(SP_ERR_ARG, "sp_row_map_i32: op %d is not an integer op", op);
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const int t = lanes_per_row(cols);
    const int c = (int)((cols + 4 * t - 1) / (4 * t));
    const int grid = row_grid(rows, t);
    rc = dispatch_tc(t, c, [&](auto T_, auto C_) {
        hipLaunchKernelGGL((row_kernel_i32<decltype(T_)::value, decltype(C_)::value>), dim3(grid), dim3(ROW_THREADS), 0,
                           (hipStream_t)stream, x, out, (long)rows, (int)cols, op);
    });
    if (rc != SP_OK) return rc;
    return check_launch(__func__);
}

extern "C" int sp_row_get_prob(int op, const float* x, const int32_t* action, float* prob_out, int64_t rows,
                               int64_t cols, int32_t mask_size, void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(action);
    SP_REQUIRE_PTR(prob_out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (!(op == SP_ROW_IDENTITY || op == SP_ROW_SOFTMAX || op == SP_ROW_MASKED_SOFTMAX ||
          op == SP_ROW_REGRET_MATCHING || op == SP_ROW_MASKED_REGRET_MATCHING || op == SP_ROW_LN_L2))
        return fail(SP_ERR_ARG, "sp_row_get_prob: op %d is not a row map", op);
    const bool masked = (op == SP_ROW_MASKED_SOFTMAX || op == SP_ROW_MASKED_REGRET_MATCHING);
    if (masked && (mask_size < 1 || mask_size > cols))
        return fail(SP_ERR_ARG, "sp_row_get_prob: mask_size must be in [1, cols], got %d", mask_size);
    RowArgs a{};
    a.x = x; a.action = action; a.prob_out = prob_out; a.rows = rows; a.cols = (int)cols; a.op = op;
    a.mask_size = masked ? mask_size : (int)cols; a.philox_mode = -1;
    return launch_row<false>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_row_binarize(const float* x, uint32_t* out, int64_t rows, int64_t cols, uint32_t modulo,
                               void* stream) {
    SP_REQUIRE_PTR(x);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, cols);
    if (rc != SP_OK) return rc;
    if (modulo == 0) return fail(SP_ERR_ARG, "sp_row_binarize: modulo must be positive");
    RowArgs a{};
    a.x = x; a.bits_out = out; a.modulo = modulo; a.rows = rows; a.cols = (int)cols; a.op = SP_ROW_IDENTITY;
    a.mask_size = (int)cols; a.philox_mode = -1;
    return launch_row<false>(a, (hipStream_t)stream, __func__);
}

extern "C" int sp_cem_resample(const float* weights_t, const int32_t* mask, const float* normals, float* out,
                               int64_t rows, int64_t ensemble, float noise, float decay, void* stream) {
    SP_REQUIRE_PTR(weights_t);
    SP_REQUIRE_PTR(mask);
    SP_REQUIRE_PTR(normals);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, ensemble);
    if (rc != SP_OK) return rc;
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const int t = lanes_per_row(ensemble);
    const int c = (int)((ensemble + 4 * t - 1) / (4 * t));
    const int grid = row_grid(rows, t);
    rc = dispatch_tc(t, c, [&](auto T_, auto C_) {
        hipLaunchKernelGGL((cem_kernel<decltype(T_)::value, decltype(C_)::value>), dim3(grid), dim3(ROW_THREADS), 0,
                           (hipStream_t)stream, weights_t, mask, normals, out, (long)rows, (int)ensemble, noise, decay,
                           0ull, 0ull);
    });
    if (rc != SP_OK) return rc;
    return check_launch(__func__);
}

extern "C" int sp_cem_resample_philox(const float* weights_t, const int32_t* mask, uint64_t seed, uint64_t offset, float* out,
                                      int64_t rows, int64_t ensemble, float noise, float decay, void* stream) {
    SP_REQUIRE_PTR(weights_t);
    SP_REQUIRE_PTR(mask);
    SP_REQUIRE_PTR(out);
    int rc = check_rows_cols(__func__, rows, ensemble);
    if (rc != SP_OK) return rc;
    if (offset % 4 != 0) return fail(SP_ERR_ARG, "sp_cem_resample_philox: offset must be a multiple of 4 draws, got %llu",
                                     (unsigned long long)offset);
    rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    const int t = lanes_per_row(ensemble);
    const int c = (int)((ensemble + 4 * t - 1) / (4 * t));
    const int grid = row_grid(rows, t);
    rc = dispatch_tc(t, c, [&](auto T_, auto C_) {
        hipLaunchKernelGGL((cem_kernel<decltype(T_)::value, decltype(C_)::value>), dim3(grid), dim3(ROW_THREADS), 0,
                           (hipStream_t)stream, weights_t, mask, (const float*)nullptr, out, (long)rows, (int)ensemble, noise,
                           decay, (unsigned long long)seed, (unsigned long long)(offset / 4));
    });
    if (rc != SP_OK) return rc;
    return check_launch(__func__);
}

// ---- one reduction per row: out[r] = map_out(reduce over j of map_in(x[r, j])) ----
// T lanes share a row (any width that is a multiple of 4: a lane walks its 4-column pieces 4 T columns apart), each
// folds its own elements in order, then the lanes' results meet in a butterfly; the order of a float sum depends on
// the width only.
template <int OP>
__device__ __forceinline__ float reduce_op(float a, float b) {
    if constexpr (OP == SP_REDUCE_SUM || OP == SP_REDUCE_AVERAGE) return a + b;
    else if constexpr (OP == SP_REDUCE_PROD) return a * b;
    else if constexpr (OP == SP_REDUCE_MAX) return fmaxf(a, b);
    else return fminf(a, b);
}

template <int T, int OP>
__global__ __launch_bounds__(ROW_THREADS) void row_reduce_kernel(const float* __restrict__ x, float* __restrict__ out, long rows,
                                                                 long cols, int map_in, int map_out) {
    constexpr int ROWS_PER_WAVE = WAVE / T;
    const float neutral = OP == SP_REDUCE_PROD ? 1.f : OP == SP_REDUCE_MAX ? -__builtin_inff() : OP == SP_REDUCE_MIN ? __builtin_inff() : 0.f;
    const int lane = threadIdx.x & (WAVE - 1);
    const int l = lane % T, sub = lane / T;
    const long wave_id = (long)blockIdx.x * (ROW_THREADS / WAVE) + (threadIdx.x / WAVE);
    const long n_waves = (long)gridDim.x * (ROW_THREADS / WAVE);
    for (long row0 = wave_id * ROWS_PER_WAVE; row0 < rows; row0 += n_waves * ROWS_PER_WAVE) {
        const long row = row0 + sub;
        float acc = neutral;
        if (row < rows) {
            const float* xr = x + row * cols;
            for (long col = 4 * l; col < cols; col += 4 * T) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(xr + col);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float e = v[k];
                    if (map_in == SP_MAP_IN_SQUARE) e = e * e;
                    else if (map_in == SP_MAP_IN_ABS) e = fabsf(e);
                    acc = reduce_op<OP>(acc, e);
                }
            }
        }
        acc = group_reduce<T>(acc, [](float a, float b) { return reduce_op<OP>(a, b); });
        if (OP == SP_REDUCE_AVERAGE) acc = acc / (float)cols;
        if (map_out == SP_MAP_OUT_SQRT) acc = sqrtf(acc);
        if (row < rows && l == 0) out[row] = acc;
    }
}

template <int OP>
static int launch_row_reduce(const float* x, float* out, int64_t rows, int64_t cols, int map_in, int map_out, hipStream_t stream) {
    int t = 1;
    while (t * 4 < cols && t < 64) t *= 2;
    const int grid = row_grid(rows, t);
#define SP_ROW_REDUCE_T(TT)                                                                                             \
    case TT: hipLaunchKernelGGL((row_reduce_kernel<TT, OP>), dim3(grid), dim3(ROW_THREADS), 0, stream, x, out, (long)rows,  \
                                (long)cols, map_in, map_out); break;
    switch (t) {
        SP_ROW_REDUCE_T(1) SP_ROW_REDUCE_T(2) SP_ROW_REDUCE_T(4) SP_ROW_REDUCE_T(8) SP_ROW_REDUCE_T(16) SP_ROW_REDUCE_T(32)
        SP_ROW_REDUCE_T(64)
    }
#undef SP_ROW_REDUCE_T
    return check_launch("sp_row_reduce_f32");
}

extern "C" int sp_row_reduce_f32(int op, int map_in, int map_out, const float* x, float* out, int64_t rows, int64_t cols,
                                 void* stream) {
    SP_REQUIRE_PTR(x);
    if (out == nullptr) return fail(SP_ERR_NULL, "sp_row_reduce_f32: out is NULL");
    if (rows <= 0 || cols <= 0 || cols % 4 != 0)
        return fail(SP_ERR_SHAPE, "sp_row_reduce_f32: rows must be positive and cols a positive multiple of 4 (got %lld, %lld)",
                    (long long)rows, (long long)cols);
    if (rows > (int64_t)1 << 40 || cols > (int64_t)1 << 40) return fail(SP_ERR_SHAPE, "sp_row_reduce_f32: tensor too large");
    if (map_in < SP_MAP_IN_IDENTITY || map_in > SP_MAP_IN_ABS) return fail(SP_ERR_ARG, "sp_row_reduce_f32: unknown map_in %d", map_in);
    if (map_out < SP_MAP_OUT_IDENTITY || map_out > SP_MAP_OUT_SQRT) return fail(SP_ERR_ARG, "sp_row_reduce_f32: unknown map_out %d", map_out);
    if (op < SP_REDUCE_SUM || op > SP_REDUCE_AVERAGE) return fail(SP_ERR_ARG, "sp_row_reduce_f32: unknown op %d", op);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (op) {
        case SP_REDUCE_SUM: return launch_row_reduce<SP_REDUCE_SUM>(x, out, rows, cols, map_in, map_out, s);
        case SP_REDUCE_PROD: return launch_row_reduce<SP_REDUCE_PROD>(x, out, rows, cols, map_in, map_out, s);
        case SP_REDUCE_MAX: return launch_row_reduce<SP_REDUCE_MAX>(x, out, rows, cols, map_in, map_out, s);
        case SP_REDUCE_MIN: return launch_row_reduce<SP_REDUCE_MIN>(x, out, rows, cols, map_in, map_out, s);
        default: return launch_row_reduce<SP_REDUCE_AVERAGE>(x, out, rows, cols, map_in, map_out, s);
    }
}

extern "C" int sp_cem_update_mask(float* rewards, int32_t* mask, int64_t ensemble, void* stream) {
    SP_REQUIRE_PTR(rewards);
    SP_REQUIRE_PTR(mask);
    if (ensemble <= 0 || ensemble > 65536)
        return fail(SP_ERR_SHAPE, "sp_cem_update_mask: ensemble must be in [1, 65536], got %lld", (long long)ensemble);
    int rc = require_gfx950(__func__);
    if (rc != SP_OK) return rc;
    hipLaunchKernelGGL(cem_mask_kernel, dim3(1), dim3(ROW_THREADS), 0, (hipStream_t)stream, rewards, mask, (int)ensemble);
    return check_launch(__func__);
}
