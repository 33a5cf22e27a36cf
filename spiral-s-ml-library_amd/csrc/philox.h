// Device-side Philox4_32_10 with cuRAND's conventions, and which draw of which stream a sampled row uses: shared by
// the row kernels (row_ops.hip) and the heads of the fused dense-stack kernels (mlp*.hip).
#pragma once
#include "common.h"

#pragma clang fp contract(off)

namespace sp {

// The stream description as the kernels carry it; RowArgs (row_ops.hip) has the same fields under the same names,
// and the functions below take either.
struct PhiloxStream {
    unsigned long long seed;
    unsigned long long draw_offset;
    unsigned long long member_draws;   // extra draw offset per run
    long member_rows;                  // 0: one run; else the rows are stacked runs of member_rows rows each
    int philox_mode;                   // sp_philox_mode, -1: none
    int tpb;
    int blocks;
    int rows_per_block;
    int cols;                          // width of the rows the sampling op works on
};

#ifdef __HIPCC__
// Philox4x32-10 (Salmon et al., SC'11) with cuRAND's counter layout: key = seed, counter =
// (group, 0, subsequence_lo, subsequence_hi); returns word `word` of the group, mapped to (0, 1]
// like curand_uniform (corecuda/random.spi:22-32,84).
__device__ __forceinline__ void philox_words(unsigned long long seed, unsigned long long subsequence,
                                             unsigned long long group, unsigned (&w)[4]) {
    unsigned c0 = (unsigned)group, c1 = (unsigned)(group >> 32), c2 = (unsigned)subsequence,
             c3 = (unsigned)(subsequence >> 32);
    unsigned k0 = (unsigned)seed, k1 = (unsigned)(seed >> 32);
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        if (r) {
            k0 += 0x9E3779B9u;
            k1 += 0xBB67AE85u;
        }
        unsigned hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        unsigned hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        unsigned n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    }
    w[0] = c0; w[1] = c1; w[2] = c2; w[3] = c3;
}

__device__ __forceinline__ float philox_uniform(unsigned long long seed, unsigned long long subsequence,
                                                unsigned long long group, int word) {
    unsigned w[4];
    philox_words(seed, subsequence, group, w);
    const unsigned v = word == 0 ? w[0] : word == 1 ? w[1] : word == 2 ? w[2] : w[3];
    return (float)v * 2.3283064e-10f + 1.1641532e-10f;
}

// Which (subsequence, 4-word group) the reference's sampling op uses for row r: every thread of
// the row draws once per element it holds and the draw attached to column 0 wins
// (ml/primitives.spi:786-791), i.e. the first draw of the row's lane 0 in that row-iteration.
template <typename A>
__device__ __forceinline__ float reference_row_uniform(const A& a, long r) {
    unsigned long long draw_offset = a.draw_offset;
    if (a.member_rows > 0) {              // stacked runs (ensemble members): each restarts the row walk, later in the stream
        draw_offset += (unsigned long long)(r / a.member_rows) * a.member_draws;
        r = r % a.member_rows;
    }
    const long t = a.cols / 4;            // threads per row in the reference
    const long per_iter = a.tpb / t;      // rows per block-iteration
    unsigned long long sub, group;
    if (a.philox_mode == SP_PHILOX_BLOCK) {
        sub = (r % per_iter) * t;
        group = r / per_iter;
    } else if (a.philox_mode == SP_PHILOX_GRID) {
        const long it = r / per_iter;
        sub = (it % a.blocks) * a.tpb + (r % per_iter) * t;
        group = it / a.blocks;
    } else if (a.philox_mode == SP_PHILOX_GATHER) {  // row r belongs to thread r
        const long lt = r % a.tpb;
        sub = (r / a.tpb) * a.tpb + (lt % per_iter) * t;
        group = lt / per_iter;
    } else {  // SP_PHILOX_LAYER: block b = r / rows_per_block walks its own slice (ml/layers.spi:339-344)
        const long b = r / a.rows_per_block, rb = r % a.rows_per_block;
        sub = b * a.tpb + (rb % per_iter) * t;
        group = rb / per_iter;
    }
    // the generator is `draw_offset` draws in; this row uses the first draw of its 4-draw group
    return philox_uniform(a.seed, sub, group + draw_offset / 4, (int)(draw_offset % 4));
}

#endif

// Checks an sp_philox_t against the tensor it is to draw for and copies it into the kernel's argument block.
template <typename A>
inline int set_philox(A& a, const sp_philox_t* philox, int64_t rows, int64_t cols, const char* fn) {
    if (philox->mode < SP_PHILOX_BLOCK || philox->mode > SP_PHILOX_LAYER)
        return fail(SP_ERR_ARG, "%s: unknown philox mode %d", fn, philox->mode);
    const int64_t t = cols / 4;
    if (philox->threads_per_block <= 0 || philox->threads_per_block % t != 0)
        return fail(SP_ERR_ARG, "%s: threads_per_block (%d) must be a positive multiple of cols/4 (%lld)", fn,
                    philox->threads_per_block, (long long)t);
    if (philox->mode == SP_PHILOX_GRID && philox->blocks_per_grid <= 0)
        return fail(SP_ERR_ARG, "%s: blocks_per_grid must be positive", fn);
    if (philox->member_rows < 0 || (philox->member_rows > 0 && rows % philox->member_rows != 0))
        return fail(SP_ERR_ARG, "%s: member_rows (%lld) must divide rows (%lld)", fn, (long long)philox->member_rows,
                    (long long)rows);
    const int64_t run_rows = philox->member_rows > 0 ? philox->member_rows : rows;
    if (philox->mode == SP_PHILOX_LAYER && (philox->rows_per_block <= 0 || run_rows % philox->rows_per_block != 0))
        return fail(SP_ERR_ARG, "%s: rows_per_block (%d) must be positive and divide the rows of a run (%lld)", fn,
                    philox->rows_per_block, (long long)run_rows);
    a.seed = philox->seed; a.philox_mode = philox->mode; a.tpb = philox->threads_per_block;
    a.blocks = philox->blocks_per_grid; a.rows_per_block = philox->rows_per_block;
    a.draw_offset = philox->offset;
    a.member_rows = philox->member_rows;
    a.member_draws = philox->member_draws;
    return SP_OK;
}


}  // namespace sp
